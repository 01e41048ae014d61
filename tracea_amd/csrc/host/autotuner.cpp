// Candidate generation and the AutoTuner.
//
// Reference behaviour kept (src/optimizer/mod.rs:625-760, src/core/tuning.rs:92-139):
// optimize / optimize_conv adapt their problem to optimize_v2, which asks the
// policy for candidates and hands them to the cache's get_or_tune: cached key
// -> cached config; otherwise every candidate is measured, the best TFLOP/s
// wins and is persisted at once.  optimize_guided is the budgeted, surrogate-
// driven loop that the reference keeps as an unused sketch (mod.rs:776-838).
#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdio>

#include "dispatch.hpp"
#include "tuner.hpp"
#include "tuning_cache.hpp"

namespace tracea_amd {

// ---- SearchSpace -------------------------------------------------------------------
std::vector<PipelineConfig> SearchSpace::enumerate() const {
  const PipelineConfig dflt;
  auto axis = [](const std::vector<uint32_t> &v, uint32_t d) {
    return v.empty() ? std::vector<uint32_t>{d} : v;
  };
  const auto tm = axis(tile_m_, dflt.m_tile), tn = axis(tile_n_, dflt.n_tile), tk = axis(tile_k_, dflt.k_tile);
  const auto ws = axis(warps_, 4), st = axis(stages_, dflt.num_stages), ku = axis(k_unroll_, dflt.k_unroll);
  const auto pf = axis(prefetch_distance_, dflt.prefetch_distance), mm = axis(micro_m_, dflt.micro_m);
  const std::vector<std::string> none{"None"};
  const auto &sw = swizzles_.empty() ? none : swizzles_;
  const auto &bm = barrier_modes_.empty() ? none : barrier_modes_;
  std::vector<PipelineConfig> out;
  for (uint32_t mt : tm)
    for (uint32_t nt : tn)
      for (uint32_t kt : tk)
        for (uint32_t w : ws)
          for (uint32_t s : st)
            for (const auto &swz : sw)
              for (const auto &bar : bm)
                for (uint32_t u : ku)
                  for (uint32_t p : pf)
                    for (uint32_t mi : mm) {
                      PipelineConfig c(s, mt, nt, kt);
                      c.has_force_num_warps = true;
                      c.force_num_warps = w;
                      c.instruction = use_tensor_core_ ? "RocmMFMA" : "None";
                      c.swizzle_mode = swz;
                      c.barrier_mode = bar;
                      c.k_unroll = u;
                      c.prefetch_distance = p;
                      c.micro_m = mi;
                      if (s > 2) c.cp_async_distance = s - 1;
                      out.push_back(c);
                    }
  return out;
}

// ---- candidates --------------------------------------------------------------------
namespace {
std::vector<PipelineConfig> propose_contraction(uint32_t m, uint32_t n, uint32_t k, bool conv) {
  std::vector<PipelineConfig> out;
  const HardwareProfile hw = HardwareProfile::mi355x();
  const int pick = select_contraction_variant((int)m, (int)n, (int)k, conv);
  if (pick >= 0) out.push_back(config_for_contraction_variant(pick));
  for (int i = 0; i < contraction_variant_count(); ++i) {
    if (i == pick) continue;
    const ContractionVariant &v = contraction_variant(i);
    if (v.lds_bytes > hw.shared_memory_per_block) continue;
    if (v.pipeline >= 4 && !conv) continue;  // patch-resident kernels compute convolutions only
    out.push_back(config_for_contraction_variant(i));
  }
  return out;
}
}  // namespace

std::vector<PipelineConfig> propose_gemm_configs(uint32_t m, uint32_t n, uint32_t k) {
  return propose_contraction(m, n, k, false);
}

std::vector<PipelineConfig> propose_conv_configs(uint32_t m, uint32_t n, uint32_t k) {
  return propose_contraction(m, n, k, true);
}

std::vector<PipelineConfig> propose_attention_configs(uint32_t head_dim) {
  std::vector<PipelineConfig> out;
  char tag[16];
  snprintf(tag, sizeof(tag), "_d%u_", head_dim);
  for (int i = 0; i < attention_variant_count(); ++i)
    if (std::string(attention_variant(i).name).find(tag) != std::string::npos)
      out.push_back(config_for_attention_variant(i));
  return out;
}

// ---- AutoTuner ---------------------------------------------------------------------
const char *magic_number_strategy_for(uint64_t divisor) {
  if (divisor > 0 && (divisor & (divisor - 1)) == 0) return "PowerOfTwo";
  if (divisor <= 65535) return "FastSmall";
  return "Standard";
}

std::string gemm_cache_key(uint64_t m, uint64_t n, uint64_t k, const std::string &device) {
  char buf[96];
  snprintf(buf, sizeof(buf), "gemm_%llu_%llu_%llu_", (unsigned long long)m, (unsigned long long)n,
           (unsigned long long)k);
  return buf + device;
}

std::string conv_cache_key(const ConvProblem &p, const std::string &device) {
  char buf[160];
  snprintf(buf, sizeof(buf), "conv_%u_%u_%u_%u_%u_%u_%u_%u_%u_", p.batch, p.h_in, p.w_in, p.c_in, p.c_out,
           p.kernel_h, p.kernel_w, p.stride, p.pad);
  return buf + device;
}

AutoTuner::AutoTuner(const HardwareProfile &profile) : gpu(profile), hardware_id(profile.name) {}

PipelineConfig AutoTuner::optimize_v2(const std::string &key, const std::vector<PipelineConfig> &candidates,
                                      const MeasureFn &measure) {
  if (candidates.empty()) return PipelineConfig(2, 64, 64, 32);
  if (key.empty()) return candidates.front();
  CacheEntry hit;
  if (tuning_cache_get(key, &hit)) {
    has_best = true;
    best_config = hit.config;
    best_score = hit.score;
    return hit.config;
  }
  PipelineConfig best = candidates.front();
  float max_score = 0.0f;
  for (const PipelineConfig &c : candidates) {
    const float score = measure(c);
    stats.total_trials += 1;
    if (score > max_score) {
      max_score = score;
      best = c;
    }
  }
  CacheEntry e;
  e.config = best;
  e.score = max_score;
  e.timestamp = (uint64_t)std::chrono::duration_cast<std::chrono::seconds>(
                    std::chrono::system_clock::now().time_since_epoch())
                    .count();
  tuning_cache_put(key, e, true);
  has_best = true;
  best_config = best;
  best_score = max_score;
  return best;
}

PipelineConfig AutoTuner::optimize(uint32_t m, uint32_t n, uint32_t k, const MeasureFn &measure,
                                   const Json &epilogue) {
  PipelineConfig c = optimize_v2(gemm_cache_key(m, n, k, hardware_id), propose_gemm_configs(m, n, k), measure);
  c.epilogue = epilogue;
  return c;
}

ConvConfig AutoTuner::optimize_conv(const ConvProblem &p, const MeasureFn &measure) {
  const uint32_t m = p.batch * p.h_out() * p.w_out();
  const uint32_t kk = p.c_in * p.kernel_h * p.kernel_w;
  ConvConfig out;
  out.magic_strategy = magic_number_strategy_for((uint64_t)p.h_out() * p.w_out());
  out.base = optimize_v2(conv_cache_key(p, hardware_id), propose_conv_configs(m, p.c_out, kk), measure);
  return out;
}

PipelineConfig AutoTuner::optimize_guided(uint32_t m, uint32_t n, uint32_t k,
                                          const std::vector<PipelineConfig> &candidates,
                                          const MeasureFn &measure, size_t iterations, AcquisitionFunction acq,
                                          uint64_t seed) {
  if (candidates.empty()) return PipelineConfig(2, 64, 64, 32);
  std::vector<int> open;  // candidates still unmeasured and not pruned
  for (size_t i = 0; i < candidates.size(); ++i) {
    const std::string reason = gpu.check_feasibility(candidates[i], m);
    if (!reason.empty()) {
      stats.log_pruning(reason);
      continue;
    }
    open.push_back((int)i);
  }
  PipelineConfig best = candidates.front();
  float best_y = 0.0f;
  uint64_t rng = seed;
  for (size_t it = 0; it < iterations && !open.empty(); ++it) {
    size_t pick = 0;
    float pick_score = -1e30f;
    for (size_t j = 0; j < open.size(); ++j) {
      const PipelineConfig &c = candidates[open[j]];
      float s;
      switch (acq) {
        case AcquisitionFunction::UCB: s = gp.ucb(m, n, k, c, gpu); break;
        case AcquisitionFunction::Thompson: s = gp.thompson_sample(m, n, k, c, gpu, &rng); break;
        default: s = gp.expected_improvement(m, n, k, c, best_y, gpu); break;
      }
      if (s > pick_score) {
        pick_score = s;
        pick = j;
      }
    }
    const PipelineConfig &c = candidates[open[pick]];
    const float y = measure(c);
    stats.total_trials += 1;
    Observation o;
    o.m = m; o.n = n; o.k = k;
    o.config = c;
    o.score = y > 0.0f ? y : 0.0f;
    gp.observe(o, gpu);
    if (y > best_y) {
      best_y = y;
      best = c;
    }
    open.erase(open.begin() + (long)pick);
  }
  has_best = true;
  best_config = best;
  best_score = best_y;
  return best;
}

float AutoTuner::calculate_score(float tflops, float latency_ms, OptimizationGoal goal, float tflops_weight) {
  const float latency_score = 1000.0f / std::max(latency_ms, 1e-6f);
  switch (goal) {
    case OptimizationGoal::MinimizeLatency: return latency_score;
    case OptimizationGoal::Balanced: return tflops * tflops_weight + latency_score * (1.0f - tflops_weight);
    default: return tflops;
  }
}

}  // namespace tracea_amd
