// C entry points of include/tracea_tuner.h: JSON in, JSON out, over the host
// tuner classes.  Exceptions never cross the boundary.
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <limits>

#include "host/dispatch.hpp"
#include "host/tuner.hpp"
#include "host/tuning_cache.hpp"
#include "tracea_tuner.h"

using namespace tracea_amd;

struct TraceaGaussianProcess {
  GaussianProcess gp;
};

namespace {

bool parse_config(const char *text, PipelineConfig *out) {
  if (text == nullptr) {
    fail(TRACEA_INVALID_PARAMS, "config JSON is NULL");
    return false;
  }
  std::string err;
  if (!PipelineConfig::from_json(text, out, &err)) {
    fail(TRACEA_INVALID_PARAMS, "config JSON: %s", err.c_str());
    return false;
  }
  return true;
}

bool parse_profile(const char *name, HardwareProfile *out) {
  if (name == nullptr || !HardwareProfile::by_name(name, out)) {
    fail(TRACEA_INVALID_PARAMS, "unknown hardware profile '%s'", name ? name : "(null)");
    return false;
  }
  return true;
}

bool parse_candidates(const char *text, std::vector<PipelineConfig> *out) {
  if (text == nullptr) {
    fail(TRACEA_INVALID_PARAMS, "candidate list is NULL");
    return false;
  }
  Json root;
  std::string err;
  if (!Json::parse(text, &root, &err) || root.type != Json::Array) {
    fail(TRACEA_INVALID_PARAMS, "candidate list must be a JSON array: %s", err.c_str());
    return false;
  }
  for (const Json &j : root.arr) {
    PipelineConfig c;
    if (!PipelineConfig::from_json_value(j, &c, &err)) {
      fail(TRACEA_INVALID_PARAMS, "candidate %zu: %s", out->size(), err.c_str());
      return false;
    }
    out->push_back(c);
  }
  return true;
}

char *configs_to_json(const std::vector<PipelineConfig> &v) {
  Json arr = Json::make_arr();
  for (const PipelineConfig &c : v) arr.arr.push_back(c.to_json_value());
  return dup_cstr(arr.dump());
}

int32_t copy_floats(const std::vector<float> &v, float *out, int32_t capacity) {
  if (out != nullptr)
    for (int32_t i = 0; i < capacity && (size_t)i < v.size(); ++i) out[i] = v[(size_t)i];
  return (int32_t)v.size();
}

std::vector<uint32_t> number_list(const Json &obj, const char *key) {
  std::vector<uint32_t> v;
  if (const Json *a = obj.find(key))
    if (a->type == Json::Array)
      for (const Json &e : a->arr)
        if (e.type == Json::Number) v.push_back((uint32_t)e.num);
  return v;
}

std::vector<std::string> string_list(const Json &obj, const char *key, bool *present) {
  std::vector<std::string> v;
  *present = false;
  if (const Json *a = obj.find(key))
    if (a->type == Json::Array) {
      *present = true;
      for (const Json &e : a->arr)
        if (e.type == Json::String) v.push_back(e.str);
    }
  return v;
}

MeasureFn wrap_measure(TraceaMeasureFn fn, void *user) {
  return [fn, user](const PipelineConfig &c) -> float {
    const std::string text = c.to_json();
    return fn(text.c_str(), user);
  };
}

const float kNaN = std::numeric_limits<float>::quiet_NaN();

}  // namespace

#define TUNER_GUARDED(fallback, ...)                                   \
  try {                                                                \
    __VA_ARGS__                                                        \
  } catch (const std::exception &e) {                                  \
    fail(TRACEA_UNKNOWN_ERROR, "internal error: %s", e.what());        \
    return fallback;                                                   \
  } catch (...) {                                                      \
    fail(TRACEA_UNKNOWN_ERROR, "internal error");                      \
    return fallback;                                                   \
  }

#pragma GCC visibility push(default)
extern "C" {

// ---- PipelineConfig ----------------------------------------------------------------
char *tracea_pipeline_config_new(uint32_t num_stages, uint32_t m_tile, uint32_t n_tile, uint32_t k_tile) {
  TUNER_GUARDED(nullptr, return dup_cstr(PipelineConfig(num_stages, m_tile, n_tile, k_tile).to_json());)
}

char *tracea_pipeline_config_normalize(const char *config_json) {
  TUNER_GUARDED(nullptr, PipelineConfig c; if (!parse_config(config_json, &c)) return nullptr;
                return dup_cstr(c.to_json());)
}

int32_t tracea_pipeline_config_validate(const char *config_json, char **message) {
  TUNER_GUARDED(-1, if (message) *message = nullptr; PipelineConfig c;
                if (!parse_config(config_json, &c)) return -1; const std::string why = c.validate();
                if (why.empty()) return 0; if (message) *message = dup_cstr(why); return 1;)
}

int32_t tracea_pipeline_config_to_vector(const char *config_json, float *out, int32_t capacity) {
  TUNER_GUARDED(-1, PipelineConfig c; if (!parse_config(config_json, &c)) return -1;
                return copy_floats(c.to_vector(), out, capacity);)
}

// ---- HardwareProfile ---------------------------------------------------------------
char *tracea_hardware_profile_json(const char *profile) {
  TUNER_GUARDED(nullptr, HardwareProfile hw; if (!parse_profile(profile, &hw)) return nullptr;
                return dup_cstr(hw.to_json_value().dump());)
}

int32_t tracea_check_feasibility(const char *profile, const char *config_json, uint64_t m, char **reason) {
  TUNER_GUARDED(-1, if (reason) *reason = nullptr; HardwareProfile hw; PipelineConfig c;
                if (!parse_profile(profile, &hw) || !parse_config(config_json, &c)) return -1;
                const std::string why = hw.check_feasibility(c, m); if (why.empty()) return 0;
                if (reason) *reason = dup_cstr(why); return 1;)
}

float tracea_estimate_occupancy(const char *profile, const char *config_json) {
  TUNER_GUARDED(-1.0f, HardwareProfile hw; PipelineConfig c;
                if (!parse_profile(profile, &hw) || !parse_config(config_json, &c)) return -1.0f;
                return hw.estimate_occupancy(c);)
}

// ---- GaussianProcess ---------------------------------------------------------------
TraceaGaussianProcess *tracea_gp_create(void) {
  TUNER_GUARDED(nullptr, return new TraceaGaussianProcess();)
}

void tracea_gp_destroy(TraceaGaussianProcess *gp) { delete gp; }

void tracea_gp_set_noise_sigma(TraceaGaussianProcess *gp, float sigma) {
  if (gp) gp->gp.noise_sigma = sigma;
}

void tracea_gp_set_exploration_beta(TraceaGaussianProcess *gp, float beta) {
  if (gp) gp->gp.exploration_beta = beta;
}

int32_t tracea_gp_observe(TraceaGaussianProcess *gp, uint32_t m, uint32_t n, uint32_t k,
                          const char *config_json, float score, const char *profile) {
  TUNER_GUARDED(-1, HardwareProfile hw; Observation o;
                if (gp == nullptr || m == 0 || n == 0 || k == 0) {
                  fail(TRACEA_INVALID_PARAMS, "gp_observe: NULL handle or zero dimension");
                  return -1;
                } if (!parse_profile(profile, &hw) || !parse_config(config_json, &o.config)) return -1;
                o.m = m; o.n = n; o.k = k; o.score = score; gp->gp.observe(o, hw); return 0;)
}

int32_t tracea_gp_predict(const TraceaGaussianProcess *gp, uint32_t m, uint32_t n, uint32_t k,
                          const char *config_json, const char *profile, float *mean, float *stddev) {
  TUNER_GUARDED(-1, HardwareProfile hw; PipelineConfig c;
                if (gp == nullptr || mean == nullptr || stddev == nullptr || m == 0 || n == 0 || k == 0) {
                  fail(TRACEA_INVALID_PARAMS, "gp_predict: NULL argument or zero dimension");
                  return -1;
                } if (!parse_profile(profile, &hw) || !parse_config(config_json, &c)) return -1;
                gp->gp.predict(m, n, k, c, hw, mean, stddev); return 0;)
}

float tracea_gp_acquisition(const TraceaGaussianProcess *gp, int32_t kind, uint32_t m, uint32_t n, uint32_t k,
                            const char *config_json, const char *profile, float best_y, uint64_t seed) {
  TUNER_GUARDED(kNaN, HardwareProfile hw; PipelineConfig c;
                if (gp == nullptr || m == 0 || n == 0 || k == 0 || kind < 0 || kind > 2) {
                  fail(TRACEA_INVALID_PARAMS, "gp_acquisition: bad argument");
                  return kNaN;
                } if (!parse_profile(profile, &hw) || !parse_config(config_json, &c)) return kNaN;
                if (kind == 0) return gp->gp.expected_improvement(m, n, k, c, best_y, hw);
                if (kind == 1) return gp->gp.ucb(m, n, k, c, hw);
                uint64_t state = seed; return gp->gp.thompson_sample(m, n, k, c, hw, &state);)
}

float tracea_gp_marginal_log_likelihood(const TraceaGaussianProcess *gp, const char *profile) {
  TUNER_GUARDED(kNaN, HardwareProfile hw; if (gp == nullptr || !parse_profile(profile, &hw)) return kNaN;
                return gp->gp.marginal_log_likelihood(hw);)
}

void tracea_gp_optimize_hyperparams(TraceaGaussianProcess *gp, const char *profile) {
  TUNER_GUARDED(, HardwareProfile hw; if (gp == nullptr || !parse_profile(profile, &hw)) return;
                gp->gp.optimize_hyperparams(hw);)
}

int32_t tracea_gp_length_scales(const TraceaGaussianProcess *gp, float *out, int32_t capacity) {
  if (gp == nullptr) return -1;
  return copy_floats(gp->gp.length_scales, out, capacity);
}

int32_t tracea_gp_features(uint32_t m, uint32_t n, uint32_t k, const char *config_json, float *out,
                           int32_t capacity) {
  TUNER_GUARDED(-1, PipelineConfig c; if (m == 0 || n == 0 || k == 0 || !parse_config(config_json, &c)) return -1;
                return copy_floats(GaussianProcess::full_features(m, n, k, c), out, capacity);)
}

float tracea_gp_roofline_prior(uint32_t m, uint32_t n, uint32_t k, const char *config_json,
                               const char *profile) {
  TUNER_GUARDED(kNaN, HardwareProfile hw; PipelineConfig c;
                if (!parse_profile(profile, &hw) || !parse_config(config_json, &c)) return kNaN;
                return GaussianProcess::roofline_prior(m, n, k, c, hw);)
}

// ---- candidates --------------------------------------------------------------------
char *tracea_propose_gemm_configs(uint32_t m, uint32_t n, uint32_t k) {
  TUNER_GUARDED(nullptr, return configs_to_json(propose_gemm_configs(m, n, k));)
}

char *tracea_propose_conv_configs(uint32_t m, uint32_t n, uint32_t k) {
  TUNER_GUARDED(nullptr, return configs_to_json(propose_conv_configs(m, n, k));)
}

char *tracea_propose_attention_configs(uint32_t head_dim) {
  TUNER_GUARDED(nullptr, return configs_to_json(propose_attention_configs(head_dim));)
}

char *tracea_search_space_enumerate(const char *space_json) {
  TUNER_GUARDED(
      nullptr, Json root; std::string err;
      if (space_json == nullptr || !Json::parse(space_json, &root, &err) || root.type != Json::Object) {
        fail(TRACEA_INVALID_PARAMS, "search space must be a JSON object: %s", err.c_str());
        return nullptr;
      } SearchSpace sp;
      sp.tile_m(number_list(root, "tile_m")).tile_n(number_list(root, "tile_n")).tile_k(number_list(root, "tile_k"));
      sp.warps(number_list(root, "warps")).k_unroll(number_list(root, "k_unroll"));
      sp.prefetch_distance(number_list(root, "prefetch_distance")).micro_m(number_list(root, "micro_m"));
      const std::vector<uint32_t> st = number_list(root, "stages"); if (!st.empty()) sp.stages(st);
      bool present = false; std::vector<std::string> sv = string_list(root, "swizzles", &present);
      if (present) sp.swizzles(sv); sv = string_list(root, "barrier_modes", &present);
      if (present) sp.barrier_modes(sv);
      if (const Json *tc = root.find("use_tensor_core")) if (tc->type == Json::Bool) sp.use_tensor_core(tc->b);
      return configs_to_json(sp.enumerate());)
}

int32_t tracea_variant_for_config(const char *config_json) {
  TUNER_GUARDED(-1, PipelineConfig c; if (!parse_config(config_json, &c)) return -1;
                return contraction_variant_for_config(c);)
}

const char *tracea_magic_number_strategy(uint64_t divisor) { return magic_number_strategy_for(divisor); }

// ---- tuning cache ------------------------------------------------------------------
char *tracea_tuning_cache_path(void) {
  TUNER_GUARDED(nullptr, return dup_cstr(tuning_cache_path());)
}

char *tracea_tuning_cache_get(const char *key) {
  TUNER_GUARDED(nullptr, CacheEntry e; if (key == nullptr || !tuning_cache_get(key, &e)) return nullptr;
                Json j = Json::make_obj(); j.set("config", e.config.to_json_value());
                j.set("score", Json::make_num(e.score)); j.set("timestamp", Json::make_num((double)e.timestamp));
                return dup_cstr(j.dump());)
}

int32_t tracea_tuning_cache_put(const char *key, const char *config_json, float score, uint64_t timestamp) {
  TUNER_GUARDED(-1, CacheEntry e; if (key == nullptr || *key == 0) {
    fail(TRACEA_INVALID_PARAMS, "tuning_cache_put: empty key");
    return -1;
  } if (!parse_config(config_json, &e.config)) return -1;
                e.score = score; e.timestamp = timestamp; tuning_cache_put(key, e, true); return 0;)
}

void tracea_tuning_cache_reload(void) { tuning_cache_reload(); }

char *tracea_tuning_history_path(void) {
  TUNER_GUARDED(nullptr, return dup_cstr(tuning_history_path());)
}

int32_t tracea_tuning_history_record(const char *key, const char *config_json, float tflops, uint64_t timestamp,
                                     const char *reason) {
  TUNER_GUARDED(-1, HistoryEntry e; if (key == nullptr || *key == 0) {
    fail(TRACEA_INVALID_PARAMS, "tuning_history_record: empty key");
    return -1;
  } if (!parse_config(config_json, &e.config)) return -1;
                e.tflops = tflops; e.timestamp = timestamp;
                e.explanation = tuning_history_explanation(e.backend, tflops, reason ? reason : "");
                tuning_history_record(key, e); return 0;)
}

char *tracea_tuning_history_query(const char *key) {
  TUNER_GUARDED(nullptr, HistoryEntry e; if (key == nullptr || !tuning_history_query(key, &e)) return nullptr;
                Json j = Json::make_obj(); j.set("backend", Json::make_str(e.backend));
                j.set("config", e.config.to_json_value()); j.set("tflops", Json::make_num(e.tflops));
                j.set("timestamp", Json::make_num((double)e.timestamp));
                j.set("explanation", Json::make_str(e.explanation)); return dup_cstr(j.dump());)
}

void tracea_tuning_history_reload(void) { tuning_history_reload(); }

char *tracea_tuning_key_gemm(uint64_t m, uint64_t n, uint64_t k, const char *device_name) {
  TUNER_GUARDED(nullptr, return dup_cstr(gemm_cache_key(m, n, k, device_name ? device_name : ""));)
}

char *tracea_tuning_key_conv2d(uint32_t batch, uint32_t h, uint32_t w, uint32_t c, uint32_t k, uint32_t r,
                               uint32_t s, uint32_t stride, uint32_t pad, const char *device_name) {
  TUNER_GUARDED(nullptr, ConvProblem p; p.batch = batch; p.h_in = h; p.w_in = w; p.c_in = c; p.c_out = k;
                p.kernel_h = r; p.kernel_w = s; p.stride = stride; p.pad = pad;
                return dup_cstr(conv_cache_key(p, device_name ? device_name : ""));)
}

// ---- AutoTuner ---------------------------------------------------------------------
TraceaResult tracea_autotune_candidates(const char *key, const char *candidates_json, TraceaMeasureFn measure,
                                        void *user) {
  TUNER_GUARDED(
      failure("internal error"), std::vector<PipelineConfig> cands;
      if (measure == nullptr) return failure("autotune: measure callback is NULL");
      if (!parse_candidates(candidates_json, &cands)) return failure("autotune: malformed candidate list");
      AutoTuner tuner(HardwareProfile::mi355x());
      const PipelineConfig best = tuner.optimize_v2(key ? key : "", cands, wrap_measure(measure, user));
      return success(best, tuner.best_score);)
}

TraceaResult tracea_autotune_guided(const char *profile, uint32_t m, uint32_t n, uint32_t k,
                                    const char *candidates_json, TraceaMeasureFn measure, void *user,
                                    uint32_t iterations, TraceaAcquisition acquisition, uint64_t seed) {
  TUNER_GUARDED(
      failure("internal error"), std::vector<PipelineConfig> cands; HardwareProfile hw;
      if (measure == nullptr || m == 0 || n == 0 || k == 0)
        return failure("autotune_guided: NULL callback or zero dimension");
      if (!parse_profile(profile, &hw)) return failure("autotune_guided: unknown hardware profile");
      if (!parse_candidates(candidates_json, &cands)) return failure("autotune_guided: malformed candidate list");
      const AcquisitionFunction acq = acquisition == TRACEA_ACQ_UCB        ? AcquisitionFunction::UCB
                                      : acquisition == TRACEA_ACQ_THOMPSON ? AcquisitionFunction::Thompson
                                                                           : AcquisitionFunction::EI;
      AutoTuner tuner(hw);
      const PipelineConfig best =
          tuner.optimize_guided(m, n, k, cands, wrap_measure(measure, user), iterations, acq, seed);
      return success(best, tuner.best_score);)
}

TraceaResult tracea_autotune_gemm(size_t m, size_t n, size_t k, uint32_t iterations) {
  TUNER_GUARDED(failure("internal error"), return autotune_gemm(m, n, k, iterations);)
}

TraceaResult tracea_autotune_conv2d(size_t n, size_t c, size_t h, size_t w, size_t k, size_t r, size_t s_kernel,
                                    size_t stride, size_t pad, size_t dilation, uint32_t iterations) {
  TUNER_GUARDED(failure("internal error"),
                return autotune_conv2d(n, c, h, w, k, r, s_kernel, stride, pad, dilation, iterations);)
}

}  // extern "C"
#pragma GCC visibility pop
