// Host-side tuner: device profile, Gaussian-process surrogate, candidate
// generation and the AutoTuner that drives micro-benchmarks.
//
// Mirrors the reference's optimizer (src/optimizer/mod.rs:15-250 HardwareProfile,
// :297-576 GaussianProcess, :578-760 AutoTuner; src/optimizer/policy.rs:15-88
// SearchSpace / estimate_smem_usage; src/policy/standard.rs:33-113 candidate
// lists) with one difference in kind: a candidate here always names a compiled
// kernel variant of this library, so every proposed PipelineConfig can be run.
#pragma once
#include <cstdint>
#include <functional>
#include <map>
#include <string>
#include <vector>

#include "pipeline_config.hpp"

namespace tracea_amd {

// ---- HardwareProfile (src/optimizer/mod.rs:15-37) ----------------------------------
struct HardwareProfile {
  std::string name;
  std::string backend;  // "Cuda" | "Rocm" | "Metal" | "Cpu"
  size_t shared_memory_per_block = 0;
  uint32_t max_registers_per_thread = 0;
  uint32_t registers_per_sm = 0;
  uint32_t max_registers_per_block = 0;
  uint32_t max_warps_per_sm = 0;  // waves per CU
  uint32_t wavefront_size = 0;
  uint32_t max_blocks_per_sm = 0;
  size_t shared_memory_per_sm = 0;
  bool has_specialized_units = false;
  std::vector<std::string> supported_intrinsic_shapes;
  size_t max_threadgroup_memory = 0;
  uint32_t preferred_tile_shape[3] = {0, 0, 0};
  uint32_t simd_width = 0;
  float peak_tflops_standard = 0.0f;
  float peak_tflops_tensor = 0.0f;
  float mem_bw_gbps = 0.0f;

  // One CU of an MI355X: 160 KB LDS, 4 SIMDs x 8 waves, 512 VGPRs per lane
  // (arch + accumulation), 128 K 32-bit registers per SIMD.
  static HardwareProfile mi355x();
  // The reference's presets, kept for its own test vectors (mod.rs:39-133).
  static HardwareProfile rtx3070();
  static HardwareProfile mi250();
  static HardwareProfile a100();
  // "mi355x" | "rtx3070" | "mi250" | "a100"; false when the name is unknown.
  static bool by_name(const std::string &name, HardwareProfile *out);

  // Empty string when the config may be tried, else the reference's pruning
  // reason spelled as its Debug form ("SharedMemoryOverflow", "LowOccupancy(31)",
  // "ForbiddenZone(\"...\")"); mod.rs:183-216.  m is the problem's row count.
  std::string check_feasibility(const PipelineConfig &c, uint64_t m) const;
  // Fraction of max_blocks_per_sm that fit by waves and by the register
  // estimate tile*stages/threads + 32 (mod.rs:218-249).
  float estimate_occupancy(const PipelineConfig &c) const;
  Json to_json_value() const;
};

// TuningPolicy::estimate_smem_usage default (policy.rs:81-87).
size_t estimate_smem_usage(const PipelineConfig &c);

struct TuningStats {
  size_t total_trials = 0;
  size_t pruned_count = 0;
  std::map<std::string, size_t> pruning_reasons;
  void log_pruning(const std::string &reason);
};

// ---- GaussianProcess (src/optimizer/mod.rs:297-576) --------------------------------
struct Observation {
  uint32_t m = 0, n = 0, k = 0;
  PipelineConfig config;
  float score = 0.0f;
};

enum class AcquisitionFunction { EI, UCB, Thompson };
enum class OptimizationGoal { MaximizeTFLOPS, MinimizeLatency, Balanced };

class GaussianProcess {
 public:
  std::vector<Observation> observations;
  std::vector<float> length_scales;
  float noise_sigma = 0.1f;
  float exploration_beta = 2.0f;

  GaussianProcess();
  // Appends; every 5th observation past the 5th re-fits the length scales.
  void observe(const Observation &obs, const HardwareProfile &gpu);
  // Coordinate search, 10 sweeps of +-10 % per dimension, clamp [0.1, 10].
  void optimize_hyperparams(const HardwareProfile &gpu);
  float marginal_log_likelihood(const HardwareProfile &gpu) const;
  // Posterior mean and standard deviation; (prior, 1) with no observations or
  // when the kernel matrix is not positive definite.
  void predict(uint32_t m, uint32_t n, uint32_t k, const PipelineConfig &c, const HardwareProfile &gpu,
               float *mean, float *stddev) const;
  float expected_improvement(uint32_t m, uint32_t n, uint32_t k, const PipelineConfig &c, float best_y,
                             const HardwareProfile &gpu) const;
  float ucb(uint32_t m, uint32_t n, uint32_t k, const PipelineConfig &c, const HardwareProfile &gpu) const;
  // One draw from N(mean, std); `state` is a splitmix64 state the call advances
  // (the reference draws from the thread RNG, so its samples are not repeatable).
  float thompson_sample(uint32_t m, uint32_t n, uint32_t k, const PipelineConfig &c,
                        const HardwareProfile &gpu, uint64_t *state) const;
  // min(peak, bandwidth * arithmetic intensity / 1000) in TFLOP/s (mod.rs:484-493).
  static float roofline_prior(uint32_t m, uint32_t n, uint32_t k, const PipelineConfig &c,
                              const HardwareProfile &gpu);
  // 5 shape features ++ config numbers ++ 3 tile ratios (mod.rs:350-361, 476-503).
  static std::vector<float> full_features(uint32_t m, uint32_t n, uint32_t k, const PipelineConfig &c);

 private:
  float ard_distance_sq(const std::vector<float> &a, const std::vector<float> &b) const;
  // Builds K + sigma^2 I over the observations, factors it, and returns
  // alpha = K^-1 (y - prior); false when the factorisation fails.
  bool factor(const HardwareProfile &gpu, std::vector<std::vector<float>> *feats, std::vector<double> *chol,
              std::vector<double> *diff) const;
};

// ---- candidate generation ----------------------------------------------------------
// SearchSpace builder (policy.rs:15-64; usage in docs/API_USAGE.md:128-140).
struct SearchSpace {
  std::vector<uint32_t> tile_m_, tile_n_, tile_k_, warps_, k_unroll_, prefetch_distance_, micro_m_;
  std::vector<uint32_t> stages_{2};
  std::vector<std::string> swizzles_{"None"};
  std::vector<std::string> barrier_modes_{"None"};
  std::vector<std::string> softmax_granularities_{"PerTile"};
  bool use_tensor_core_ = true;
  bool enable_swizzle_ = false;

  SearchSpace &tile_m(std::vector<uint32_t> v) { tile_m_ = std::move(v); return *this; }
  SearchSpace &tile_n(std::vector<uint32_t> v) { tile_n_ = std::move(v); return *this; }
  SearchSpace &tile_k(std::vector<uint32_t> v) { tile_k_ = std::move(v); return *this; }
  SearchSpace &warps(std::vector<uint32_t> v) { warps_ = std::move(v); return *this; }
  SearchSpace &use_tensor_core(bool v) { use_tensor_core_ = v; return *this; }
  SearchSpace &enable_swizzle(bool v) { enable_swizzle_ = v; return *this; }
  SearchSpace &k_unroll(std::vector<uint32_t> v) { k_unroll_ = std::move(v); return *this; }
  SearchSpace &prefetch_distance(std::vector<uint32_t> v) { prefetch_distance_ = std::move(v); return *this; }
  SearchSpace &micro_m(std::vector<uint32_t> v) { micro_m_ = std::move(v); return *this; }
  SearchSpace &stages(std::vector<uint32_t> v) { stages_ = std::move(v); return *this; }
  SearchSpace &swizzles(std::vector<std::string> v) { swizzles_ = std::move(v); return *this; }
  SearchSpace &barrier_modes(std::vector<std::string> v) { barrier_modes_ = std::move(v); return *this; }

  // Cartesian product as PipelineConfigs (the loop nest of mod.rs:791-836);
  // an empty axis contributes the PipelineConfig default for that field.
  std::vector<PipelineConfig> enumerate() const;
};

// Candidate configs for a GEMM (or the implicit GEMM of a conv): one per
// compiled contraction variant that is feasible for the problem, the cost
// model's pick first (the role of policy/standard.rs:33-113).
std::vector<PipelineConfig> propose_gemm_configs(uint32_t m, uint32_t n, uint32_t k);
std::vector<PipelineConfig> propose_conv_configs(uint32_t m, uint32_t n, uint32_t k);
std::vector<PipelineConfig> propose_attention_configs(uint32_t head_dim);

// ---- AutoTuner (mod.rs:578-760) ----------------------------------------------------
// MagicNumberStrategy::select_for (src/core/config.rs:470-478).
const char *magic_number_strategy_for(uint64_t divisor);

struct ConvProblem {
  uint32_t batch = 1, h_in = 1, w_in = 1, c_in = 1, c_out = 1, kernel_h = 1, kernel_w = 1;
  uint32_t stride = 1, pad = 0, dilation = 1;
  uint32_t h_out() const { return (h_in + 2 * pad - dilation * (kernel_h - 1) - 1) / stride + 1; }
  uint32_t w_out() const { return (w_in + 2 * pad - dilation * (kernel_w - 1) - 1) / stride + 1; }
};

struct ConvConfig {
  PipelineConfig base;
  bool use_tensor_core = true;
  bool use_nhwc = true;
  std::string magic_strategy = "Standard";
};

// TFLOP/s of one candidate; <= 0 when it could not be run.
using MeasureFn = std::function<float(const PipelineConfig &)>;

class AutoTuner {
 public:
  HardwareProfile gpu;
  GaussianProcess gp;
  bool has_best = false;
  PipelineConfig best_config;
  float best_score = 0.0f;
  std::string hardware_id;
  TuningStats stats;

  explicit AutoTuner(const HardwareProfile &profile);

  // Cache lookup under `key`, else a grid search over `candidates` with the
  // best TFLOP/s winning and the entry persisted (optimize_v2 + get_or_tune:
  // mod.rs:704-760, src/core/tuning.rs:92-139).  An empty key skips the cache
  // and returns the first candidate unmeasured, as the reference does for
  // operators without a key (tuning.rs:95-98).  No candidates: the reference's
  // fallback PipelineConfig(2, 64, 64, 32).
  PipelineConfig optimize_v2(const std::string &key, const std::vector<PipelineConfig> &candidates,
                             const MeasureFn &measure);
  // GEMM adapter (mod.rs:625-636): key gemm_{m}_{n}_{k}_{device}; the epilogue
  // list is stored on the returned config.
  PipelineConfig optimize(uint32_t m, uint32_t n, uint32_t k, const MeasureFn &measure,
                          const Json &epilogue = Json::make_arr());
  // Conv adapter (mod.rs:639-660): implicit-GEMM dims, magic strategy from Ho*Wo.
  ConvConfig optimize_conv(const ConvProblem &p, const MeasureFn &measure);
  // Budgeted search: measures at most `iterations` candidates, the first by
  // roofline prior and each next one the arg-max of the acquisition function
  // over the unmeasured feasible candidates (the loop the reference sketches
  // in propose_candidate, mod.rs:776-838).  Observations feed `gp`.
  PipelineConfig optimize_guided(uint32_t m, uint32_t n, uint32_t k,
                                 const std::vector<PipelineConfig> &candidates, const MeasureFn &measure,
                                 size_t iterations, AcquisitionFunction acq, uint64_t seed = 1);
  // Goal-weighted score of one measurement (mod.rs:763-773).
  static float calculate_score(float tflops, float latency_ms, OptimizationGoal goal, float tflops_weight);
};

// Cache keys (src/core/tuning.rs:66-78).
std::string gemm_cache_key(uint64_t m, uint64_t n, uint64_t k, const std::string &device);
std::string conv_cache_key(const ConvProblem &p, const std::string &device);

}  // namespace tracea_amd
