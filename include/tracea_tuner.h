/* Tuner surface of libtracea.so: tuning records, device profile, Gaussian-process
 * surrogate, candidate lists and the auto-tuner loop, as a C ABI.
 *
 * The reference keeps these as Rust types without an FFI; each entry point
 * names the Rust item whose behaviour it carries.  Configurations cross the
 * boundary as the reference's own PipelineConfig JSON (src/core/config.rs:297-340),
 * so a record produced by either side is readable by the other.
 *
 * Every `char *` returned is owned by the caller and released with
 * tracea_free_string; NULL means failure with the reason in
 * tracea_get_last_error.  Nothing in this header touches the GPU except
 * tracea_autotune_gemm / tracea_autotune_conv2d. */
#ifndef TRACEA_TUNER_H
#define TRACEA_TUNER_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#include "tracea.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- PipelineConfig: src/core/config.rs:342-448 ------------------------------------ */
/* PipelineConfig::new(num_stages, m_tile, n_tile, k_tile) as JSON. */
char *tracea_pipeline_config_new(uint32_t num_stages, uint32_t m_tile, uint32_t n_tile, uint32_t k_tile);
/* from_json followed by to_json: fills the fields an older record lacks with
 * their defaults and emits the canonical field order. */
char *tracea_pipeline_config_normalize(const char *config_json);
/* validate() (config.rs:376-396): 0 when valid; 1 when invalid with the
 * reference's message in *message (caller frees); -1 on malformed JSON. */
int32_t tracea_pipeline_config_validate(const char *config_json, char **message);
/* to_vector() (config.rs:399-433): writes up to `capacity` floats and returns
 * the full length, or -1 on malformed JSON. */
int32_t tracea_pipeline_config_to_vector(const char *config_json, float *out, int32_t capacity);

/* ---- HardwareProfile: src/optimizer/mod.rs:15-250 ---------------------------------- */
/* `profile` is "mi355x", or one of the reference's presets "rtx3070", "mi250",
 * "a100" (kept for its test vectors). */
char *tracea_hardware_profile_json(const char *profile);
/* check_feasibility (mod.rs:183-216) for a problem with m rows: 0 feasible;
 * 1 pruned with the reason ("SharedMemoryOverflow", "LowOccupancy(n)",
 * "ForbiddenZone(..)") in *reason (caller frees); -1 bad argument. */
int32_t tracea_check_feasibility(const char *profile, const char *config_json, uint64_t m, char **reason);
/* estimate_occupancy (mod.rs:218-249); negative on a bad argument. */
float tracea_estimate_occupancy(const char *profile, const char *config_json);

/* ---- GaussianProcess: src/optimizer/mod.rs:297-576 --------------------------------- */
typedef struct TraceaGaussianProcess TraceaGaussianProcess;
TraceaGaussianProcess *tracea_gp_create(void); /* noise_sigma 0.1, exploration_beta 2.0 */
void tracea_gp_destroy(TraceaGaussianProcess *gp);
void tracea_gp_set_noise_sigma(TraceaGaussianProcess *gp, float sigma);
void tracea_gp_set_exploration_beta(TraceaGaussianProcess *gp, float beta);
/* observe(Observation{m,n,k,config,score}, gpu); 0 ok, -1 bad argument. */
int32_t tracea_gp_observe(TraceaGaussianProcess *gp, uint32_t m, uint32_t n, uint32_t k,
                          const char *config_json, float score, const char *profile);
/* predict -> (mean, std); 0 ok, -1 bad argument. */
int32_t tracea_gp_predict(const TraceaGaussianProcess *gp, uint32_t m, uint32_t n, uint32_t k,
                          const char *config_json, const char *profile, float *mean, float *stddev);
/* Acquisition value of one candidate.  kind: 0 expected improvement over
 * `best_y`, 1 upper confidence bound, 2 Thompson sample (drawn from a stream
 * seeded with `seed`).  NaN on a bad argument. */
float tracea_gp_acquisition(const TraceaGaussianProcess *gp, int32_t kind, uint32_t m, uint32_t n, uint32_t k,
                            const char *config_json, const char *profile, float best_y, uint64_t seed);
float tracea_gp_marginal_log_likelihood(const TraceaGaussianProcess *gp, const char *profile);
void tracea_gp_optimize_hyperparams(TraceaGaussianProcess *gp, const char *profile);
/* Copies up to `capacity` length scales, returns their count. */
int32_t tracea_gp_length_scales(const TraceaGaussianProcess *gp, float *out, int32_t capacity);
/* Feature vector the kernel sees for (m, n, k, config): full length returned. */
int32_t tracea_gp_features(uint32_t m, uint32_t n, uint32_t k, const char *config_json, float *out,
                           int32_t capacity);
/* Roofline prior in TFLOP/s (mod.rs:484-493); NaN on a bad argument. */
float tracea_gp_roofline_prior(uint32_t m, uint32_t n, uint32_t k, const char *config_json,
                               const char *profile);

/* ---- candidates: src/policy/standard.rs:33-113, src/optimizer/policy.rs:15-64 ------- */
/* JSON arrays of PipelineConfig, one per compiled kernel variant, the cost
 * model's choice first.  (m, n, k) is the GEMM, or the implicit GEMM of the
 * convolution: m = N*Ho*Wo, n = K filters, k = R*S*C. */
char *tracea_propose_gemm_configs(uint32_t m, uint32_t n, uint32_t k);
char *tracea_propose_conv_configs(uint32_t m, uint32_t n, uint32_t k);
char *tracea_propose_attention_configs(uint32_t head_dim);
/* SearchSpace product: `space_json` is an object with optional arrays tile_m,
 * tile_n, tile_k, warps, stages, k_unroll, prefetch_distance, micro_m
 * (numbers), swizzles, barrier_modes (strings) and the bool use_tensor_core;
 * returns the JSON array of configs in the reference's loop order. */
char *tracea_search_space_enumerate(const char *space_json);
/* Index of the compiled contraction variant a config names, or -1. */
int32_t tracea_variant_for_config(const char *config_json);
/* MagicNumberStrategy::select_for (src/core/config.rs:470-478); library-owned string. */
const char *tracea_magic_number_strategy(uint64_t divisor);

/* ---- tuning cache: src/core/tuning.rs:14-139 --------------------------------------- */
/* Path in use (TRACEA_TUNING_CACHE or .tracea/tuning_cache_v2.json). */
char *tracea_tuning_cache_path(void);
/* Entry {config, score, timestamp} as JSON, or NULL when the key is absent. */
char *tracea_tuning_cache_get(const char *key);
/* Inserts / replaces and rewrites the file; 0 ok, -1 bad argument. */
int32_t tracea_tuning_cache_put(const char *key, const char *config_json, float score, uint64_t timestamp);
/* Forgets the in-memory copy; the next access re-reads the file. */
void tracea_tuning_cache_reload(void);
/* ---- tuning history: src/optimizer/history.rs:7-51 ----------------------------------- */
/* The reference's second record of tuning results, tuning_history.json in the working directory
 * (override: TRACEA_TUNING_HISTORY): a map key -> {backend, config, tflops, timestamp, explanation},
 * keys "HardwareId:OpFingerprint:Precision" (history.rs:17).  tracea_tune_* record the winner of every
 * measurement here under "<device name>:<cache key>:<F16|BF16|FP32>" with backend "Rocm". */
char *tracea_tuning_history_path(void);
/* TuningHistory::record (history.rs:38-41): inserts / replaces and rewrites the file.  The explanation is
 * generate_explanation's sentence (history.rs:47-52) built from backend, tflops and `reason`.  0 ok, -1 bad
 * argument. */
int32_t tracea_tuning_history_record(const char *key, const char *config_json, float tflops, uint64_t timestamp,
                                     const char *reason);
/* TuningHistory::query (history.rs:43-45): the entry as JSON, or NULL when the key is absent. */
char *tracea_tuning_history_query(const char *key);
/* Forgets the in-memory copy; the next access re-reads the file (load_or_create, history.rs:22-29). */
void tracea_tuning_history_reload(void);

/* Keys as the reference spells them (tuning.rs:66-78). */
char *tracea_tuning_key_gemm(uint64_t m, uint64_t n, uint64_t k, const char *device_name);
char *tracea_tuning_key_conv2d(uint32_t batch, uint32_t h, uint32_t w, uint32_t c, uint32_t k, uint32_t r,
                               uint32_t s, uint32_t stride, uint32_t pad, const char *device_name);

/* ---- AutoTuner: src/optimizer/mod.rs:578-760 --------------------------------------- */
/* Caller-supplied micro-benchmark: TFLOP/s of one candidate, <= 0 if it failed. */
typedef float (*TraceaMeasureFn)(const char *config_json, void *user);
typedef enum {
  TRACEA_ACQ_EI = 0,
  TRACEA_ACQ_UCB = 1,
  TRACEA_ACQ_THOMPSON = 2,
} TraceaAcquisition;

/* optimize_v2 + get_or_tune: a cached `key` wins, otherwise every candidate of
 * the JSON array is measured, the best is cached under `key` and returned.
 * key NULL or "": no cache, first candidate returned unmeasured (the
 * reference's behaviour for operators without a key). */
TraceaResult tracea_autotune_candidates(const char *key, const char *candidates_json, TraceaMeasureFn measure,
                                        void *user);
/* Budgeted search: measures at most `iterations` candidates, each chosen by the
 * acquisition function over a Gaussian process fed with the earlier results. */
TraceaResult tracea_autotune_guided(const char *profile, uint32_t m, uint32_t n, uint32_t k,
                                    const char *candidates_json, TraceaMeasureFn measure, void *user,
                                    uint32_t iterations, TraceaAcquisition acquisition, uint64_t seed);
/* AutoTuner::optimize / optimize_conv on the device: candidates from the
 * variant table, the library's own event-timed benchmark as the measure, and
 * the tuning cache consulted first (unlike tracea_tune_*, which always
 * measures).  iterations 0 measures every candidate; otherwise at most that
 * many, chosen by expected improvement. */
TraceaResult tracea_autotune_gemm(size_t m, size_t n, size_t k, uint32_t iterations);
TraceaResult tracea_autotune_conv2d(size_t n, size_t c, size_t h, size_t w, size_t k, size_t r, size_t s_kernel,
                                    size_t stride, size_t pad, size_t dilation, uint32_t iterations);

#ifdef __cplusplus
}
#endif
#endif /* TRACEA_TUNER_H */
