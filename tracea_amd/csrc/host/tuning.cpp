// Tuning cache and the exhaustive micro-benchmark tuner behind
// tracea_tune_gemm / tracea_tune_conv2d / tracea_tune_fa2.
//
// Reference behaviour kept: TuningCache::get_or_tune is a grid search over
// the candidate list with the best TFLOP/s winning and the entry persisted
// at once (src/core/tuning.rs:92-139); the benchmark protocol is warm-up
// launches followed by timed launches of the real kernel on device buffers
// (src/optimizer/benchmark.rs:255-343, 814-868); GEMM flops = 2MNK
// (benchmark.rs:188-190), conv flops = 2*M*N*K of the implicit GEMM
// (benchmark.rs:466-469), attention flops = 4*B*H*S^2*D for causal and dense
// alike (benchmark.rs:954-957).  Timing uses HIP events on one stream instead
// of the reference's host clock.
#include <sys/stat.h>

#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <map>
#include <mutex>
#include <sstream>

#include "dispatch.hpp"
#include "tuner.hpp"
#include "tuning_cache.hpp"

namespace tracea_amd {

namespace {
std::mutex g_mu;
std::map<std::string, CacheEntry> g_cache;
bool g_loaded = false;
std::string g_device_name;

void load_locked() {
  if (g_loaded) return;
  g_loaded = true;
  std::ifstream f(tuning_cache_path());
  if (!f) return;
  std::stringstream ss;
  ss << f.rdbuf();
  Json root;
  std::string err;
  if (!Json::parse(ss.str(), &root, &err) || root.type != Json::Object) return;
  for (const auto &kv : root.obj) {
    const Json *cfg = kv.second.find("config");
    CacheEntry e;
    if (!cfg || !PipelineConfig::from_json_value(*cfg, &e.config, &err)) continue;
    if (const Json *s = kv.second.find("score")) e.score = (float)s->num;
    if (const Json *t = kv.second.find("timestamp")) e.timestamp = (uint64_t)t->num;
    if (const Json *t = kv.second.find("operand_dtype")) e.operand_dtype = t->str;
    if (const Json *t = kv.second.find("b_layout")) e.b_layout = t->str;
    g_cache[kv.first] = e;
  }
}

void save_locked() {
  const std::string path = tuning_cache_path();
  const size_t slash = path.find_last_of('/');
  if (slash != std::string::npos) mkdir(path.substr(0, slash).c_str(), 0755);
  Json root = Json::make_obj();
  for (const auto &kv : g_cache) {
    Json e = Json::make_obj();
    e.set("config", kv.second.config.to_json_value());
    e.set("score", Json::make_num(kv.second.score));
    e.set("timestamp", Json::make_num((double)kv.second.timestamp));
    if (!kv.second.operand_dtype.empty()) e.set("operand_dtype", Json::make_str(kv.second.operand_dtype));
    if (!kv.second.b_layout.empty()) e.set("b_layout", Json::make_str(kv.second.b_layout));
    root.set(kv.first, e);
  }
  std::ofstream f(path);
  if (f) f << root.dump(2) << "\n";
}
}  // namespace

const char *tuning_device_name() {
  std::lock_guard<std::mutex> lk(g_mu);
  if (g_device_name.empty() && runtime_ready()) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, 0) == hipSuccess) g_device_name = prop.name;
  }
  return g_device_name.c_str();
}

std::string tuning_cache_path() {
  const char *env = getenv("TRACEA_TUNING_CACHE");
  return env && *env ? std::string(env) : std::string(".tracea/tuning_cache_v2.json");
}

bool tuning_cache_get(const std::string &key, CacheEntry *out) {
  std::lock_guard<std::mutex> lk(g_mu);
  load_locked();
  auto it = g_cache.find(key);
  if (it == g_cache.end()) return false;
  if (out) *out = it->second;
  return true;
}

void tuning_cache_put(const std::string &key, const CacheEntry &e, bool persist) {
  std::lock_guard<std::mutex> lk(g_mu);
  load_locked();
  g_cache[key] = e;
  if (persist) save_locked();
}

void tuning_cache_reload() {
  std::lock_guard<std::mutex> lk(g_mu);
  g_cache.clear();
  g_loaded = false;
}

// ---- tuning history (src/optimizer/history.rs) ----
namespace {
std::mutex g_hist_mu;
std::map<std::string, HistoryEntry> g_hist;
bool g_hist_loaded = false;

void hist_load_locked() {
  if (g_hist_loaded) return;
  g_hist_loaded = true;
  std::ifstream f(tuning_history_path());
  if (!f) return;
  std::stringstream ss;
  ss << f.rdbuf();
  Json root;
  std::string err;
  // (a file that does not parse is an empty history, as load_or_create has it)
  if (!Json::parse(ss.str(), &root, &err) || root.type != Json::Object) return;
  for (const auto &kv : root.obj) {
    const Json *cfg = kv.second.find("config");
    HistoryEntry e;
    if (!cfg || !PipelineConfig::from_json_value(*cfg, &e.config, &err)) continue;
    if (const Json *b = kv.second.find("backend")) e.backend = b->str;
    if (const Json *t = kv.second.find("tflops")) e.tflops = (float)t->num;
    if (const Json *t = kv.second.find("timestamp")) e.timestamp = (uint64_t)t->num;
    if (const Json *x = kv.second.find("explanation")) e.explanation = x->str;
    g_hist[kv.first] = e;
  }
}
}  // namespace

std::string tuning_history_path() {
  const char *env = getenv("TRACEA_TUNING_HISTORY");
  return env && *env ? std::string(env) : std::string("tuning_history.json");
}

std::string tuning_history_explanation(const std::string &backend, float tflops, const std::string &reason) {
  char buf[96];
  snprintf(buf, sizeof(buf), "%.2f", (double)tflops);
  return "Selected " + backend + " because it achieved " + buf + " TFLOPS. Reason: " + reason;
}

bool tuning_history_query(const std::string &key, HistoryEntry *out) {
  std::lock_guard<std::mutex> lk(g_hist_mu);
  hist_load_locked();
  auto it = g_hist.find(key);
  if (it == g_hist.end()) return false;
  if (out) *out = it->second;
  return true;
}

void tuning_history_record(const std::string &key, const HistoryEntry &e) {
  std::lock_guard<std::mutex> lk(g_hist_mu);
  hist_load_locked();
  g_hist[key] = e;
  Json root = Json::make_obj();
  for (const auto &kv : g_hist) {
    Json j = Json::make_obj();
    j.set("backend", Json::make_str(kv.second.backend));
    j.set("config", kv.second.config.to_json_value());
    j.set("tflops", Json::make_num(kv.second.tflops));
    j.set("timestamp", Json::make_num((double)kv.second.timestamp));
    j.set("explanation", Json::make_str(kv.second.explanation));
    root.set(kv.first, j);
  }
  std::ofstream f(tuning_history_path());
  if (f) f << root.dump(2) << "\n";
}

void tuning_history_reload() {
  std::lock_guard<std::mutex> lk(g_hist_mu);
  g_hist.clear();
  g_hist_loaded = false;
}

int tuning_cache_lookup_variant(const std::string &key, int dtype, bool b_ncontig) {
  CacheEntry e;
  if (!tuning_cache_get(key, &e) || !e.matches(dtype, b_ncontig)) return -1;
  return contraction_variant_for_config(e.config);
}

// A contraction variant as a PipelineConfig: tiles, LDS stages, wave count
// (force_num_warps) and the per-wave tile (micro_m x micro_n).  The reference's
// IntrinsicShape enum has no 32x32x16 entry; M32N32K2 names the 32x32 MFMA
// family, the only spelling a reference build would accept.
PipelineConfig config_for_contraction_variant(int index) {
  const ContractionVariant &v = contraction_variant(index);
  PipelineConfig c((uint32_t)v.stages, (uint32_t)v.bm, (uint32_t)v.bn, (uint32_t)v.bk);
  c.instruction = "RocmMFMA";
  c.swizzle_mode = "Xor8";
  c.layout_policy = "XorSwizzled";
  c.has_force_num_warps = true;
  c.force_num_warps = (uint32_t)(v.waves_m * v.waves_n);
  c.micro_m = (uint32_t)(v.bm / v.waves_m);
  c.micro_n = (uint32_t)(v.bn / v.waves_n);
  // v_mfma_f32_32x32x16 or v_mfma_f32_16x16x32 under the reference's names for a 32x32 and a 16x16 MFMA
  // block (src/core/config.rs:166-181)
  c.intrinsic_shape = v.mfma == 16 ? "M16N16K4" : "M32N32K2";
  c.gemm_variant = "Simd";
  c.double_buffer = true;
  c.cp_async_distance = (uint32_t)v.pipeline;  // operand prefetch distance in k-steps
  c.bank_conflict_padding = 0;
  return c;
}

int contraction_variant_for_config(const PipelineConfig &c) {
  for (int i = 0; i < contraction_variant_count(); ++i) {
    const ContractionVariant &v = contraction_variant(i);
    if ((uint32_t)v.bm != c.m_tile || (uint32_t)v.bn != c.n_tile || (uint32_t)v.bk != c.k_tile) continue;
    if ((uint32_t)v.stages != c.num_stages) continue;
    if (c.has_force_num_warps && (uint32_t)(v.waves_m * v.waves_n) != c.force_num_warps) continue;
    if (c.micro_m > 1 && (uint32_t)(v.bm / v.waves_m) != c.micro_m) continue;
    if (c.cp_async_distance != (uint32_t)v.pipeline) continue;
    if ((c.intrinsic_shape == "M16N16K4") != (v.mfma == 16)) continue;
    return i;
  }
  return -1;
}

PipelineConfig config_for_attention_variant(int index) {
  const AttentionVariant &v = attention_variant(index);
  PipelineConfig c((uint32_t)v.stages, (uint32_t)v.block_q, (uint32_t)v.block_kv, 32);
  c.instruction = "RocmMFMA";
  c.swizzle_mode = "Xor8";
  c.has_force_num_warps = true;
  c.force_num_warps = (uint32_t)v.waves;
  c.intrinsic_shape = v.mfma == 16 ? "M16N16K4" : "M32N32K2";
  c.attention_variant = "FlashV2";
  c.softmax_granularity = "PerTile";
  c.double_buffer = true;
  c.bank_conflict_padding = 0;
  c.fusion_count = (uint32_t)v.items;  // tiles of the output a workgroup takes (src/optimizer/benchmark.rs:131-132)
  // two wave groups handing the vector ALU and the matrix pipe to each other across a barrier per phase
  c.barrier_mode = v.offset_groups ? "ProducerConsumer" : "None";
  return c;
}

int attention_variant_for_config(const PipelineConfig &c, const AttentionArgs &a) {
  for (int i = 0; i < attention_variant_count(); ++i) {
    const AttentionVariant &v = attention_variant(i);
    if ((uint32_t)v.block_q != c.m_tile || (uint32_t)v.stages != c.num_stages) continue;
    if (c.has_force_num_warps && (uint32_t)v.waves != c.force_num_warps) continue;
    if ((c.intrinsic_shape == "M16N16K4") != (v.mfma == 16)) continue;
    if ((uint32_t)v.items != (c.fusion_count > 1 ? c.fusion_count : 1u)) continue;
    if ((v.offset_groups != 0) != (c.barrier_mode == "ProducerConsumer")) continue;
    if (v.feasible(a)) return i;
  }
  return -1;
}

std::string attention_cache_key(size_t b, size_t s, size_t h, size_t d, bool causal) {
  char key[200];
  snprintf(key, sizeof(key), "fa2_kernel:b%zu_s%zu_h%zu_d%zu_%s", b, s, h, d, causal ? "causal" : "dense");
  return key;
}

int tuning_cache_lookup_attention(const AttentionArgs &a) {
  CacheEntry e;
  if (!tuning_cache_get(attention_cache_key((size_t)a.B, (size_t)a.S, (size_t)a.H, (size_t)a.D, a.causal != 0), &e)) return -1;
  return attention_variant_for_config(e.config, a);
}

char *dup_cstr(const std::string &s) {
  char *p = (char *)malloc(s.size() + 1);
  if (p) memcpy(p, s.c_str(), s.size() + 1);
  return p;
}

TraceaResult failure(const std::string &msg) {
  TraceaResult r;
  r.success = false;
  r.error_msg = dup_cstr(msg);
  r.score = 0.0f;
  r.config_ptr = nullptr;
  return r;
}

TraceaResult success(const PipelineConfig &cfg, float tflops) {
  TraceaResult r;
  r.success = true;
  r.error_msg = nullptr;
  r.score = tflops;
  r.config_ptr = dup_cstr(cfg.to_json());
  return r;
}

// ---- micro-benchmarks ------------------------------------------------------------
namespace {

struct DeviceBuffer {
  void *p = nullptr;
  ~DeviceBuffer() {
    if (p) (void)hipFree(p);
  }
  bool alloc(size_t bytes) { return hipMalloc(&p, bytes ? bytes : 16) == hipSuccess; }
};

std::string last_error_text() {
  uint8_t buf[512];
  const int n = tracea_get_last_error(buf, sizeof(buf));
  return n > 0 ? std::string((const char *)buf, (size_t)n) : std::string("unknown error");
}

// Times `launch` (which must enqueue exactly one kernel on the default stream):
// warm-up launches, then `iters` launches between two events.  Returns seconds
// per launch, or a negative value on error.
template <typename F>
double time_launches(F &&launch, int warmup, int iters) {
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess) return -1.0;
  if (hipEventCreate(&e1) != hipSuccess) {
    (void)hipEventDestroy(e0);
    return -1.0;
  }
  double result = -1.0;
  bool ok = true;
  for (int i = 0; i < warmup && ok; ++i) ok = launch();
  if (ok && hipDeviceSynchronize() == hipSuccess) {
    (void)hipEventRecord(e0, nullptr);
    for (int i = 0; i < iters && ok; ++i) ok = launch();
    (void)hipEventRecord(e1, nullptr);
    if (ok && hipEventSynchronize(e1) == hipSuccess) {
      float ms = 0.0f;
      if (hipEventElapsedTime(&ms, e0, e1) == hipSuccess) result = (double)ms * 1e-3 / iters;
    }
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  return result;
}

uint64_t now_seconds() {
  return (uint64_t)std::chrono::duration_cast<std::chrono::seconds>(
             std::chrono::system_clock::now().time_since_epoch())
      .count();
}

}  // namespace

// ---- micro-benchmarks as objects (the reference's MicroBenchmark / Conv2dBenchmark
// traits: src/optimizer/benchmark.rs:140-200, 420-470) ----------------------------
namespace {

// fp16 GEMM, A row-major [M,K], B column-major (stored [N,K]), C fp16 row-major.
struct GemmBenchmark {
  size_t m = 0, n = 0, k = 0;
  DeviceBuffer a, b, c;
  std::string error;

  bool init(size_t m_, size_t n_, size_t k_) {
    m = m_; n = n_; k = k_;
    if (!a.alloc(m * k * 2) || !b.alloc(n * k * 2) || !c.alloc(m * n * 2)) {
      (void)hipGetLastError();
      error = "device allocation failed";
      return false;
    }
    const float amp = sqrtf(3.0f / (float)k);  // unit-variance dot products
    launch_fill_uniform(a.p, m * k, DT_F16, 1u, amp, nullptr);
    launch_fill_uniform(b.p, n * k, DT_F16, 2u, amp, nullptr);
    return true;
  }
  // TFLOP/s of one contraction variant, <= 0 when it did not run.
  float measure(int variant) {
    const uint64_t sa[2] = {m, k}, sb[2] = {k, n}, sc[2] = {m, n};
    const int64_t ta[2] = {(int64_t)k, 1}, tb[2] = {1, (int64_t)k}, tcs[2] = {(int64_t)n, 1};
    TraceaTensorView va{a.p, 2, sa, ta, TRACEA_DTYPE_FLOAT16, 0};
    TraceaTensorView vb{b.p, 2, sb, tb, TRACEA_DTYPE_FLOAT16, 0};
    TraceaTensorView vc{c.p, 2, sc, tcs, TRACEA_DTYPE_FLOAT16, 0};
    TraceaGemmParams gp{TRACEA_EPILOGUE_IDENTITY, nullptr};
    const int saved = forced_variant("gemm");
    set_forced_variant("gemm", variant);
    const double t = time_launches(
        [&]() { return dispatch_gemm_kind(va, vb, nullptr, nullptr, &vc, gp) == TRACEA_SUCCESS; }, 3, 10);
    set_forced_variant("gemm", saved);
    if (t <= 0.0) {
      error = last_error_text();
      return 0.0f;
    }
    // the dispatcher replaces a variant that cannot run the problem by the nearest one that can: such a
    // time belongs to that other variant and must not be recorded under this one
    if (last_variant("gemm") != variant) {
      error = "the dispatcher ran another variant in its place";
      return 0.0f;
    }
    return (float)(2.0 * (double)m * (double)n * (double)k / t * 1e-12);
  }
};

// fp16 NHWC convolution with a ReLU epilogue, square stride / padding / dilation.
struct ConvBenchmark {
  size_t n = 0, c = 0, h = 0, w = 0, k = 0, r = 0, s = 0, stride = 1, pad = 0, dilation = 1;
  ConvGeometry g;
  DeviceBuffer x, wt, y;
  std::string error;

  bool init(size_t n_, size_t c_, size_t h_, size_t w_, size_t k_, size_t r_, size_t s_, size_t stride_,
            size_t pad_, size_t dilation_) {
    n = n_; c = c_; h = h_; w = w_; k = k_; r = r_; s = s_;
    stride = stride_; pad = pad_; dilation = dilation_;
    if (make_conv_geometry((int)n, (int)h, (int)w, (int)c, (int)k, (int)r, (int)s, (int)stride,
                           (int)stride, (int)pad, (int)pad, (int)dilation, (int)dilation,
                           &g) != TRACEA_SUCCESS) {
      error = last_error_text();
      return false;
    }
    const size_t ho = (size_t)g.block.h_out, wo = (size_t)g.block.w_out;
    if (!x.alloc(n * h * w * c * 2) || !wt.alloc(k * r * s * c * 2) || !y.alloc(n * ho * wo * k * 2)) {
      (void)hipGetLastError();
      error = "device allocation failed";
      return false;
    }
    launch_fill_uniform(x.p, n * h * w * c, DT_F16, 3u, 1.0f, nullptr);
    launch_fill_uniform(wt.p, k * r * s * c, DT_F16, 4u, sqrtf(3.0f / (float)(r * s * c)), nullptr);
    return true;
  }
  float measure(int variant) {
    const size_t ho = (size_t)g.block.h_out, wo = (size_t)g.block.w_out;
    const uint64_t sx[4] = {n, h, w, c}, sw[4] = {k, r, s, c}, sy[4] = {n, ho, wo, k};
    TraceaTensorView vx{x.p, 4, sx, nullptr, TRACEA_DTYPE_FLOAT16, 0};
    TraceaTensorView vw{wt.p, 4, sw, nullptr, TRACEA_DTYPE_FLOAT16, 0};
    TraceaTensorView vy{y.p, 4, sy, nullptr, TRACEA_DTYPE_FLOAT16, 0};
    TraceaConv2dParams cp{(uint32_t)stride, (uint32_t)stride, (uint32_t)pad, (uint32_t)pad,
                          (uint32_t)dilation, (uint32_t)dilation, 1, TRACEA_EPILOGUE_RELU, nullptr};
    const int saved = forced_variant("conv2d");
    set_forced_variant("conv2d", variant);
    const double t = time_launches(
        [&]() { return dispatch_conv2d_kind(vx, vw, nullptr, nullptr, &vy, cp) == TRACEA_SUCCESS; }, 3, 10);
    set_forced_variant("conv2d", saved);
    if (t <= 0.0) {
      error = last_error_text();
      return 0.0f;
    }
    if (last_variant("conv2d") != variant) {  // (as for the GEMM: a substitute's time is not this variant's)
      error = "the dispatcher ran another variant in its place";
      return 0.0f;
    }
    return (float)(2.0 * (double)g.m_gemm * (double)g.n_gemm * (double)g.k_gemm / t * 1e-12);
  }
};

bool gemm_dims_ok(size_t m, size_t n, size_t k) {
  return m != 0 && n != 0 && k != 0 && k % 8 == 0 && m < (1u << 31) && n < (1u << 31) && k < (1u << 31);
}

bool conv_dims_ok(size_t n, size_t c, size_t h, size_t w, size_t k, size_t r, size_t s, size_t stride,
                  size_t dilation, std::string *why) {
  if (n == 0 || c == 0 || h == 0 || w == 0 || k == 0 || r == 0 || s == 0 || stride == 0 || dilation == 0) {
    *why = "dimensions, stride and dilation must be positive";
    return false;
  }
  if (c % 8 != 0) {
    *why = "input channels must be a multiple of 8";
    return false;
  }
  return true;
}

}  // namespace

// The winner of a measurement, in the tuning history as well (the reference's orchestrator records what
// it selects, src/optimizer/orchestrator.rs:68-81): key "HardwareId:OpFingerprint:Precision".
static void record_history(const std::string &cache_key, const CacheEntry &e, const char *precision) {
  HistoryEntry h;
  h.config = e.config;
  h.tflops = e.score;
  h.timestamp = e.timestamp;
  h.explanation = tuning_history_explanation(h.backend, h.tflops, "Selected based on highest benchmarking score in real-time.");
  tuning_history_record(std::string(tuning_device_name()) + ":" + cache_key + ":" + precision, h);
}

TraceaResult tune_gemm(size_t m, size_t n, size_t k) {
  if (!runtime_ready()) return failure("tracea_init has not been called");
  if (!gemm_dims_ok(m, n, k)) return failure("tune_gemm: dimensions must be positive, K a multiple of 8");
  GemmBenchmark bench;
  if (!bench.init(m, n, k)) return failure("tune_gemm: " + bench.error);
  int best = -1;
  float best_tflops = 0.0f;
  for (int i = 0; i < contraction_variant_count(); ++i) {
    const float tf = bench.measure(i);
    if (tf > best_tflops) {
      best_tflops = tf;
      best = i;
    }
  }
  if (best < 0) return failure("tune_gemm: no variant ran: " + bench.error);
  CacheEntry e;
  e.config = config_for_contraction_variant(best);
  e.score = best_tflops;
  e.timestamp = now_seconds();
  e.operand_dtype = "f16";
  e.b_layout = "k_contiguous";
  tuning_cache_put(gemm_cache_key(m, n, k, tuning_device_name()), e, true);
  record_history(gemm_cache_key(m, n, k, tuning_device_name()), e, "F16");
  return success(e.config, e.score);
}

TraceaResult tune_conv2d(size_t n, size_t c, size_t h, size_t w, size_t k, size_t r, size_t s,
                         size_t stride, size_t pad, size_t dilation) {
  if (!runtime_ready()) return failure("tracea_init has not been called");
  std::string why;
  if (!conv_dims_ok(n, c, h, w, k, r, s, stride, dilation, &why)) return failure("tune_conv2d: " + why);
  ConvBenchmark bench;
  if (!bench.init(n, c, h, w, k, r, s, stride, pad, dilation)) return failure("tune_conv2d: " + bench.error);
  int best = -1;
  float best_tflops = 0.0f;
  for (int i = 0; i < contraction_variant_count(); ++i) {
    const float tf = bench.measure(i);
    if (tf > best_tflops) {
      best_tflops = tf;
      best = i;
    }
  }
  if (best < 0) return failure("tune_conv2d: no variant ran: " + bench.error);
  CacheEntry e;
  e.config = config_for_contraction_variant(best);
  e.config.layout_policy = "NHWC";
  e.score = best_tflops;
  e.timestamp = now_seconds();
  e.operand_dtype = "f16";
  e.b_layout = "k_contiguous";
  ConvProblem p;
  p.batch = (uint32_t)n; p.h_in = (uint32_t)h; p.w_in = (uint32_t)w; p.c_in = (uint32_t)c;
  p.c_out = (uint32_t)k; p.kernel_h = (uint32_t)r; p.kernel_w = (uint32_t)s;
  p.stride = (uint32_t)stride; p.pad = (uint32_t)pad; p.dilation = (uint32_t)dilation;
  tuning_cache_put(conv_cache_key(p, tuning_device_name()), e, true);
  record_history(conv_cache_key(p, tuning_device_name()), e, "F16");
  return success(e.config, e.score);
}

// AutoTuner::optimize on the device: cache first, then every candidate
// (iterations 0) or an expected-improvement-guided subset of them.
TraceaResult autotune_gemm(size_t m, size_t n, size_t k, uint32_t iterations) {
  if (!runtime_ready()) return failure("tracea_init has not been called");
  if (!gemm_dims_ok(m, n, k)) return failure("autotune_gemm: dimensions must be positive, K a multiple of 8");
  GemmBenchmark bench;
  bool ready = false;
  auto measure = [&](const PipelineConfig &cfg) -> float {
    const int vi = contraction_variant_for_config(cfg);
    if (vi < 0) return 0.0f;
    if (!ready) {
      if (!bench.init(m, n, k)) return 0.0f;
      ready = true;
    }
    return bench.measure(vi);
  };
  AutoTuner tuner(HardwareProfile::mi355x());
  tuner.hardware_id = tuning_device_name();
  PipelineConfig best;
  if (iterations == 0) {
    best = tuner.optimize((uint32_t)m, (uint32_t)n, (uint32_t)k, measure);
  } else {
    const std::string key = gemm_cache_key(m, n, k, tuner.hardware_id);
    CacheEntry hit;
    if (tuning_cache_get(key, &hit)) return success(hit.config, hit.score);
    best = tuner.optimize_guided((uint32_t)m, (uint32_t)n, (uint32_t)k,
                                 propose_gemm_configs((uint32_t)m, (uint32_t)n, (uint32_t)k), measure,
                                 iterations, AcquisitionFunction::EI);
    if (tuner.best_score > 0.0f) {
      CacheEntry e;
      e.config = best;
      e.score = tuner.best_score;
      e.timestamp = now_seconds();
      tuning_cache_put(key, e, true);
    }
  }
  if (!(tuner.best_score > 0.0f)) return failure("autotune_gemm: no candidate ran: " + bench.error);
  return success(best, tuner.best_score);
}

TraceaResult autotune_conv2d(size_t n, size_t c, size_t h, size_t w, size_t k, size_t r, size_t s,
                             size_t stride, size_t pad, size_t dilation, uint32_t iterations) {
  if (!runtime_ready()) return failure("tracea_init has not been called");
  std::string why;
  if (!conv_dims_ok(n, c, h, w, k, r, s, stride, dilation, &why)) return failure("autotune_conv2d: " + why);
  ConvProblem p;
  p.batch = (uint32_t)n; p.h_in = (uint32_t)h; p.w_in = (uint32_t)w; p.c_in = (uint32_t)c;
  p.c_out = (uint32_t)k; p.kernel_h = (uint32_t)r; p.kernel_w = (uint32_t)s;
  p.stride = (uint32_t)stride; p.pad = (uint32_t)pad; p.dilation = (uint32_t)dilation;
  ConvBenchmark bench;
  bool ready = false;
  auto measure = [&](const PipelineConfig &cfg) -> float {
    const int vi = contraction_variant_for_config(cfg);
    if (vi < 0) return 0.0f;
    if (!ready) {
      if (!bench.init(n, c, h, w, k, r, s, stride, pad, dilation)) return 0.0f;
      ready = true;
    }
    return bench.measure(vi);
  };
  AutoTuner tuner(HardwareProfile::mi355x());
  tuner.hardware_id = tuning_device_name();
  PipelineConfig best;
  if (iterations == 0) {
    best = tuner.optimize_conv(p, measure).base;
  } else {
    const std::string key = conv_cache_key(p, tuner.hardware_id);
    CacheEntry hit;
    if (tuning_cache_get(key, &hit)) return success(hit.config, hit.score);
    const uint32_t mg = p.batch * p.h_out() * p.w_out(), kg = p.c_in * p.kernel_h * p.kernel_w;
    best = tuner.optimize_guided(mg, p.c_out, kg, propose_conv_configs(mg, p.c_out, kg), measure, iterations,
                                 AcquisitionFunction::EI);
    if (tuner.best_score > 0.0f) {
      CacheEntry e;
      e.config = best;
      e.score = tuner.best_score;
      e.timestamp = now_seconds();
      tuning_cache_put(key, e, true);
    }
  }
  if (!(tuner.best_score > 0.0f)) return failure("autotune_conv2d: no candidate ran: " + bench.error);
  best.layout_policy = "NHWC";
  return success(best, tuner.best_score);
}

TraceaResult tune_fa2(size_t b, size_t h, size_t s, size_t d, bool causal) {
  if (!runtime_ready()) return failure("tracea_init has not been called");
  if (b == 0 || h == 0 || s == 0 || (d != 64 && d != 128))
    return failure("tune_fa2: B, H, S must be positive and D 64 or 128");
  const size_t elems = b * h * s * d;
  DeviceBuffer q, k, v, o;
  if (!q.alloc(elems * 2) || !k.alloc(elems * 2) || !v.alloc(elems * 2) || !o.alloc(elems * 2)) {
    (void)hipGetLastError();
    return failure("tune_fa2: device allocation failed");
  }
  launch_fill_uniform(q.p, elems, DT_BF16, 5u, 1.7f, nullptr);
  launch_fill_uniform(k.p, elems, DT_BF16, 6u, 1.7f, nullptr);
  launch_fill_uniform(v.p, elems, DT_BF16, 7u, 1.7f, nullptr);
  const uint64_t sh[4] = {b, h, s, d};
  TraceaTensorView vq{q.p, 4, sh, nullptr, TRACEA_DTYPE_BFLOAT16, 0};
  TraceaTensorView vk{k.p, 4, sh, nullptr, TRACEA_DTYPE_BFLOAT16, 0};
  TraceaTensorView vv{v.p, 4, sh, nullptr, TRACEA_DTYPE_BFLOAT16, 0};
  TraceaTensorView vo{o.p, 4, sh, nullptr, TRACEA_DTYPE_BFLOAT16, 0};
  TraceaAttentionParams ap{(uint8_t)(causal ? 1 : 0), TRACEA_SOFTMAX_AUTO, 0.0f, nullptr};
  const int saved = forced_variant("attention");
  const double flops = 4.0 * (double)b * (double)h * (double)s * (double)s * (double)d;
  int best = -1;
  double best_tflops = 0.0;
  std::string err;
  for (int i = 0; i < attention_variant_count(); ++i) {
    AttentionArgs probe{};
    probe.D = (int)d;
    probe.S = (int)s;
    probe.k_ss = probe.v_ss = (long long)d;
    probe.scale_log2 = 1.0f;
    probe.causal = causal ? 1 : 0;
    if (!attention_variant(i).feasible(probe)) continue;
    set_forced_variant("attention", i);
    const double t = time_launches(
        [&]() { return dispatch_attention(vq, vk, vv, &vo, ap) == TRACEA_SUCCESS; }, 2, 5);
    if (t <= 0.0) {
      err = last_error_text();
      continue;
    }
    // (a member that cannot run the problem gives way to the rule's choice: that time is not this member's)
    if (last_variant("attention") != i) continue;
    const double tf = flops / t * 1e-12;
    if (tf > best_tflops) {
      best_tflops = tf;
      best = i;
    }
  }
  set_forced_variant("attention", saved);
  if (best < 0) return failure("tune_fa2: no variant ran: " + err);
  CacheEntry e;
  e.config = config_for_attention_variant(best);
  e.score = (float)best_tflops;
  e.timestamp = now_seconds();
  // key of the reference's attention adapter (src/kernels/attention/cuda_adapter.rs)
  const std::string key = attention_cache_key(b, s, h, d, causal);
  tuning_cache_put(key, e, true);
  record_history(key, e, "BF16");
  return success(e.config, e.score);
}

}  // namespace tracea_amd
