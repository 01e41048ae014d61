// Argument checking and kernel dispatch for tracea_gemm / tracea_conv2d /
// tracea_attention.  Validation order and status codes follow the reference's
// FFI layer (tracea-ffi/src/lib.rs:151-181; src/interface/c_bindings.rs:206-495):
// runtime not initialised -> UNKNOWN_ERROR; NULL pointers and wrong ranks ->
// INVALID_PARAMS; groups/dtype/layout the kernels do not cover ->
// UNSUPPORTED_CONFIG; host pointers -> CPU_ERROR; HIP failures -> CUDA_ERROR.
#include "dispatch.hpp"
#include "tile_graph.hpp"

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstring>
#include <map>
#include <mutex>

#include "tuner.hpp"
#include "tuning_cache.hpp"

namespace tracea_amd {

namespace {

struct View {
  void *ptr = nullptr;
  int rank = 0;
  long long shape[4] = {0, 0, 0, 0};
  long long stride[4] = {0, 0, 0, 0};
  int dtype = 0;
  int device = -1;
};

// Copies a TraceaTensorView; a NULL stride array means contiguous row-major.
TraceaStatus read_view(const char *what, const TraceaTensorView &t, int want_rank, View *v) {
  if (t.ptr == nullptr) return fail(TRACEA_INVALID_PARAMS, "%s: data pointer is NULL", what);
  if (t.shape == nullptr) return fail(TRACEA_INVALID_PARAMS, "%s: shape pointer is NULL", what);
  if ((int)t.rank != want_rank)
    return fail(TRACEA_INVALID_PARAMS, "%s: expected rank %d, got %u", what, want_rank, t.rank);
  v->ptr = t.ptr;
  v->rank = (int)t.rank;
  for (int i = 0; i < want_rank; ++i) v->shape[i] = (long long)t.shape[i];
  if (t.stride != nullptr) {
    for (int i = 0; i < want_rank; ++i) v->stride[i] = (long long)t.stride[i];
  } else {
    long long s = 1;
    for (int i = want_rank - 1; i >= 0; --i) {
      v->stride[i] = s;
      s *= v->shape[i];
    }
  }
  v->dtype = (int)t.dtype;
  v->device = t.device_id;
  return TRACEA_SUCCESS;
}

bool is_half(int dt) { return dt == TRACEA_DTYPE_FLOAT16 || dt == TRACEA_DTYPE_BFLOAT16; }
bool is_float_type(int dt) { return dt == TRACEA_DTYPE_FLOAT32 || is_half(dt); }
int elem_size(int dt) { return dt == TRACEA_DTYPE_FLOAT32 ? 4 : 2; }
bool aligned(const void *p, size_t a) { return (((uintptr_t)p) & (a - 1)) == 0; }

const char *dtype_name(int dt) {
  switch (dt) {
    case TRACEA_DTYPE_FLOAT32: return "f32";
    case TRACEA_DTYPE_FLOAT16: return "f16";
    case TRACEA_DTYPE_BFLOAT16: return "bf16";
    case TRACEA_DTYPE_INT32: return "i32";
    case TRACEA_DTYPE_INT8: return "i8";
    default: return "?";
  }
}

TraceaStatus check_device(const char *what, int device) {
  if (device < 0)
    return fail(TRACEA_CPU_ERROR,
                "%s: host memory (device_id -1) is not supported; this library has no CPU arm",
                what);
  if (device >= runtime_device_count())
    return fail(TRACEA_INVALID_PARAMS, "%s: device_id %d out of range (%d devices)", what, device,
                runtime_device_count());
  return TRACEA_SUCCESS;
}

// Makes `device` current for the lifetime of the object.
struct DeviceScope {
  int prev = -1;
  bool switched = false;
  hipError_t err = hipSuccess;
  explicit DeviceScope(int device) {
    err = hipGetDevice(&prev);
    if (err == hipSuccess && prev != device) {
      err = hipSetDevice(device);
      switched = err == hipSuccess;
    }
  }
  ~DeviceScope() {
    if (switched) (void)hipSetDevice(prev);
  }
};

// ---- epilogue chains ---------------------------------------------------------

// TraceaEpilogueKind -> operator list, as src/interface/c_bindings.rs:144-197:
// an operator whose tensor is absent is dropped, not an error.
int kind_to_ops(int kind, const TraceaTensorView *bias, const TraceaTensorView *residual,
                TraceaEpilogueOp *ops) {
  int n = 0;
  auto bias_op = [&](TraceaEpilogueOpKind k) {
    if (bias == nullptr) return;
    ops[n] = TraceaEpilogueOp{k, bias->dtype, bias->ptr, nullptr, nullptr, nullptr, 0.0f, 0};
    ++n;
  };
  auto res_op = [&]() {
    if (residual == nullptr) return;
    ops[n] = TraceaEpilogueOp{TRACEA_EPI_OP_RESIDUAL_ADD, residual->dtype, residual->ptr, nullptr,
                              nullptr, nullptr, 0.0f, -1 /* resolved from the view */};
    ++n;
  };
  auto plain = [&](TraceaEpilogueOpKind k) {
    ops[n] = TraceaEpilogueOp{k, TRACEA_DTYPE_FLOAT32, nullptr, nullptr, nullptr, nullptr, 0.0f, 0};
    ++n;
  };
  switch (kind) {
    case TRACEA_EPILOGUE_IDENTITY: break;
    case TRACEA_EPILOGUE_BIAS_ADD: bias_op(TRACEA_EPI_OP_BIAS_ADD); break;
    case TRACEA_EPILOGUE_RELU: plain(TRACEA_EPI_OP_RELU); break;
    case TRACEA_EPILOGUE_GELU: plain(TRACEA_EPI_OP_GELU); break;
    case TRACEA_EPILOGUE_SILU: plain(TRACEA_EPI_OP_SILU); break;
    case TRACEA_EPILOGUE_BIAS_RELU: bias_op(TRACEA_EPI_OP_BIAS_ADD); plain(TRACEA_EPI_OP_RELU); break;
    case TRACEA_EPILOGUE_BIAS_SILU: bias_op(TRACEA_EPI_OP_BIAS_ADD_SILU); break;
    case TRACEA_EPILOGUE_RESIDUAL: res_op(); break;
    case TRACEA_EPILOGUE_RESIDUAL_RELU: res_op(); plain(TRACEA_EPI_OP_RELU); break;
    default: return -1;
  }
  return n;
}

// Validates a caller-supplied chain and lowers it to device form.  `rows` and
// `channels` are the GEMM view of the output; res_ld_default is the row stride
// assumed for a residual whose ld is 0.
TraceaStatus lower_chain(const char *what, const TraceaEpilogueOp *ops, uint32_t n_ops,
                         long long channels, long long res_ld_default, EpilogueChain *chain) {
  if (n_ops > TRACEA_MAX_EPILOGUE_OPS)
    return fail(TRACEA_INVALID_PARAMS, "%s: %u epilogue operators, at most %d are supported", what,
                n_ops, TRACEA_MAX_EPILOGUE_OPS);
  if (n_ops > 0 && ops == nullptr)
    return fail(TRACEA_INVALID_PARAMS, "%s: epilogue operator list is NULL", what);
  chain->n_ops = 0;
  for (uint32_t i = 0; i < n_ops; ++i) {
    const TraceaEpilogueOp &op = ops[i];
    EpilogueOpDev d{};
    d.kind = (int)op.kind;
    d.dtype = DT_F32;
    d.epsilon = op.epsilon;
    d.ld = 0;
    switch (op.kind) {
      case TRACEA_EPI_OP_NONE: continue;
      case TRACEA_EPI_OP_RELU:
      case TRACEA_EPI_OP_GELU:
      case TRACEA_EPI_OP_SILU: break;
      case TRACEA_EPI_OP_BIAS_ADD:
      case TRACEA_EPI_OP_BIAS_ADD_SILU:
      case TRACEA_EPI_OP_RESIDUAL_ADD:
        if (op.p0 == nullptr)
          return fail(TRACEA_INVALID_PARAMS, "%s: epilogue operator %u has a NULL tensor", what, i);
        if (!is_float_type(op.dtype))
          return fail(TRACEA_UNSUPPORTED_CONFIG, "%s: epilogue operator %u: dtype %s unsupported",
                      what, i, dtype_name(op.dtype));
        d.dtype = op.dtype;
        d.p0 = op.p0;
        if (op.kind == TRACEA_EPI_OP_RESIDUAL_ADD) d.ld = op.ld > 0 ? op.ld : res_ld_default;
        break;
      case TRACEA_EPI_OP_BATCHNORM:
        if (!op.p0 || !op.p1 || !op.p2 || !op.p3)
          return fail(TRACEA_INVALID_PARAMS, "%s: BatchNorm needs gamma, beta, mean and var", what);
        // the kernels read these vectors as fp32 whatever the operator says: anything else is refused
        if (op.dtype != TRACEA_DTYPE_FLOAT32)
          return fail(TRACEA_UNSUPPORTED_CONFIG, "%s: epilogue operator %u: BatchNorm parameters must be float32, not %s",
                      what, i, dtype_name(op.dtype));
        d.p0 = op.p0; d.p1 = op.p1; d.p2 = op.p2; d.p3 = op.p3;
        break;
      case TRACEA_EPI_OP_SCALE_SHIFT:
        if (!op.p0 || !op.p1)
          return fail(TRACEA_INVALID_PARAMS, "%s: ScaleShift needs scale and shift", what);
        if (op.dtype != TRACEA_DTYPE_FLOAT32)
          return fail(TRACEA_UNSUPPORTED_CONFIG, "%s: epilogue operator %u: scale and shift must be float32, not %s",
                      what, i, dtype_name(op.dtype));
        d.p0 = op.p0; d.p1 = op.p1;
        break;
      default:
        return fail(TRACEA_INVALID_PARAMS, "%s: unknown epilogue operator kind %d", what,
                    (int)op.kind);
    }
    chain->ops[chain->n_ops++] = d;
  }
  (void)channels;
  return TRACEA_SUCCESS;
}

// Checks the optional bias / residual views of the TraceaEpilogueKind calls
// against the output geometry and fills the residual row stride.
TraceaStatus check_bias_residual(const char *what, const TraceaTensorView *bias,
                                 const TraceaTensorView *residual, long long channels,
                                 const View &out_view, int device, TraceaEpilogueOp *ops, int n) {
  if (bias != nullptr) {
    if (bias->ptr == nullptr || bias->shape == nullptr)
      return fail(TRACEA_INVALID_PARAMS, "%s: bias view has a NULL pointer", what);
    if (bias->rank != 1 || (long long)bias->shape[0] != channels)
      return fail(TRACEA_INVALID_PARAMS, "%s: bias must have shape [%lld]", what, channels);
    if (bias->stride != nullptr && bias->stride[0] != 1)
      return fail(TRACEA_UNSUPPORTED_CONFIG, "%s: bias must be contiguous", what);
    if (!is_float_type(bias->dtype))
      return fail(TRACEA_UNSUPPORTED_CONFIG, "%s: bias dtype %s unsupported", what,
                  dtype_name(bias->dtype));
    if (bias->device_id != device)
      return fail(TRACEA_INVALID_PARAMS, "%s: bias lives on device %d, output on %d", what,
                  bias->device_id, device);
  }
  if (residual != nullptr) {
    View r;
    TraceaStatus st = read_view("residual", *residual, out_view.rank, &r);
    if (st != TRACEA_SUCCESS) return st;
    for (int i = 0; i < r.rank; ++i)
      if (r.shape[i] != out_view.shape[i])
        return fail(TRACEA_INVALID_PARAMS, "%s: residual shape differs from the output shape", what);
    if (!is_float_type(r.dtype))
      return fail(TRACEA_UNSUPPORTED_CONFIG, "%s: residual dtype %s unsupported", what,
                  dtype_name(r.dtype));
    if (r.device != device)
      return fail(TRACEA_INVALID_PARAMS, "%s: residual lives on device %d, output on %d", what,
                  r.device, device);
    // channel-contiguous rows with one row stride across all leading dims
    const int last = r.rank - 1;
    if (r.stride[last] != 1)
      return fail(TRACEA_UNSUPPORTED_CONFIG, "%s: residual channels must be contiguous", what);
    const long long ld = r.rank >= 2 ? r.stride[last - 1] : channels;
    long long expect = ld;
    for (int i = last - 1; i >= 0; --i) {
      if (r.stride[i] != expect)
        return fail(TRACEA_UNSUPPORTED_CONFIG, "%s: residual must be densely strided over rows", what);
      expect *= r.shape[i];
    }
    for (int i = 0; i < n; ++i)
      if (ops[i].kind == TRACEA_EPI_OP_RESIDUAL_ADD && ops[i].ld < 0) ops[i].ld = ld;
  }
  return TRACEA_SUCCESS;
}

// A forced variant belongs to the thread that set it: the tuner (and a test) forces a variant around its own
// launches, and another thread dispatching meanwhile must keep its own choice.
thread_local int t_forced_contraction = -1, t_forced_conv = -1, t_forced_attention = -1;
std::atomic<bool> g_split_k_enabled{true};
std::atomic<bool> g_split_k_one_launch{true};
std::atomic<bool> g_conv_transpose_by_phase{true};
// variant the calling thread's latest launch of each operator used (-1: none,
// or a kernel outside the variant tables)
thread_local int t_last_contraction = -1, t_last_conv = -1, t_last_attention = -1;
thread_local int t_last_splits = 1;  // K ranges of the calling thread's latest gemm / conv2d launch
thread_local int t_last_split_launches = 1;  // kernels that launch took: 2 when a reduction kernel followed

TraceaStatus hip_status(const char *what, int e) {
  if (e == 0) return TRACEA_SUCCESS;
  return fail(TRACEA_CUDA_ERROR, "%s: %s", what, hipGetErrorString((hipError_t)e));
}

}  // namespace

TraceaStatus dispatch_lower_chain(const char *what, const TraceaEpilogueOp *ops, uint32_t n_ops, long long channels,
                                  EpilogueChain *chain) {
  return lower_chain(what, ops, n_ops, channels, channels, chain);
}

void set_split_k_enabled(bool on) { g_split_k_enabled.store(on); }
void set_split_k_one_launch(bool on) { g_split_k_one_launch.store(on); }
int last_split_k_launches() { return t_last_split_launches; }
void set_conv_transpose_by_phase(bool on) { g_conv_transpose_by_phase.store(on); }

// Regrouped filter banks of the by-phase transposed convolution, kept between calls when the caller
// has switched the cache on (tracea_set_conv_transpose_filter_cache).
namespace {
std::atomic<bool> g_ct_filter_cache{false};
// (one array of equal words: a struct of mixed members has padding bytes, which a copy into the map need
// not preserve and a bytewise comparison would read)
struct CtFilterKey {
  long long v[17];  // device, filter pointer, dims[4], strides[4], dtype, stride h/w, padding h/w, output h/w
  bool operator<(const CtFilterKey &o) const {
    for (int i = 0; i < 17; ++i)
      if (v[i] != o.v[i]) return v[i] < o.v[i];
    return false;
  }
};
std::mutex g_ct_filter_mu;
std::map<CtFilterKey, void *> g_ct_filters;
}  // namespace
void set_conv_transpose_filter_cache(bool on) { g_ct_filter_cache.store(on); }
void conv_transpose_filter_cache_clear() {
  std::lock_guard<std::mutex> lk(g_ct_filter_mu);
  if (g_ct_filters.empty()) return;
  int prev = 0;
  const bool have_prev = hipGetDevice(&prev) == hipSuccess;
  for (auto &kv : g_ct_filters) {
    if (hipSetDevice((int)kv.first.v[0]) == hipSuccess) {
      (void)hipDeviceSynchronize();  // a launch that reads the copy may still be in flight
      (void)hipFree(kv.second);
    }
  }
  g_ct_filters.clear();
  if (have_prev) (void)hipSetDevice(prev);
}
int last_split_k() { return t_last_splits; }

void set_forced_variant(const char *op, int index) {
  if (!strcmp(op, "gemm")) t_forced_contraction = index;
  else if (!strcmp(op, "conv2d")) t_forced_conv = index;
  else if (!strcmp(op, "attention")) t_forced_attention = index;
}
int last_variant(const char *op) {
  if (!strcmp(op, "gemm")) return t_last_contraction;
  if (!strcmp(op, "conv2d")) return t_last_conv;
  if (!strcmp(op, "attention")) return t_last_attention;
  return -1;
}
int forced_variant(const char *op) {
  if (!strcmp(op, "gemm")) return t_forced_contraction;
  if (!strcmp(op, "conv2d")) return t_forced_conv;
  if (!strcmp(op, "attention")) return t_forced_attention;
  return -1;
}

// ---- reciprocals ---------------------------------------------------------------
// The reference's magic_u32 (src/emitter/cuda/conv.rs:6-16) always ends at
// p = 32, i.e. magic = ceil(2^32/d) with no extra shift, which is exact only
// while n*d < 2^32.  That pair is kept whenever it is exact for the largest
// dividend (so the packed block equals the reference's bit for bit); beyond
// it the shift floor(log2 d) is used, which is exact for every n < 2^31.
void magic_for_divisor(uint32_t d, uint64_t n_max, uint32_t *magic, uint32_t *shift) {
  *magic = 0;
  *shift = 0;
  if (d <= 1) return;
  if ((d & (d - 1)) == 0) {
    *shift = (uint32_t)__builtin_ctz(d);
    return;
  }
  if (n_max * (uint64_t)d < (1ull << 32)) {
    *magic = (uint32_t)(((1ull << 32) + d - 1) / d);
    return;
  }
  const uint32_t s = 31u - (uint32_t)__builtin_clz(d);
  *magic = (uint32_t)((((unsigned __int128)1 << (32 + s)) + d - 1) / d);
  *shift = s;
}

TraceaStatus make_conv_geometry(int n, int h, int w, int c, int k, int r, int s, int stride_h,
                                int stride_w, int pad_h, int pad_w, int dil_h, int dil_w,
                                ConvGeometry *out) {
  if (n <= 0 || h <= 0 || w <= 0 || c <= 0 || k <= 0 || r <= 0 || s <= 0)
    return fail(TRACEA_INVALID_PARAMS, "conv2d: every dimension must be positive");
  if (stride_h <= 0 || stride_w <= 0 || dil_h <= 0 || dil_w <= 0 || pad_h < 0 || pad_w < 0)
    return fail(TRACEA_INVALID_PARAMS, "conv2d: stride and dilation must be >= 1, padding >= 0");
  const long long ho = ((long long)h + 2 * pad_h - (long long)dil_h * (r - 1) - 1) / stride_h + 1;
  const long long wo = ((long long)w + 2 * pad_w - (long long)dil_w * (s - 1) - 1) / stride_w + 1;
  if ((long long)h + 2 * pad_h < (long long)dil_h * (r - 1) + 1 ||
      (long long)w + 2 * pad_w < (long long)dil_w * (s - 1) + 1 || ho <= 0 || wo <= 0)
    return fail(TRACEA_INVALID_PARAMS, "conv2d: filter larger than the padded input");
  const long long m_gemm = (long long)n * ho * wo, k_gemm = (long long)r * s * c;
  if (m_gemm >= (1ll << 31) || k_gemm >= (1ll << 31) || (long long)n * h * w * c >= (1ll << 40))
    return fail(TRACEA_UNSUPPORTED_CONFIG, "conv2d: problem too large for 32-bit row indices");
  TraceaConvParamsBlock &b = out->block;
  b.batch = n; b.h_in = h; b.w_in = w; b.c_in = c; b.k_out = k;
  b.h_out = (int)ho; b.w_out = (int)wo; b.r_sz = r; b.s_sz = s;
  b.stride = stride_h; b.pad = pad_h; b.dilation = dil_h;
  magic_for_divisor((uint32_t)(ho * wo), (uint64_t)m_gemm, &b.hw_m, &b.hw_s);
  magic_for_divisor((uint32_t)wo, (uint64_t)(ho * wo), &b.w_m, &b.w_s);
  magic_for_divisor((uint32_t)(s * c), (uint64_t)k_gemm + 1024, &b.sic_m, &b.sic_s);
  magic_for_divisor((uint32_t)c, (uint64_t)s * c, &b.c_m, &b.c_s);
  out->stride_h = stride_h; out->stride_w = stride_w;
  out->pad_h = pad_h; out->pad_w = pad_w;
  out->dil_h = dil_h; out->dil_w = dil_w;
  out->m_gemm = (int)m_gemm; out->n_gemm = k; out->k_gemm = (int)k_gemm;
  return TRACEA_SUCCESS;
}

// ---- variant choice --------------------------------------------------------------
// Cost model: the tile grid is executed in rounds over the 256 compute units;
// a round costs the tile area divided by the efficiency prior of the variant
// (operand re-use of the tile shape x measured gain of its pipeline).  Partial
// tiles at the edges are paid in full through the tile count.  A tuning-cache
// entry, when present, wins over this.
// What the selector knows of the device: CU count, LDS per workgroup and shader clock from the device
// properties of device 0, read once after tracea_init; before that (variant queries without a device)
// the figures of an MI355X.  The rate of a workgroup slot was calibrated at the MI355X's 2.4 GHz and
// scales with the clock; a tuning-cache record of the calibration product (the 4096^3 GEMM on a
// 256x256 direct-to-LDS tile) replaces it by what that device measured.
const DeviceLimits &device_limits() {
  static std::mutex mu;
  static DeviceLimits lim;
  static std::atomic<bool> settled{false};  // read from the device: from then on nothing changes and nobody locks
  static bool from_device = false;
  if (settled.load(std::memory_order_acquire)) return lim;
  std::lock_guard<std::mutex> lk(mu);
  if (!from_device && runtime_ready()) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, 0) == hipSuccess) {
      if (prop.multiProcessorCount > 0) lim.cus = prop.multiProcessorCount;
      if (prop.sharedMemPerBlockOptin >= 64 * 1024) lim.lds_bytes = (long long)prop.sharedMemPerBlockOptin;
      if (prop.clockRate > 0) lim.clock_ghz = prop.clockRate * 1e-6;
      lim.slot_rate = 1.43e6 * lim.clock_ghz / 2.4;
      CacheEntry e;
      if (tuning_cache_get(gemm_cache_key(4096, 4096, 4096, prop.name), &e) && e.score > 0.0f) {
        const int vi = contraction_variant_for_config(e.config);
        // (a record of the 32x32x16 member only: the selector gives the 16x16x32 members further factors, and a
        // rate divided by less than the selector multiplies by would come out too high)
        if (vi >= 0 && contraction_variant(vi).bm == 256 && contraction_variant(vi).bn == 256 &&
            contraction_variant(vi).pipeline == 2 && contraction_variant(vi).mfma == 32)
          // score TFLOP/s = 2 MAC: MAC per microsecond and CU at the variant's efficiency prior (1.5, x1.04 on 8 waves)
          lim.slot_rate = (double)e.score * 1e6 / 2.0 / lim.cus /
                          (1.5 * (contraction_variant(vi).waves_m * contraction_variant(vi).waves_n == 8 ? 1.04 : 1.0));
      }
    }
    from_device = true;
    settled.store(true, std::memory_order_release);
  }
  return lim;
}

namespace {
// Number of K ranges for a launch of variant v (1: no split) and the extent of one range.
// Pipelines 4 and 5 are convolution kernels of their own (input patch in LDS): they need the
// convolution geometry (plan_conv_patch / plan_conv_filter_resident), never split K and run no GEMM.
inline bool conv_only(const ContractionVariant &v) { return v.pipeline >= 4; }

constexpr int kOneLaunchMaxSplits = 4;  // finest split that runs as one launch (see launch_maybe_split)

int choose_split(const ContractionVariant &v, int M, int N, int K, int *k_split, int min_tiles = 4) {
  const long long tiles = (long long)((M + v.bm - 1) / v.bm) * ((N + v.bn - 1) / v.bn);
  const int nk = (K + v.bk - 1) / v.bk;
  const long long cus = device_limits().cus;
  if (v.bk >= 128 && min_tiles == 4) min_tiles = 2;  // (a range is at least 256 deep, whatever the K tile)
  if (conv_only(v) || tiles * 2 > cus || nk < 2 * min_tiles) return 1;
  long long splits = cus / tiles;
  if (splits > nk / min_tiles) splits = nk / min_tiles;  // at least min_tiles K tiles per range
  if (splits < 2) return 1;
  const int per = (int)((nk + splits - 1) / splits);
  *k_split = per * v.bk;
  return (nk + per - 1) / per;
}

}  // namespace

// Estimated time in microseconds of each variant on the problem, smallest wins:
//   rounds of workgroups over the 256 CUs x multiply-accumulates of one workgroup
//   / (rate of a workgroup slot x the variant's efficiency), plus, for a launch that
//   would be split along K, the reduction pass (launch and fp32 partials at ~3 TB/s).
// The slot rate is calibrated on the 4096^3 GEMM (256x256 tiles, one round, 120 us);
// the estimate then reads 52.8 / 25.9 us for a 3x3 convolution on N32 7x7x512 with
// unsplit 64x64 tiles / 128x128 tiles split four ways, where 53.7 / 29.6 us were measured.
int select_contraction_variant(int m, int n, int k, bool conv, bool b_ncontig) {
  (void)conv;
  const DeviceLimits &dev = device_limits();
  const double cus = (double)dev.cus, slot_rate = dev.slot_rate;  // multiply-accumulates per microsecond and CU at efficiency 1
  int best = -1;
  double best_cost = 0.0;
  for (int i = 0; i < contraction_variant_count(); ++i) {
    const ContractionVariant &v = contraction_variant(i);
    if (conv_only(v)) continue;  // needs the convolution geometry: see plan_conv_patch
    const double gm = (double)((m + v.bm - 1) / v.bm), gn = (double)((n + v.bn - 1) / v.bn);
    int k_split = 0;
    const int splits = g_split_k_enabled.load() ? choose_split(v, m, n, k, &k_split) : 1;
    const double units = gm * gn * splits;
    const double k_per = splits > 1 ? (double)k_split : (double)(k > 0 ? k : 1);
    const double exact = units / cus > 1.0 ? units / cus : 1.0;
    const double rounds = 0.5 * std::ceil(units / cus) + 0.5 * exact;  // co-resident workgroups soften the step
    // operand reuse of the tile relative to 256x256; its square root matches the measured
    // ranking of the tile shapes better than the ratio itself, which overrates large tiles
    // (smaller tiles put more waves on a CU and hide more latency)
    const double reuse = (double)(v.bm * v.bn) / (double)(v.bm + v.bn) / 128.0;
    double prior = reuse > 1.0 ? 1.0 : std::sqrt(reuse);
    // measured on MI355X at 4096^3: the pipelined loops gain ~35 % over the plain
    // one, direct-to-LDS loads a further ~10 %, eight waves ~4 % over four
    prior *= v.pipeline == 2 ? 1.5 : (v.pipeline == 1 ? 1.35 : (v.pipeline == 3 ? 1.25 : 1.0));
    if (v.waves_m * v.waves_n == 8) prior *= 1.04;
    // (256x64 tiles on four waves of 64x64: never the best member in the sweeps over GEMM and ResNet layer shapes,
    // and 74.5 us against 47.2 for 128x64 tiles where the reuse term preferred it: N32 224x224 8->64 7x7 s2)
    if (v.bm == 256 && v.bn == 64 && v.waves_m * v.waves_n == 4) prior *= 0.85;
    // K tiles of 128: a row of an operand tile is 256 contiguous bytes instead of 128, which memory beyond the L2
    // delivers better.  Replayed graphs, K-tile 64 -> 128: M 6272 N 256 K 2304 (ResNet's 14x14 stage at batch 32)
    // 22.3-23.4 -> 17.8-18.4 us, M 1568 N 512 K 4608 (the 7x7 stage) 37.8-40.3 -> 26.3-31.3; from K = 1152 up
    // the deeper tile wins on 64x64 and 128x64 tiles, from 2304 up on 128x128; below it is level or 3 % behind.
    // Only where a CU has one workgroup anyway: with more workgroups than CUs the doubled LDS footprint costs
    // the co-resident workgroups that hide each other's waits (2048^3 on 128x64 tiles 33.4 us against 23.4-24,
    // 1024x4096x1024 17.9 against 13.1).
    if (v.bk == 128) prior *= units <= cus && k >= (v.bm * v.bn >= 128 * 128 ? 2048 : 1024) ? 1.2 : 0.85;
    // The same loop on 16x16x32 MFMAs.  Measured against the 32x32x16 twin (replayed graphs, same box):
    // 256x256 tiles on four waves 104.2-108.7 us, on eight 107.7-110.3, against 116.1-119.6 at 4096^3;
    // 128x128 tiles 5 % faster at 4096^3, 8 % slower at 2048^3, 27 % slower at 1024^3; 128x64 tiles slower
    // everywhere.  (Convolutions and calls with operands of 2 GiB run on the twin: resolve_variant.)
    // Four waves against eight on 16x16x32: 781 against 836 us at 8192^3, 198 against 203 at 8192x2048x8192,
    // 36.3 against 35.0 at 4096x4096x1024 (the four-wave factor also undoes the few-waves penalty below).
    if (v.mfma == 16) prior *= v.bm * v.bn >= 256 * 256 ? (v.waves_m * v.waves_n == 4 ? (k >= 2048 ? 1.35 : 1.2) : 1.06) : 0.9;
    // An N-contiguous B is fetched with two transposing LDS reads per fragment, and four waves have twice the
    // B fragments of eight.  4096^3 with this layout, operands N(0,1)/sqrt(K), replayed graphs, one box: eight
    // waves on 16x16x32 112.6 us, eight on 32x32x16 116.2-119.8, four on 16x16x32 129.6 (the library GEMM itself
    // 107.8): the eight-wave 16x16x32 member runs this layout.  (Before the transposing reads were written as
    // instructions the compiler put a vmcnt(0) in front of each one that followed a tile request: 128-132 and
    // 209 us for the two 16x16x32 members.)
    if (b_ncontig && !conv && v.bm * v.bn >= 256 * 256 && v.waves_m * v.waves_n == 4) prior *= 0.8;
    {
      // A CU with fewer than 8 resident waves (one 4-wave workgroup, the launch too small or
      // the tile's LDS too large for a second) hides less latency.  The fourth root is fitted
      // on 48 convolution shapes (ResNet-18/50 layers at batch 1, 8, 32) and 17 GEMM shapes,
      // every variant timed inside a replayed HIP graph: it moves the choice from 128x128 to
      // 128x64 tiles where the former leave CUs idle, and leaves the other choices alone
      // (defaults within 1.4 % / 1.6 % of the per-shape best in total on the two sets).
      const double lds = (double)v.stages * (v.bm + v.bn) * v.bk * 2.0;
      const double fit = std::floor((double)dev.lds_bytes / lds) < 1.0 ? 1.0 : std::floor((double)dev.lds_bytes / lds);
      const double per_cu = units / cus < 1.0 ? 1.0 : (units / cus > fit ? fit : units / cus);
      const double waves = per_cu * v.waves_m * v.waves_n;
      if (waves < 8.0) prior *= std::sqrt(std::sqrt(waves / 8.0));
    }
    double cost = rounds * (double)v.bm * (double)v.bn * k_per / (slot_rate * prior);
    // (a coarse split on a tile up to 128x128 runs as one launch, see launch_maybe_split: about a microsecond less)
    const bool one_launch = splits <= kOneLaunchMaxSplits && v.bm * v.bn <= 128 * 128 && v.mfma == 32 && g_split_k_one_launch.load();
    if (splits > 1) cost += (one_launch ? 3.0 : 4.0) + (double)splits * m * n * 4.0 / 3.0e6;
    if (best < 0 || cost < best_cost) {
      best_cost = cost;
      best = i;
    }
  }
  return best;
}

namespace {

int pick_contraction(const char *op, const std::string &cache_key, int m, int n, int k, bool conv, int dtype,
                     bool b_ncontig = false) {
  const int forced = forced_variant(op);
  if (forced >= 0) return forced;
  int cached = tuning_cache_lookup_variant(cache_key, dtype, b_ncontig);
  if (cached >= 0) return cached;
  return select_contraction_variant(m, n, k, conv, b_ncontig);
}

// The variant (on 32x32x16 MFMAs) with the same tile shape and the given pipeline mode, or -1.
int twin(int vi, int pipeline) {
  const ContractionVariant &p = contraction_variant(vi);
  for (int i = 0; i < contraction_variant_count(); ++i) {
    const ContractionVariant &v = contraction_variant(i);
    if (v.pipeline == pipeline && v.mfma == 32 && v.bm == p.bm && v.bn == p.bn && v.bk == p.bk &&
        v.waves_m == p.waves_m && v.waves_n == p.waves_n)
      return i;
  }
  return -1;
}

// Replaces a variant that cannot run the problem by the nearest one that can:
// direct-to-LDS loads (pipelines 2 and 3) address operands with 32-bit byte
// offsets, so operands of 2 GiB and more go through registers (`staged`); the
// register-staged pipelined loop (pipeline 1) has no K-tail masking for a GEMM; the members on 16x16x32
// MFMAs exist for a GEMM on pipeline 2.
int resolve_variant(int vi, bool conv, bool staged, bool k_exact, bool b_ncontig) {
  (void)b_ncontig;
  if (contraction_variant(vi).mfma == 16 && (conv || staged)) {
    const int t = twin(vi, 2);  // the member with the same tile on 32x32x16 MFMAs
    if (t >= 0) vi = t;
    else return select_contraction_variant(1024, 1024, 1024, conv);  // (every such member has a twin; not reached)
  }
  int pipe = contraction_variant(vi).pipeline;
  if (pipe >= 4) pipe = 2;  // a convolution-only kernel asked for a GEMM: same tile with streamed operands, if any
  if (pipe >= 2 && staged) pipe = 1;
  if (pipe == 1 && !conv && !k_exact) pipe = 0;
  if (pipe == contraction_variant(vi).pipeline) return vi;
  for (int want = pipe; want >= 0; --want) {
    if (want == 1 && !conv && !k_exact) continue;
    const int t = twin(vi, want);
    if (t >= 0) return t;
  }
  for (int i = 0; i < contraction_variant_count(); ++i)
    if (contraction_variant(i).pipeline == 0) return i;
  return vi;
}

void fill_grid(ContractionArgs *a, const ContractionVariant &v) {
  a->grid_m = (a->M + v.bm - 1) / v.bm;
  a->grid_n = (a->N + v.bn - 1) / v.bn;
  // 8 XCDs each take total/8 consecutive tiles; a group height of 4 (256-row
  // tiles) or 8 (smaller) keeps an XCD's run inside a near-square patch.
  a->group_m = v.bm >= 256 ? 4 : 8;
  if (a->group_m > a->grid_m) a->group_m = a->grid_m;
}

// ---- split-K ---------------------------------------------------------------------
// A problem with few output tiles and a long K leaves most of the 256 CUs idle while a
// handful of workgroups walk K serially (a 3x3 convolution on a 7x7 image with 512
// channels: 8 tiles, 72 K tiles each).  Such a launch is split along K over blockIdx.y;
// the fp32 partial products go to a scratch buffer and a second kernel sums them and runs
// the operator chain.  The scratch buffer is kept per (device, stream), grows on demand up
// to 64 MiB, is never allocated while the stream is being captured into a graph and is
// never freed.
constexpr size_t kSplitScratchCap = 64u << 20;
std::mutex g_scratch_mu;
std::map<std::pair<int, void *>, std::pair<void *, size_t>> g_scratch;

void *splitk_scratch(int device, hipStream_t stream, size_t bytes) {
  if (bytes > kSplitScratchCap) return nullptr;
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  auto &slot = g_scratch[{device, (void *)stream}];
  if (slot.second >= bytes) return slot.first;
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) {
    (void)hipGetLastError();
    return nullptr;
  }
  // A buffer that is outgrown is not freed: launches queued on the stream, and HIP graphs
  // captured from it, may still hold its address.  Sizes double, so everything ever
  // allocated for one stream stays below twice the cap.
  size_t want = 1u << 20;
  while (want < bytes) want <<= 1;
  void *p = nullptr;
  if (hipMalloc(&p, want) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  slot = {p, want};
  return p;
}

// Buffer of the padded operand copies (run_gemm), per (device, stream) like the split-K workspace and by the same
// rules: grows on demand up to a cap, never while its stream is being captured, never freed.
constexpr size_t kPadScratchCap = 1u << 30;
std::map<std::pair<int, void *>, std::pair<void *, size_t>> g_pad_scratch;
void *pad_scratch(int device, hipStream_t stream, size_t bytes) {
  if (bytes > kPadScratchCap) return nullptr;
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  auto &slot = g_pad_scratch[{device, (void *)stream}];
  if (slot.second >= bytes) return slot.first;
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) {
    (void)hipGetLastError();
    return nullptr;
  }
  size_t want = 1u << 20;
  while (want < bytes) want <<= 1;
  void *p = nullptr;
  if (hipMalloc(&p, want) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  slot = {p, want};
  return p;
}

// Ticket counters of the one-launch split, one per tile, kept per (device, stream) like the scratch
// buffer: zero when allocated, and every launch leaves them at zero again.  Null while the stream is
// being captured and the counters do not exist yet.
constexpr int kFuseTiles = 16384;
std::map<std::pair<int, void *>, unsigned *> g_fuse_counters;
unsigned *fuse_counters(int device, hipStream_t stream) {
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  auto &slot = g_fuse_counters[{device, (void *)stream}];
  if (slot != nullptr) return slot;
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) {
    (void)hipGetLastError();
    return nullptr;
  }
  void *p = nullptr;
  if (hipMalloc(&p, kFuseTiles * sizeof(unsigned)) != hipSuccess || hipMemset(p, 0, kFuseTiles * sizeof(unsigned)) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  slot = (unsigned *)p;
  return slot;
}

// A one-launch split whose launch was refused may leave tickets behind (some workgroups ran, some did
// not): the counters of the stream go back to zero, in stream order, unless the stream is being captured
// (then nothing was launched yet and the capture fails as a whole).
void reset_fuse_counters(unsigned *cnt, hipStream_t stream) {
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (cnt == nullptr || hipStreamIsCapturing(stream, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) {
    (void)hipGetLastError();
    return;
  }
  if (hipMemsetAsync(cnt, 0, kFuseTiles * sizeof(unsigned), stream) != hipSuccess) (void)hipGetLastError();
}

// Launches `args` on variant v, split along K when that pays; `chain` is the operator chain
// of the call (args.epi is ignored).
// The workspace of a launch split `splits` ways: the per-stream buffer (null when it cannot be had:
// the launch then runs unsplit), or, for the entry point that must not allocate, the static one,
// where a workspace that does not fit is an error (*st).
void *split_workspace(const char *what, bool static_only, int device, hipStream_t stream, int splits, long long M,
                      long long N, TraceaStatus *st) {
  *st = TRACEA_SUCCESS;
  if (splits <= 1) return nullptr;
  const size_t bytes = (size_t)splits * (size_t)M * (size_t)N * 4;
  if (!static_only) return splitk_scratch(device, stream, bytes);
  if (bytes > (size_t)TRACEA_STATIC_SCRATCH_BYTES) {
    *st = fail(TRACEA_UNSUPPORTED_CONFIG,
               "%s: the launch is split %d ways along K and needs a workspace of %zu bytes; the static workspace "
               "of the no-allocation entry point holds %zu", what, splits, bytes, (size_t)TRACEA_STATIC_SCRATCH_BYTES);
    return nullptr;
  }
  void *p = nullptr;
  const int e = static_scratch_address(device, &p);
  if (e != 0) *st = hip_status("static workspace address", e);
  return p;
}

TraceaStatus launch_maybe_split(const char *what, const ContractionVariant &v, ContractionArgs args,
                                const EpilogueChain &chain, bool conv, int dtype, bool b_ncontig, int device,
                                hipStream_t stream, bool static_only = false) {
  int k_split = 0;
  const int splits = g_split_k_enabled.load() ? choose_split(v, args.M, args.N, args.K, &k_split) : 1;
  t_last_split_launches = 1;
  // One launch: the tile's last workgroup sums the partial products and runs the chain (tiles up to
  // 128x128: the larger kernels do not carry the code; never for the entry point that must not allocate).
  // Up to kOneLaunchMaxSplits K ranges only: one workgroup reads all of a tile's partial products through
  // one CU, where the reduction kernel spreads them over the device.  Measured, 20 launches in a graph:
  // 2 ranges 6.6 us against 7.6, 4 ranges 7.2-7.8 against 8.0-9.3, 9 ranges 8.9 against 7.7, 18 ranges
  // 12.8 against 8.5.
  const long long tiles = (long long)args.grid_m * args.grid_n;
  if (splits > 1 && splits <= kOneLaunchMaxSplits && g_split_k_one_launch.load() && !static_only && v.bm * v.bn <= 128 * 128 && v.mfma == 32 && args.phases <= 1 &&
      args.out_map == 0 && args.tile_list == nullptr && tiles <= kFuseTiles) {
    const size_t bytes = (size_t)tiles * (size_t)splits * (size_t)(v.bm * v.bn) * 4;
    void *fws = splitk_scratch(device, stream, bytes);
    unsigned *cnt = fws != nullptr ? fuse_counters(device, stream) : nullptr;
    if (cnt != nullptr) {
      args.epi = chain;
      args.k_split = k_split;
      args.fuse_ws = (float *)fws;
      args.fuse_count = cnt;
      t_last_splits = splits;
      const TraceaStatus st = hip_status(what, v.launch(args, conv, dtype, b_ncontig, stream));
      if (st != TRACEA_SUCCESS) reset_fuse_counters(cnt, stream);
      return st;
    }
  }
  TraceaStatus ws = TRACEA_SUCCESS;
  void *scratch = split_workspace(what, static_only, device, stream, splits, args.M, args.N, &ws);
  if (ws != TRACEA_SUCCESS) return ws;
  t_last_splits = scratch != nullptr ? splits : 1;
  if (scratch == nullptr) {
    args.epi = chain;
    args.k_split = 0;
    return hip_status(what, v.launch(args, conv, dtype, b_ncontig, stream));
  }
  SplitKReduceArgs r{};
  r.partial = (const float *)scratch;
  r.out = args.C; r.out_dtype = args.out_dtype;
  r.splits = splits; r.M = args.M; r.N = args.N; r.ldc = args.ldc;
  r.epi = chain;
  args.C = scratch;
  args.ldc = args.N;
  args.out_dtype = DT_F32;
  args.epi = EpilogueChain{};
  args.k_split = k_split;
  TraceaStatus st = hip_status(what, v.launch(args, conv, dtype, b_ncontig, stream));
  if (st != TRACEA_SUCCESS) return st;
  t_last_split_launches = 2;
  return hip_status("split-K reduction launch", launch_splitk_reduce(r, stream));
}

// ---- GEMM ----------------------------------------------------------------------
TraceaStatus run_gemm(const View &a, const View &b, const View &c, const EpilogueChain &chain,
                      hipStream_t stream, bool static_only = false) {
  const long long M = a.shape[0], K = a.shape[1], N = b.shape[1];
  t_last_contraction = -1;
  if (M == 0 || N == 0) return TRACEA_SUCCESS;
  DeviceScope scope(c.device);
  if (scope.err != hipSuccess) return hip_status("hipSetDevice", (int)scope.err);

  if (is_half(a.dtype) && b.dtype == a.dtype && K > 0) {
    const bool a_ok = a.stride[1] == 1 && a.stride[0] % 8 == 0 && K % 8 == 0 && aligned(a.ptr, 16);
    const bool b_kcontig = b.stride[0] == 1 && b.stride[1] % 8 == 0 && aligned(b.ptr, 16);
    const bool b_ncontig = b.stride[1] == 1 && b.stride[0] % 8 == 0 && N % 8 == 0 && aligned(b.ptr, 16);
    const bool c_ok = c.stride[1] == 1;
    if (a_ok && (b_kcontig || b_ncontig) && c_ok) {
      ContractionArgs args{};
      args.A = a.ptr; args.B = b.ptr; args.C = c.ptr;
      args.M = (int)M; args.N = (int)N; args.K = (int)K;
      args.lda = a.stride[0];
      args.ldb = b_kcontig ? b.stride[1] : b.stride[0];
      args.ldc = c.stride[0];
      args.out_dtype = c.dtype;
      args.epi = chain;
      char key[160];
      snprintf(key, sizeof(key), "gemm_%lld_%lld_%lld_%s", M, N, K, tuning_device_name());
      int vi = pick_contraction("gemm", key, (int)M, (int)N, (int)K, false, a.dtype, !b_kcontig);
      if (vi < 0) return fail(TRACEA_UNKNOWN_ERROR, "gemm: no kernel variant available");
      // direct-to-LDS variants address operands with 32-bit byte offsets below 2 GiB
      const long long a_extent = ((M - 1) * a.stride[0] + K) * 2;
      const long long b_extent = b_kcontig ? ((N - 1) * b.stride[1] + K) * 2 : ((K - 1) * b.stride[0] + N) * 2;
      const bool small = a_extent < (1ll << 31) && b_extent < (1ll << 31);
      vi = resolve_variant(vi, false, !small, K % contraction_variant(vi).bk == 0, !b_kcontig);
      const ContractionVariant &v = contraction_variant(vi);
      args.a_bytes = (unsigned)(small ? a_extent : 0);
      args.b_bytes = (unsigned)(small ? b_extent : 0);
      fill_grid(&args, v);
      t_last_contraction = vi;
      return launch_maybe_split("gemm launch", v, args, chain, false, a.dtype, !b_kcontig, c.device, stream, static_only);
    }
  }
  if (a.dtype == TRACEA_DTYPE_FLOAT32 && b.dtype == TRACEA_DTYPE_FLOAT32 && c.dtype == TRACEA_DTYPE_FLOAT32 && K > 0 &&
      a.stride[1] == 1 && b.stride[1] == 1 && c.stride[1] == 1 && K % 4 == 0 &&
      (N % 4 == 0 || ((K - 1) * b.stride[0] + N) * 4 < (1ll << 31)) &&
      a.stride[0] % 4 == 0 && b.stride[0] % 4 == 0 && aligned(a.ptr, 16) && aligned(b.ptr, 16)) {
    // (N itself may be ragged where B is read through a buffer descriptor, i.e. below 2 GiB: a piece that starts
    // inside N is read whole -- what lies behind N in the row only reaches output columns that are never stored,
    // and behind the last row the descriptor returns zeros -- and the epilogue stores by valid channels)
    ContractionArgs args{};
    args.A = a.ptr; args.B = b.ptr; args.C = c.ptr;
    args.M = (int)M; args.N = (int)N; args.K = (int)K;
    args.lda = a.stride[0]; args.ldb = b.stride[0]; args.ldc = c.stride[0];
    args.out_dtype = DT_F32;
    // the direct-to-LDS form addresses operands with 32-bit byte offsets
    const long long a_extent = ((M - 1) * a.stride[0] + K) * 4, b_extent = ((K - 1) * b.stride[0] + N) * 4;
    if (a_extent < (1ll << 31) && b_extent < (1ll << 31)) {
      args.a_bytes = (unsigned)a_extent;
      args.b_bytes = (unsigned)b_extent;
    }
    // Two tile shapes, 128x128x16 and (direct-to-LDS form only) 64x64x16.  A CU works through its
    // share of the tiles at one 128x128 tile per 4 units of time or one 64x64 tile per 1.06 units
    // (the small tile reads its operands from LDS twice as often): the shape whose busiest CU
    // finishes first is taken.  Measured, 128 / 64, in us: 1024^3 68 / 24.7, 1536^3 102 / 77,
    // 3072^3 558 / 441, 2048^3 134.7 / 133.4, 4096^3 972 / 1033.  (A 128x64 tile was never the fastest:
    // 477 at 3072^3, 1003 at 4096^3.)
    static const ContractionVariant f32_tile128 = {"f32_128x128x16", 128, 128, 16, 2, 2, 1, 0, 0, nullptr, 32};
    const long long tiles128 = ((M + 127) / 128) * ((N + 127) / 128), tiles64 = ((M + 63) / 64) * ((N + 63) / 64);
    const long long ncu = device_limits().cus;
    int tile = args.a_bytes != 0 && (double)((tiles64 + ncu - 1) / ncu) * 1.06 < (double)((tiles128 + ncu - 1) / ncu) * 4.0 ? 64 : 128;
    int k_split = 0, splits = 1;
    t_last_split_launches = 1;
    const bool can_fuse = args.a_bytes != 0 && !static_only && g_split_k_enabled.load() && g_split_k_one_launch.load();
    const int nk = (int)((K + 15) / 16);
    if (tile == 64) {
      // (the same K ranges whether the sum then runs in the launch or, for the entry point that must not
      // allocate or with one-launch splits switched off, in a reduction kernel: the results are the same bits)
      // The 64x64 tile splits in one launch (the tile's last workgroup sums, see the kernel).  Up to four ranges
      // of at least 16 K tiles, and no more than 4.5 workgroups per CU; among those the count with the least
      // estimated time, in K tiles of one workgroup: rounds of workgroups over the CUs x K tiles per range,
      // x 0.9 where at least two workgroups share a CU (one's MFMAs run under the other's waits), x 0.92 where
      // there is at most one per CU (it then runs K tiles of 32: half the barriers, and the 64 KB of LDS
      // displace nobody), + 3 for a split + 4 per range beyond two (partial tiles written and read again).
      // Measured (us, replayed graphs, 1 / 2 / 4 ranges): 1024^3 24.7 (22.8 on K tiles of 32) / 23.9 / 26.8,
      // 1024x1024x2048 42.5 (41.8) / 40.3 / 42.3, 768x1024x1024 23.5 / 23.5 / 20.1, 1536^3 76.9 / 67.7 / -,
      // 2048^3 133.4 / 137.5 / -.
      int best = 1;
      if (g_split_k_enabled.load()) {
        double best_cost = 0.0;
        for (int s = 1; s <= kOneLaunchMaxSplits && (s == 1 || (s <= nk / 16 && tiles64 * s * 2 <= 9 * ncu)); ++s) {
          const long long wgs = tiles64 * s;
          const double share = wgs >= 2 * ncu ? 0.9 : wgs <= ncu ? 0.92 : 1.0;
          const double cost = (double)((wgs + ncu - 1) / ncu) * (double)((nk + s - 1) / s) * share + (s > 1 ? 3.0 + 4.0 * (s - 2) : 0.0);
          if (s == 1 || cost < best_cost) { best = s; best_cost = cost; }
        }
      }
      if (tiles64 * best <= ncu) tile = 6432;
      if (best >= 2) {
        int per = (nk + best - 1) / best;
        if (tile == 6432) per += per & 1;  // whole K tiles of 32
        k_split = per * 16;
        splits = (nk + per - 1) / per;
      }
    } else {
      splits = g_split_k_enabled.load() ? choose_split(f32_tile128, (int)M, (int)N, (int)K, &k_split, 4) : 1;
    }
    const long long tiles = tile == 128 ? tiles128 : tiles64;
    const size_t tile_elts = tile == 128 ? 128 * 128 : 64 * 64;
    if (can_fuse && splits > 1 && splits <= kOneLaunchMaxSplits && tiles <= kFuseTiles) {
      void *fws = splitk_scratch(c.device, stream, (size_t)tiles * (size_t)splits * tile_elts * 4);
      unsigned *cnt = fws != nullptr ? fuse_counters(c.device, stream) : nullptr;
      if (cnt != nullptr) {
        args.epi = chain;
        args.k_split = k_split;
        args.fuse_ws = (float *)fws;
        args.fuse_count = cnt;
        t_last_splits = splits;
        const TraceaStatus fst = hip_status("gemm_f32 launch", launch_gemm_f32(args, tile, stream));
        if (fst != TRACEA_SUCCESS) reset_fuse_counters(cnt, stream);
        return fst;
      }
    }
    TraceaStatus ws = TRACEA_SUCCESS;
    void *scratch = split_workspace("gemm_f32 launch", static_only, c.device, stream, splits, M, N, &ws);
    if (ws != TRACEA_SUCCESS) return ws;
    t_last_splits = scratch != nullptr ? splits : 1;
    if (scratch == nullptr) {
      args.epi = chain;
      return hip_status("gemm_f32 launch", launch_gemm_f32(args, tile, stream));
    }
    SplitKReduceArgs r{};
    r.partial = (const float *)scratch;
    r.out = c.ptr; r.out_dtype = DT_F32;
    r.splits = splits; r.M = (int)M; r.N = (int)N; r.ldc = c.stride[0];
    r.epi = chain;
    args.C = scratch;
    args.ldc = N;
    args.k_split = k_split;
    TraceaStatus st = hip_status("gemm_f32 launch", launch_gemm_f32(args, tile, stream));
    if (st != TRACEA_SUCCESS) return st;
    t_last_split_launches = 2;
    return hip_status("split-K reduction launch", launch_splitk_reduce(r, stream));
  }
  // Operands the tile kernels cannot read as they lie -- a K (or the N of a row-major B) that is not a whole
  // number of 16-byte pieces, rows that do not start on 16 bytes, strides along K -- are copied once into
  // padded, zero-filled rows and multiplied from there: two copy launches in front of a tile kernel instead of
  // the any-layout kernel on the vector ALU (fp32 1000 x 900 x 1030: 794 us there).  Half precision: both as
  // K-contiguous rows (a row-major B is transposed on the way); fp32: A by rows, B row-major.  Not for the entry
  // point that must not allocate, nor while the buffer cannot grow (a stream under capture).
  static thread_local bool in_padded = false;
  const bool same_half = is_half(a.dtype) && b.dtype == a.dtype;
  const bool all_f32 = a.dtype == TRACEA_DTYPE_FLOAT32 && b.dtype == TRACEA_DTYPE_FLOAT32 && c.dtype == TRACEA_DTYPE_FLOAT32;
  if (!in_padded && !static_only && K > 0 && (same_half || all_f32) && c.stride[1] == 1 && M < (1ll << 31) && N < (1ll << 31) &&
      K < (1ll << 31)) {
    const int esz = same_half ? 2 : 4;
    const long long Kp = (K + 31) / 32 * 32, Np = (N + 31) / 32 * 32;
    const size_t a_bytes = (size_t)M * (size_t)Kp * esz;
    const size_t b_bytes = same_half ? (size_t)N * (size_t)Kp * esz : (size_t)Kp * (size_t)Np * esz;
    const size_t a_room = (a_bytes + 255) / 256 * 256;
    unsigned char *buf = (unsigned char *)pad_scratch(c.device, stream, a_room + b_bytes);
    if (buf != nullptr) {
      int e = launch_pad_copy(a.ptr, buf, esz, M, K, a.stride[0], a.stride[1], M, Kp, stream);
      if (e == 0) {
        if (same_half) e = launch_pad_copy(b.ptr, buf + a_room, esz, N, K, b.stride[1], b.stride[0], N, Kp, stream);
        else e = launch_pad_copy(b.ptr, buf + a_room, esz, K, N, b.stride[0], b.stride[1], Kp, Np, stream);
      }
      if (e != 0) return hip_status("operand copy launch", e);
      View ap = a, bp = b;
      ap.ptr = buf; ap.shape[1] = Kp; ap.stride[0] = Kp; ap.stride[1] = 1;
      bp.ptr = buf + a_room; bp.shape[0] = Kp;
      if (same_half) { bp.stride[0] = 1; bp.stride[1] = Kp; }
      else { bp.stride[0] = Np; bp.stride[1] = 1; }
      in_padded = true;
      const TraceaStatus st = run_gemm(ap, bp, c, chain, stream, static_only);
      in_padded = false;
      return st;
    }
  }
  GenericGemmArgs g{};
  g.A = a.ptr; g.B = b.ptr; g.C = c.ptr;
  g.M = (int)M; g.N = (int)N; g.K = (int)K;
  g.sam = a.stride[0]; g.sak = a.stride[1];
  g.sbk = b.stride[0]; g.sbn = b.stride[1];
  g.scm = c.stride[0]; g.scn = c.stride[1];
  g.a_dtype = a.dtype; g.b_dtype = b.dtype; g.c_dtype = c.dtype;
  g.epi = chain;
  return hip_status("gemm_generic launch", launch_gemm_generic(g, stream));
}

TraceaStatus gemm_common(const TraceaTensorView &ta, const TraceaTensorView &tb,
                         TraceaTensorView *tc, View *a, View *b, View *c) {
  if (!runtime_ready()) return fail(TRACEA_UNKNOWN_ERROR, "tracea_gemm: tracea_init has not been called");
  if (tc == nullptr) return fail(TRACEA_INVALID_PARAMS, "tracea_gemm: output view is NULL");
  TraceaStatus st;
  if ((st = read_view("tracea_gemm: a", ta, 2, a)) != TRACEA_SUCCESS) return st;
  if ((st = read_view("tracea_gemm: b", tb, 2, b)) != TRACEA_SUCCESS) return st;
  if ((st = read_view("tracea_gemm: c", *tc, 2, c)) != TRACEA_SUCCESS) return st;
  if (!is_float_type(a->dtype) || !is_float_type(b->dtype) || !is_float_type(c->dtype))
    return fail(TRACEA_UNSUPPORTED_CONFIG, "tracea_gemm: dtypes %s x %s -> %s unsupported",
                dtype_name(a->dtype), dtype_name(b->dtype), dtype_name(c->dtype));
  if (a->shape[1] != b->shape[0] || c->shape[0] != a->shape[0] || c->shape[1] != b->shape[1])
    return fail(TRACEA_INVALID_PARAMS,
                "tracea_gemm: shapes a[%lld,%lld] b[%lld,%lld] c[%lld,%lld] do not agree",
                a->shape[0], a->shape[1], b->shape[0], b->shape[1], c->shape[0], c->shape[1]);
  if ((st = check_device("tracea_gemm", c->device)) != TRACEA_SUCCESS) return st;
  if (a->device != c->device || b->device != c->device)
    return fail(TRACEA_INVALID_PARAMS, "tracea_gemm: operands live on different devices");
  if (a->shape[0] >= (1ll << 31) || a->shape[1] >= (1ll << 31) || b->shape[1] >= (1ll << 31))
    return fail(TRACEA_UNSUPPORTED_CONFIG, "tracea_gemm: dimension exceeds 2^31-1");
  return TRACEA_SUCCESS;
}

}  // namespace

TraceaStatus dispatch_gemm_kind(const TraceaTensorView &ta, const TraceaTensorView &tb,
                                const TraceaTensorView *bias, const TraceaTensorView *residual,
                                TraceaTensorView *tc, const TraceaGemmParams &params, bool static_only) {
  View a, b, c;
  TraceaStatus st = gemm_common(ta, tb, tc, &a, &b, &c);
  if (st != TRACEA_SUCCESS) return st;
  TraceaEpilogueOp ops[TRACEA_MAX_EPILOGUE_OPS];
  const int n = kind_to_ops((int)params.epilogue, bias, residual, ops);
  if (n < 0) return fail(TRACEA_INVALID_PARAMS, "tracea_gemm: unknown epilogue kind %d", (int)params.epilogue);
  st = check_bias_residual("tracea_gemm", bias, residual, c.shape[1], c, c.device, ops, n);
  if (st != TRACEA_SUCCESS) return st;
  EpilogueChain chain{};
  st = lower_chain("tracea_gemm", ops, (uint32_t)n, c.shape[1], c.shape[1], &chain);
  if (st != TRACEA_SUCCESS) return st;
  return run_gemm(a, b, c, chain, (hipStream_t)params.stream, static_only);
}

TraceaStatus dispatch_gemm_ops(const TraceaTensorView &ta, const TraceaTensorView &tb,
                               TraceaTensorView *tc, const TraceaGemmParams &params,
                               const TraceaEpilogueOp *ops, uint32_t n_ops) {
  View a, b, c;
  TraceaStatus st = gemm_common(ta, tb, tc, &a, &b, &c);
  if (st != TRACEA_SUCCESS) return st;
  EpilogueChain chain{};
  st = lower_chain("tracea_gemm_ex", ops, n_ops, c.shape[1], c.shape[1], &chain);
  if (st != TRACEA_SUCCESS) return st;
  return run_gemm(a, b, c, chain, (hipStream_t)params.stream);
}

// ---- GEMM over a tile list ---------------------------------------------------------
// The tile extents of the layout name the kernel: a compiled variant with that macro-tile
// runs one workgroup per listed record.  Output tiles without a record are not written.
// When several records share a tile (a K split written out as records), every tile must
// have the same number of them: their partial products go to the split-K workspace and
// the reduction kernel sums them and applies the operator chain.
TraceaStatus dispatch_gemm_tiles(const TraceaTensorView &ta, const TraceaTensorView &tb,
                                 const TraceaTensorView *bias, const TraceaTensorView *residual,
                                 TraceaTensorView *tc, const TraceaGemmParams &params,
                                 const TraceaEpilogueOp *ops_in, uint32_t n_ops, const TileLayout &layout,
                                 const DeviceTileTables &tables) {
  const char *what = "tracea_gemm_ttg";
  View a, b, c;
  TraceaStatus st = gemm_common(ta, tb, tc, &a, &b, &c);
  if (st != TRACEA_SUCCESS) return st;
  EpilogueChain chain{};
  if (ops_in == nullptr) {
    TraceaEpilogueOp ops[TRACEA_MAX_EPILOGUE_OPS];
    const int n = kind_to_ops((int)params.epilogue, bias, residual, ops);
    if (n < 0) return fail(TRACEA_INVALID_PARAMS, "%s: unknown epilogue kind %d", what, (int)params.epilogue);
    st = check_bias_residual(what, bias, residual, c.shape[1], c, c.device, ops, n);
    if (st != TRACEA_SUCCESS) return st;
    st = lower_chain(what, ops, (uint32_t)n, c.shape[1], c.shape[1], &chain);
  } else {
    st = lower_chain(what, ops_in, n_ops, c.shape[1], c.shape[1], &chain);
  }
  if (st != TRACEA_SUCCESS) return st;

  const long long M = a.shape[0], K = a.shape[1], N = b.shape[1];
  if (M != layout.m || N != layout.n || K != layout.k)
    return fail(TRACEA_INVALID_PARAMS, "%s: operands are %lldx%lldx%lld, the layout was built for %ux%ux%u", what, M,
                N, K, layout.m, layout.n, layout.k);
  t_last_contraction = -1;
  t_last_splits = 1;
  if (tables.count == 0) return TRACEA_SUCCESS;  // nothing listed: nothing written
  if (tables.l1 == nullptr || tables.l2 == nullptr || (tables.slices > 1 && tables.slice == nullptr))
    return fail(TRACEA_INVALID_PARAMS, "%s: the layout has no tables on device %d", what, c.device);

  const bool a_ok = a.stride[1] == 1 && a.stride[0] % 8 == 0 && K % 8 == 0 && aligned(a.ptr, 16);
  const bool b_kcontig = b.stride[0] == 1 && b.stride[1] % 8 == 0 && aligned(b.ptr, 16);
  const bool b_ncontig = b.stride[1] == 1 && b.stride[0] % 8 == 0 && N % 8 == 0 && aligned(b.ptr, 16);
  if (!(is_half(a.dtype) && b.dtype == a.dtype && a_ok && (b_kcontig || b_ncontig) && c.stride[1] == 1))
    return fail(TRACEA_UNSUPPORTED_CONFIG,
                "%s: needs fp16 or bf16 operands of one type, 16-byte aligned, K-contiguous A with K and the row "
                "stride multiples of 8, B contiguous along K or N, unit column stride of C", what);
  if (tables.k_gcd % 8 != 0 || tables.start_gcd % 8 != 0)
    return fail(TRACEA_UNSUPPORTED_CONFIG, "%s: every k_start and k range length must be a multiple of 8", what);

  const long long a_extent = ((M - 1) * a.stride[0] + K) * 2;
  const long long b_extent = b_kcontig ? ((N - 1) * b.stride[1] + K) * 2 : ((K - 1) * b.stride[0] + N) * 2;
  const bool small = a_extent < (1ll << 31) && b_extent < (1ll << 31);
  // the variant: forced if its tile fits, else the most pipelined one with this macro-tile
  int vi = -1;
  const int forced = forced_variant("gemm");
  if (forced >= 0 && !conv_only(contraction_variant(forced)) && contraction_variant(forced).bm == (int)layout.mt &&
      contraction_variant(forced).bn == (int)layout.nt)
    vi = forced;
  static const int rank_of_pipeline[5] = {0, 1, 3, 2, -1};
  const bool use_forced = vi >= 0;
  for (int i = 0; !use_forced && i < contraction_variant_count(); ++i) {
    const ContractionVariant &v = contraction_variant(i);
    if (conv_only(v) || v.mfma != 32 || v.bm != (int)layout.mt || v.bn != (int)layout.nt) continue;
    if (vi < 0) { vi = i; continue; }
    const ContractionVariant &best = contraction_variant(vi);
    const int r = rank_of_pipeline[v.pipeline], rb = rank_of_pipeline[best.pipeline];
    if (r > rb || (r == rb && v.waves_m * v.waves_n > best.waves_m * best.waves_n)) vi = i;
  }
  if (vi < 0)
    return fail(TRACEA_UNSUPPORTED_CONFIG, "%s: no kernel with a %ux%u macro-tile (compiled: 64x64, 128x64, 128x128, "
                "256x64, 256x128, 256x256)", what, layout.mt, layout.nt);
  vi = resolve_variant(vi, false, !small, tables.k_gcd % contraction_variant(vi).bk == 0, !b_kcontig);
  const ContractionVariant &v = contraction_variant(vi);

  DeviceScope scope(c.device);
  if (scope.err != hipSuccess) return hip_status("hipSetDevice", (int)scope.err);
  hipStream_t stream = (hipStream_t)params.stream;
  ContractionArgs args{};
  args.A = a.ptr; args.B = b.ptr; args.C = c.ptr;
  args.M = (int)M; args.N = (int)N; args.K = (int)K;
  args.lda = a.stride[0];
  args.ldb = b_kcontig ? b.stride[1] : b.stride[0];
  args.ldc = c.stride[0];
  args.out_dtype = c.dtype;
  args.a_bytes = (unsigned)(small ? a_extent : 0);
  args.b_bytes = (unsigned)(small ? b_extent : 0);
  fill_grid(&args, v);
  args.tile_list = tables.l1;
  args.tile_records = tables.l2;
  args.tile_count = (int)tables.count;
  t_last_contraction = vi;
  if (tables.slices <= 1) {
    args.epi = chain;
    return hip_status("gemm tile-list launch", v.launch(args, false, a.dtype, !b_kcontig, stream));
  }
  // (tiles with different numbers of records: tables.counts tells the reduction how many planes each
  // tile has, and to leave unlisted tiles alone)
  if (tables.counts == nullptr && (long long)tables.count != (long long)tables.slices * args.grid_m * args.grid_n)
    return fail(TRACEA_INVALID_PARAMS, "%s: the layout's tables carry no per-tile record counts", what);
  void *scratch = splitk_scratch(c.device, stream, (size_t)tables.slices * M * N * 4);
  if (scratch == nullptr)
    return fail(TRACEA_UNSUPPORTED_CONFIG, "%s: %u partial products of %lldx%lld exceed the 64 MiB workspace", what,
                tables.slices, M, N);
  t_last_splits = (int)tables.slices;
  SplitKReduceArgs r{};
  r.partial = (const float *)scratch;
  r.out = c.ptr; r.out_dtype = c.dtype;
  r.splits = (int)tables.slices; r.M = (int)M; r.N = (int)N; r.ldc = c.stride[0];
  r.epi = chain;
  r.tile_counts = tables.counts;
  r.mt = (int)layout.mt; r.nt = (int)layout.nt; r.grid_n = args.grid_n;
  args.C = scratch;
  args.ldc = N;
  args.out_dtype = DT_F32;
  args.tile_slice = tables.slice;
  st = hip_status("gemm tile-list launch", v.launch(args, false, a.dtype, !b_kcontig, stream));
  if (st != TRACEA_SUCCESS) return st;
  return hip_status("split-K reduction launch", launch_splitk_reduce(r, stream));
}

// ---- low-rank MLP ------------------------------------------------------------------
// C = chain((X A) B): the rank-r product T = X A is rounded to the operands' type, as the
// reference's kernel keeps it (half sT, src/emitter/cuda/low_rank.rs:28-31, 86-94), and
// lives in a stream-ordered allocation for the duration of the call; both products run
// on the GEMM kernels.
TraceaStatus dispatch_low_rank_mlp(const TraceaTensorView &tx, const TraceaTensorView &ta,
                                   const TraceaTensorView &tb, const TraceaTensorView *bias,
                                   const TraceaTensorView *residual, TraceaTensorView *tc,
                                   const TraceaGemmParams &params) {
  const char *what = "tracea_low_rank_mlp";
  if (!runtime_ready()) return fail(TRACEA_UNKNOWN_ERROR, "%s: tracea_init has not been called", what);
  if (tc == nullptr) return fail(TRACEA_INVALID_PARAMS, "%s: output view is NULL", what);
  View x, a, b, c;
  TraceaStatus st;
  if ((st = read_view("tracea_low_rank_mlp: x", tx, 2, &x)) != TRACEA_SUCCESS) return st;
  if ((st = read_view("tracea_low_rank_mlp: a", ta, 2, &a)) != TRACEA_SUCCESS) return st;
  if ((st = read_view("tracea_low_rank_mlp: b", tb, 2, &b)) != TRACEA_SUCCESS) return st;
  if ((st = read_view("tracea_low_rank_mlp: c", *tc, 2, &c)) != TRACEA_SUCCESS) return st;
  if (!is_float_type(x.dtype) || a.dtype != x.dtype || b.dtype != x.dtype || !is_float_type(c.dtype))
    return fail(TRACEA_UNSUPPORTED_CONFIG, "%s: x, a and b must share one floating type (%s, %s, %s)", what,
                dtype_name(x.dtype), dtype_name(a.dtype), dtype_name(b.dtype));
  const long long M = x.shape[0], K = x.shape[1], R = a.shape[1], N = b.shape[1];
  if (a.shape[0] != K || b.shape[0] != R || c.shape[0] != M || c.shape[1] != N)
    return fail(TRACEA_INVALID_PARAMS, "%s: shapes x[%lld,%lld] a[%lld,%lld] b[%lld,%lld] c[%lld,%lld] do not agree",
                what, M, K, a.shape[0], R, b.shape[0], N, c.shape[0], c.shape[1]);
  if ((st = check_device(what, c.device)) != TRACEA_SUCCESS) return st;
  if (x.device != c.device || a.device != c.device || b.device != c.device)
    return fail(TRACEA_INVALID_PARAMS, "%s: operands live on different devices", what);
  if (M >= (1ll << 31) || K >= (1ll << 31) || N >= (1ll << 31) || R >= (1ll << 31))
    return fail(TRACEA_UNSUPPORTED_CONFIG, "%s: dimension exceeds 2^31-1", what);
  TraceaEpilogueOp ops[TRACEA_MAX_EPILOGUE_OPS];
  const int n = kind_to_ops((int)params.epilogue, bias, residual, ops);
  if (n < 0) return fail(TRACEA_INVALID_PARAMS, "%s: unknown epilogue kind %d", what, (int)params.epilogue);
  st = check_bias_residual(what, bias, residual, N, c, c.device, ops, n);
  if (st != TRACEA_SUCCESS) return st;
  EpilogueChain chain{};
  st = lower_chain(what, ops, (uint32_t)n, N, N, &chain);
  if (st != TRACEA_SUCCESS) return st;
  if (M == 0 || N == 0) return TRACEA_SUCCESS;

  hipStream_t stream = (hipStream_t)params.stream;
  DeviceScope scope(c.device);
  if (scope.err != hipSuccess) return hip_status("hipSetDevice", (int)scope.err);
  const long long ldt = (R + 7) / 8 * 8;  // rows of T start 16-byte aligned
  void *t_mem = nullptr;
  hipError_t e = hipMallocAsync(&t_mem, (size_t)std::max(1ll, M * ldt) * elem_size(x.dtype), stream);
  if (e != hipSuccess) return hip_status("tracea_low_rank_mlp: workspace allocation", (int)e);
  View t{};
  t.ptr = t_mem; t.dtype = x.dtype; t.device = c.device; t.rank = 2;
  t.shape[0] = M; t.shape[1] = R; t.stride[0] = ldt; t.stride[1] = 1;
  st = run_gemm(x, a, t, EpilogueChain{}, stream);
  if (st == TRACEA_SUCCESS) st = run_gemm(t, b, c, chain, stream);
  e = hipFreeAsync(t_mem, stream);
  if (st == TRACEA_SUCCESS && e != hipSuccess) st = hip_status("tracea_low_rank_mlp: workspace release", (int)e);
  return st;
}

// ---- operators that are not contractions (src/emitter/cuda/nn.rs:3-135) -------------
namespace {

// A contiguous tensor whose last axis is the channel axis: rows x channels.
TraceaStatus rows_by_channels(const char *what, const TraceaTensorView &t, long long *rows, long long *channels,
                              View *v) {
  if (t.rank < 1 || t.rank > 4) return fail(TRACEA_INVALID_PARAMS, "%s: rank %u, expected 1 to 4", what, t.rank);
  TraceaStatus st = read_view(what, t, (int)t.rank, v);
  if (st != TRACEA_SUCCESS) return st;
  if (!is_float_type(v->dtype)) return fail(TRACEA_UNSUPPORTED_CONFIG, "%s: dtype %s unsupported", what, dtype_name(v->dtype));
  long long expect = 1, r = 1;
  for (int i = v->rank - 1; i >= 0; --i) {
    if (v->shape[i] > 1 && v->stride[i] != expect)
      return fail(TRACEA_UNSUPPORTED_CONFIG, "%s: the tensor must be contiguous with the channel axis last "
                  "(NHWC); axis %d has stride %lld, expected %lld", what, i, v->stride[i], expect);
    expect *= v->shape[i];
    if (i < v->rank - 1) r *= v->shape[i];
  }
  *rows = r;
  *channels = v->shape[v->rank - 1];
  if (*channels >= (1ll << 31)) return fail(TRACEA_UNSUPPORTED_CONFIG, "%s: more than 2^31-1 channels", what);
  return TRACEA_SUCCESS;
}

bool same_shape(const View &a, const View &b) {
  if (a.rank != b.rank) return false;
  for (int i = 0; i < a.rank; ++i)
    if (a.shape[i] != b.shape[i]) return false;
  return true;
}

}  // namespace

// out = chain(x), element by element with per-channel operands: standalone BatchNorm
// (nn.rs:37-70, channel axis last here), ReLU, bias, residual Add as one pass over the tensor.
TraceaStatus dispatch_apply_epilogue(const TraceaTensorView &tx, TraceaTensorView *tout, const TraceaEpilogueOp *ops,
                                     uint32_t n_ops, void *stream) {
  const char *what = "tracea_apply_epilogue";
  if (!runtime_ready()) return fail(TRACEA_UNKNOWN_ERROR, "%s: tracea_init has not been called", what);
  if (tout == nullptr) return fail(TRACEA_INVALID_PARAMS, "%s: output view is NULL", what);
  View x, out;
  long long rows, channels, orows, ochannels;
  TraceaStatus st;
  if ((st = rows_by_channels("tracea_apply_epilogue: x", tx, &rows, &channels, &x)) != TRACEA_SUCCESS) return st;
  if ((st = rows_by_channels("tracea_apply_epilogue: out", *tout, &orows, &ochannels, &out)) != TRACEA_SUCCESS) return st;
  if (!same_shape(x, out)) return fail(TRACEA_INVALID_PARAMS, "%s: x and out differ in shape", what);
  if ((st = check_device(what, out.device)) != TRACEA_SUCCESS) return st;
  if (x.device != out.device) return fail(TRACEA_INVALID_PARAMS, "%s: operands live on different devices", what);
  ChainApplyArgs a{};
  st = lower_chain(what, ops, n_ops, channels, channels, &a.epi);
  if (st != TRACEA_SUCCESS) return st;
  a.x = x.ptr; a.out = out.ptr;
  a.x_dtype = x.dtype; a.out_dtype = out.dtype;
  a.rows = rows; a.channels = (int)channels;
  DeviceScope scope(out.device);
  if (scope.err != hipSuccess) return hip_status("hipSetDevice", (int)scope.err);
  return hip_status("operator chain launch", launch_chain_apply(a, (hipStream_t)stream));
}

// Softmax over the last axis (nn.rs:3-35), fp32 arithmetic whatever the storage type.
TraceaStatus dispatch_softmax(const TraceaTensorView &tx, TraceaTensorView *tout, void *stream) {
  const char *what = "tracea_softmax";
  if (!runtime_ready()) return fail(TRACEA_UNKNOWN_ERROR, "%s: tracea_init has not been called", what);
  if (tout == nullptr) return fail(TRACEA_INVALID_PARAMS, "%s: output view is NULL", what);
  View x, out;
  long long rows, cols, orows, ocols;
  TraceaStatus st;
  if ((st = rows_by_channels("tracea_softmax: x", tx, &rows, &cols, &x)) != TRACEA_SUCCESS) return st;
  if ((st = rows_by_channels("tracea_softmax: out", *tout, &orows, &ocols, &out)) != TRACEA_SUCCESS) return st;
  if (!same_shape(x, out)) return fail(TRACEA_INVALID_PARAMS, "%s: x and out differ in shape", what);
  if ((st = check_device(what, out.device)) != TRACEA_SUCCESS) return st;
  if (x.device != out.device) return fail(TRACEA_INVALID_PARAMS, "%s: operands live on different devices", what);
  DeviceScope scope(out.device);
  if (scope.err != hipSuccess) return hip_status("hipSetDevice", (int)scope.err);
  return hip_status("softmax launch",
                    launch_softmax_rows(x.ptr, out.ptr, x.dtype, out.dtype, rows, (int)cols, (hipStream_t)stream));
}

// out[n, c] = mean over (h, w) of x[n, h, w, c] (nn.rs:72-100; the reference indexes NCHW).
TraceaStatus dispatch_global_avg_pool(const TraceaTensorView &tx, TraceaTensorView *tout, void *stream) {
  const char *what = "tracea_global_avg_pool";
  if (!runtime_ready()) return fail(TRACEA_UNKNOWN_ERROR, "%s: tracea_init has not been called", what);
  if (tout == nullptr) return fail(TRACEA_INVALID_PARAMS, "%s: output view is NULL", what);
  if (tx.rank != 4 || tout->rank != 2)
    return fail(TRACEA_INVALID_PARAMS, "%s: x must be [N,H,W,C] and out [N,C]", what);
  View x, out;
  long long rows, channels, orows, ochannels;
  TraceaStatus st;
  if ((st = rows_by_channels("tracea_global_avg_pool: x", tx, &rows, &channels, &x)) != TRACEA_SUCCESS) return st;
  if ((st = rows_by_channels("tracea_global_avg_pool: out", *tout, &orows, &ochannels, &out)) != TRACEA_SUCCESS) return st;
  if (out.shape[0] != x.shape[0] || ochannels != channels)
    return fail(TRACEA_INVALID_PARAMS, "%s: out is [%lld,%lld], expected [%lld,%lld]", what, out.shape[0], ochannels,
                x.shape[0], channels);
  if ((st = check_device(what, out.device)) != TRACEA_SUCCESS) return st;
  if (x.device != out.device) return fail(TRACEA_INVALID_PARAMS, "%s: operands live on different devices", what);
  const long long hw = x.shape[1] * x.shape[2];
  if (x.shape[0] > 65535 || hw >= (1ll << 31))
    return fail(TRACEA_UNSUPPORTED_CONFIG, "%s: batch above 65535 or more than 2^31-1 pixels", what);
  if (hw == 0) return fail(TRACEA_INVALID_PARAMS, "%s: empty spatial extent", what);
  DeviceScope scope(out.device);
  if (scope.err != hipSuccess) return hip_status("hipSetDevice", (int)scope.err);
  return hip_status("global average pool launch",
                    launch_global_avg_pool(x.ptr, out.ptr, x.dtype, out.dtype, (int)x.shape[0], (int)hw, (int)channels,
                                           (hipStream_t)stream));
}

// c[b] = epilogue(a[b] w[b]) for every batch b (nn.rs:102-135: A [B,M,K], B [B,K,N], C [B,M,N]);
// a weight of rank 2 is shared by all batches, and the batch then folds into the rows.
TraceaStatus dispatch_linear(const TraceaTensorView &ta, const TraceaTensorView &tw, const TraceaTensorView *bias,
                             TraceaTensorView *tc, const TraceaGemmParams &params) {
  const char *what = "tracea_linear";
  if (!runtime_ready()) return fail(TRACEA_UNKNOWN_ERROR, "%s: tracea_init has not been called", what);
  if (tc == nullptr) return fail(TRACEA_INVALID_PARAMS, "%s: output view is NULL", what);
  if (ta.rank != 3 || tc->rank != 3 || (tw.rank != 2 && tw.rank != 3))
    return fail(TRACEA_INVALID_PARAMS, "%s: a and c must have rank 3 ([B,M,K], [B,M,N]), w rank 2 or 3", what);
  View a, w, c;
  TraceaStatus st;
  if ((st = read_view("tracea_linear: a", ta, 3, &a)) != TRACEA_SUCCESS) return st;
  if ((st = read_view("tracea_linear: w", tw, (int)tw.rank, &w)) != TRACEA_SUCCESS) return st;
  if ((st = read_view("tracea_linear: c", *tc, 3, &c)) != TRACEA_SUCCESS) return st;
  const long long B = a.shape[0], M = a.shape[1], K = a.shape[2];
  const bool shared = w.rank == 2;
  const long long wk = w.shape[w.rank - 2], N = w.shape[w.rank - 1];
  if (wk != K || c.shape[0] != B || c.shape[1] != M || c.shape[2] != N || (!shared && w.shape[0] != B))
    return fail(TRACEA_INVALID_PARAMS, "%s: shapes a[%lld,%lld,%lld], w[..,%lld,%lld], c[%lld,%lld,%lld] do not agree",
                what, B, M, K, wk, N, c.shape[0], c.shape[1], c.shape[2]);
  if (!is_float_type(a.dtype) || !is_float_type(w.dtype) || !is_float_type(c.dtype))
    return fail(TRACEA_UNSUPPORTED_CONFIG, "%s: dtypes %s x %s -> %s unsupported", what, dtype_name(a.dtype),
                dtype_name(w.dtype), dtype_name(c.dtype));
  if ((st = check_device(what, c.device)) != TRACEA_SUCCESS) return st;
  if (a.device != c.device || w.device != c.device)
    return fail(TRACEA_INVALID_PARAMS, "%s: operands live on different devices", what);
  if (M >= (1ll << 31) || K >= (1ll << 31) || N >= (1ll << 31) || B * M >= (1ll << 31))
    return fail(TRACEA_UNSUPPORTED_CONFIG, "%s: dimension exceeds 2^31-1", what);
  if (params.epilogue == TRACEA_EPILOGUE_RESIDUAL || params.epilogue == TRACEA_EPILOGUE_RESIDUAL_RELU)
    return fail(TRACEA_UNSUPPORTED_CONFIG, "%s: residual epilogues are not defined for a batched product", what);
  TraceaEpilogueOp ops[TRACEA_MAX_EPILOGUE_OPS];
  const int n = kind_to_ops((int)params.epilogue, bias, nullptr, ops);
  if (n < 0) return fail(TRACEA_INVALID_PARAMS, "%s: unknown epilogue kind %d", what, (int)params.epilogue);
  View c2{};
  c2.ptr = c.ptr; c2.rank = 2; c2.dtype = c.dtype; c2.device = c.device;
  c2.shape[0] = M; c2.shape[1] = N; c2.stride[0] = c.stride[1]; c2.stride[1] = c.stride[2];
  st = check_bias_residual(what, bias, nullptr, N, c2, c.device, ops, n);
  if (st != TRACEA_SUCCESS) return st;
  EpilogueChain chain{};
  st = lower_chain(what, ops, (uint32_t)n, N, N, &chain);
  if (st != TRACEA_SUCCESS) return st;
  hipStream_t stream = (hipStream_t)params.stream;
  View a2 = c2, w2 = c2;
  a2.ptr = a.ptr; a2.dtype = a.dtype; a2.shape[0] = M; a2.shape[1] = K; a2.stride[0] = a.stride[1]; a2.stride[1] = a.stride[2];
  w2.ptr = w.ptr; w2.dtype = w.dtype; w2.shape[0] = K; w2.shape[1] = N;
  w2.stride[0] = w.stride[w.rank - 2]; w2.stride[1] = w.stride[w.rank - 1];
  // one launch when the weight is shared and the batches of a and c are evenly spaced rows
  if (shared && (B <= 1 || (a.stride[0] == M * a.stride[1] && c.stride[0] == M * c.stride[1]))) {
    a2.shape[0] = c2.shape[0] = B * M;
    return run_gemm(a2, w2, c2, chain, stream);
  }
  for (long long b = 0; b < B; ++b) {
    View ab = a2, wb = w2, cb = c2;
    ab.ptr = (char *)a.ptr + b * a.stride[0] * elem_size(a.dtype);
    cb.ptr = (char *)c.ptr + b * c.stride[0] * elem_size(c.dtype);
    if (!shared) wb.ptr = (char *)w.ptr + b * w.stride[0] * elem_size(w.dtype);
    if ((st = run_gemm(ab, wb, cb, chain, stream)) != TRACEA_SUCCESS) return st;
  }
  return TRACEA_SUCCESS;
}

// ---- Conv2d ----------------------------------------------------------------------
namespace {

struct ConvPlan {
  View x, w, out;
  ConvGeometry geo;
  bool w_ncontig;  // filters stored [R,S,C,K]
  long long ldb, ldc;
  bool pad_c = false;  // channels not a multiple of 8, or operands not on 16 bytes: run from padded copies
};

TraceaStatus conv_common(const TraceaTensorView &tx, const TraceaTensorView &tw,
                         TraceaTensorView *tout, const TraceaConv2dParams &p, ConvPlan *plan) {
  if (!runtime_ready()) return fail(TRACEA_UNKNOWN_ERROR, "tracea_conv2d: tracea_init has not been called");
  if (tout == nullptr) return fail(TRACEA_INVALID_PARAMS, "tracea_conv2d: output view is NULL");
  if (tx.ptr == nullptr || tw.ptr == nullptr || tout->ptr == nullptr)
    return fail(TRACEA_INVALID_PARAMS, "tracea_conv2d: NULL data pointer");
  if (p.groups != 1)
    return fail(TRACEA_UNSUPPORTED_CONFIG, "tracea_conv2d: groups=%u (only groups=1)", p.groups);
  TraceaStatus st;
  View &x = plan->x, &w = plan->w, &out = plan->out;
  if ((st = read_view("tracea_conv2d: x", tx, 4, &x)) != TRACEA_SUCCESS) return st;
  if ((st = read_view("tracea_conv2d: w", tw, 4, &w)) != TRACEA_SUCCESS) return st;
  if ((st = read_view("tracea_conv2d: out", *tout, 4, &out)) != TRACEA_SUCCESS) return st;
  if (!is_half(x.dtype) || w.dtype != x.dtype)
    return fail(TRACEA_UNSUPPORTED_CONFIG,
                "tracea_conv2d: activations %s / filters %s; f16 or bf16 (both alike) required",
                dtype_name(x.dtype), dtype_name(w.dtype));
  if (out.dtype != x.dtype && out.dtype != TRACEA_DTYPE_FLOAT32)
    return fail(TRACEA_UNSUPPORTED_CONFIG, "tracea_conv2d: output dtype %s unsupported",
                dtype_name(out.dtype));
  if ((st = check_device("tracea_conv2d", out.device)) != TRACEA_SUCCESS) return st;
  if (x.device != out.device || w.device != out.device)
    return fail(TRACEA_INVALID_PARAMS, "tracea_conv2d: operands live on different devices");
  const long long N = x.shape[0], H = x.shape[1], W = x.shape[2], C = x.shape[3];
  const long long K = w.shape[0], R = w.shape[1], S = w.shape[2];
  if (w.shape[3] != C)
    return fail(TRACEA_INVALID_PARAMS, "tracea_conv2d: x has %lld channels, w expects %lld", C, w.shape[3]);
  if (N >= (1ll << 31) || H >= (1ll << 31) || W >= (1ll << 31) || C >= (1ll << 31) || K >= (1ll << 31))
    return fail(TRACEA_UNSUPPORTED_CONFIG, "tracea_conv2d: dimension exceeds 2^31-1");
  st = make_conv_geometry((int)N, (int)H, (int)W, (int)C, (int)K, (int)R, (int)S, (int)p.stride_h,
                          (int)p.stride_w, (int)p.padding_h, (int)p.padding_w, (int)p.dilation_h,
                          (int)p.dilation_w, &plan->geo);
  if (st != TRACEA_SUCCESS) return st;
  const ConvGeometry &g = plan->geo;
  if (out.shape[0] != N || out.shape[1] != g.block.h_out || out.shape[2] != g.block.w_out || out.shape[3] != K)
    return fail(TRACEA_INVALID_PARAMS, "tracea_conv2d: output shape must be [%lld,%d,%d,%lld]", N,
                g.block.h_out, g.block.w_out, K);
  // layouts
  if (!(x.stride[3] == 1 && x.stride[2] == C && x.stride[1] == W * C && x.stride[0] == H * W * C))
    return fail(TRACEA_UNSUPPORTED_CONFIG,
                "tracea_conv2d: activations must be contiguous NHWC (shape [N,H,W,C])");
  if (w.stride[3] == 1 && w.stride[2] == C && w.stride[1] == S * C && w.stride[0] == R * S * C) {
    plan->w_ncontig = false;
    plan->ldb = R * S * C;
  } else if (w.stride[0] == 1 && w.stride[3] == K && w.stride[2] == C * K && w.stride[1] == S * C * K) {
    plan->w_ncontig = true;
    plan->ldb = K;
  } else {
    return fail(TRACEA_UNSUPPORTED_CONFIG,
                "tracea_conv2d: filters must be stored [K,R,S,C] or [R,S,C,K] (dims always [K,R,S,C])");
  }
  const long long ldc = out.stride[2];
  if (!(out.stride[3] == 1 && ldc >= K && out.stride[1] == g.block.w_out * ldc &&
        out.stride[0] == (long long)g.block.h_out * g.block.w_out * ldc))
    return fail(TRACEA_UNSUPPORTED_CONFIG, "tracea_conv2d: output must be channel-contiguous NHWK");
  plan->ldc = ldc;
  // (what the kernels cannot read in place runs from padded copies where a buffer for them can be had: see
  // run_conv_padded; these messages are what the caller reads where it cannot)
  plan->pad_c = false;
  if (C % 8 != 0 || (plan->w_ncontig && K % 8 != 0) || !aligned(x.ptr, 16) || !aligned(w.ptr, 16)) plan->pad_c = true;
  return TRACEA_SUCCESS;
}

// Fills the patch-resident convolution fields of `a` for variant `v` and sets
// the grid; false when the kernel cannot run this problem (then nothing the
// caller relies on has been changed).
//   * K-contiguous filters, C a multiple of 16 (a 16-wide k-step stays inside
//     one tap);
//   * one image and the filter bank each below 2 GiB (32-bit buffer offsets);
//   * the patch of the worst tile plus the filter ring fits in LDS.
// The patch bound: BM consecutive output pixels take at most nw row wraps; a
// step inside a row advances the padded linear index by stride_w, a wrap by
// stride_h*PW - (Wo-1)*stride_w; the taps add (R-1)*dil_h*PW + (S-1)*dil_w.
bool plan_conv_patch(const ConvGeometry &g, const ContractionVariant &v, bool w_ncontig, ContractionArgs *a) {
  const TraceaConvParamsBlock &b = g.block;
  const int C = b.c_in;
  if (v.pipeline != 4 || w_ncontig || C % 16 != 0) return false;
  const long long img_bytes = (long long)b.h_in * b.w_in * C * 2;
  const long long w_bytes = (long long)g.n_gemm * g.k_gemm * 2;
  if (img_bytes >= (1ll << 31) || w_bytes >= (1ll << 31)) return false;
  const long long pw = (long long)b.w_in + 2ll * g.pad_w;
  const long long ph = (long long)b.h_in + 2ll * g.pad_h;
  if (pw * ph >= (1ll << 30)) return false;
  const int hw = b.h_out * b.w_out;
  const int tm = v.bm < hw ? v.bm : hw;
  const long long steps = tm - 1;
  long long nw = (steps + b.w_out - 1) / b.w_out;
  if (nw > steps) nw = steps;
  if (nw > b.h_out - 1) nw = b.h_out - 1;
  const long long in_row = g.stride_w;
  long long wrap = (long long)g.stride_h * pw - (long long)(b.w_out - 1) * g.stride_w;
  if (wrap < in_row) wrap = in_row;
  const long long span = (steps - nw) * in_row + nw * wrap;
  const long long taps = (long long)(b.r_sz - 1) * g.dil_h * pw + (long long)(b.s_sz - 1) * g.dil_w;
  const long long np = span + taps + 1;
  const int cpp = (C / 8) | 1;
  const int nt = v.waves_m * v.waves_n * 64;
  const long long chunks = np * cpp;
  const long long iters = (chunks + nt - 1) / nt;
  const long long patch_bytes = iters * nt * 16;
  const long long ring = (long long)v.stages * v.bn * 128;
  if (patch_bytes + ring > device_limits().lds_bytes) return false;
  a->r_sz = b.r_sz;
  a->p_tiles = (hw + v.bm - 1) / v.bm;
  a->p_pw = (int)pw;
  a->p_cpp = cpp;
  a->p_iters = (int)iters;
  a->p_np_bytes = (int)patch_bytes;
  magic_for_divisor((uint32_t)cpp, (uint64_t)(iters * nt), &a->p_cpp_m, &a->p_cpp_s);
  magic_for_divisor((uint32_t)pw, (uint64_t)(pw * ph + np), &a->p_pw_m, &a->p_pw_s);
  a->grid_m = b.batch * a->p_tiles;
  a->grid_n = (g.n_gemm + v.bn - 1) / v.bn;
  a->group_m = 1;
  a->b_bytes = (unsigned)w_bytes;
  a->a_bytes = 0;
  return true;
}

// The same for the kernel that keeps patch and filter bank in LDS together (pipeline 5,
// conv_resident_kernel.hpp): K-contiguous filters, C a multiple of 16, K = 16 * stages exactly;
// a workgroup takes p_tm consecutive output pixels of one image and 64 filters.  p_tm: every
// workgroup costs the same whatever its tile holds (the kernel runs all its pixel blocks), so
// the fewest rounds over the CUs win, and within that the most workgroups (smaller patches,
// more CUs busy): N32 56x56 -> 8 tiles of 392 pixels per image, 256 workgroups.
bool plan_conv_filter_resident(const ConvGeometry &g, const ContractionVariant &v, bool w_ncontig, ContractionArgs *a) {
  const TraceaConvParamsBlock &b = g.block;
  const int C = b.c_in;
  // (the compiled member walks K as taps of 64 channels: 3x3x64; another split of K = 576 is not its problem)
  if (v.pipeline != 5 || w_ncontig || C != 64 || g.k_gemm != 16 * v.stages) return false;
  const long long img_bytes = (long long)b.h_in * b.w_in * C * 2;
  const long long w_bytes = (long long)g.n_gemm * g.k_gemm * 2;
  if (img_bytes >= (1ll << 31) || w_bytes >= (1ll << 31)) return false;
  const long long pw = (long long)b.w_in + 2ll * g.pad_w;
  const long long ph = (long long)b.h_in + 2ll * g.pad_h;
  if (pw * ph >= (1ll << 30)) return false;
  const int hw = b.h_out * b.w_out;
  const int grid_n = (g.n_gemm + v.bn - 1) / v.bn;
  const long long cus = device_limits().cus;
  const long long t_min = (hw + v.bm - 1) / v.bm;
  const long long rounds = ((long long)b.batch * t_min * grid_n + cus - 1) / cus;
  long long tiles = rounds * cus / ((long long)b.batch * grid_n);
  if (tiles < t_min) tiles = t_min;
  if (tiles > (hw + 15) / 16) tiles = (hw + 15) / 16;
  const int tm = (int)((hw + tiles - 1) / tiles);
  tiles = (hw + tm - 1) / tm;
  const int cpp = (C / 8) | 1;
  // the patch holds whole padded rows: p_seg load instructions of ppi pixels each per row; the largest
  // tile whose rows fit the kernel's fixed number of load instructions and the LDS left beside the
  // filters (shrinking the tile makes more workgroups)
  const int ppi = 64 / cpp;
  if (ppi < 1) return false;
  const int seg = (int)((pw + ppi - 1) / ppi);
  int tm_fit = tm;
  long long rows = 0, iters = 0, patch_bytes = 0;
  for (;;) {
    // most output rows one of the image's tiles spans (tiles start at multiples of tm_fit), then padded input rows
    long long out_rows = 1;
    for (int p0 = 0; p0 < hw; p0 += tm_fit) {
      const int last = (p0 + tm_fit < hw ? p0 + tm_fit : hw) - 1;
      const long long span = last / b.w_out - p0 / b.w_out + 1;
      if (span > out_rows) out_rows = span;
    }
    rows = (out_rows - 1) * g.stride_h + (long long)(b.r_sz - 1) * g.dil_h + 1;
    iters = (rows * seg + 7) / 8;
    patch_bytes = (rows * pw * cpp + 1) * 16;  // (+1: the repeated first part behind the last pixel)
    patch_bytes = (patch_bytes + 1023) / 1024 * 1024;
    if (patch_bytes + (long long)v.lds_bytes <= device_limits().lds_bytes) break;
    if (tm_fit <= 32) return false;
    int next = tm_fit * 7 / 8 / 32 * 32;  // strictly smaller: rounded down to whole pixel blocks
    if (next >= tm_fit) next = tm_fit - 32;
    tm_fit = next < 32 ? 32 : next;
  }
  if ((long long)b.h_in * b.w_in >= (1ll << 24)) return false;
  a->r_sz = b.r_sz;
  a->p_tm = tm_fit;
  a->p_tiles = (hw + tm_fit - 1) / tm_fit;
  a->p_pw = (int)pw;
  a->p_cpp = cpp;
  a->p_iters = (int)iters;
  a->p_np_bytes = (int)patch_bytes;
  a->p_seg = seg;
  a->p_ppi = ppi;
  magic_for_divisor((uint32_t)cpp, 64, &a->p_cpp_m, &a->p_cpp_s);
  a->p_pw_m = a->p_pw_s = 0;
  a->grid_m = b.batch * a->p_tiles;
  a->grid_n = grid_n;
  a->group_m = 1;
  a->b_bytes = (unsigned)w_bytes;
  a->a_bytes = 0;
  return true;
}

// The same for the kernels on 16x16x32 MFMAs (pipelines 7 and 8, conv_wave16_kernel.hpp): K-contiguous
// filters, exactly v.bk input channels, a workgroup takes p_tm <= v.bm consecutive output pixels of one
// image and 64 filters; beside the patch LDS holds the whole 64 x K filter slab (pipeline 7) or a ring of
// v.stages one-tap stages (pipeline 8).  p_tm as for the kernel above: fewest rounds over the CUs, then the
// most workgroups; N32 56x56 -> 8 tiles of 392 pixels per image, N32 28x28 with 128 filters -> 4 tiles of
// 196 pixels x 2 filter slabs, 256 workgroups each.
bool plan_conv_wave16(const ConvGeometry &g, const ContractionVariant &v, bool w_ncontig, ContractionArgs *a) {
  const TraceaConvParamsBlock &b = g.block;
  const int C = b.c_in;
  if ((v.pipeline != 7 && v.pipeline != 8) || w_ncontig || C != v.bk || g.k_gemm != b.r_sz * b.s_sz * C) return false;
  const long long img_bytes = (long long)b.h_in * b.w_in * C * 2;
  const long long w_bytes = (long long)g.n_gemm * g.k_gemm * 2;
  if (img_bytes >= (1ll << 31) || w_bytes >= (1ll << 31)) return false;
  const long long pw = (long long)b.w_in + 2ll * g.pad_w;
  const long long ph = (long long)b.h_in + 2ll * g.pad_h;
  if (pw * ph >= (1ll << 30) || (long long)b.h_in * b.w_in >= (1ll << 24)) return false;
  // (pipeline 7: the slab of all taps of 64 filters, 128 bytes per filter and tap, no padding)
  const long long filter_bytes =
      v.pipeline == 7 ? 64ll * g.k_gemm * 2 : (long long)v.lds_bytes - TRACEA_MAX_EPILOGUE_OPS * 2 * 64 * 4;
  const long long table_bytes = TRACEA_MAX_EPILOGUE_OPS * 2 * 64 * 4;
  const int hw = b.h_out * b.w_out;
  const int grid_n = (g.n_gemm + v.bn - 1) / v.bn;
  const long long cus = device_limits().cus;
  const long long t_min = (hw + v.bm - 1) / v.bm;
  const long long rounds = ((long long)b.batch * t_min * grid_n + cus - 1) / cus;
  long long tiles = rounds * cus / ((long long)b.batch * grid_n);
  if (tiles < t_min) tiles = t_min;
  if (tiles > (hw + 15) / 16) tiles = (hw + 15) / 16;
  const int tm = (int)((hw + tiles - 1) / tiles);
  const int cpp = (C / 8) | 1;
  const int ppi = 64 / cpp;
  if (ppi < 1) return false;
  const int seg = (int)((pw + ppi - 1) / ppi);
  // LDS bytes of the patch of the worst tile when tiles hold t pixels (tiles start at multiples of t): the
  // most output rows a tile spans, then padded input rows
  auto patch_for = [&](int t) -> long long {
    long long out_rows = 1;
    for (int p0 = 0; p0 < hw; p0 += t) {
      const int last = (p0 + t < hw ? p0 + t : hw) - 1;
      const long long span = last / b.w_out - p0 / b.w_out + 1;
      if (span > out_rows) out_rows = span;
    }
    const long long rows = (out_rows - 1) * g.stride_h + (long long)(b.r_sz - 1) * g.dil_h + 1;
    const long long bytes = (rows * pw * cpp + 64) * 16;
    return (bytes + 1023) / 1024 * 1024;
  };
  const long long room = (long long)device_limits().lds_bytes - filter_bytes - table_bytes;
  // the largest tile up to the balanced one that fits; failing that (few, wide rows: a smaller tile still
  // straddles two rows) the smallest larger one
  int tm_fit = 0;
  for (int t = tm < v.bm ? tm : v.bm; t >= 16 && tm_fit == 0; --t)
    if (patch_for(t) <= room) tm_fit = t;
  for (int t = tm + 1; t <= v.bm && t <= hw && tm_fit == 0; ++t)
    if (patch_for(t) <= room) tm_fit = t;
  if (tm_fit == 0) return false;
  const long long patch_bytes = patch_for(tm_fit);
  a->r_sz = b.r_sz;
  a->p_tm = tm_fit;
  a->p_tiles = (hw + tm_fit - 1) / tm_fit;
  a->p_pw = (int)pw;
  a->p_cpp = cpp;
  a->p_iters = 0;
  a->p_np_bytes = (int)patch_bytes;
  a->p_seg = seg;
  a->p_ppi = ppi;
  magic_for_divisor((uint32_t)cpp, 64, &a->p_cpp_m, &a->p_cpp_s);
  a->p_pw_m = 0; a->p_pw_s = 0;
  a->grid_m = b.batch * a->p_tiles;
  a->grid_n = grid_n;
  magic_for_divisor((uint32_t)grid_n, (uint64_t)a->grid_m * grid_n, &a->gn_m, &a->gn_s);
  magic_for_divisor((uint32_t)a->p_tiles, (uint64_t)a->grid_m, &a->pt_m, &a->pt_s);
  a->group_m = 1;
  a->b_bytes = (unsigned)w_bytes;
  a->a_bytes = 0;
  return true;
}

// Plan of the K-split kernel (pipeline 9): as plan_conv_wave16, with the patch rows fetched as flat runs
// of 16-byte chunks (a pixel may be wider than one 64-lane load) and the ring's fixed stage size.
bool plan_conv_ksplit16(const ConvGeometry &g, const ContractionVariant &v, bool w_ncontig, ContractionArgs *a) {
  const TraceaConvParamsBlock &b = g.block;
  const int C = b.c_in;
  if (v.pipeline != 9 || w_ncontig || C != v.bk || C % 256 != 0 || g.k_gemm != b.r_sz * b.s_sz * C) return false;
  const long long img_bytes = (long long)b.h_in * b.w_in * C * 2;
  const long long w_bytes = (long long)g.n_gemm * g.k_gemm * 2;
  if (img_bytes >= (1ll << 31) || w_bytes >= (1ll << 31)) return false;
  const long long pw = (long long)b.w_in + 2ll * g.pad_w;
  const long long ph = (long long)b.h_in + 2ll * g.pad_h;
  if (pw * ph >= (1ll << 30) || (long long)b.h_in * b.w_in >= (1ll << 24)) return false;
  const long long table_bytes = TRACEA_MAX_EPILOGUE_OPS * 2 * 64 * 4;
  const long long ring_bytes = (long long)v.lds_bytes - table_bytes;
  const int hw = b.h_out * b.w_out;
  const int grid_n = (g.n_gemm + v.bn - 1) / v.bn;
  const long long cus = device_limits().cus;
  const long long t_min = (hw + v.bm - 1) / v.bm;
  const long long rounds = ((long long)b.batch * t_min * grid_n + cus - 1) / cus;
  long long tiles = rounds * cus / ((long long)b.batch * grid_n);
  if (tiles < t_min) tiles = t_min;
  if (tiles > (hw + 15) / 16) tiles = (hw + 15) / 16;
  const int tm = (int)((hw + tiles - 1) / tiles);
  const int cpp = (C / 8) | 1;
  const long long row_chunks = pw * cpp;
  if (row_chunks >= (1ll << 20)) return false;
  const int seg = (int)((row_chunks + 63) / 64);
  auto patch_for = [&](int t) -> long long {
    long long out_rows = 1;
    for (int p0 = 0; p0 < hw; p0 += t) {
      const int last = (p0 + t < hw ? p0 + t : hw) - 1;
      const long long span = last / b.w_out - p0 / b.w_out + 1;
      if (span > out_rows) out_rows = span;
    }
    const long long rows = (out_rows - 1) * g.stride_h + (long long)(b.r_sz - 1) * g.dil_h + 1;
    return (rows * row_chunks * 16 + 1023) / 1024 * 1024;
  };
  const long long room = (long long)device_limits().lds_bytes - ring_bytes - table_bytes;
  int tm_fit = 0;
  for (int t = tm < v.bm ? tm : v.bm; t >= 16 && tm_fit == 0; --t)
    if (patch_for(t) <= room) tm_fit = t;
  for (int t = tm + 1; t <= v.bm && t <= hw && tm_fit == 0; ++t)
    if (patch_for(t) <= room) tm_fit = t;
  if (tm_fit == 0) return false;
  a->r_sz = b.r_sz;
  a->p_tm = tm_fit;
  a->p_tiles = (hw + tm_fit - 1) / tm_fit;
  a->p_pw = (int)pw;
  a->p_cpp = cpp;
  a->p_iters = 0;
  a->p_np_bytes = (int)patch_for(tm_fit);
  a->p_seg = seg;
  a->p_ppi = 0;
  magic_for_divisor((uint32_t)cpp, (uint64_t)seg * 64, &a->p_cpp_m, &a->p_cpp_s);
  a->p_pw_m = 0; a->p_pw_s = 0;
  a->grid_m = b.batch * a->p_tiles;
  a->grid_n = grid_n;
  magic_for_divisor((uint32_t)grid_n, (uint64_t)a->grid_m * grid_n, &a->gn_m, &a->gn_s);
  magic_for_divisor((uint32_t)a->p_tiles, (uint64_t)a->grid_m, &a->pt_m, &a->pt_s);
  a->group_m = 1;
  a->b_bytes = (unsigned)w_bytes;
  a->a_bytes = 0;
  return true;
}

// Plan of the 8-channel first-layer kernel (pipeline 10): tiles of whole output rows (up to 128 pixels; flat
// runs of 128 pixels for wider rows) whose patch fits LDS twice beside the staging area; rows of RP 16-byte
// pixels, RP a multiple of 8 that covers the padded row and the 8 taps read for the last output pixel; one
// workgroup per CU and filter slab at most, walking the tiles.
bool plan_conv_thin8(const ConvGeometry &g, const ContractionVariant &v, bool w_ncontig, ContractionArgs *a) {
  const TraceaConvParamsBlock &b = g.block;
  if (v.pipeline != 10 || w_ncontig || b.c_in != 8 || b.r_sz != v.stages || b.s_sz > 8 || g.dil_w != 1 ||
      g.k_gemm != b.r_sz * b.s_sz * 8)
    return false;
  const long long img_bytes = (long long)b.h_in * b.w_in * 8 * 2;
  const long long w_bytes = (long long)g.n_gemm * g.k_gemm * 2;
  if (img_bytes >= (1ll << 31) || w_bytes >= (1ll << 31)) return false;
  long long pw = (long long)b.w_in + 2ll * g.pad_w;
  const long long reach = (long long)(b.w_out - 1) * g.stride_w + 8;
  if (reach > pw) pw = reach;
  const long long rp = (pw + 7) / 8 * 8;
  const long long ph = (long long)b.h_in + 2ll * g.pad_h;
  if (rp * ph >= (1ll << 26) || (long long)b.h_in * b.w_in >= (1ll << 24)) return false;
  const long long table_bytes = TRACEA_MAX_EPILOGUE_OPS * 2 * 64 * 4;
  const long long frag_bytes = (long long)b.r_sz * 8 * 1024;
  const int hw = b.h_out * b.w_out;
  const int grid_n = (g.n_gemm + v.bn - 1) / v.bn;
  auto patch_for = [&](int t) -> long long {
    long long out_rows = 1;
    for (int p0 = 0; p0 < hw; p0 += t) {
      const int last = (p0 + t < hw ? p0 + t : hw) - 1;
      const long long span = last / b.w_out - p0 / b.w_out + 1;
      if (span > out_rows) out_rows = span;
    }
    const long long rows = (out_rows - 1) * g.stride_h + (long long)(b.r_sz - 1) * g.dil_h + 1;
    return (rows * rp * 16 + 1023) / 1024 * 1024;
  };
  auto lds_for = [&](int t) -> long long {
    const long long pb = patch_for(t);
    const long long staging = (long long)t * 68 * 4, spill = frag_bytes - pb;
    return 2 * pb + (staging > spill ? staging : spill) + table_bytes;
  };
  // candidates: whole rows, most first; then flat tiles
  int tm_fit = 0;
  if (b.w_out <= v.bm) {
    for (int rows = v.bm / b.w_out; rows >= 1 && tm_fit == 0; --rows) {
      const int t = rows * b.w_out < hw ? rows * b.w_out : hw;
      if (lds_for(t) <= (long long)device_limits().lds_bytes) tm_fit = t;
    }
  }
  for (int t = v.bm < hw ? v.bm : hw; t >= 16 && tm_fit == 0; t -= 16)
    if (lds_for(t) <= (long long)device_limits().lds_bytes) tm_fit = t;
  if (tm_fit == 0) return false;
  a->r_sz = b.r_sz;
  a->p_tm = tm_fit;
  a->p_tiles = (hw + tm_fit - 1) / tm_fit;
  a->p_pw = (int)rp;
  a->p_cpp = 1;
  a->p_np_bytes = (int)patch_for(tm_fit);
  a->p_seg = (int)((rp + 63) / 64);
  a->p_ppi = 0;
  a->p_cpp_m = 0; a->p_cpp_s = 0; a->p_pw_m = 0; a->p_pw_s = 0;
  a->grid_m = b.batch * a->p_tiles;
  a->grid_n = grid_n;
  long long slots = device_limits().cus / grid_n;
  if (slots < 1) slots = 1;
  if (slots > a->grid_m) slots = a->grid_m;
  a->p_iters = (int)slots;  // workgroups per filter slab
  magic_for_divisor((uint32_t)grid_n, (uint64_t)slots * grid_n, &a->gn_m, &a->gn_s);
  magic_for_divisor((uint32_t)a->p_tiles, (uint64_t)a->grid_m, &a->pt_m, &a->pt_s);
  a->group_m = 1;
  a->b_bytes = (unsigned)w_bytes;
  a->a_bytes = 0;
  return true;
}

// The operator chain in the fast form of the filter-resident kernel: [affine] [ReLU] [residual] [ReLU],
// each part at most once and in this order, affine = bias / scale-shift / BatchNorm; every tile has all 64
// channels, output rows and residual rows are 8-byte aligned and addressable with 32-bit byte offsets
// inside a tile, output and residual have the operand type.  Anything else: sig = -1 (general path).
void fast_epilogue_form(const EpilogueChain &chain, int dtype, ContractionArgs *a) {
  ContractionArgs::FastEpilogue fe{};
  fe.sig = -1;
  a->fe = fe;
  bool ok = a->N % 64 == 0 && (a->ldc & 3) == 0 && aligned(a->C, 8) && a->out_dtype == dtype &&
            (long long)a->p_tm * a->ldc * 2 < (1ll << 31);
  int sig = 0, stage = 0;
  for (int o = 0; o < chain.n_ops && ok; ++o) {
    const EpilogueOpDev &op = chain.ops[o];
    const bool aff = op.kind == TRACEA_EPI_OP_BIAS_ADD || op.kind == TRACEA_EPI_OP_SCALE_SHIFT || op.kind == TRACEA_EPI_OP_BATCHNORM;
    int part;
    if (op.kind == TRACEA_EPI_OP_NONE) continue;
    else if (aff) part = 0;
    else if (op.kind == TRACEA_EPI_OP_RELU) part = stage <= 2 ? 1 : 3;
    else if (op.kind == TRACEA_EPI_OP_RESIDUAL_ADD) part = 2;
    else { ok = false; break; }
    if (part < stage) { ok = false; break; }
    sig |= 1 << part;
    stage = part + 1;
    if (aff) {
      fe.aff_kind = op.kind; fe.aff_dtype = op.dtype;
      fe.p0 = op.p0; fe.p1 = op.p1; fe.p2 = op.p2; fe.p3 = op.p3; fe.epsilon = op.epsilon;
    }
    if (part == 2) {
      fe.res = op.p0; fe.res_ld = op.ld;
      ok = op.dtype == dtype && (op.ld & 3) == 0 && aligned(op.p0, 8) && (long long)a->p_tm * op.ld * 2 < (1ll << 31);
    }
  }
  if (!ok) return;
  fe.sig = sig;
  a->fe = fe;
}

bool plan_conv_resident(const ConvGeometry &g, const ContractionVariant &v, bool w_ncontig, ContractionArgs *a) {
  if (v.pipeline == 7 || v.pipeline == 8) return plan_conv_wave16(g, v, w_ncontig, a);
  if (v.pipeline == 9) return plan_conv_ksplit16(g, v, w_ncontig, a);
  if (v.pipeline == 10) return plan_conv_thin8(g, v, w_ncontig, a);
  return v.pipeline == 5 ? plan_conv_filter_resident(g, v, w_ncontig, a) : plan_conv_patch(g, v, w_ncontig, a);
}

TraceaStatus run_conv(const ConvPlan &plan, const EpilogueChain &chain, hipStream_t stream) {
  const ConvGeometry &g = plan.geo;
  DeviceScope scope(plan.out.device);
  if (scope.err != hipSuccess) return hip_status("hipSetDevice", (int)scope.err);
  ContractionArgs a{};
  a.A = plan.x.ptr; a.B = plan.w.ptr; a.C = plan.out.ptr;
  a.M = g.m_gemm; a.N = g.n_gemm; a.K = g.k_gemm;
  a.lda = 0; a.ldb = plan.ldb; a.ldc = plan.ldc;
  a.out_dtype = plan.out.dtype;
  a.h_in = g.block.h_in; a.w_in = g.block.w_in; a.c_in = g.block.c_in;
  a.h_out = g.block.h_out; a.w_out = g.block.w_out; a.s_sz = g.block.s_sz;
  a.stride_h = g.stride_h; a.stride_w = g.stride_w;
  a.pad_h = g.pad_h; a.pad_w = g.pad_w; a.dil_h = g.dil_h; a.dil_w = g.dil_w;
  a.hw_m = g.block.hw_m; a.hw_s = g.block.hw_s; a.w_m = g.block.w_m; a.w_s = g.block.w_s;
  a.sc_m = g.block.sic_m; a.sc_s = g.block.sic_s; a.c_m = g.block.c_m; a.c_s = g.block.c_s;
  a.epi = chain;
  char key[200];
  snprintf(key, sizeof(key), "conv_%d_%d_%d_%d_%d_%d_%d_%d_%d_%s", g.block.batch, g.block.h_in,
           g.block.w_in, g.block.c_in, g.block.k_out, g.block.r_sz, g.block.s_sz, g.stride_h,
           g.pad_h, tuning_device_name());
  int vi = pick_contraction("conv2d", key, a.M, a.N, a.K, true, plan.x.dtype, plan.w_ncontig);
  if (vi < 0) return fail(TRACEA_UNKNOWN_ERROR, "conv2d: no kernel variant available");
  // Default choice of the filter-resident variant (patch and 64 filters of K = 576 in LDS together, no
  // barrier in its main loop): wherever it can run and the launch fills most of the device with tiles of
  // at least 10 pixel blocks.  Measured in a replayed HIP graph against the best other variant: N32
  // 56x56x64->64 14.1 us / 16.7; N64 25.2 / 28.6; N32 64->128 24.5 / 28.8; N8 10.3 / 9.5 (not taken).
  bool resident_chosen = false;
  // First choice: the kernels on 16x16x32 MFMAs with the patch in LDS and the filter slab resident or in a
  // ring (pipelines 7 to 10), where their plan fits, the launch fills most of the device and a workgroup's
  // tile is at least three quarters of the kernel's largest (smaller tiles leave its waves' blocks empty).
  if (forced_variant("conv2d") < 0 && tuning_cache_lookup_variant(key, plan.x.dtype, plan.w_ncontig) < 0) {
    for (int i = 0; i < contraction_variant_count() && !resident_chosen; ++i) {
      const ContractionVariant &cv = contraction_variant(i);
      if (cv.pipeline < 7 || cv.pipeline > 10) continue;
      ContractionArgs probe = a;
      // (the K-split members with tiles of one or two pixel blocks are for small launches: 14x14x256 at batch 1
      // 6.4 us on 52 workgroups against 8.4 streamed and split along K; the stride-2 3x3 and 1x1 layers from
      // 14x14x256 to 7x7x512 at batch 1, 32 workgroups, 6.5 and 3.8 us against 7.8 and 5.1; from 32 workgroups on)
      const long long enough = cv.pipeline == 9 && cv.bm <= 32 ? 32 * 4 : device_limits().cus * 3;
      // (tile at least three quarters of the member's largest; the larger K-split members, whose waves all work
      // on every pixel block there is, from two fifths: 14x14x256 at batch 16, tiles of 49 of 112 pixels, 11.8 us
      // against 13.1 on the 32-pixel member)
      if (!plan_conv_resident(g, cv, plan.w_ncontig, &probe)) continue;
      const bool tile_ok = cv.pipeline == 9 && cv.bm > 32 ? probe.p_tm * 5 >= cv.bm * 2 : probe.p_tm * 4 >= cv.bm * 3;
      if ((long long)probe.grid_m * probe.grid_n * 4 >= enough && tile_ok) {
        vi = i;
        resident_chosen = true;
      }
    }
  }
  if (!resident_chosen && forced_variant("conv2d") < 0 && tuning_cache_lookup_variant(key, plan.x.dtype, plan.w_ncontig) < 0) {
    for (int i = 0; i < contraction_variant_count() && !resident_chosen; ++i) {
      const ContractionVariant &cv = contraction_variant(i);
      if (cv.pipeline != 5) continue;
      ContractionArgs probe = a;
      if (plan_conv_resident(g, cv, plan.w_ncontig, &probe) && (long long)probe.grid_m * probe.grid_n * 4 >= device_limits().cus * 3 &&
          probe.p_tm >= 320) {
        vi = i;
        resident_chosen = true;
      }
    }
  }
  // Default choice of a patch-resident variant: stride-1 convolutions with a real filter
  // window whose K fits 40 filter tiles (the kernel has no split along K).  Fitted on the
  // ResNet-18/50 layer shapes at batch 1, 8 and 32, every variant timed inside a replayed
  // HIP graph (eager launches from a host loop cost 9-15 us apiece here and hide differences
  // between kernels shorter than that): the 256-pixel tile (eight waves of 32 pixels) wins
  // with at least 256 workgroups of mostly real pixels (N32 56x56x64->64: 15.0 us against
  // 17.8 for the best streamed variant; N32 28x28 128->128: 14.0 against 15.3); the
  // 128-pixel tile (eight waves of 32 pixels x 32 filters) wins on small launches with a
  // short K (one 56x56x64->64 image: 7.4 us against 8.4).  Everywhere else the streamed
  // 8-wave 128x64 and pipelined 64x64 tiles are as fast or faster.  A tuning-cache entry or
  // a forced variant wins over this rule, and tracea_autotune_conv2d measures every variant.
  if (!resident_chosen && forced_variant("conv2d") < 0 && tuning_cache_lookup_variant(key, plan.x.dtype, plan.w_ncontig) < 0 && g.stride_h == 1 &&
      g.stride_w == 1 && g.block.r_sz * g.block.s_sz > 1 && a.K % 64 == 0 && a.K / 64 <= 40) {
    const long long hw = (long long)g.block.h_out * g.block.w_out;
    int chosen = -1;
    for (int i = 0; i < contraction_variant_count() && chosen < 0; ++i) {
      const ContractionVariant &cv = contraction_variant(i);
      if (cv.pipeline != 4 || cv.bm != 256 || cv.bn != 64) continue;
      ContractionArgs probe = a;
      if (plan_conv_patch(g, cv, plan.w_ncontig, &probe) && (long long)probe.grid_m * probe.grid_n >= device_limits().cus &&
          hw * 4 >= (long long)probe.p_tiles * cv.bm * 3)
        chosen = i;
    }
    for (int i = 0; i < contraction_variant_count() && chosen < 0; ++i) {
      const ContractionVariant &cv = contraction_variant(i);
      if (cv.pipeline != 4 || cv.bm != 128 || cv.bn != 64) continue;
      ContractionArgs probe = a;
      if (plan_conv_patch(g, cv, plan.w_ncontig, &probe) && (long long)probe.grid_m * probe.grid_n < 100 &&
          a.K / 64 <= 9)
        chosen = i;
    }
    if (chosen >= 0) vi = chosen;
  }
  const long long x_extent = (long long)g.block.batch * g.block.h_in * g.block.w_in * g.block.c_in * 2;
  const long long w_extent = (long long)g.n_gemm * g.k_gemm * 2;
  const bool small = x_extent < (1ll << 31) && w_extent < (1ll << 31);
  if (conv_only(contraction_variant(vi)) && plan_conv_resident(g, contraction_variant(vi), plan.w_ncontig, &a)) {
    if (contraction_variant(vi).pipeline == 5 || contraction_variant(vi).pipeline >= 7) fast_epilogue_form(chain, plan.x.dtype, &a);
    const int e = contraction_variant(vi).launch(a, true, plan.x.dtype, false, stream);
    // a member that refuses the arguments its plan accepted (it launched nothing) gives way to the
    // selector's choice below, like one whose plan failed
    if (e != (int)hipErrorInvalidValue) {
      t_last_conv = vi;
      return hip_status("conv2d launch", e);
    }
    (void)hipGetLastError();
  }
  // a patch-resident variant that cannot run this problem (asked for by a forced
  // index or a cache entry) gives way to the selector's choice, not to whatever
  // shares its tile shape
  if (conv_only(contraction_variant(vi))) {
    vi = select_contraction_variant(a.M, a.N, a.K, true);
    if (vi < 0) return fail(TRACEA_UNKNOWN_ERROR, "conv2d: no kernel variant available");
  }
  vi = resolve_variant(vi, true, !small, true, plan.w_ncontig);
  const ContractionVariant &v = contraction_variant(vi);
  a.a_bytes = (unsigned)(small ? x_extent : 0);
  a.b_bytes = (unsigned)(small ? w_extent : 0);
  fill_grid(&a, v);
  t_last_conv = vi;
  return launch_maybe_split("conv2d launch", v, a, chain, true, plan.x.dtype, plan.w_ncontig, plan.out.device, stream);
}

// A convolution whose operands the kernels cannot read in place -- input channels that are not a multiple of 8
// (an RGB first layer), [R,S,C,K] filters with a ragged K, operands that do not start on 16 bytes -- runs from
// copies with the channels padded to a multiple of 8 with zeros (they add nothing to any sum), activations
// NHWC and filters [K,R,S,C], in the per-(device, stream) buffer of run_gemm's padded operands.  (The
// reference's kernel reads such channels element by element: src/emitter/cuda/conv.rs:228-240.)
TraceaStatus run_conv_maybe_padded(const ConvPlan &plan, const TraceaTensorView *tout_c, const TraceaConv2dParams &params,
                                   const EpilogueChain &chain, hipStream_t stream) {
  if (!plan.pad_c) return run_conv(plan, chain, stream);
  const View &x = plan.x, &w = plan.w;
  const long long N = x.shape[0], H = x.shape[1], W = x.shape[2], C = x.shape[3];
  const long long K = w.shape[0], R = w.shape[1], S = w.shape[2];
  const long long Cp = (C + 7) / 8 * 8;
  const size_t x_bytes = (size_t)(N * H * W) * (size_t)Cp * 2, w_bytes = (size_t)(K * R * S) * (size_t)Cp * 2;
  const size_t x_room = (x_bytes + 255) / 256 * 256;
  DeviceScope scope(plan.out.device);
  if (scope.err != hipSuccess) return hip_status("hipSetDevice", (int)scope.err);
  unsigned char *buf = (unsigned char *)pad_scratch(plan.out.device, stream, x_room + w_bytes);
  if (buf == nullptr)
    return fail(TRACEA_UNSUPPORTED_CONFIG,
                "tracea_conv2d: input channels (%lld) must be a multiple of 8 ([R,S,C,K] filters: output channels too) and x, "
                "w 16-byte aligned where no buffer for padded copies can be had (stream under capture, or above 1 GiB)", C);
  int e = launch_pad_copy(x.ptr, buf, 2, N * H * W, C, C, 1, N * H * W, Cp, stream);
  if (e == 0) {
    if (!plan.w_ncontig) e = launch_pad_copy(w.ptr, buf + x_room, 2, K * R * S, C, C, 1, K * R * S, Cp, stream);
    else e = launch_pad_copy(w.ptr, buf + x_room, 2, K * R * S, C, 1, K, K * R * S, Cp, stream, R * S, C * K);
  }
  if (e != 0) return hip_status("operand copy launch", e);
  const uint64_t xs[4] = {(uint64_t)N, (uint64_t)H, (uint64_t)W, (uint64_t)Cp}, ws[4] = {(uint64_t)K, (uint64_t)R, (uint64_t)S, (uint64_t)Cp};
  TraceaTensorView tx{}, tw{};
  tx.ptr = buf; tx.rank = 4; tx.shape = xs; tx.stride = nullptr; tx.dtype = (TraceaDType)x.dtype; tx.device_id = x.device;
  tw.ptr = buf + x_room; tw.rank = 4; tw.shape = ws; tw.stride = nullptr; tw.dtype = (TraceaDType)w.dtype; tw.device_id = w.device;
  TraceaTensorView tout = *tout_c;
  ConvPlan padded;
  const TraceaStatus st = conv_common(tx, tw, &tout, params, &padded);
  if (st != TRACEA_SUCCESS) return st;
  if (padded.pad_c) return fail(TRACEA_UNKNOWN_ERROR, "tracea_conv2d: padded operands still not readable");
  return run_conv(padded, chain, stream);
}

}  // namespace

TraceaStatus dispatch_conv2d_kind(const TraceaTensorView &tx, const TraceaTensorView &tw,
                                  const TraceaTensorView *bias, const TraceaTensorView *residual,
                                  TraceaTensorView *tout, const TraceaConv2dParams &params) {
  ConvPlan plan;
  TraceaStatus st = conv_common(tx, tw, tout, params, &plan);
  if (st != TRACEA_SUCCESS) return st;
  TraceaEpilogueOp ops[TRACEA_MAX_EPILOGUE_OPS];
  const int n = kind_to_ops((int)params.epilogue, bias, residual, ops);
  if (n < 0) return fail(TRACEA_INVALID_PARAMS, "tracea_conv2d: unknown epilogue kind %d", (int)params.epilogue);
  st = check_bias_residual("tracea_conv2d", bias, residual, plan.out.shape[3], plan.out,
                           plan.out.device, ops, n);
  if (st != TRACEA_SUCCESS) return st;
  EpilogueChain chain{};
  st = lower_chain("tracea_conv2d", ops, (uint32_t)n, plan.out.shape[3], plan.out.shape[3], &chain);
  if (st != TRACEA_SUCCESS) return st;
  return run_conv_maybe_padded(plan, tout, params, chain, (hipStream_t)params.stream);
}

TraceaStatus dispatch_conv2d_ops(const TraceaTensorView &tx, const TraceaTensorView &tw,
                                 TraceaTensorView *tout, const TraceaConv2dParams &params,
                                 const TraceaEpilogueOp *ops, uint32_t n_ops) {
  ConvPlan plan;
  TraceaStatus st = conv_common(tx, tw, tout, params, &plan);
  if (st != TRACEA_SUCCESS) return st;
  EpilogueChain chain{};
  st = lower_chain("tracea_conv2d_ex", ops, n_ops, plan.out.shape[3], plan.out.shape[3], &chain);
  if (st != TRACEA_SUCCESS) return st;
  return run_conv_maybe_padded(plan, tout, params, chain, (hipStream_t)params.stream);
}

// ---- ConvTranspose2d ---------------------------------------------------------------
// cols = x[(b,hi,wi), c] . w[c, (k,r,s)] on the GEMM kernels, then the gather
// kernel sums the taps that land on each output pixel and runs the chain.
namespace {

// The filter bank [K,R,S,C] seen as the matrix B[c, j], j running densely over
// (k, r, s) in whatever order the strides give.
struct FilterMatrix {
  bool c_inner;        // true: B is K-contiguous (element (c, j) at j*ld + c); false: row-major, (c, j) at c*ld + j
  long long ld;
  long long col[3];    // column of one step of k, r, s
  long long columns;   // K*R*S
};

bool dense_block(const View &w, long long unit, long long *col) {
  int order[3] = {0, 1, 2};
  for (int i = 0; i < 3; ++i)
    for (int j = i + 1; j < 3; ++j)
      if (w.stride[order[j]] < w.stride[order[i]]) std::swap(order[i], order[j]);
  long long expect = unit;
  for (int i = 0; i < 3; ++i) {
    const int d = order[i];
    col[d] = 0;
    if (w.shape[d] == 1) continue;
    if (w.stride[d] != expect) return false;
    col[d] = expect / unit;
    expect *= w.shape[d];
  }
  return true;
}

bool filter_as_matrix(const View &w, FilterMatrix *f) {
  const long long C = w.shape[3], J = w.shape[0] * w.shape[1] * w.shape[2];
  f->columns = J;
  // input channels outermost: the reference kernel's [C*R*S, K] rows (C, R, S, K), or (C, K, R, S)
  if (dense_block(w, 1, f->col) && (C == 1 || w.stride[3] >= J)) {
    f->c_inner = false;
    f->ld = C == 1 ? J : w.stride[3];
    return true;
  }
  // input channels innermost, e.g. contiguous [K,R,S,C]
  if (C == 1 || w.stride[3] == 1) {
    long long unit = 0;
    for (int d = 0; d < 3; ++d)
      if (w.shape[d] > 1 && (unit == 0 || w.stride[d] < unit)) unit = w.stride[d];
    if (unit == 0) unit = C;
    if (unit >= C && dense_block(w, unit, f->col)) {
      f->c_inner = true;
      f->ld = unit;
      return true;
    }
  }
  return false;
}

struct ConvTransposePlan {
  View x, w, out;
  FilterMatrix fm;
  int stride_h, stride_w, pad_h, pad_w;
  long long ldx, ldc;
};

TraceaStatus conv_transpose_common(const TraceaTensorView &tx, const TraceaTensorView &tw, TraceaTensorView *tout,
                                   const TraceaConvTranspose2dParams &p, ConvTransposePlan *plan) {
  const char *me = "tracea_conv_transpose2d";
  if (!runtime_ready()) return fail(TRACEA_UNKNOWN_ERROR, "%s: tracea_init has not been called", me);
  if (tout == nullptr) return fail(TRACEA_INVALID_PARAMS, "%s: output view is NULL", me);
  // the reference states groups = 1 and dilation = 1 as constraints and reads neither
  // field (src/emitter/conv_transpose.rs:26-29); 0 is taken as "left unset"
  if (p.groups > 1) return fail(TRACEA_UNSUPPORTED_CONFIG, "%s: groups=%u (only groups=1)", me, p.groups);
  if (p.dilation_h > 1 || p.dilation_w > 1)
    return fail(TRACEA_UNSUPPORTED_CONFIG, "%s: dilation %ux%u (only 1)", me, p.dilation_h, p.dilation_w);
  if (p.stride_h == 0 || p.stride_w == 0) return fail(TRACEA_INVALID_PARAMS, "%s: stride must be at least 1", me);
  TraceaStatus st;
  View &x = plan->x, &w = plan->w, &out = plan->out;
  if ((st = read_view("tracea_conv_transpose2d: x", tx, 4, &x)) != TRACEA_SUCCESS) return st;
  if ((st = read_view("tracea_conv_transpose2d: w", tw, 4, &w)) != TRACEA_SUCCESS) return st;
  if ((st = read_view("tracea_conv_transpose2d: out", *tout, 4, &out)) != TRACEA_SUCCESS) return st;
  if (!is_float_type(x.dtype) || w.dtype != x.dtype)
    return fail(TRACEA_UNSUPPORTED_CONFIG, "%s: activations %s / filters %s; f32, f16 or bf16 (both alike) required",
                me, dtype_name(x.dtype), dtype_name(w.dtype));
  if (!is_float_type(out.dtype))
    return fail(TRACEA_UNSUPPORTED_CONFIG, "%s: output dtype %s unsupported", me, dtype_name(out.dtype));
  if ((st = check_device(me, out.device)) != TRACEA_SUCCESS) return st;
  if (x.device != out.device || w.device != out.device)
    return fail(TRACEA_INVALID_PARAMS, "%s: operands live on different devices", me);
  const long long N = x.shape[0], H = x.shape[1], W = x.shape[2], C = x.shape[3];
  const long long K = w.shape[0], R = w.shape[1], S = w.shape[2];
  if (w.shape[3] != C) return fail(TRACEA_INVALID_PARAMS, "%s: x has %lld channels, w expects %lld", me, C, w.shape[3]);
  if (N <= 0 || H <= 0 || W <= 0 || C <= 0 || K <= 0 || R <= 0 || S <= 0)
    return fail(TRACEA_INVALID_PARAMS, "%s: empty dimension", me);
  const long long big = 1ll << 31;
  if (N >= big || H >= big || W >= big || C >= big || K >= big || R >= big || S >= big || K * R * S >= big)
    return fail(TRACEA_UNSUPPORTED_CONFIG, "%s: dimension exceeds 2^31-1", me);
  // H_out = (H_in - 1) * stride - 2 * pad + kernel + output_padding (conv_transpose.rs:36-37)
  const long long Ho = (H - 1) * p.stride_h - 2ll * p.padding_h + R + p.output_padding_h;
  const long long Wo = (W - 1) * p.stride_w - 2ll * p.padding_w + S + p.output_padding_w;
  if (Ho <= 0 || Wo <= 0) return fail(TRACEA_INVALID_PARAMS, "%s: output would be %lldx%lld", me, Ho, Wo);
  if (Ho >= big || Wo >= big) return fail(TRACEA_UNSUPPORTED_CONFIG, "%s: dimension exceeds 2^31-1", me);
  if (out.shape[0] != N || out.shape[1] != Ho || out.shape[2] != Wo || out.shape[3] != K)
    return fail(TRACEA_INVALID_PARAMS, "%s: output shape must be [%lld,%lld,%lld,%lld]", me, N, Ho, Wo, K);
  const long long ldx = x.stride[2];
  if (!(x.stride[3] == 1 && ldx >= C && x.stride[1] == W * ldx && x.stride[0] == H * W * ldx))
    return fail(TRACEA_UNSUPPORTED_CONFIG, "%s: activations must be channel-contiguous NHWC", me);
  const long long ldc = out.stride[2];
  if (!(out.stride[3] == 1 && ldc >= K && out.stride[1] == Wo * ldc && out.stride[0] == Ho * Wo * ldc))
    return fail(TRACEA_UNSUPPORTED_CONFIG, "%s: output must be channel-contiguous NHWK", me);
  if (!filter_as_matrix(w, &plan->fm))
    return fail(TRACEA_UNSUPPORTED_CONFIG,
                "%s: filters (dims [K,R,S,C]) must be stored with the input channels outermost or innermost "
                "and the other three dims dense, e.g. [C,R,S,K], [C,K,R,S] or [K,R,S,C]", me);
  plan->stride_h = (int)p.stride_h; plan->stride_w = (int)p.stride_w;
  plan->pad_h = (int)p.padding_h; plan->pad_w = (int)p.padding_w;
  plan->ldx = ldx; plan->ldc = ldc;
  return TRACEA_SUCCESS;
}

// ---- transposed convolution by output phase ----------------------------------------
// Output pixels whose row is congruent to a modulo stride_h (and column to b modulo stride_w)
// are reached by the taps r = r0 + stride_h*t, r0 = (a + pad_h) mod stride_h, only, from input
// rows q + d - t with oh = a + stride_h*q, d = (a + pad_h - r0) / stride_h: each of the
// stride_h*stride_w phases is an ordinary stride-1 convolution of the input with the flipped
// sub-filter (taps_r x taps_s taps), top padding taps_r - 1 - d, whose output pixels are
// written into their places of the full output by the kernel's row map.  Against the
// formulation through partial products (a GEMM to [pixels, R*S*K] fp32 and a gather) nothing
// but the input, the filters and the output touches memory.
struct PhaseAxis {
  int taps, pad, out;  // taps of the sub-filter, top/left padding, output extent of the phase
  int first_tap;       // r0
};

PhaseAxis phase_axis(int a, int stride, int pad, int filter, long long out_extent) {
  PhaseAxis p{};
  p.first_tap = (a + pad) % stride;
  p.taps = p.first_tap < filter ? (filter - p.first_tap + stride - 1) / stride : 0;
  const int d = (a + pad - p.first_tap) / stride;
  p.pad = p.taps - 1 - d;
  p.out = a < out_extent ? (int)((out_extent - a + stride - 1) / stride) : 0;
  return p;
}

// True when every phase is a convolution the streamed kernels take: taps in every phase, no
// negative padding, half-precision dense NHWC input with channels in 16-byte groups.
bool conv_transpose_by_phase_ok(const ConvTransposePlan &plan) {
  const View &x = plan.x, &w = plan.w, &out = plan.out;
  const long long C = x.shape[3], R = w.shape[1], S = w.shape[2];
  if (!is_half(x.dtype) || C % 8 != 0 || plan.ldx != C || !aligned(x.ptr, 16) || R * S > 64) return false;
  if (x.shape[0] * x.shape[1] * x.shape[2] * C * 2 >= (1ll << 40)) return false;
  for (int a = 0; a < plan.stride_h; ++a) {
    const PhaseAxis p = phase_axis(a, plan.stride_h, plan.pad_h, (int)R, out.shape[1]);
    if (p.taps <= 0 || p.pad < 0 || p.out <= 0) return false;
  }
  for (int b = 0; b < plan.stride_w; ++b) {
    const PhaseAxis p = phase_axis(b, plan.stride_w, plan.pad_w, (int)S, out.shape[2]);
    if (p.taps <= 0 || p.pad < 0 || p.out <= 0) return false;
  }
  return (long long)plan.stride_h * plan.stride_w <= 16;
}

TraceaStatus run_conv_transpose_by_phase(const ConvTransposePlan &plan, const EpilogueChain &chain,
                                         hipStream_t stream) {
  const View &x = plan.x, &w = plan.w, &out = plan.out;
  const int N = (int)x.shape[0], H = (int)x.shape[1], W = (int)x.shape[2], C = (int)x.shape[3];
  const int K = (int)w.shape[0], R = (int)w.shape[1], S = (int)w.shape[2];
  const long long Ho = out.shape[1], Wo = out.shape[2];
  const int sh = plan.stride_h, sw = plan.stride_w;
  // the filter bank, regrouped: phase (a, b) holds [K][taps_r][taps_s][C], flipped
  PhaseFilterArgs f{};
  f.w = w.ptr; f.C = C; f.K = K; f.R = R; f.S = S;
  f.sk = w.stride[0]; f.sr = w.stride[1]; f.ss = w.stride[2]; f.sc = w.stride[3];
  std::vector<long long> phase_off((size_t)sh * sw);
  long long total = 0;
  for (int a = 0; a < sh; ++a)
    for (int b = 0; b < sw; ++b) {
      const PhaseAxis pr = phase_axis(a, sh, plan.pad_h, R, Ho), ps = phase_axis(b, sw, plan.pad_w, S, Wo);
      phase_off[(size_t)a * sw + b] = total;
      for (int t = 0; t < pr.taps; ++t)
        for (int u = 0; u < ps.taps; ++u) {
          const int r = pr.first_tap + sh * t, s_ = ps.first_tap + sw * u;
          const int z = r * S + s_;
          f.tap_base[z] = total + ((long long)(pr.taps - 1 - t) * ps.taps + (ps.taps - 1 - u)) * C;
          f.tap_kstride[z] = pr.taps * ps.taps * C;
        }
      total += (long long)K * pr.taps * ps.taps * C;
    }
  // The regrouped filters live in the per-(device, stream) scratch buffer that split-K launches use
  // (no launch of this path splits K, and work on one stream is ordered); a bank beyond its 64 MiB
  // cap, or a first use while the stream is being captured, takes a stream-ordered allocation.
  hipError_t e = hipSuccess;
  void *filt = nullptr;
  bool pooled = true, regroup = true;
  if (g_ct_filter_cache.load()) {
    // cached copy of this bank: built once (the stream is drained before the copy is published, so that
    // calls on other streams may read it), then no helper launch and no allocation per call
    CtFilterKey key;
    key.v[0] = out.device; key.v[1] = (long long)(uintptr_t)w.ptr; key.v[10] = w.dtype;
    for (int i = 0; i < 4; ++i) { key.v[2 + i] = w.shape[i]; key.v[6 + i] = w.stride[i]; }
    key.v[11] = sh; key.v[12] = sw; key.v[13] = plan.pad_h; key.v[14] = plan.pad_w; key.v[15] = Ho; key.v[16] = Wo;
    std::lock_guard<std::mutex> lk(g_ct_filter_mu);
    auto it = g_ct_filters.find(key);
    if (it != g_ct_filters.end()) {
      filt = it->second;
      regroup = false;
    } else {
      hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
      if (g_ct_filters.size() < 64 && hipStreamIsCapturing(stream, &cap) == hipSuccess && cap == hipStreamCaptureStatusNone &&
          hipMalloc(&filt, (size_t)total * 2 + 256) == hipSuccess) {
        f.out = filt;
        TraceaStatus fs = hip_status("phase filter launch", launch_phase_filters(f, stream));
        if (fs == TRACEA_SUCCESS && hipStreamSynchronize(stream) != hipSuccess) fs = TRACEA_UNKNOWN_ERROR;
        if (fs != TRACEA_SUCCESS) {
          (void)hipFree(filt);
          return fs == TRACEA_UNKNOWN_ERROR ? fail(TRACEA_UNKNOWN_ERROR, "tracea_conv_transpose2d: regrouping the filters failed") : fs;
        }
        g_ct_filters[key] = filt;
        regroup = false;
      } else {
        filt = nullptr;  // (cache full, stream under capture or out of memory: per-call regrouping below)
      }
    }
  }
  if (filt == nullptr) {
    filt = splitk_scratch(out.device, stream, (size_t)total * 2 + 256);
    pooled = filt != nullptr;
    if (!pooled) {
      e = hipMallocAsync(&filt, (size_t)total * 2 + 256, stream);
      if (e != hipSuccess) return hip_status("tracea_conv_transpose2d: workspace allocation", (int)e);
    }
  }
  f.out = filt;
  TraceaStatus st = regroup ? hip_status("phase filter launch", launch_phase_filters(f, stream)) : TRACEA_SUCCESS;
  const long long x_extent = (long long)N * H * W * C * 2;
  // Phases that are alike but for their padding (even filter extents divided by the stride: the 4x4
  // stride-2 decoder layer) go out as one launch with the phase in blockIdx.z.
  bool uniform = sh <= 4 && sw <= 4 && sh * sw > 1;
  for (int a = 1; a < sh && uniform; ++a) {
    const PhaseAxis p0 = phase_axis(0, sh, plan.pad_h, R, Ho), pa = phase_axis(a, sh, plan.pad_h, R, Ho);
    uniform = p0.taps == pa.taps && p0.out == pa.out;
  }
  for (int b = 1; b < sw && uniform; ++b) {
    const PhaseAxis p0 = phase_axis(0, sw, plan.pad_w, S, Wo), pb = phase_axis(b, sw, plan.pad_w, S, Wo);
    uniform = p0.taps == pb.taps && p0.out == pb.out;
  }
  for (int a = 0; a < sh && st == TRACEA_SUCCESS; ++a)
    for (int b = 0; b < sw && st == TRACEA_SUCCESS; ++b) {
      if (uniform && (a > 0 || b > 0)) continue;  // phase (0, 0) launched all of them
      const PhaseAxis pr = phase_axis(a, sh, plan.pad_h, R, Ho), ps = phase_axis(b, sw, plan.pad_w, S, Wo);
      const long long m = (long long)N * pr.out * ps.out, kg = (long long)pr.taps * ps.taps * C;
      if (m >= (1ll << 31) || kg >= (1ll << 31)) {
        st = fail(TRACEA_UNSUPPORTED_CONFIG, "tracea_conv_transpose2d: problem too large for 32-bit row indices");
        break;
      }
      ContractionArgs c{};
      c.A = x.ptr;
      c.B = (const unsigned short *)filt + phase_off[(size_t)a * sw + b];
      c.C = out.ptr;
      c.M = (int)m; c.N = K; c.K = (int)kg;
      c.ldb = kg; c.ldc = plan.ldc;
      c.out_dtype = out.dtype;
      c.h_in = H; c.w_in = W; c.c_in = C;
      c.h_out = pr.out; c.w_out = ps.out; c.s_sz = ps.taps;
      c.stride_h = c.stride_w = 1; c.dil_h = c.dil_w = 1;
      c.pad_h = pr.pad; c.pad_w = ps.pad;
      magic_for_divisor((uint32_t)(pr.out * ps.out), (uint64_t)m, &c.hw_m, &c.hw_s);
      magic_for_divisor((uint32_t)ps.out, (uint64_t)pr.out * ps.out, &c.w_m, &c.w_s);
      magic_for_divisor((uint32_t)(ps.taps * C), (uint64_t)kg + 1024, &c.sc_m, &c.sc_s);
      magic_for_divisor((uint32_t)C, (uint64_t)ps.taps * C, &c.c_m, &c.c_s);
      c.out_map = 1;
      c.o_sh = sh; c.o_sw = sw; c.o_a = a; c.o_b = b; c.o_wo = (int)Wo;
      c.o_img = Ho * Wo;
      if (uniform) {
        c.phases = sh * sw;
        c.phase_b_stride = (long long)K * kg;
        for (int i = 0; i < sh; ++i) c.phase_pad_h[i] = phase_axis(i, sh, plan.pad_h, R, Ho).pad;
        for (int i = 0; i < sw; ++i) c.phase_pad_w[i] = phase_axis(i, sw, plan.pad_w, S, Wo).pad;
      }
      c.epi = chain;
      // uniform phases go out as one launch: the selector sees the rows of all of them
      // (VAE layer 65.2 -> 53.8 us on 128x128 tiles instead of 128x64)
      const long long m_launch = uniform ? (long long)c.M * sh * sw : (long long)c.M;
      int vi = select_contraction_variant((int)(m_launch < (1ll << 31) - 1 ? m_launch : (1ll << 31) - 1), c.N, c.K, true);
      if (vi < 0) { st = fail(TRACEA_UNKNOWN_ERROR, "tracea_conv_transpose2d: no kernel variant available"); break; }
      const long long w_extent = (long long)K * kg * 2;
      const bool small = x_extent < (1ll << 31) && w_extent < (1ll << 31);
      vi = resolve_variant(vi, true, !small, true, false);
      const ContractionVariant &v = contraction_variant(vi);
      c.a_bytes = (unsigned)(small ? x_extent : 0);
      c.b_bytes = (unsigned)(small ? w_extent : 0);
      fill_grid(&c, v);
      t_last_conv = vi;
      st = hip_status("conv_transpose2d phase launch", v.launch(c, true, x.dtype, false, stream));
    }
  if (!pooled) {
    e = hipFreeAsync(filt, stream);
    if (st == TRACEA_SUCCESS && e != hipSuccess) st = hip_status("tracea_conv_transpose2d: workspace release", (int)e);
  }
  return st;
}

TraceaStatus run_conv_transpose(const ConvTransposePlan &plan, const EpilogueChain &chain, hipStream_t stream) {
  const View &x = plan.x, &w = plan.w, &out = plan.out;
  const long long N = x.shape[0], H = x.shape[1], W = x.shape[2], C = x.shape[3];
  const long long K = w.shape[0], Ho = out.shape[1], Wo = out.shape[2];
  const long long J = plan.fm.columns;
  DeviceScope scope(out.device);
  if (scope.err != hipSuccess) return hip_status("hipSetDevice", (int)scope.err);
  // tracea_last_variant afterwards names what THIS call launched: a convolution variant (by phase) or a
  // GEMM variant (partial products), the other one reads -1
  t_last_contraction = -1;
  t_last_conv = -1;
  if (g_conv_transpose_by_phase.load() && conv_transpose_by_phase_ok(plan))
    return run_conv_transpose_by_phase(plan, chain, stream);
  // Images per pass: the partial products of a pass stay below 512 MiB, the GEMM
  // rows and the gather kernel's thread count below 2^31.
  const long long per_image = H * W * J * 4;
  long long nb = per_image > 0 ? (512ll << 20) / per_image : N;
  if (nb < 1) nb = 1;
  if (nb > N) nb = N;
  const long long lim = (1ll << 31) - 1;
  while (nb > 1 && (nb * H * W > lim || nb * Ho * Wo * K > lim)) nb = (nb + 1) / 2;
  if (H * W > lim || Ho * Wo * K > lim || per_image / 4 >= (1ll << 40))
    return fail(TRACEA_UNSUPPORTED_CONFIG, "tracea_conv_transpose2d: one image is too large");
  // Filters already stored in the order the GEMM reads are used in place; any other order is
  // copied into it (C*R*S*K elements, next to the partial products in the temporary buffer).
  const long long R = w.shape[1], S = w.shape[2];
  // The gather kernel wants the columns ordered (r, s, k).  The half-precision GEMM kernels
  // read either orientation of B at nearly the same speed, so [R,S,K,C] and [C,R,S,K] (the
  // reference's own order) are both used in place; the fp32 kernel reads a row-major B only.
  const bool cols_ok = (K == 1 || plan.fm.col[0] == 1) && (S == 1 || plan.fm.col[2] == K) &&
                       (R == 1 || plan.fm.col[1] == S * K);
  const bool half = is_half(x.dtype);
  const bool in_place = cols_ok && (plan.fm.c_inner ? (half && plan.fm.ld == C)
                                                    : (plan.fm.ld % 8 == 0 && aligned(w.ptr, 16)));
  const bool c_inner = in_place ? plan.fm.c_inner : half;
  const long long ldw = in_place ? plan.fm.ld : (c_inner ? C : J);
  const size_t cols_bytes = (size_t)(nb * per_image);
  const size_t cols_padded = (cols_bytes + 255) & ~(size_t)255;
  const size_t filt_bytes = in_place ? 0 : (size_t)(J * C) * elem_size(w.dtype);
  char *ws = nullptr;
  hipError_t e = hipMallocAsync((void **)&ws, cols_padded + filt_bytes, stream);
  if (e != hipSuccess) return hip_status("tracea_conv_transpose2d: workspace allocation", (int)e);
  float *cols = (float *)ws;
  const void *filt = w.ptr;
  TraceaStatus st = TRACEA_SUCCESS;
  if (!in_place) {
    FilterRepackArgs f{};
    f.w = w.ptr; f.out = ws + cols_padded; f.elem_bytes = elem_size(w.dtype);
    f.c_inner = c_inner ? 1 : 0;
    f.C = (int)C; f.K = (int)K; f.R = (int)R; f.S = (int)S;
    f.sk = w.stride[0]; f.sr = w.stride[1]; f.ss = w.stride[2]; f.sc = w.stride[3];
    st = hip_status("conv_transpose2d filter repack launch", launch_filter_repack(f, stream));
    filt = f.out;
  }
  for (long long b0 = 0; b0 < N && st == TRACEA_SUCCESS; b0 += nb) {
    const long long cnt = N - b0 < nb ? N - b0 : nb;
    View a = x, b = w, c{};
    a.rank = b.rank = c.rank = 2;
    a.ptr = (char *)x.ptr + b0 * x.stride[0] * elem_size(x.dtype);
    a.shape[0] = cnt * H * W; a.shape[1] = C;
    a.stride[0] = plan.ldx; a.stride[1] = 1;
    b.ptr = (void *)filt;
    b.shape[0] = C; b.shape[1] = J;
    if (c_inner) { b.stride[0] = 1; b.stride[1] = ldw; }
    else { b.stride[0] = ldw; b.stride[1] = 1; }
    c.ptr = cols; c.dtype = TRACEA_DTYPE_FLOAT32; c.device = out.device;
    c.shape[0] = a.shape[0]; c.shape[1] = J;
    c.stride[0] = J; c.stride[1] = 1;
    EpilogueChain none{};
    st = run_gemm(a, b, c, none, stream);
    if (st != TRACEA_SUCCESS) break;
    Col2imArgs g{};
    g.cols = cols; g.out = out.ptr; g.out_dtype = out.dtype;
    g.ld_cols = J; g.ldc = plan.ldc;
    g.st_k = 1; g.st_s = K; g.st_r = S * K;
    g.b0 = (int)b0; g.nb = (int)cnt;
    g.h_in = (int)H; g.w_in = (int)W; g.h_out = (int)Ho; g.w_out = (int)Wo; g.k_out = (int)K;
    g.r_sz = (int)R; g.s_sz = (int)S;
    g.stride_h = plan.stride_h; g.stride_w = plan.stride_w; g.pad_h = plan.pad_h; g.pad_w = plan.pad_w;
    g.epi = chain;
    st = hip_status("conv_transpose2d gather launch", launch_col2im_epilogue(g, stream));
  }
  e = hipFreeAsync(ws, stream);
  if (st == TRACEA_SUCCESS && e != hipSuccess) st = hip_status("tracea_conv_transpose2d: workspace release", (int)e);
  return st;
}

}  // namespace

TraceaStatus dispatch_conv_transpose2d_kind(const TraceaTensorView &tx, const TraceaTensorView &tw,
                                            const TraceaTensorView *bias, const TraceaTensorView *residual,
                                            TraceaTensorView *tout, const TraceaConvTranspose2dParams &params) {
  ConvTransposePlan plan;
  TraceaStatus st = conv_transpose_common(tx, tw, tout, params, &plan);
  if (st != TRACEA_SUCCESS) return st;
  TraceaEpilogueOp ops[TRACEA_MAX_EPILOGUE_OPS];
  const int n = kind_to_ops((int)params.epilogue, bias, residual, ops);
  if (n < 0)
    return fail(TRACEA_INVALID_PARAMS, "tracea_conv_transpose2d: unknown epilogue kind %d", (int)params.epilogue);
  st = check_bias_residual("tracea_conv_transpose2d", bias, residual, plan.out.shape[3], plan.out, plan.out.device,
                           ops, n);
  if (st != TRACEA_SUCCESS) return st;
  EpilogueChain chain{};
  st = lower_chain("tracea_conv_transpose2d", ops, (uint32_t)n, plan.out.shape[3], plan.out.shape[3], &chain);
  if (st != TRACEA_SUCCESS) return st;
  return run_conv_transpose(plan, chain, (hipStream_t)params.stream);
}

TraceaStatus dispatch_conv_transpose2d_ops(const TraceaTensorView &tx, const TraceaTensorView &tw,
                                           TraceaTensorView *tout, const TraceaConvTranspose2dParams &params,
                                           const TraceaEpilogueOp *ops, uint32_t n_ops) {
  ConvTransposePlan plan;
  TraceaStatus st = conv_transpose_common(tx, tw, tout, params, &plan);
  if (st != TRACEA_SUCCESS) return st;
  EpilogueChain chain{};
  st = lower_chain("tracea_conv_transpose2d_ex", ops, n_ops, plan.out.shape[3], plan.out.shape[3], &chain);
  if (st != TRACEA_SUCCESS) return st;
  return run_conv_transpose(plan, chain, (hipStream_t)params.stream);
}

// ---- attention ---------------------------------------------------------------------
TraceaStatus dispatch_attention(const TraceaTensorView &tq, const TraceaTensorView &tk,
                                const TraceaTensorView &tv, TraceaTensorView *to,
                                const TraceaAttentionParams &params) {
  if (!runtime_ready()) return fail(TRACEA_UNKNOWN_ERROR, "tracea_attention: tracea_init has not been called");
  if (to == nullptr) return fail(TRACEA_INVALID_PARAMS, "tracea_attention: output view is NULL");
  View q, k, v, o;
  TraceaStatus st;
  if ((st = read_view("tracea_attention: q", tq, 4, &q)) != TRACEA_SUCCESS) return st;
  if ((st = read_view("tracea_attention: k", tk, 4, &k)) != TRACEA_SUCCESS) return st;
  if ((st = read_view("tracea_attention: v", tv, 4, &v)) != TRACEA_SUCCESS) return st;
  if ((st = read_view("tracea_attention: o", *to, 4, &o)) != TRACEA_SUCCESS) return st;
  if (!is_half(q.dtype) || k.dtype != q.dtype || v.dtype != q.dtype || o.dtype != q.dtype)
    return fail(TRACEA_UNSUPPORTED_CONFIG,
                "tracea_attention: q/k/v/o must all be f16 or all bf16 (got %s,%s,%s,%s)",
                dtype_name(q.dtype), dtype_name(k.dtype), dtype_name(v.dtype), dtype_name(o.dtype));
  for (int i = 0; i < 4; ++i)
    if (k.shape[i] != q.shape[i] || v.shape[i] != q.shape[i] || o.shape[i] != q.shape[i])
      return fail(TRACEA_INVALID_PARAMS, "tracea_attention: q, k, v and o must share one [B,H,S,D] shape");
  if ((st = check_device("tracea_attention", o.device)) != TRACEA_SUCCESS) return st;
  if (q.device != o.device || k.device != o.device || v.device != o.device)
    return fail(TRACEA_INVALID_PARAMS, "tracea_attention: operands live on different devices");
  const long long B = q.shape[0], H = q.shape[1], S = q.shape[2], D = q.shape[3];
  if (B == 0 || H == 0 || S == 0) return TRACEA_SUCCESS;
  if (D < 1 || D > 128)
    return fail(TRACEA_UNSUPPORTED_CONFIG, "tracea_attention: head dim %lld (1 to 128 supported)", D);
  if (S >= (1ll << 31) || B * H * ((S + 127) / 128) >= (1ll << 31))
    return fail(TRACEA_UNSUPPORTED_CONFIG, "tracea_attention: problem too large");
  float scale = params.scale;
  if (scale == 0.0f) scale = 1.0f / sqrtf((float)D);
  if (!(scale == scale) || std::isinf(scale))
    return fail(TRACEA_INVALID_PARAMS, "tracea_attention: scale is not finite");
  const View *views[4] = {&q, &k, &v, &o};
  bool in_place = D == 64 || D == 128;
  for (const View *t : views)
    if (t->stride[3] != 1 || t->stride[2] % 8 != 0 || t->stride[1] % 8 != 0 || t->stride[0] % 8 != 0 || !aligned(t->ptr, 16))
      in_place = false;
  if (!in_place) {
    // Head dimensions other than 64 and 128 (the kernels' two), and tensors the kernels cannot read in place
    // (head dimension strided, other strides off a multiple of 8 elements, bases off 16 bytes): Q, K and V are
    // copied into dense [B,H,S,Dp] tensors, Dp = 64 or 128, zeros behind the data -- they add nothing to a score
    // and give zero output columns -- the kernels run on those with the caller's scale, and the first D columns
    // of the result are copied out.  In the per-(device, stream) buffer of the padded GEMM operands; where it
    // cannot be had the call is refused.  (The reference compiles its kernel for the head dimension at hand:
    // src/kernels/attention/cuda_emitter.rs:39-58.)
    static thread_local bool in_padded = false;
    const long long Dp = D <= 64 ? 64 : 128;
    const size_t one = (size_t)(B * H * S) * (size_t)Dp * 2;
    DeviceScope pad_scope(o.device);
    if (pad_scope.err != hipSuccess) return hip_status("hipSetDevice", (int)pad_scope.err);
    unsigned char *buf = in_padded ? nullptr : (unsigned char *)pad_scratch(o.device, (hipStream_t)params.stream, 4 * one);
    if (buf == nullptr)
      return fail(TRACEA_UNSUPPORTED_CONFIG,
                  "tracea_attention: head dim %lld / these strides need padded copies, and no buffer for them can be had "
                  "(stream under capture, or above 1 GiB); in place: head dim 64 or 128, contiguous, other strides "
                  "multiples of 8 elements, bases 16-byte aligned", D);
    hipStream_t stream = (hipStream_t)params.stream;
    const View *src[3] = {&q, &k, &v};
    for (int i = 0; i < 3; ++i) {
      const int e = launch_pad_copy(src[i]->ptr, buf + i * one, 2, B * H * S, D, src[i]->stride[0], src[i]->stride[3], B * H * S, Dp,
                                    stream, H, src[i]->stride[1], S, src[i]->stride[2]);
      if (e != 0) return hip_status("operand copy launch", e);
    }
    const uint64_t shape[4] = {(uint64_t)B, (uint64_t)H, (uint64_t)S, (uint64_t)Dp};
    TraceaTensorView pq = tq, pk = tk, pv = tv, po = *to;
    pq.ptr = buf; pk.ptr = buf + one; pv.ptr = buf + 2 * one; po.ptr = buf + 3 * one;
    pq.shape = pk.shape = pv.shape = po.shape = shape;
    pq.stride = pk.stride = pv.stride = po.stride = nullptr;
    TraceaAttentionParams pp = params;
    pp.scale = scale;
    in_padded = true;
    st = dispatch_attention(pq, pk, pv, &po, pp);
    in_padded = false;
    if (st != TRACEA_SUCCESS) return st;
    return hip_status("result copy launch", launch_unpad_copy(buf + 3 * one, o.ptr, 2, B * H * S, D, o.stride[0], o.stride[3], Dp, stream,
                                                              H, o.stride[1], S, o.stride[2]));
  }

  AttentionArgs a{};
  a.Q = q.ptr; a.K = k.ptr; a.V = v.ptr; a.O = o.ptr;
  a.B = (int)B; a.H = (int)H; a.S = (int)S; a.D = (int)D;
  a.q_sb = q.stride[0]; a.q_sh = q.stride[1]; a.q_ss = q.stride[2];
  a.k_sb = k.stride[0]; a.k_sh = k.stride[1]; a.k_ss = k.stride[2];
  a.v_sb = v.stride[0]; a.v_sh = v.stride[1]; a.v_ss = v.stride[2];
  a.o_sb = o.stride[0]; a.o_sh = o.stride[1]; a.o_ss = o.stride[2];
  a.scale_log2 = scale * 1.4426950408889634f;
  a.causal = params.causal ? 1 : 0;

  // Choice of the family member: a forced one, else the tuner's record of this problem, else by rule.
  int vi = forced_variant("attention");
  if (vi >= 0 && !attention_variant(vi).feasible(a)) vi = -1;
  if (vi < 0) vi = tuning_cache_lookup_attention(a);
  auto member = [&](int block_q, int waves, int items) {
    for (int i = 0; i < attention_variant_count(); ++i) {
      const AttentionVariant &v = attention_variant(i);
      if (v.block_q == block_q && v.waves == waves && v.stages == 2 && v.mfma == 32 && v.items == items && v.offset_groups == 0 && v.feasible(a)) return i;
    }
    return -1;
  };
  const long long cus = device_limits().cus, bh = (long long)(B * H);
  // Two query blocks per workgroup where the pairs alone fill the device: the second block starts on tiles and
  // queries already requested, and under a causal mask a heavy block is paired with a light one.  Sweep over
  // B*H in {8, 32, 128, 512} and S in {512 ... 8192}, replayed graphs: with at least one pair per CU the paired
  // member wins or ties (causal B4 H32 S4096 D128 585 -> 553 us, B1 H32 S2048 63.8 -> 52.2; dense B4 H32 S4096
  // 1002 -> 980 on eight waves), with fewer it loses (causal B1 H32 S1024 26.2 -> 30.1).
  // (Dense attention no longer takes the pairs by rule: with the softmax shift folded into the score product,
  // which the paired members at head dimension 128 have no registers for, the one-block eight-wave member below
  // is ahead -- B4 H32 S4096 D128 904 us against 964, B8 H32 S2048 D64 294 against 302, same box.)
  if (vi < 0 && a.causal && bh * (((S + 127) / 128) / 2) >= cus) vi = member(128, 4, 2);
  // Dense attention over a long sequence with enough workgroups to go round: 256 queries on eight waves share
  // every K/V tile (B4 H32 S4096 D128: 997-999 us against 1013 for 128 queries on four).  Under a causal mask
  // the smaller block wins (584 against 624 us: less masked work on the diagonal, finer load balance).
  if (vi < 0 && !a.causal && S >= 2048 && bh * ((S + 255) / 256) >= 2 * cus) vi = member(256, 8, 1);
  if (vi < 0) {
    for (int i = 0; i < attention_variant_count(); ++i)
      if (attention_variant(i).feasible(a)) {
        vi = i;
        break;
      }
  }
  if (vi < 0) return fail(TRACEA_UNSUPPORTED_CONFIG, "tracea_attention: no kernel variant fits");
  DeviceScope scope(o.device);
  if (scope.err != hipSuccess) return hip_status("hipSetDevice", (int)scope.err);
  t_last_attention = vi;
  return hip_status("attention launch",
                    attention_variant(vi).launch(a, q.dtype, (hipStream_t)params.stream));
}

TraceaStatus dispatch_clock_probe(void *out, int32_t samples, int32_t gap, void *stream) {
  if (!runtime_ready()) return fail(TRACEA_UNKNOWN_ERROR, "tracea_init has not been called");
  if (out == nullptr || samples <= 0 || samples > (1 << 20) || gap < 0 || gap > 4096)
    return fail(TRACEA_INVALID_PARAMS, "tracea_clock_probe: out must be a device buffer of 2*samples 64-bit words, "
                                       "samples in 1..2^20, gap in 0..4096");
  return hip_status("clock probe launch", launch_clock_probe((unsigned long long *)out, samples, gap, (hipStream_t)stream));
}

}  // namespace tracea_amd
