// extern "C" entry points of the MI355X Tracea library: argument validation,
// thread-local error reporting and dispatch to the precompiled HIP kernels.
// Declarations and the reference interfaces they replace: include/tracea.h.
#include <atomic>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "common.hpp"
#include "host/dispatch.hpp"

using namespace tracea_amd;

// ---------------------------------------------------------------------------
// last-error slot (reference: tracea-ffi/src/lib.rs:13-15, 77-109)
// ---------------------------------------------------------------------------
namespace {
thread_local std::string g_last_error;
std::atomic<bool> g_initialised{false};
std::atomic<int> g_device_count{0};
}  // namespace

namespace tracea_amd {
TraceaStatus fail(TraceaStatus st, const char *fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return st;
}
bool runtime_ready() { return g_initialised.load(); }
int runtime_device_count() { return g_device_count.load(); }
}  // namespace tracea_amd

#pragma GCC visibility push(default)
extern "C" {

int32_t tracea_get_last_error(uint8_t *buf, size_t len) {
  if (buf == nullptr || len == 0) return -1;
  const size_t n = g_last_error.size() < len - 1 ? g_last_error.size() : len - 1;
  memcpy(buf, g_last_error.data(), n);
  buf[n] = 0;
  return (int32_t)n;
}

void tracea_clear_error(void) { g_last_error.clear(); }

uint32_t tracea_version_major(void) { return 0; }
uint32_t tracea_version_minor(void) { return 1; }
uint32_t tracea_version_patch(void) { return 0; }

int tracea_init(void) {
  if (g_initialised.load()) return 0;
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess || n <= 0) {
    (void)hipGetLastError();
    fail(TRACEA_CUDA_ERROR, "tracea_init: no HIP device available (%s)",
         e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
    return 1;
  }
  g_device_count.store(n);
  g_initialised.store(true);
  return 0;
}

void tracea_shutdown(void) { g_initialised.store(false); }

void tracea_free_string(char *s) { free(s); }

// ---------------------------------------------------------------------------
// compute entry points: catch everything, report through the status code
// ---------------------------------------------------------------------------
#define TRACEA_GUARDED(expr)                                                    \
  try {                                                                         \
    return (expr);                                                              \
  } catch (const std::exception &ex) {                                          \
    return fail(TRACEA_UNKNOWN_ERROR, "internal error: %s", ex.what());         \
  } catch (...) {                                                               \
    return fail(TRACEA_UNKNOWN_ERROR, "internal error: unknown exception");     \
  }

TraceaStatus tracea_gemm(TraceaTensorView a, TraceaTensorView b, const TraceaTensorView *bias,
                         const TraceaTensorView *residual, TraceaTensorView *c,
                         TraceaGemmParams params) {
  TRACEA_GUARDED(dispatch_gemm_kind(a, b, bias, residual, c, params))
}

TraceaStatus tracea_gemm_noalloc(TraceaTensorView a, TraceaTensorView b, const TraceaTensorView *bias,
                                 const TraceaTensorView *residual, TraceaTensorView *c,
                                 TraceaGemmParams params) {
  TRACEA_GUARDED(dispatch_gemm_kind(a, b, bias, residual, c, params, true))
}

TraceaStatus tracea_gemm_ex(TraceaTensorView a, TraceaTensorView b, TraceaTensorView *c,
                            TraceaGemmParams params, const TraceaEpilogueOp *ops, uint32_t n_ops) {
  TRACEA_GUARDED(dispatch_gemm_ops(a, b, c, params, ops, n_ops))
}

TraceaStatus tracea_apply_epilogue(TraceaTensorView x, TraceaTensorView *out, const TraceaEpilogueOp *ops,
                                   uint32_t n_ops, void *stream) {
  TRACEA_GUARDED(dispatch_apply_epilogue(x, out, ops, n_ops, stream))
}

TraceaStatus tracea_softmax(TraceaTensorView x, TraceaTensorView *out, void *stream) {
  TRACEA_GUARDED(dispatch_softmax(x, out, stream))
}

TraceaStatus tracea_global_avg_pool(TraceaTensorView x, TraceaTensorView *out, void *stream) {
  TRACEA_GUARDED(dispatch_global_avg_pool(x, out, stream))
}

TraceaStatus tracea_linear(TraceaTensorView a, TraceaTensorView w, const TraceaTensorView *bias, TraceaTensorView *c,
                           TraceaGemmParams params) {
  TRACEA_GUARDED(dispatch_linear(a, w, bias, c, params))
}

TraceaStatus tracea_low_rank_mlp(TraceaTensorView x, TraceaTensorView a, TraceaTensorView b,
                                 const TraceaTensorView *bias, const TraceaTensorView *residual,
                                 TraceaTensorView *c, TraceaGemmParams params) {
  TRACEA_GUARDED(dispatch_low_rank_mlp(x, a, b, bias, residual, c, params))
}

TraceaStatus tracea_conv2d(TraceaTensorView x, TraceaTensorView w, const TraceaTensorView *b,
                           const TraceaTensorView *residual, TraceaTensorView *out,
                           TraceaConv2dParams params) {
  TRACEA_GUARDED(dispatch_conv2d_kind(x, w, b, residual, out, params))
}

TraceaStatus tracea_conv2d_ex(TraceaTensorView x, TraceaTensorView w, TraceaTensorView *out,
                              TraceaConv2dParams params, const TraceaEpilogueOp *ops,
                              uint32_t n_ops) {
  TRACEA_GUARDED(dispatch_conv2d_ops(x, w, out, params, ops, n_ops))
}

TraceaStatus tracea_conv_transpose2d(TraceaTensorView x, TraceaTensorView w, const TraceaTensorView *b,
                                     const TraceaTensorView *residual, TraceaTensorView *out,
                                     TraceaConvTranspose2dParams params) {
  TRACEA_GUARDED(dispatch_conv_transpose2d_kind(x, w, b, residual, out, params))
}

TraceaStatus tracea_conv_transpose2d_ex(TraceaTensorView x, TraceaTensorView w, TraceaTensorView *out,
                                        TraceaConvTranspose2dParams params, const TraceaEpilogueOp *ops,
                                        uint32_t n_ops) {
  TRACEA_GUARDED(dispatch_conv_transpose2d_ops(x, w, out, params, ops, n_ops))
}

TraceaStatus tracea_attention(TraceaTensorView q, TraceaTensorView k, TraceaTensorView v,
                              TraceaTensorView *o, TraceaAttentionParams params) {
  TRACEA_GUARDED(dispatch_attention(q, k, v, o, params))
}

void tracea_set_split_k(int32_t enabled) { set_split_k_enabled(enabled != 0); }
void tracea_set_split_k_one_launch(int32_t enabled) { set_split_k_one_launch(enabled != 0); }
int32_t tracea_last_split_k_launches(void) { return last_split_k_launches(); }
void tracea_set_conv_transpose_by_phase(int32_t enabled) { set_conv_transpose_by_phase(enabled != 0); }
void tracea_set_conv_transpose_filter_cache(int32_t enabled) { set_conv_transpose_filter_cache(enabled != 0); }
void tracea_conv_transpose_filter_cache_clear(void) { conv_transpose_filter_cache_clear(); }
int32_t tracea_last_split_k(void) { return last_split_k(); }

TraceaStatus tracea_clock_probe(void *out, int32_t samples, int32_t gap, void *stream) {
  TRACEA_GUARDED(dispatch_clock_probe(out, samples, gap, stream))
}

int32_t tracea_variant_count(const char *op) {
  if (op == nullptr) return -1;
  if (!strcmp(op, "gemm") || !strcmp(op, "conv2d")) return contraction_variant_count();
  if (!strcmp(op, "attention")) return attention_variant_count();
  return -1;
}

const char *tracea_variant_name(const char *op, int32_t index) {
  const int n = tracea_variant_count(op);
  if (n < 0 || index < 0 || index >= n) return nullptr;
  if (!strcmp(op, "attention")) return attention_variant(index).name;
  return contraction_variant(index).name;
}

int32_t tracea_force_variant(const char *op, int32_t index) {
  const int n = tracea_variant_count(op);
  if (n < 0 || index < -1 || index >= n) return -1;
  set_forced_variant(op, index);
  return 0;
}

int32_t tracea_last_variant(const char *op) { return op == nullptr ? -1 : last_variant(op); }

int32_t tracea_select_variant(const char *op, int64_t m, int64_t n, int64_t k) {
  if (op == nullptr || m <= 0 || n <= 0 || k <= 0 || m >= (1ll << 31) || n >= (1ll << 31) || k >= (1ll << 31))
    return -1;
  const bool conv = !strcmp(op, "conv2d");
  if (!conv && strcmp(op, "gemm") != 0) return -1;
  return select_contraction_variant((int)m, (int)n, (int)k, conv);
}

TraceaStatus tracea_conv_params_pack(int32_t n, int32_t h, int32_t w, int32_t c, int32_t k,
                                     int32_t r, int32_t s, int32_t stride, int32_t pad,
                                     int32_t dilation, TraceaConvParamsBlock *out) {
  if (out == nullptr) return fail(TRACEA_INVALID_PARAMS, "tracea_conv_params_pack: out is NULL");
  ConvGeometry g;
  TraceaStatus st = make_conv_geometry(n, h, w, c, k, r, s, stride, stride, pad, pad, dilation,
                                       dilation, &g);
  if (st != TRACEA_SUCCESS) return st;
  *out = g.block;
  return TRACEA_SUCCESS;
}

TraceaStatus tracea_conv_coords_device(const TraceaConvParamsBlock *p, int32_t *rows,
                                       int64_t *base_off, int32_t *cols, void *stream) {
  if (!runtime_ready()) return fail(TRACEA_UNKNOWN_ERROR, "tracea_init has not been called");
  if (p == nullptr || rows == nullptr || base_off == nullptr || cols == nullptr)
    return fail(TRACEA_INVALID_PARAMS, "tracea_conv_coords_device: NULL argument");
  const int e = launch_conv_coords(*p, rows, base_off, cols, (hipStream_t)stream);
  if (e != 0) return fail(TRACEA_CUDA_ERROR, "conv_coords launch: %s", hipGetErrorString((hipError_t)e));
  return TRACEA_SUCCESS;
}

TraceaResult tracea_tune_gemm(size_t m, size_t n, size_t k) { return tune_gemm(m, n, k); }
TraceaResult tracea_tune_fa2(size_t b, size_t h, size_t s, size_t d, bool causal) {
  return tune_fa2(b, h, s, d, causal);
}
TraceaResult tracea_tune_conv2d(size_t n, size_t c, size_t h, size_t w, size_t k, size_t r,
                                size_t s_kernel, size_t stride, size_t pad, size_t dilation) {
  return tune_conv2d(n, c, h, w, k, r, s_kernel, stride, pad, dilation);
}

}  // extern "C"
#pragma GCC visibility pop
