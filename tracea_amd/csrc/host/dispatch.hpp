// Host side of the library above the kernels: argument checking, operator
// chains, kernel-variant selection, tuning.  C++ counterpart of the reference's
// Rust host layer for this path (src/interface/c_bindings.rs,
// src/core/tuning.rs, src/optimizer/mod.rs).
#pragma once
#include <string>

#include "../common.hpp"

namespace tracea_amd {

// error slot / lifecycle (defined in abi.cpp)
TraceaStatus fail(TraceaStatus st, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
bool runtime_ready();
int runtime_device_count();

// Device figures the variant selector and the convolution plans work with (see device_limits()).
struct DeviceLimits {
  long long cus = 256;              // compute units
  long long lds_bytes = 160 * 1024; // LDS a workgroup may use
  double clock_ghz = 2.4;           // shader clock the device reports
  double slot_rate = 1.43e6;        // multiply-accumulates per microsecond of one workgroup slot at efficiency 1
};
const DeviceLimits &device_limits();

// Convolution geometry with the reciprocal ("magic") numbers of every divisor
// the coordinate mapping uses.
struct ConvGeometry {
  TraceaConvParamsBlock block;  // reference-compatible 80-byte block (symmetric form)
  int stride_h, stride_w, pad_h, pad_w, dil_h, dil_w;
  int m_gemm, n_gemm, k_gemm;
};
TraceaStatus make_conv_geometry(int n, int h, int w, int c, int k, int r, int s, int stride_h,
                                int stride_w, int pad_h, int pad_w, int dil_h, int dil_w,
                                ConvGeometry *out);

// magic = ceil(2^(32+shift)/d) (0 for powers of two, shift = log2 d), chosen so
// that fast_divmod is exact for every 0 <= n <= n_max.
void magic_for_divisor(uint32_t d, uint64_t n_max, uint32_t *magic, uint32_t *shift);

void set_forced_variant(const char *op, int index);
int forced_variant(const char *op);
// Variant index the calling thread's latest launch of `op` used, -1 if none.
int last_variant(const char *op);
// Split-K of launches with few output tiles and a long K (on by default), and the number of
// K ranges the calling thread's latest gemm / conv2d launch was split into (1: not split).
void set_split_k_enabled(bool on);
void set_split_k_one_launch(bool on);  // default on: the tile's last workgroup reduces, no second kernel
int last_split_k_launches();            // 1 or 2: kernels the calling thread's latest gemm / conv2d launch took
// Transposed convolutions as one stride-1 convolution per output phase where that applies (on by
// default); off: always the GEMM to partial products followed by the gather.
void set_conv_transpose_by_phase(bool on);
void set_conv_transpose_filter_cache(bool on);
void conv_transpose_filter_cache_clear();
int last_split_k();

TraceaStatus dispatch_gemm_kind(const TraceaTensorView &a, const TraceaTensorView &b,
                                const TraceaTensorView *bias, const TraceaTensorView *residual,
                                TraceaTensorView *c, const TraceaGemmParams &params, bool static_only = false);
TraceaStatus dispatch_gemm_ops(const TraceaTensorView &a, const TraceaTensorView &b,
                               TraceaTensorView *c, const TraceaGemmParams &params,
                               const TraceaEpilogueOp *ops, uint32_t n_ops);
// A caller's operator list, checked and in device form, for an output of rows of `channels` elements
// (a residual without a row stride of its own has that one).
TraceaStatus dispatch_lower_chain(const char *what, const TraceaEpilogueOp *ops, uint32_t n_ops, long long channels,
                                  EpilogueChain *chain);
// GEMM over a tile list.  `tables` are the device copies of a TileLayout's tables on the
// device of c: level-1 map in launch order, records, and (slices > 1 only) the workspace
// row block of every workgroup.  Exactly one of (ops, n_ops) and the kind in params is used:
// ops == nullptr selects the kind.
struct TileLayout;
struct DeviceTileTables {
  const unsigned *l1 = nullptr;
  const unsigned *l2 = nullptr;
  const unsigned *slice = nullptr;
  const unsigned *counts = nullptr;  // records per tile of the grid, when tiles differ in that (else nullptr)
  uint32_t count = 0;   // workgroups
  uint32_t slices = 1;  // most records any tile has
  uint32_t k_gcd = 0;      // gcd of the k range lengths (k_end clipped to K) of all listed records
  uint32_t start_gcd = 0;  // gcd of their k_start (0: all start at 0)
};
TraceaStatus dispatch_gemm_tiles(const TraceaTensorView &a, const TraceaTensorView &b,
                                 const TraceaTensorView *bias, const TraceaTensorView *residual,
                                 TraceaTensorView *c, const TraceaGemmParams &params,
                                 const TraceaEpilogueOp *ops, uint32_t n_ops, const TileLayout &layout,
                                 const DeviceTileTables &tables);
TraceaStatus dispatch_apply_epilogue(const TraceaTensorView &x, TraceaTensorView *out, const TraceaEpilogueOp *ops,
                                     uint32_t n_ops, void *stream);
TraceaStatus dispatch_softmax(const TraceaTensorView &x, TraceaTensorView *out, void *stream);
TraceaStatus dispatch_global_avg_pool(const TraceaTensorView &x, TraceaTensorView *out, void *stream);
TraceaStatus dispatch_linear(const TraceaTensorView &a, const TraceaTensorView &w, const TraceaTensorView *bias,
                             TraceaTensorView *c, const TraceaGemmParams &params);
TraceaStatus dispatch_low_rank_mlp(const TraceaTensorView &x, const TraceaTensorView &a,
                                   const TraceaTensorView &b, const TraceaTensorView *bias,
                                   const TraceaTensorView *residual, TraceaTensorView *c,
                                   const TraceaGemmParams &params);
TraceaStatus dispatch_conv2d_kind(const TraceaTensorView &x, const TraceaTensorView &w,
                                  const TraceaTensorView *bias, const TraceaTensorView *residual,
                                  TraceaTensorView *out, const TraceaConv2dParams &params);
TraceaStatus dispatch_conv2d_ops(const TraceaTensorView &x, const TraceaTensorView &w,
                                 TraceaTensorView *out, const TraceaConv2dParams &params,
                                 const TraceaEpilogueOp *ops, uint32_t n_ops);
TraceaStatus dispatch_conv_transpose2d_kind(const TraceaTensorView &x, const TraceaTensorView &w,
                                            const TraceaTensorView *bias, const TraceaTensorView *residual,
                                            TraceaTensorView *out, const TraceaConvTranspose2dParams &params);
TraceaStatus dispatch_conv_transpose2d_ops(const TraceaTensorView &x, const TraceaTensorView &w,
                                           TraceaTensorView *out, const TraceaConvTranspose2dParams &params,
                                           const TraceaEpilogueOp *ops, uint32_t n_ops);
TraceaStatus dispatch_attention(const TraceaTensorView &q, const TraceaTensorView &k,
                                const TraceaTensorView &v, TraceaTensorView *o,
                                const TraceaAttentionParams &params);

// Shader-clock probe (tracea_clock_probe): argument checks, then the one-wave sampling kernel on `stream`.
TraceaStatus dispatch_clock_probe(void *out, int32_t samples, int32_t gap, void *stream);

// Heuristic choice among the feasible contraction variants (used when neither a
// forced variant nor a tuning-cache entry decides).  Returns -1 if none fits.
int select_contraction_variant(int m, int n, int k, bool conv, bool b_ncontig = false);

// TraceaResult builders: strings are malloc'ed, released by tracea_free_string.
struct PipelineConfig;
char *dup_cstr(const std::string &s);
TraceaResult failure(const std::string &msg);
TraceaResult success(const PipelineConfig &cfg, float tflops);

TraceaResult tune_gemm(size_t m, size_t n, size_t k);
TraceaResult autotune_gemm(size_t m, size_t n, size_t k, uint32_t iterations);
TraceaResult autotune_conv2d(size_t n, size_t c, size_t h, size_t w, size_t k, size_t r, size_t s,
                             size_t stride, size_t pad, size_t dilation, uint32_t iterations);
TraceaResult tune_fa2(size_t b, size_t h, size_t s, size_t d, bool causal);
TraceaResult tune_conv2d(size_t n, size_t c, size_t h, size_t w, size_t k, size_t r, size_t s,
                         size_t stride, size_t pad, size_t dilation);

}  // namespace tracea_amd
