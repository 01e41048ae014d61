/*
 * Tracea C ABI, MI355X (gfx950) implementation.
 *
 * Every declaration below keeps the name, argument order, field order and
 * enumerator values of the interface it replaces in the reference, so that a
 * program compiled against the reference's headers links against this
 * library unchanged.  The reference file and line of each item is cited.
 * Entry points that have no counterpart in the reference are grouped at the
 * end and say so.
 *
 * Conventions shared by all calls
 *   - pointers, shape arrays and stride arrays are borrowed for the duration
 *     of the call and never freed by the library;
 *   - strides are in ELEMENTS; a NULL stride array means contiguous row-major;
 *   - device_id >= 0 names the HIP device that owns `ptr`; device_id == -1
 *     (host memory) is rejected with TRACEA_CPU_ERROR: there is no CPU arm;
 *   - `stream` is a hipStream_t passed through as void* (NULL = the default
 *     stream); calls enqueue work and return without synchronising;
 *   - a failing call returns a status other than TRACEA_SUCCESS and leaves a
 *     human-readable message in a thread-local slot read with
 *     tracea_get_last_error(); no C++ exception crosses the boundary.
 */
#ifndef TRACEA_H
#define TRACEA_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* reference: include/tracea.hpp:16-23.  TRACEA_CUDA_ERROR keeps its name for
 * source compatibility; here it reports any HIP runtime / device failure. */
typedef enum {
  TRACEA_SUCCESS = 0,
  TRACEA_INVALID_PARAMS = 1,
  TRACEA_UNSUPPORTED_CONFIG = 2,
  TRACEA_CUDA_ERROR = 3,
  TRACEA_CPU_ERROR = 4,
  TRACEA_UNKNOWN_ERROR = 99
} TraceaStatus;

/* reference: include/tracea.hpp:29-35 */
typedef enum {
  TRACEA_DTYPE_FLOAT32 = 0,
  TRACEA_DTYPE_FLOAT16 = 1,
  TRACEA_DTYPE_BFLOAT16 = 2,
  TRACEA_DTYPE_INT32 = 3,
  TRACEA_DTYPE_INT8 = 4
} TraceaDType;

/* reference: include/tracea.hpp:37-47; expansion into operator chains:
 * src/interface/c_bindings.rs:144-197 */
typedef enum {
  TRACEA_EPILOGUE_IDENTITY = 0,
  TRACEA_EPILOGUE_BIAS_ADD = 1,
  TRACEA_EPILOGUE_RELU = 2,
  TRACEA_EPILOGUE_GELU = 3,
  TRACEA_EPILOGUE_SILU = 4,
  TRACEA_EPILOGUE_BIAS_RELU = 5,
  TRACEA_EPILOGUE_BIAS_SILU = 6,
  TRACEA_EPILOGUE_RESIDUAL = 7,
  TRACEA_EPILOGUE_RESIDUAL_RELU = 8
} TraceaEpilogueKind;

/* reference: include/tracea.hpp:49-53.  Accepted and ignored: the online
 * softmax here always rescales once per key/value tile. */
typedef enum {
  TRACEA_SOFTMAX_AUTO = 0,
  TRACEA_SOFTMAX_PER_TILE = 1,
  TRACEA_SOFTMAX_PER_TWO_TILES = 2
} TraceaSoftmaxGranularity;

/* reference: include/tracea.hpp:59-66 */
typedef struct {
  void *ptr;
  uint32_t rank;
  const uint64_t *shape;
  const int64_t *stride;
  TraceaDType dtype;
  int32_t device_id;
} TraceaTensorView;

/* reference: include/tracea.hpp:72-82 */
typedef struct {
  uint32_t stride_h;
  uint32_t stride_w;
  uint32_t padding_h;
  uint32_t padding_w;
  uint32_t dilation_h;
  uint32_t dilation_w;
  uint32_t groups;
  TraceaEpilogueKind epilogue;
  void *stream;
} TraceaConv2dParams;

/* reference: include/tracea.hpp:119-131 */
typedef struct {
  uint32_t stride_h;
  uint32_t stride_w;
  uint32_t padding_h;
  uint32_t padding_w;
  uint32_t output_padding_h;
  uint32_t output_padding_w;
  uint32_t dilation_h;
  uint32_t dilation_w;
  uint32_t groups;
  TraceaEpilogueKind epilogue;
  void *stream;
} TraceaConvTranspose2dParams;

/* reference: include/tracea.hpp:84-87 */
typedef struct {
  TraceaEpilogueKind epilogue;
  void *stream;
} TraceaGemmParams;

/* reference: include/tracea.hpp:89-94.  scale == 0 selects 1/sqrt(D). */
typedef struct {
  uint8_t causal;
  TraceaSoftmaxGranularity softmax_mode;
  float scale;
  void *stream;
} TraceaAttentionParams;

/* reference: include/tracea.h:15-20 */
typedef struct {
  bool success;
  char *error_msg;
  float score;      /* TFLOP/s of the winning configuration */
  void *config_ptr; /* char*: PipelineConfig JSON; free with tracea_free_string */
} TraceaResult;

/* ---- lifecycle: reference include/tracea.h:26-31, src/interface/c_bindings.rs:105-125.
 * tracea_init returns 0 on success.  It is idempotent.  Compute entry points
 * called before it return TRACEA_UNKNOWN_ERROR (c_bindings.rs:212). */
int tracea_init(void);
void tracea_shutdown(void);
void tracea_free_string(char *s);

/* ---- implicit-GEMM convolution: reference include/tracea.hpp:107-110,
 * src/interface/c_bindings.rs:206-290.
 *   x   [N,H,W,C]   activations, channels innermost (NHWC)
 *   w   [K,R,S,C]   filters as the reference reads the dims (c_bindings.rs:219-227);
 *                   the physical order is taken from the strides, so both the
 *                   K-major [K,R,S,C] and the [R,S,C,K] storage the reference's
 *                   kernel indexes (src/emitter/cuda/conv.rs:253) are accepted
 *   b   [K]         optional bias (f32, or the activation dtype)
 *   residual        optional, shape of out
 *   out [N,Ho,Wo,K] pre-allocated, Ho = (H + 2p - d(R-1) - 1)/s + 1
 * groups must be 1; stride/padding/dilation may differ between h and w. */
TraceaStatus tracea_conv2d(TraceaTensorView x, TraceaTensorView w, const TraceaTensorView *b,
                           const TraceaTensorView *residual, TraceaTensorView *out,
                           TraceaConv2dParams params);

/* ---- transposed convolution: reference include/tracea.hpp:112-137,
 * src/interface/c_bindings.rs:292-368, kernel src/emitter/conv_transpose.rs:178-266.
 *   x   [N,H,W,C]   activations, channels innermost (NHWC)
 *   w   [K,R,S,C]   filters as the reference reads the dims (c_bindings.rs:303-311:
 *                   K = output channels); the physical order is taken from the
 *                   strides.  The reference kernel indexes the storage as
 *                   [C*R*S, K] rows (conv_transpose.rs:236), i.e. strides
 *                   {1, S*K, K, R*S*K}; that order, torch's [C,K,R,S] and a
 *                   contiguous [K,R,S,C] are accepted (input channels outermost
 *                   or innermost, the other three dims dense)
 *   b   [K]         optional bias; residual optional, shape of out
 *   out [N,Ho,Wo,K] pre-allocated, Ho = (H-1)*stride - 2*pad + R + output_padding
 * x and w are both f32 (the reference's only case), both f16 or both bf16;
 * sums are kept in fp32.  groups and dilation must be 1 (0 = unset), as the
 * reference states (conv_transpose.rs:26-29).  Stride, padding and output
 * padding may differ between h and w (the reference reads the _h fields for both).
 * The call takes a temporary device buffer from the stream-ordered allocator
 * (hipMallocAsync on params.stream) for the per-tap partial products. */
TraceaStatus tracea_conv_transpose2d(TraceaTensorView x, TraceaTensorView w,
                                     const TraceaTensorView *b, const TraceaTensorView *residual,
                                     TraceaTensorView *out, TraceaConvTranspose2dParams params);

/* ---- GEMM C = epilogue(A.B): reference include/tracea.hpp:141-144,
 * src/interface/c_bindings.rs:371-440.  a [M,K], b [K,N], c [M,N]; a
 * column-major B is expressed through b's strides ({1, K}). */
TraceaStatus tracea_gemm(TraceaTensorView a, TraceaTensorView b, const TraceaTensorView *bias,
                         const TraceaTensorView *residual, TraceaTensorView *c,
                         TraceaGemmParams params);

/* ---- Low-rank MLP: the reference's UnifiedOpType::LowRankMlp {m, n, k, r}
 * (src/emitter/traits.rs:95-100; kernel sketch src/emitter/cuda/low_rank.rs:4-150, whose
 * matrix steps are left empty; expected value k*r for all-ones operands in
 * examples/low_rank_mlp_test.rs:96-98).  c[M,N] = epilogue((x[M,K] a[K,R]) b[R,N]);
 * the rank-r product is rounded to the operands' type before the second product,
 * as the reference keeps it in a half-precision tile.  x, a, b share one floating
 * type; strides and epilogue as for tracea_gemm.  The intermediate lives in a
 * stream-ordered allocation: the call must not be captured into a HIP graph. */
TraceaStatus tracea_low_rank_mlp(TraceaTensorView x, TraceaTensorView a, TraceaTensorView b,
                                 const TraceaTensorView *bias, const TraceaTensorView *residual,
                                 TraceaTensorView *c, TraceaGemmParams params);

/* ---- FlashAttention-2 forward: reference include/tracea.hpp:147-149,
 * src/interface/c_bindings.rs:443-495.  q,k,v,o [B,H,S,D], f16 or bf16, D <= 128.
 * The kernels read D = 64 or 128 with a contiguous head dimension, other strides
 * multiples of 8 elements and bases on 16 bytes in place.  Any other D from 1 to
 * 128 (the reference compiles its kernel for the head dimension at hand:
 * src/kernels/attention/cuda_emitter.rs:39-58) and any other strides or bases
 * run from zero-padded copies of q, k and v in the padded road's per-(device,
 * stream) buffer (four tensors of B*H*S rows of 64 or 128 elements, at most
 * 1 GiB, not grown under capture), the result copied out to o; scale 0 stays
 * 1/sqrt(D) of the true D. */
TraceaStatus tracea_attention(TraceaTensorView q, TraceaTensorView k, TraceaTensorView v,
                              TraceaTensorView *o, TraceaAttentionParams params);

/* ---- errors and version: reference include/tracea.hpp:151-164,
 * tracea-ffi/src/lib.rs:77-109, 244-251.  tracea_get_last_error copies at most
 * len-1 bytes plus a NUL and returns the number of bytes copied, or -1 when
 * buf is NULL or len is 0. */
int32_t tracea_get_last_error(uint8_t *buf, size_t len);
void tracea_clear_error(void);
uint32_t tracea_version_major(void);
uint32_t tracea_version_minor(void);
uint32_t tracea_version_patch(void);

/* ---- tuning: reference include/tracea.h:41-71 (the reference's bodies are
 * stubs returning success=false, src/interface/c_bindings.rs:499-513).  Each
 * call times every feasible kernel variant for the problem on synthetic
 * device buffers, records the winner in the tuning cache and returns its
 * PipelineConfig as JSON. */
TraceaResult tracea_tune_gemm(size_t m, size_t n, size_t k);
TraceaResult tracea_tune_fa2(size_t b, size_t h, size_t s, size_t d, bool causal);
TraceaResult tracea_tune_conv2d(size_t n, size_t c, size_t h, size_t w, size_t k, size_t r,
                                size_t s_kernel, size_t stride, size_t pad, size_t dilation);

/* ======================================================================== */
/* Additions.  None of these has a counterpart in the reference's headers.   */
/* ======================================================================== */

/* Operator vocabulary of the reference's EpilogueOp (src/core/op.rs:70-90)
 * exposed one-to-one, plus the folded form of BatchNorm.  Applied to the fp32
 * accumulator in list order before the conversion to the output dtype. */
typedef enum {
  TRACEA_EPI_OP_NONE = 0,
  TRACEA_EPI_OP_BIAS_ADD = 1,      /* p0 = bias[channel] */
  TRACEA_EPI_OP_RELU = 2,
  TRACEA_EPI_OP_GELU = 3,
  TRACEA_EPI_OP_SILU = 4,
  TRACEA_EPI_OP_RESIDUAL_ADD = 5,  /* p0 = residual[row*ld + channel] */
  TRACEA_EPI_OP_BIAS_ADD_SILU = 6, /* p0 = bias */
  TRACEA_EPI_OP_BATCHNORM = 7,     /* p0..p3 = gamma, beta, mean, var (f32); epsilon */
  TRACEA_EPI_OP_SCALE_SHIFT = 8    /* p0 = scale, p1 = shift (f32): folded BatchNorm */
} TraceaEpilogueOpKind;

typedef struct {
  TraceaEpilogueOpKind kind;
  TraceaDType dtype; /* element type of p0 for BIAS_ADD / RESIDUAL_ADD / BIAS_ADD_SILU */
  const void *p0;
  const void *p1;
  const void *p2;
  const void *p3;
  float epsilon;
  int64_t ld; /* RESIDUAL_ADD: row stride in elements; 0 = number of channels */
} TraceaEpilogueOp;

#define TRACEA_MAX_EPILOGUE_OPS 4

/* tracea_conv2d / tracea_gemm / tracea_conv_transpose2d with an explicit operator chain (at most
 * TRACEA_MAX_EPILOGUE_OPS entries) instead of a TraceaEpilogueKind; the
 * `epilogue` field of params is ignored.  This is how BatchNorm, which
 * TraceaEpilogueKind cannot name, reaches the fused epilogue
 * (fusion rules: src/core/optimizer.rs:122-150). */
TraceaStatus tracea_conv2d_ex(TraceaTensorView x, TraceaTensorView w, TraceaTensorView *out,
                              TraceaConv2dParams params, const TraceaEpilogueOp *ops,
                              uint32_t n_ops);
TraceaStatus tracea_gemm_ex(TraceaTensorView a, TraceaTensorView b, TraceaTensorView *c,
                            TraceaGemmParams params, const TraceaEpilogueOp *ops, uint32_t n_ops);
TraceaStatus tracea_conv_transpose2d_ex(TraceaTensorView x, TraceaTensorView w, TraceaTensorView *out,
                                        TraceaConvTranspose2dParams params,
                                        const TraceaEpilogueOp *ops, uint32_t n_ops);

/* ---- Operators that are not contractions: the reference's Softmax, BatchNorm,
 * GlobalAveragePool and Linear kernels (src/emitter/cuda/nn.rs:3-135) and its
 * element-wise ReLU / Add nodes.  Activations are contiguous with the channel
 * axis last (NHWC), the layout of every other entry point here; the reference's
 * BatchNorm and pooling kernels index NCHW, and a tensor strided that way is
 * TRACEA_UNSUPPORTED_CONFIG.  Storage may be f32, f16 or bf16 (in and out
 * independently); arithmetic is fp32.  `stream` is a hipStream_t (NULL: default).
 *
 * tracea_apply_epilogue: out = chain(x) in one pass; x and out of equal shape, rank 1-4.
 *   Standalone BatchNorm is {TRACEA_EPI_OP_BATCHNORM, p0..p3 = gamma, beta, mean, var (f32), epsilon}:
 *   (x - mean) * rsqrt(var + eps) * gamma + beta (nn.rs:56-66); ReLU and a residual Add likewise.
 * tracea_softmax: over the last axis, max-subtracted (nn.rs:14-32).
 * tracea_global_avg_pool: x [N,H,W,C] -> out [N,C], the mean over H*W (nn.rs:84-97).
 * tracea_linear: c[b] = epilogue(a[b] w[b]) with a [B,M,K], c [B,M,N] and w [B,K,N] (nn.rs:113-131)
 *   or a shared w [K,N]; any strides within a batch as for tracea_gemm; epilogue kinds without a
 *   residual. */
TraceaStatus tracea_apply_epilogue(TraceaTensorView x, TraceaTensorView *out, const TraceaEpilogueOp *ops,
                                   uint32_t n_ops, void *stream);
TraceaStatus tracea_softmax(TraceaTensorView x, TraceaTensorView *out, void *stream);
TraceaStatus tracea_global_avg_pool(TraceaTensorView x, TraceaTensorView *out, void *stream);
TraceaStatus tracea_linear(TraceaTensorView a, TraceaTensorView w, const TraceaTensorView *bias, TraceaTensorView *c,
                           TraceaGemmParams params);


/* Split-K.  A gemm / conv2d launch with few output tiles and a long K (tiles * 2 <= 256 CUs,
 * at least 8 K tiles; the 64x64 tile of the fp32 GEMM: one to four ranges of at least 16 K tiles of 16, at
 * most 4.5 workgroups per CU, the count with the least estimated time) is split along K
 * over more workgroups; fp32 partial products go to a
 * scratch buffer the library keeps per (device, stream) (grown on demand up to 64 MiB, never
 * while the stream is being captured, never freed) and a second kernel sums them and applies
 * the operator chain.  On by default; tracea_set_split_k(0) turns it off.
 * tracea_last_split_k: K ranges of the calling thread's latest gemm / conv2d launch (1: not split).
 * Half-precision launches on tiles up to 128x128 and fp32 launches that are split at most four ways need no second kernel: every workgroup leaves its partial
 * product in the scratch buffer and takes a ticket from a per-tile counter (4 bytes per tile, per (device,
 * stream), zero between launches); the workgroup that draws a tile's last ticket sums the partial products in
 * K order, applies the operator chain and writes the tile.  Results equal those of the two-kernel form bit for
 * bit (same order of summation).  tracea_set_split_k_one_launch(0) goes back to two kernels everywhere (the
 * larger half-precision tiles, finer splits and tracea_gemm_noalloc always use two: with many K ranges the
 * reduction kernel, which spreads the sum over the device, is faster than one workgroup per tile);
 * tracea_last_split_k_launches says which
 * form the calling thread's latest gemm / conv2d launch took (1 or 2).  (The reference has no split along K:
 * its GEMM grid is one block per output tile, src/emitter/cuda/gemm.rs:92-207.) */
/* Operands of tracea_gemm / tracea_gemm_ex that the tile kernels cannot read in place -- a K, or the N of a
 * row-major B, that is not a whole number of 16-byte pieces; rows that do not start on 16 bytes; an A strided
 * along K -- are copied into padded, zero-filled rows of a second per-(device, stream) buffer (at most 1 GiB,
 * same rules as the one above) and multiplied from there.  Where that buffer cannot be had
 * (tracea_gemm_noalloc, a stream under capture that made no such call before, A and B of different types) a
 * kernel on the vector ALU that reads any layout runs instead: same results, far slower.  (The reference's
 * kernels take M, N, K as they come: src/emitter/cuda/gemm.rs:92-207 guards every element.) */
void tracea_set_split_k(int32_t enabled);
void tracea_set_split_k_one_launch(int32_t enabled);
int32_t tracea_last_split_k_launches(void);
/* tracea_conv_transpose2d runs as one stride-1 convolution per output phase (stride_h * stride_w
 * launches on a regrouped copy of the filter bank, the outputs written in place) when every phase
 * has taps and no negative padding and the input is dense half-precision NHWC with a multiple of 8
 * channels; otherwise, and always after tracea_set_conv_transpose_by_phase(0), as a GEMM to fp32
 * partial products followed by a gather.  The two formulations agree within the tolerance of the
 * operator (fp32 accumulation in a different order). */
void tracea_set_conv_transpose_by_phase(int32_t enabled);
/* The by-phase formulation regroups the filter bank at every call (one helper launch).  With the filter
 * cache on, the regrouped bank of a (device, filter pointer, shape, strides, stride, padding) is built once,
 * kept in device memory of its own and reused by later calls, which then launch nothing but the phase
 * convolutions and allocate nothing: for callers whose filters do not change between calls (inference).
 * Off by default: the library cannot see an in-place update of the filters, nor that a filter tensor was freed
 * and another of the same shape now lives at its address (the usual outcome of reloading weights under a
 * caching allocator): both would be served the old bank.  After changing filters in place or replacing them
 * call tracea_conv_transpose_filter_cache_clear (also frees the copies; it waits for the device).  At most 64
 * banks are kept; a miss while the stream is being captured regroups per call as without the cache.  (The
 * reference's kernel indexes its [C*R*S, K] bank in place, src/emitter/conv_transpose.rs:207-236, and has
 * no such state.) */
void tracea_set_conv_transpose_filter_cache(int32_t enabled);
void tracea_conv_transpose_filter_cache_clear(void);
int32_t tracea_last_split_k(void);

/* Shader-clock probe for measurements (no counterpart in the reference).  Enqueues on `stream` a one-wave
 * kernel that writes `samples` pairs of 64-bit counters to the device buffer `out` (2 * samples entries):
 * the shader's clock ticks and the device's constant 100 MHz counter, one pair about every gap * 64 clocks
 * (gap 0..4096).  Run on a stream of its own beside the kernels under measurement, the ratio of the two
 * counters' increments is the clock frequency the device ran them at.  Returns TRACEA_INVALID_PARAMS for
 * a null buffer or counts out of range, TRACEA_CUDA_ERROR when the launch fails. */
TraceaStatus tracea_clock_probe(void *out, int32_t samples, int32_t gap, void *stream);

/* tracea_gemm for callers that cannot allocate device memory: code whose stream is being
 * captured into a HIP graph, tight serving loops, harnesses that forbid hipMalloc.  No
 * counterpart in the reference (its runtime allocates freely).  Arguments, results and errors
 * are those of tracea_gemm, and the same kernels run; the only difference is where the fp32
 * partial products of a launch split along K go: into a workspace of
 * TRACEA_STATIC_SCRATCH_BYTES that is part of the library's device image (one copy per GPU,
 * held until the process ends) instead of the per-stream buffer that tracea_gemm grows on
 * demand.  The call makes no hipMalloc / hipFree and no allocating library call.  A launch
 * whose split would need more than the workspace holds (splits * M * N * 4 bytes) returns
 * TRACEA_UNSUPPORTED_CONFIG with the two sizes in the error text; launches that are not split
 * need no workspace and have no limit.  All calls on one GPU share that GPU's workspace, on
 * every stream: two such calls that may overlap in time on one GPU race on it, so issue them on
 * one stream or order them with events.  Nothing in the workspace needs to start at zero (every
 * element the reduction reads is written by the launch before it). */
#define TRACEA_STATIC_SCRATCH_BYTES (16u << 20)
TraceaStatus tracea_gemm_noalloc(TraceaTensorView a, TraceaTensorView b, const TraceaTensorView *bias,
                                 const TraceaTensorView *residual, TraceaTensorView *c,
                                 TraceaGemmParams params);

/* Kernel-variant control for tuners and benchmarks.  `op` is "gemm", "conv2d"
 * or "attention".  A variant forced with tracea_force_variant (index >= 0) is
 * used by every later call of that operator FROM THE CALLING THREAD whenever it
 * is feasible for the problem (other threads keep their own choice, so a tuner
 * timing variants does not steer calls made elsewhere in the process); -1
 * restores automatic selection. */
int32_t tracea_variant_count(const char *op);
const char *tracea_variant_name(const char *op, int32_t index); /* library-owned */
int32_t tracea_force_variant(const char *op, int32_t index);    /* 0 ok, -1 bad argument */
/* The variant automatic selection would run for a "gemm" or "conv2d" problem in
 * its implicit-GEMM view (m rows, n channels, k reduction), K-contiguous B, before
 * any forced variant is applied; -1 on a bad argument. */
int32_t tracea_select_variant(const char *op, int64_t m, int64_t n, int64_t k);
/* The variant the calling thread's most recent call of `op` actually launched
 * (a forced or cached variant that cannot run a problem is replaced by the
 * nearest one that can); -1 before any call, or when the call was served by a
 * kernel outside the variant table (fp32 and strided GEMM). */
int32_t tracea_last_variant(const char *op);

/* The 80-byte ConvParams block of the reference (src/emitter/cuda/conv.rs:134-142;
 * packing src/interface/python.rs:423-435) as this library computes it, for
 * callers and tests that compare coordinate arithmetic bit for bit.  The
 * shifts are those fast_divmod consumes (shift beyond 32). */
typedef struct {
  int32_t batch, h_in, w_in, c_in, k_out;
  int32_t h_out, w_out, r_sz, s_sz;
  int32_t stride, pad, dilation;
  uint32_t hw_m, hw_s, w_m, w_s, sic_m, sic_s, c_m, c_s;
} TraceaConvParamsBlock;
TraceaStatus tracea_conv_params_pack(int32_t n, int32_t h, int32_t w, int32_t c, int32_t k,
                                     int32_t r, int32_t s, int32_t stride, int32_t pad,
                                     int32_t dilation, TraceaConvParamsBlock *out);

/* Runs the device-side coordinate mapping of the convolution kernel for every
 * GEMM row m and column k and writes {bn,ho,wo} per row, the batch base offset
 * per row and {r,s,ci} per k into DEVICE buffers rows[M*3], base_off[M],
 * cols[K*3]. */
TraceaStatus tracea_conv_coords_device(const TraceaConvParamsBlock *p, int32_t *rows,
                                       int64_t *base_off, int32_t *cols, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* TRACEA_H */
