// Shared host/device declarations of the MI355X Tracea library.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "tracea.h"

namespace tracea_amd {

// Element types the matrix-core kernels compute in (fp32 accumulate always).
enum DataType : int { DT_F32 = 0, DT_F16 = 1, DT_BF16 = 2 };

// One fused epilogue operator; mirrors TraceaEpilogueOp with device pointers.
struct EpilogueOpDev {
  int kind;   // TraceaEpilogueOpKind
  int dtype;  // DataType of p0 when p0 is a bias or residual
  const void *p0, *p1, *p2, *p3;
  float epsilon;
  long long ld;  // residual row stride, elements
};

struct EpilogueChain {
  int n_ops;
  EpilogueOpDev ops[TRACEA_MAX_EPILOGUE_OPS];
};

// Problem description handed to the contraction kernels.  For a convolution
// the GEMM view is M = batch*h_out*w_out, N = k_out, K = r*s*c_in, A is the
// NHWC activation tensor and B the filter bank.
struct ContractionArgs {
  const void *A;
  const void *B;
  void *C;
  int M, N, K;
  long long lda;       // A row stride (GEMM only), elements
  long long ldb;       // B: stride between consecutive n (K-contiguous B) or k (N-contiguous B)
  long long ldc;       // C row stride, elements
  int out_dtype;       // DataType of C
  unsigned a_bytes, b_bytes;  // extent of A and B in bytes (bounds of the direct-to-LDS buffer loads)
  int grid_m, grid_n;  // tiles along M and N
  int k_split;         // 0: one workgroup per tile runs all of K; else the K extent of one split (a multiple
                       // of the variant's BK): grid.y = ceil(K / k_split), C is the [splits][M][ldc] workspace
  // One-launch split (k_split > 0 and fuse_ws set): C, out_dtype and epi are the call's own; every workgroup
  // leaves its fp32 partial product, in accumulator order, in block (blockIdx.x*splits + blockIdx.y) of fuse_ws
  // and takes a ticket from fuse_count[blockIdx.x]; the last one of a tile sums the blocks in split order, runs
  // the operator chain, writes C and puts the counter back to zero.
  float *fuse_ws;
  unsigned *fuse_count;
  int group_m;         // tile-order group height
  // GEMM over a tile list (null: the dense grid_m x grid_n grid): workgroup p of the
  // launch (grid.x = list length) runs record tile_list[p]; a record is 5 words
  // {tile row, tile column, first k, end k, role}; tile_slice[p], if given, is the row
  // block of the fp32 workspace C = [slices][M][ldc] its partial product goes to
  const unsigned *tile_list;
  const unsigned *tile_records;
  const unsigned *tile_slice;
  int tile_count;
  // convolution geometry (ConvParams of the reference, h/w split)
  int h_in, w_in, c_in, h_out, w_out, s_sz;
  int stride_h, stride_w, pad_h, pad_w, dil_h, dil_w;
  unsigned hw_m, hw_s, w_m, w_s, sc_m, sc_s, c_m, c_s;
  // streamed convolution only (out_map != 0): output pixel (q, p) of image b is written to row
  // b*o_img + (o_a + o_sh*q)*o_wo + o_b + o_sw*p of C instead of row m (one phase of a transposed
  // convolution); residual operands are indexed by the same row.  Not combined with a K split.
  int out_map, o_sh, o_sw, o_a, o_b, o_wo;
  long long o_img;
  // phases > 1: grid.z = phases = o_sh*o_sw launches all phases at once; workgroups with
  // blockIdx.z = z work on phase (o_a, o_b) = (z / o_sw, z % o_sw) with the filter bank at
  // B + z*phase_b_stride elements and the padding phase_pad_h[o_a], phase_pad_w[o_b] (strides up to 4)
  int phases;
  long long phase_b_stride;
  int phase_pad_h[4], phase_pad_w[4];
  // patch-resident convolution (pipeline 4) only: filter rows, M tiles per image,
  // padded row width W + 2 pad_w, 16-byte chunks per patch pixel (odd), patch
  // load iterations per thread, LDS bytes reserved for the patch, and the
  // reciprocals of the chunk count and of the padded width
  int r_sz, p_tiles, p_pw, p_cpp, p_iters, p_np_bytes;
  // pipeline 5 only: output pixels per workgroup (pipeline 4 has them in its tile shape), load
  // instructions per padded patch row, pixels per load instruction
  int p_tm, p_seg, p_ppi;
  unsigned p_cpp_m, p_cpp_s, p_pw_m, p_pw_s;
  // pipelines 7 and 8 only: reciprocals of grid_n and p_tiles (workgroup index -> filter slab, tile, image)
  unsigned gn_m, gn_s, pt_m, pt_s;
  // pipeline 5 only: the chain in the fast form of conv_resident_kernel.hpp, or sig < 0
  struct FastEpilogue {
    int sig;                  // bit 0 affine, 1 ReLU, 2 residual, 3 ReLU (in this order); < 0: not of this form
    int aff_kind, aff_dtype;  // TraceaEpilogueOpKind of the affine part and the DataType of a bias
    const void *p0, *p1, *p2, *p3;
    float epsilon;
    const void *res;          // residual tensor (operand type), row stride res_ld elements
    long long res_ld;
  } fe;
  EpilogueChain epi;
};

struct AttentionArgs {
  const void *Q, *K, *V;
  void *O;
  int B, H, S, D;
  long long q_sb, q_sh, q_ss;  // element strides of batch, head, row (D contiguous)
  long long k_sb, k_sh, k_ss;
  long long v_sb, v_sh, v_ss;
  long long o_sb, o_sh, o_ss;
  float scale_log2;  // softmax scale * log2(e)
  int causal;
};

// A precompiled kernel variant and the rule that says when it applies.
struct ContractionVariant {
  const char *name;
  int bm, bn, bk, waves_m, waves_n, stages;
  int pipeline;  // 0: operands read just in time; 1: read one k-step ahead, across the barrier;
                 // 2: as 1, with direct-to-LDS tile loads (an N-contiguous B is kept [k][n] in LDS
                 //    and fetched with transposing LDS reads);
                 // 3: ring of `stages` LDS buffers, direct-to-LDS loads stages-1 tiles ahead
                 // 4: convolution only: input patch resident in LDS, filter tiles through a ring of `stages`
                 // (the build's mode 6 is pipeline 2 with mfma = 16)
                 // 5: convolution only: input patch and filter bank both resident in LDS
                 //    (conv_resident_kernel.hpp); bm = most pixels per workgroup, K = 16 * stages exactly
  size_t lds_bytes;
  // launch: returns hipError_t as int
  int (*launch)(const ContractionArgs &, bool conv, int dtype, bool b_ncontig, hipStream_t);
  int mfma;  // MFMA shape of the half-precision kernels: 32 (32x32x16) or 16 (16x16x32: GEMM on pipeline 2 only)
};

int contraction_variant_count();
const ContractionVariant &contraction_variant(int i);

// fp32 MFMA GEMM (row-major A [M,K], row-major B [K,N]).
int launch_gemm_f32(const ContractionArgs &args, int tile, hipStream_t stream);  // tile: 128, 64 or 6432 (64x64 with K tiles of 32)
// Any dtype/stride combination, no alignment requirement (VALU, slow).
struct GenericGemmArgs {
  const void *A, *B;
  void *C;
  int M, N, K;
  long long sam, sak, sbk, sbn, scm, scn;
  int a_dtype, b_dtype, c_dtype;
  EpilogueChain epi;
};
int launch_gemm_generic(const GenericGemmArgs &args, hipStream_t stream);
// An operand as the tile kernels can read it: dst[r][c] (rows_dst rows of `pitch` elements of elt_bytes = 2 or 4)
// = src[r0 * rs + r1 * s1 + r2 * s2 + c * cs] for r = (r0 * n1 + r1) * n2 + r2 < rows_src and c < cols_src, zero
// elsewhere (rows on 16 bytes, a whole number of 16-byte pieces, zeros behind the data), from up to four strides.
int launch_pad_copy(const void *src, void *dst, int elt_bytes, long long rows_src, long long cols_src, long long rs,
                    long long cs, long long rows_dst, long long pitch, hipStream_t stream, long long n1 = 1, long long s1 = 0,
                    long long n2 = 1, long long s2 = 0);
// The way back for a result: dst[r0 * rs + r1 * s1 + r2 * s2 + c * cs] = src[r][c] for r < rows, c < cols.
int launch_unpad_copy(const void *src, void *dst, int elt_bytes, long long rows, long long cols, long long rs, long long cs,
                      long long pitch, hipStream_t stream, long long n1 = 1, long long s1 = 0, long long n2 = 1, long long s2 = 0);

// Second stage of a split-K contraction: out[m, n] = chain(sum over z of partial[z][m][n]).
struct SplitKReduceArgs {
  const float *partial;  // [splits][M][N] fp32
  void *out;
  int out_dtype;
  int splits, M, N;
  long long ldc;
  EpilogueChain epi;
  // Tile lists whose tiles have different numbers of records: tile_counts[tile row * grid_n + tile column]
  // planes are summed for an element of that mt x nt tile, and a tile with none is left untouched.
  // nullptr: every element sums `splits` planes.
  const unsigned *tile_counts;
  int mt, nt, grid_n;
};
int launch_splitk_reduce(const SplitKReduceArgs &args, hipStream_t stream);

// Device address of the calling process's copy of the static split-K workspace
// (TRACEA_STATIC_SCRATCH_BYTES) on `device`; returns hipError_t as int.
int static_scratch_address(int device, void **ptr);

// Second stage of the transposed convolution: gathers the per-tap partial
// products `cols` (one row per input pixel, one column per (r, s, k)) into the
// output pixels and applies the operator chain.
struct Col2imArgs {
  const float *cols;
  void *out;
  int out_dtype;
  long long ld_cols;           // row stride of cols, elements
  long long ldc;               // output pixel pitch, elements
  long long st_r, st_s, st_k;  // column of (r, s, k) inside a row of cols
  int b0, nb;                  // images this launch covers: b0 .. b0+nb-1 (cols row 0 is image b0)
  int h_in, w_in, h_out, w_out, k_out, r_sz, s_sz;
  int stride_h, stride_w, pad_h, pad_w;
  EpilogueChain epi;
};
int launch_col2im_epilogue(const Col2imArgs &args, hipStream_t stream);

// Copies a filter bank with dims [K,R,S,C] and arbitrary element strides into
// the B operand of the transposed convolution's GEMM, columns ordered (r, s, k):
// [R][S][K][C] (K-contiguous B, for the half-precision kernels) when c_inner,
// else [C][R][S][K] (row-major B, for the fp32 kernel).
// Filters of a transposed convolution regrouped by output phase: tap (r, s) of the filter bank
// goes to out + tap_base[r*S + s] + k * tap_kstride[r*S + s] + c (half precision only), which
// makes every phase a [K, taps_r, taps_s, C] filter bank for the convolution kernels.
struct PhaseFilterArgs {
  const void *w;
  void *out;
  int C, K, R, S;
  long long sc, sk, sr, ss;  // element strides of c, k, r, s in w
  long long tap_base[64];
  int tap_kstride[64];
};
int launch_phase_filters(const PhaseFilterArgs &args, hipStream_t stream);

struct FilterRepackArgs {
  const void *w;
  void *out;
  int elem_bytes;  // 2 or 4
  int c_inner;
  int C, K, R, S;
  long long sc, sk, sr, ss;  // element strides of c, k, r, s in w
};
int launch_filter_repack(const FilterRepackArgs &args, hipStream_t stream);

// Operators of a graph that were not merged into a contraction (standalone ReLU,
// BatchNorm, Add: src/policy/types.rs:60-84) run as an operator chain over an
// existing tensor: out[m, n] = chain(x[m, n]), rows of `channels` elements.
struct ChainApplyArgs {
  const void *x;
  void *out;
  int x_dtype, out_dtype;
  long long rows;
  int channels;
  EpilogueChain epi;
};
int launch_chain_apply(const ChainApplyArgs &args, hipStream_t stream);
// out[b, c] = mean over hw of x[b, hw, c] (NHWC), fp32 sums.
int launch_global_avg_pool(const void *x, void *out, int dtype, int out_dtype, int batch, int hw, int channels,
                           hipStream_t stream);
// Pooling and the linear layer behind it in one launch: out[b, j] = chain(sum_k mean_hw(x[b, hw, k]) * w[k, j]),
// the means rounded through `dtype` (and stored to `pooled` [batch, channels] when it is not null).
struct PoolLinearArgs {
  const void *x, *w;
  void *out, *pooled;
  int dtype, out_dtype;  // x, w and pooled; out
  int batch, hw, channels, n_out;
  long long w_ld;        // elements between rows of w (its other stride is 1)
  EpilogueChain epi;
};
int launch_pool_linear(const PoolLinearArgs &args, bool k_contiguous, hipStream_t stream);
// Row-wise softmax over the last axis, fp32 arithmetic.
int launch_softmax_rows(const void *x, void *out, int dtype, int out_dtype, long long rows, int cols,
                        hipStream_t stream);

struct AttentionVariant {
  const char *name;
  int block_q, block_kv, waves;
  int stages;  // LDS stages per K and per V ring
  int (*launch)(const AttentionArgs &, int dtype, hipStream_t);
  bool (*feasible)(const AttentionArgs &);
  int mfma;   // MFMA shape: 32 (32x32x16) or 16 (16x16x32)
  int items;  // query blocks a workgroup takes one after the other (1 or 2)
  int offset_groups;  // 1: the two waves of a SIMD run half an iteration apart, two barriers per tile (else 0)
};
int attention_variant_count();
const AttentionVariant &attention_variant(int i);

// Fills n elements with a counter-based pseudo-random sequence, uniform in
// [-amplitude, amplitude] (synthetic operands for the tuner).
int launch_fill_uniform(void *ptr, size_t n, int dtype, unsigned seed, float amplitude,
                        hipStream_t stream);

// One-wave kernel that samples (shader clock ticks, 100 MHz counter) `samples` times, about gap*64 clocks
// apart, into out[2*samples]; returns hipError_t as int.
int launch_clock_probe(unsigned long long *out, int samples, int gap, hipStream_t stream);

int launch_conv_coords(const TraceaConvParamsBlock &p, int32_t *rows, int64_t *base_off,
                       int32_t *cols, hipStream_t stream);

}  // namespace tracea_amd
