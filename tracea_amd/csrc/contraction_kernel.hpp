// MFMA contraction kernel for gfx950: one template covers the fp16/bf16 GEMM
// and the implicit-GEMM convolution (they differ only in how a 16-byte piece
// of the A operand is located in global memory).
//
// Behaviour it replaces in the reference: gemm_mma_kernel
// (src/emitter/cuda/gemm.rs:92-207) and kernel_main / conv2d_implicit_gemm
// (src/emitter/cuda/conv.rs:153-331); epilogue functors
// src/kernels/gpu/epilogue.cuh:12-63.
//
// Structure
//   * block tile BM x BN x BK, WM x WN wavefronts of 64 lanes, each wave owns
//     (BM/WM) x (BN/WN) of C as 32x32 MFMA blocks (v_mfma_f32_32x32x16);
//   * both operands are staged K-contiguous in LDS ([row][BK] halves) with an
//     XOR swizzle of the 16-byte column index so that the ds_read_b128 operand
//     fetches of 16 consecutive rows fall in 16 different bank groups;
//   * global memory is read in 16-byte pieces, 8 lanes per 128-byte row
//     segment; the next K tile is fetched into registers while the current one
//     is multiplied, then written to the other LDS stage (one barrier per K
//     tile);
//   * the MFMA is issued with the operands swapped (D = B_frag x A_frag) so a
//     lane ends up with 4 consecutive output channels of one row; the epilogue
//     regroups the accumulators through LDS into 8 consecutive channels per
//     lane, applies the fused operator chain on fp32 and stores 16 bytes.
#pragma once
#include <type_traits>

#include "common.hpp"

namespace tracea_amd {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// Compile-time loop: body(std::integral_constant<int, I>) for I = 0..N-1.  Used where an
// accumulator array must be indexed by constants however large the loop body is
// (a run-time index would move the whole array to scratch memory).
template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F &&body) {
  if constexpr (I < N) {
    body(std::integral_constant<int, I>{});
    static_for<I + 1, N>(body);
  }
}

template <int DT>
struct Mfma32;
template <>
struct Mfma32<DT_F16> {
  static __device__ __forceinline__ f32x16 run(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};
template <>
struct Mfma32<DT_BF16> {
  static __device__ __forceinline__ f32x16 run(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};

// The 16x16x32 shape: four times the blocks of a quarter the size, 16 cycles each.  A fragment is 16 rows
// by 32 k (lane l: row l & 15, k = 8 * (l >> 4) .. + 7), the result a column of 4 per lane (lane l: column
// l & 15 of the second operand, rows 4 * (l >> 4) .. + 3 of the first).
template <int DT>
struct Mfma16;
template <>
struct Mfma16<DT_F16> {
  static __device__ __forceinline__ f32x4 run(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};
template <>
struct Mfma16<DT_BF16> {
  static __device__ __forceinline__ f32x4 run(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};

// q = n / d, r = n % d through a precomputed reciprocal: m = ceil(2^(32+s)/d),
// or m == 0 for a power-of-two d with s = log2(d).  Same arithmetic as the
// reference's device fast_divmod (src/emitter/cuda/conv.rs:144-151).
// One expression for all cases (n >= 0), because a branch on the kind of divisor, uniform as
// it is, splits the tile loaders of the convolution into basic blocks that the MFMAs cannot
// be interleaved with: umulhi(n, m) is the scaled quotient for a real reciprocal and 0 for
// m == 0, where n itself takes its place (d == 1 is the power of two with s == 0).
__device__ __forceinline__ void fast_divmod(int n, unsigned m, unsigned s, int d, int &q, int &r) {
  const unsigned scaled = __umulhi((unsigned)n, m) + (m == 0 ? (unsigned)n : 0u);
  q = (int)(scaled >> s);
  r = n - q * d;
}

// ---- epilogue helpers -------------------------------------------------------

// Loads V (1, 4 or 8) consecutive elements starting at index idx as floats;
// elements at or beyond nvalid read as zero.  One vector load when the run is
// complete and naturally aligned, scalar loads otherwise.
template <int V>
__device__ __forceinline__ void load_as_float(const void *base, int dtype, long long idx,
                                              int nvalid, float (&out)[V]) {
  if (dtype == DT_F32) {
    const float *p = (const float *)base + idx;
    if (V > 1 && nvalid >= V && (((uintptr_t)p) & 15) == 0) {
#pragma unroll
      for (int q = 0; q < V / 4; ++q) {
        f32x4 v = ((const f32x4 *)p)[q];
#pragma unroll
        for (int e = 0; e < 4; ++e) out[q * 4 + e] = v[e];
      }
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e) out[e] = e < nvalid ? p[e] : 0.0f;
    }
  } else if (dtype == DT_F16) {
    const _Float16 *p = (const _Float16 *)base + idx;
    if (V > 1 && nvalid >= V && (((uintptr_t)p) & (V * 2 - 1)) == 0) {
#pragma unroll
      for (int q = 0; q < V / 4; ++q) {
        f16x4 v = ((const f16x4 *)p)[q];
#pragma unroll
        for (int e = 0; e < 4; ++e) out[q * 4 + e] = (float)v[e];
      }
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e) out[e] = e < nvalid ? (float)p[e] : 0.0f;
    }
  } else {
    const __bf16 *p = (const __bf16 *)base + idx;
    if (V > 1 && nvalid >= V && (((uintptr_t)p) & (V * 2 - 1)) == 0) {
#pragma unroll
      for (int q = 0; q < V / 4; ++q) {
        bf16x4 v = ((const bf16x4 *)p)[q];
#pragma unroll
        for (int e = 0; e < 4; ++e) out[q * 4 + e] = (float)v[e];
      }
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e) out[e] = e < nvalid ? (float)p[e] : 0.0f;
    }
  }
}

// Applies one operator to V consecutive channels n..n+V-1 of output row m
// (fp32 in, fp32 out), reading its operands from global memory.
template <int V>
__device__ __forceinline__ void apply_epilogue_one(float (&v)[V], long long m, int n, int nvalid,
                                                   const EpilogueOpDev &op) {
  {
    float t[V];
    switch (op.kind) {
      case TRACEA_EPI_OP_BIAS_ADD:
        load_as_float<V>(op.p0, op.dtype, n, nvalid, t);
#pragma unroll
        for (int e = 0; e < V; ++e) v[e] = v[e] + t[e];
        break;
      case TRACEA_EPI_OP_RELU:
#pragma unroll
        for (int e = 0; e < V; ++e) v[e] = fmaxf(0.0f, v[e]);
        break;
      case TRACEA_EPI_OP_GELU:
#pragma unroll
        for (int e = 0; e < V; ++e)
          v[e] = 0.5f * v[e] * (1.0f + tanhf(0.79788456f * (v[e] + 0.044715f * v[e] * v[e] * v[e])));
        break;
      case TRACEA_EPI_OP_SILU:
#pragma unroll
        for (int e = 0; e < V; ++e) v[e] = v[e] / (1.0f + expf(-v[e]));
        break;
      case TRACEA_EPI_OP_RESIDUAL_ADD:
        load_as_float<V>(op.p0, op.dtype, m * op.ld + n, nvalid, t);
#pragma unroll
        for (int e = 0; e < V; ++e) v[e] = v[e] + t[e];
        break;
      case TRACEA_EPI_OP_BIAS_ADD_SILU:
        load_as_float<V>(op.p0, op.dtype, n, nvalid, t);
#pragma unroll
        for (int e = 0; e < V; ++e) {
          float x = v[e] + t[e];
          v[e] = x / (1.0f + expf(-x));
        }
        break;
      case TRACEA_EPI_OP_BATCHNORM: {
        float b[V], mu[V], var[V];
        load_as_float<V>(op.p0, DT_F32, n, nvalid, t);
        load_as_float<V>(op.p1, DT_F32, n, nvalid, b);
        load_as_float<V>(op.p2, DT_F32, n, nvalid, mu);
        load_as_float<V>(op.p3, DT_F32, n, nvalid, var);
#pragma unroll
        for (int e = 0; e < V; ++e)
          v[e] = (v[e] - mu[e]) * (1.0f / sqrtf(var[e] + op.epsilon)) * t[e] + b[e];
      } break;
      case TRACEA_EPI_OP_SCALE_SHIFT: {
        float sh[V];
        load_as_float<V>(op.p0, DT_F32, n, nvalid, t);
        load_as_float<V>(op.p1, DT_F32, n, nvalid, sh);
#pragma unroll
        for (int e = 0; e < V; ++e) v[e] = v[e] * t[e] + sh[e];
      } break;
      default:
        break;
    }
  }
}

// Applies the operator chain, in order, to V consecutive channels n..n+V-1 of
// output row m (fp32 in, fp32 out), every operand read from global memory.
template <int V>
__device__ __forceinline__ void apply_epilogue(float (&v)[V], long long m, int n, int nvalid,
                                               const EpilogueChain &chain) {
  for (int o = 0; o < chain.n_ops; ++o) apply_epilogue_one<V>(v, m, n, nvalid, chain.ops[o]);
}

// Converts V floats to the output type (round to nearest even) and stores
// them at element index idx; only the first nvalid are written.
template <int V>
__device__ __forceinline__ void store_from_float(void *base, int dtype, long long idx, int nvalid,
                                                 const float (&v)[V]) {
  if (dtype == DT_F32) {
    float *p = (float *)base + idx;
    if (V > 1 && nvalid >= V && (((uintptr_t)p) & 15) == 0) {
#pragma unroll
      for (int q = 0; q < V / 4; ++q) {
        f32x4 o = {v[q * 4], v[q * 4 + 1], v[q * 4 + 2], v[q * 4 + 3]};
        ((f32x4 *)p)[q] = o;
      }
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e)
        if (e < nvalid) p[e] = v[e];
    }
  } else if (dtype == DT_F16) {
    _Float16 *p = (_Float16 *)base + idx;
    _Float16 h[V];
#pragma unroll
    for (int e = 0; e < V; ++e) h[e] = (_Float16)v[e];
    if (V == 8 && nvalid >= 8 && (((uintptr_t)p) & 15) == 0) {
      f16x8 o = {h[0], h[1], h[2], h[3], h[V > 4 ? 4 : 0], h[V > 5 ? 5 : 0], h[V > 6 ? 6 : 0], h[V > 7 ? 7 : 0]};
      *(f16x8 *)p = o;
    } else if (V == 4 && nvalid >= 4 && (((uintptr_t)p) & 7) == 0) {
      f16x4 o = {h[0], h[1], h[2], h[3]};
      *(f16x4 *)p = o;
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e)
        if (e < nvalid) p[e] = h[e];
    }
  } else {
    __bf16 *p = (__bf16 *)base + idx;
    __bf16 h[V];
#pragma unroll
    for (int e = 0; e < V; ++e) h[e] = (__bf16)v[e];
    if (V == 8 && nvalid >= 8 && (((uintptr_t)p) & 15) == 0) {
      bf16x8 o = {h[0], h[1], h[2], h[3], h[V > 4 ? 4 : 0], h[V > 5 ? 5 : 0], h[V > 6 ? 6 : 0], h[V > 7 ? 7 : 0]};
      *(bf16x8 *)p = o;
    } else if (V == 4 && nvalid >= 4 && (((uintptr_t)p) & 7) == 0) {
      bf16x4 o = {h[0], h[1], h[2], h[3]};
      *(bf16x4 *)p = o;
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e)
        if (e < nvalid) p[e] = h[e];
    }
  }
}

// ---- per-channel operands of the chain, staged in LDS ----------------------------
// In the tile epilogue every row a lane stores needs the same per-channel
// operands (bias, BatchNorm or scale/shift vectors).  Reading them from global
// memory inside the row loop makes that loop a chain of dependent L2 round
// trips, one per row.  Instead each thread loads a few entries of a small
// table before the main loop (the loads complete under it), the table is
// written to LDS once the main loop has released it, and the row loop reads its
// operands from there.  Layout: table[(o * 2 + which) * BN + channel], fp32;
// which 0 = bias or scale, which 1 = shift.  BatchNorm is folded to
// scale = gamma / sqrt(var + eps), shift = beta - mean * scale (one fp32
// rounding away from the unfolded form).
__device__ __forceinline__ float chain_table_value(const EpilogueChain &chain, int o, int which, int n, int N) {
  if (o >= chain.n_ops || n >= N) return 0.0f;
  const EpilogueOpDev &op = chain.ops[o];
  float one[1];
  if (op.kind == TRACEA_EPI_OP_BIAS_ADD || op.kind == TRACEA_EPI_OP_BIAS_ADD_SILU) {
    if (which != 0) return 0.0f;
    load_as_float<1>(op.p0, op.dtype, n, 1, one);
    return one[0];
  }
  if (op.kind == TRACEA_EPI_OP_SCALE_SHIFT) return ((const float *)(which == 0 ? op.p0 : op.p1))[n];
  if (op.kind == TRACEA_EPI_OP_BATCHNORM) {
    const float scale = ((const float *)op.p0)[n] * (1.0f / sqrtf(((const float *)op.p3)[n] + op.epsilon));
    return which == 0 ? scale : ((const float *)op.p1)[n] - ((const float *)op.p2)[n] * scale;
  }
  return 0.0f;
}

// The chain as the row loop needs it, read once from the kernel arguments: the
// operator kinds and the descriptor of the first residual operator.  Indexing
// args.epi.ops[] with a run-time operator number inside the row loop re-reads
// kind, pointer, dtype and stride through dependent scalar loads for every
// (row, operator) pair, which cost more than everything else in the epilogue.
struct ChainPlan {
  unsigned kinds;      // operator o in bits 4o..4o+3 (TraceaEpilogueOpKind < 16), 0 past the end
  int n_ops;
  int res_index;       // first residual operator, -1 if none
  const void *res_ptr;
  int res_dtype;
  long long res_ld;
};

__device__ __forceinline__ ChainPlan chain_plan(const EpilogueChain &chain) {
  ChainPlan p;
  p.kinds = 0;
  p.n_ops = chain.n_ops;
  p.res_index = -1;
  p.res_ptr = nullptr;
  p.res_dtype = DT_F32;
  p.res_ld = 0;
#pragma unroll
  for (int o = TRACEA_MAX_EPILOGUE_OPS - 1; o >= 0; --o) {
    const int kind = o < chain.n_ops ? chain.ops[o].kind : (int)TRACEA_EPI_OP_NONE;
    p.kinds |= (unsigned)(kind & 15) << (4 * o);
    if (kind == TRACEA_EPI_OP_RESIDUAL_ADD) {
      p.res_index = o;
      p.res_ptr = chain.ops[o].p0;
      p.res_dtype = chain.ops[o].dtype;
      p.res_ld = chain.ops[o].ld;
    }
  }
  return p;
}

// The chain on 8 consecutive channels of row m; per-channel operands come from
// the LDS table (tab points at this lane's first channel, vectors bn apart),
// the first residual tensor through the plan, any further one from the
// kernel arguments.  The operator loop is a real loop (its body is emitted
// once) over kinds held in one scalar.
__device__ __forceinline__ void apply_epilogue_tab(float (&v)[8], long long m, int n, int nvalid,
                                                   const EpilogueChain &chain, const ChainPlan &plan,
                                                   const float *tab, int bn) {
#pragma nounroll
  for (int o = 0; o < plan.n_ops; ++o) {
    const int kind = (int)((plan.kinds >> (4 * o)) & 15u);
    if (kind == TRACEA_EPI_OP_RELU) {
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = fmaxf(0.0f, v[e]);
    } else if (kind == TRACEA_EPI_OP_BIAS_ADD || kind == TRACEA_EPI_OP_BIAS_ADD_SILU ||
               kind == TRACEA_EPI_OP_SCALE_SHIFT || kind == TRACEA_EPI_OP_BATCHNORM) {
      const float *pa = tab + (o * 2) * bn;
      const f32x4 a0 = *(const f32x4 *)pa, a1 = *(const f32x4 *)(pa + 4);
      const f32x4 b0 = *(const f32x4 *)(pa + bn), b1 = *(const f32x4 *)(pa + bn + 4);  // zeros for a bias
      const float a[8] = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
      const float b[8] = {b0[0], b0[1], b0[2], b0[3], b1[0], b1[1], b1[2], b1[3]};
      if (kind == TRACEA_EPI_OP_BIAS_ADD) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = v[e] + a[e];
      } else if (kind == TRACEA_EPI_OP_BIAS_ADD_SILU) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float x = v[e] + a[e];
          v[e] = x / (1.0f + expf(-x));
        }
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = v[e] * a[e] + b[e];
      }
    } else if (kind == TRACEA_EPI_OP_RESIDUAL_ADD && o == plan.res_index) {
      float t[8];
      load_as_float<8>(plan.res_ptr, plan.res_dtype, m * plan.res_ld + n, nvalid, t);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = v[e] + t[e];
    } else {
      apply_epilogue_one<8>(v, m, n, nvalid, chain.ops[o]);  // GELU, SiLU, a second residual
    }
  }
}

// ---- specialised row body ------------------------------------------------------------
// The general row body above carries every fallback inline (partial channel
// vectors, unaligned rows, per-element loads and stores, GELU / SiLU): several
// thousand instructions and hundreds of branches per row, more than the
// instruction cache holds.  Nearly every call needs none of it: all 8 channels
// of every lane exist, rows of C (and of the residual) are 16-byte aligned, and
// the chain is made of bias / scale-shift / BatchNorm / ReLU / one residual.
// Whether that holds is the same for the whole workgroup, so it is decided
// once and the row loops are emitted twice, each behind a uniform branch.
__device__ __forceinline__ bool chain_is_simple(const ChainPlan &plan, const ContractionArgs &args, int n0, int bn) {
  bool ok = n0 + bn <= args.N && (args.ldc & 7) == 0 && (((uintptr_t)args.C) & 15) == 0;
#pragma unroll
  for (int o = 0; o < TRACEA_MAX_EPILOGUE_OPS; ++o) {
    const int kind = (int)((plan.kinds >> (4 * o)) & 15u);
    ok = ok && (kind == TRACEA_EPI_OP_NONE || kind == TRACEA_EPI_OP_BIAS_ADD || kind == TRACEA_EPI_OP_RELU ||
                kind == TRACEA_EPI_OP_SCALE_SHIFT || kind == TRACEA_EPI_OP_BATCHNORM ||
                (kind == TRACEA_EPI_OP_RESIDUAL_ADD && o == plan.res_index));
  }
  if (plan.res_index >= 0)
    ok = ok && plan.res_dtype != DT_F32 && (plan.res_ld & 7) == 0 && (((uintptr_t)plan.res_ptr) & 15) == 0;
  return ok;
}

// The specialised path for the 32 staged rows of one accumulator block: the
// rows a lane handles (er, er+RPI, ...) are processed GROUP at a time -- all
// their staged values are read first, each operator's operands are read once
// and applied to every row of the group, residual loads are issued together,
// stores come last.  One row at a time, every row paid an LDS round trip for
// its staged values and one more per operator, back to back.
// row_of(r) gives the output row of staged row r, or -1 if it does not exist.
// F32OUT: C holds fp32 (two 16-byte stores per lane and row) instead of DT.
template <int DT, int TN, bool F32OUT = false, typename RowOf>
__device__ __forceinline__ void simple_rows(const float *stage, int lane, int n, const ContractionArgs &args,
                                            const ChainPlan &plan, const float *tab, int bn, RowOf row_of) {
  constexpr int EP_PITCH = TN + 4, LPR = TN / 8, RPI = 64 / LPR, NIT = 32 / RPI;
  constexpr int GROUP = NIT < 4 ? NIT : 4;
  const int er = lane / LPR, ec = (lane % LPR) * 8;
  static_for<0, NIT / GROUP>([&](auto grp) {
    constexpr int it0 = decltype(grp)::value * GROUP;
    float v[GROUP][8];
    long long m[GROUP];
#pragma unroll
    for (int g = 0; g < GROUP; ++g) {
      const int r = er + (it0 + g) * RPI;
      m[g] = row_of(r);
      const f32x4 lo = *(const f32x4 *)(stage + r * EP_PITCH + ec);
      const f32x4 hi = *(const f32x4 *)(stage + r * EP_PITCH + ec + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        v[g][e] = lo[e];
        v[g][4 + e] = hi[e];
      }
    }
#pragma nounroll
    for (int o = 0; o < plan.n_ops; ++o) {
      const int kind = (int)((plan.kinds >> (4 * o)) & 15u);
      if (kind == TRACEA_EPI_OP_RELU) {
#pragma unroll
        for (int g = 0; g < GROUP; ++g)
#pragma unroll
          for (int e = 0; e < 8; ++e) v[g][e] = fmaxf(0.0f, v[g][e]);
      } else if (kind == TRACEA_EPI_OP_RESIDUAL_ADD) {
        u32x4 raw[GROUP];
#pragma unroll
        for (int g = 0; g < GROUP; ++g) {
          const long long mm = m[g] >= 0 ? m[g] : 0;  // a row that does not exist re-reads row 0, result discarded
          raw[g] = *(const u32x4 *)((const unsigned short *)plan.res_ptr + mm * plan.res_ld + n);
        }
#pragma unroll
        for (int g = 0; g < GROUP; ++g) {
          if (plan.res_dtype == DT_F16) {
            const f16x8 h = __builtin_bit_cast(f16x8, raw[g]);
#pragma unroll
            for (int e = 0; e < 8; ++e) v[g][e] = v[g][e] + (float)h[e];
          } else {
            const bf16x8 h = __builtin_bit_cast(bf16x8, raw[g]);
#pragma unroll
            for (int e = 0; e < 8; ++e) v[g][e] = v[g][e] + (float)h[e];
          }
        }
      } else {  // bias: v + a; scale/shift and BatchNorm: v * a + b
        const float *pa = tab + (o * 2) * bn;
        const f32x4 a0 = *(const f32x4 *)pa, a1 = *(const f32x4 *)(pa + 4);
        const f32x4 b0 = *(const f32x4 *)(pa + bn), b1 = *(const f32x4 *)(pa + bn + 4);  // zeros for a bias
        const float a[8] = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
        const float b[8] = {b0[0], b0[1], b0[2], b0[3], b1[0], b1[1], b1[2], b1[3]};
        if (kind == TRACEA_EPI_OP_BIAS_ADD) {
#pragma unroll
          for (int g = 0; g < GROUP; ++g)
#pragma unroll
            for (int e = 0; e < 8; ++e) v[g][e] = v[g][e] + a[e];
        } else {
#pragma unroll
          for (int g = 0; g < GROUP; ++g)
#pragma unroll
            for (int e = 0; e < 8; ++e) v[g][e] = v[g][e] * a[e] + b[e];
        }
      }
    }
#pragma unroll
    for (int g = 0; g < GROUP; ++g) {
      if (m[g] >= 0) {
        unsigned short *dst = (unsigned short *)args.C + m[g] * args.ldc + n;
        if constexpr (F32OUT) {
          float *dst32 = (float *)args.C + m[g] * args.ldc + n;
          const f32x4 lo = {v[g][0], v[g][1], v[g][2], v[g][3]}, hi = {v[g][4], v[g][5], v[g][6], v[g][7]};
          *(f32x4 *)dst32 = lo;
          *(f32x4 *)(dst32 + 4) = hi;
        } else if constexpr (DT == DT_F16) {
          f16x8 h;
#pragma unroll
          for (int e = 0; e < 8; ++e) h[e] = (_Float16)v[g][e];
          *(f16x8 *)dst = h;
        } else {
          bf16x8 h;
#pragma unroll
          for (int e = 0; e < 8; ++e) h[e] = (__bf16)v[g][e];
          *(bf16x8 *)dst = h;
        }
      }
    }
  });
}

// ---- tile order ---------------------------------------------------------------
// Consecutive workgroup ids are dealt round-robin to the 8 XCDs, each with its
// own L2.  The id is first regrouped so that one XCD receives a contiguous run
// of tile indices, then the run is laid out in column-major groups of
// `group_m` tile rows, which gives every XCD a compact rectangle of C and
// therefore a small set of A and B panels to keep in its L2.
__device__ __forceinline__ void tile_coordinates(const ContractionArgs &a, int &tile_m,
                                                 int &tile_n) {
  int bid = blockIdx.x;
  const int total = a.grid_m * a.grid_n;
  if ((total & 7) == 0) bid = (bid & 7) * (total >> 3) + (bid >> 3);
  const int gsz = a.group_m * a.grid_n;
  const int group = bid / gsz;
  const int first = group * a.group_m;
  const int rows = min(a.grid_m - first, a.group_m);
  const int in_group = bid - group * gsz;
  tile_m = first + in_group % rows;
  tile_n = in_group / rows;
}

// ---- instruction interleaving --------------------------------------------------
// Emits a scheduling pipeline for the current region: kMfmas MFMAs, before each
// of which the shares of kCountA instructions of class kClassA and kCountB of
// class kClassB are placed (classes as __builtin_amdgcn_sched_group_barrier defines them:
// 0x008 MFMA, 0x020 VMEM read, 0x100 LDS read, 0x200 LDS write).
template <int kStep, int kMfmas, int kClassA, int kCountA, int kClassB, int kCountB>
struct Interleave {
  static __device__ __forceinline__ void run() {
    constexpr int na = ((kStep + 1) * kCountA) / kMfmas - (kStep * kCountA) / kMfmas;
    constexpr int nb = ((kStep + 1) * kCountB) / kMfmas - (kStep * kCountB) / kMfmas;
    if constexpr (na > 0) __builtin_amdgcn_sched_group_barrier(kClassA, na, 0);
    if constexpr (nb > 0) __builtin_amdgcn_sched_group_barrier(kClassB, nb, 0);
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    if constexpr (kStep + 1 < kMfmas)
      Interleave<kStep + 1, kMfmas, kClassA, kCountA, kClassB, kCountB>::run();
  }
};

// The same for two classes that must keep their order (every instruction of the
// first class ahead of every instruction of the second): the kFirst + kSecond
// instructions are spread evenly over the MFMAs in that order.  Used where LDS
// reads precede direct-to-LDS loads in program order: the compiler cannot tell
// that the two touch different buffers and will not move one across the other,
// so a pipeline that alternates the classes cannot be satisfied and is dropped.
template <int kStep, int kMfmas, int kClassFirst, int kFirst, int kClassSecond, int kSecond>
struct Sequenced {
  static __device__ __forceinline__ void run() {
    constexpr int total = kFirst + kSecond;
    constexpr int lo = (kStep * total) / kMfmas, hi = ((kStep + 1) * total) / kMfmas;  // items [lo, hi) go here
    constexpr int nf = (hi < kFirst ? hi : kFirst) - (lo < kFirst ? lo : kFirst);
    constexpr int ns = (hi - lo) - nf;
    if constexpr (nf > 0) __builtin_amdgcn_sched_group_barrier(kClassFirst, nf, 0);
    if constexpr (ns > 0) __builtin_amdgcn_sched_group_barrier(kClassSecond, ns, 0);
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    if constexpr (kStep + 1 < kMfmas)
      Sequenced<kStep + 1, kMfmas, kClassFirst, kFirst, kClassSecond, kSecond>::run();
  }
};

// ---- the kernel -----------------------------------------------------------------
// MS: the MFMA shape, 32 (v_mfma_f32_32x32x16) or 16 (v_mfma_f32_16x16x32; GEMM on pipeline 2 only).
template <int DT, int BM, int BN, int BK, int WM, int WN, int NS, int PIPE, int MS, bool CONV, bool B_NCONTIG>
__global__ void __launch_bounds__(WM *WN * 64) contraction_kernel(const ContractionArgs args) {
  static_assert(MS == 32 || (MS == 16 && PIPE == 2 && !CONV && BK % 32 == 0), "the 16x16x32 form exists for a GEMM on pipeline 2");
  constexpr int NT = WM * WN * 64;
  constexpr int CH = BK / 8;       // 16-byte pieces per tile row
  constexpr int ROW_BYTES = BK * 2;
  constexpr int RP = (256 / ROW_BYTES) > 0 ? (256 / ROW_BYTES) : 1;  // rows per 256 B
  constexpr int TM = BM / WM, TN = BN / WN, FM = TM / 32, FN = TN / 32;
  constexpr int A_STAGE = BM * ROW_BYTES, B_STAGE = BN * ROW_BYTES;
  constexpr int STAGE = A_STAGE + B_STAGE;
  constexpr int NA = BM * CH / NT;  // A pieces per thread per K tile
  constexpr int NB = BN * CH / NT;  // B pieces per thread per K tile
  static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0, "wave tile must be 32-aligned");
  static_assert((BM * CH) % NT == 0 && (BN * CH) % NT == 0, "pieces must divide over threads");
  static_assert(NT % CH == 0 && BK % 16 == 0, "bad BK");
  static_assert(!B_NCONTIG || (NT % (BN / 8) == 0), "bad BN for N-contiguous B");

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  // Everything the prologue reads from the kernel arguments, asked for HERE in one batch of scalar loads.
  // Left to itself the compiler loads each field where it is first used, behind the branch that needs it:
  // eight or more dependent round trips to the scalar cache's backing memory in front of the first tile
  // request (4.1 k cycles from kernel entry to that request in the 4096^3 launch).
  // (Not in the eight-wave 256x256 kernels: at 256 registers a wave they have none to hold the batch in.)
  constexpr bool BATCH_ARGS = !(WM * WN == 8 && BM * BN >= 256 * 256);
  if constexpr (BATCH_ARGS)
  asm volatile("" ::"s"(args.A), "s"(args.B), "s"(args.M), "s"(args.N), "s"(args.K), "s"(args.lda), "s"(args.ldb),
               "s"(args.a_bytes), "s"(args.b_bytes), "s"(args.grid_m), "s"(args.grid_n), "s"(args.k_split),
               "s"(args.fuse_ws), "s"(args.group_m), "s"(args.tile_list), "s"(args.epi.n_ops));
  if constexpr (CONV && BATCH_ARGS) {
    asm volatile("" ::"s"(args.h_in), "s"(args.w_in), "s"(args.c_in), "s"(args.h_out), "s"(args.w_out), "s"(args.s_sz),
                 "s"(args.stride_h), "s"(args.stride_w), "s"(args.pad_h), "s"(args.pad_w), "s"(args.dil_h), "s"(args.dil_w),
                 "s"(args.hw_m), "s"(args.hw_s), "s"(args.w_m), "s"(args.w_s), "s"(args.sc_m), "s"(args.sc_s),
                 "s"(args.c_m), "s"(args.c_s), "s"(args.phases));
  }

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave % WM, wn = wave / WM;

  const int M = args.M, N = args.N;
  // Split-K: workgroups with blockIdx.y = z multiply the K range [z*k_split, (z+1)*k_split)
  // and write their fp32 partial product to rows z*M.. of C, which is then a workspace that
  // a reduction kernel sums.  kb is added to every K offset below; K is the end of the range.
  int tile_m, tile_n;
  int kb = args.k_split > 0 ? (int)blockIdx.y * args.k_split : 0;
  int K = args.k_split > 0 ? min(args.K, kb + args.k_split) : args.K;
  // (tiles above 128x128 are never split in one launch: their kernels do not carry that code)
  constexpr bool FUSE_OK = BM * BN <= 128 * 128 && MS == 32;
  const bool fused = FUSE_OK && args.k_split > 0 && args.fuse_ws != nullptr;
  if (!FUSE_OK && args.k_split > 0 && args.fuse_ws != nullptr) return;  // (a launch the dispatcher never makes: C is not a workspace)
  long long zrow = args.k_split > 0 && !fused ? (long long)blockIdx.y * M : 0ll;
  if (!CONV && args.tile_list != nullptr) {
    // Tile list (the reference's two-level tile table, src/core/ttg.rs:3-11 and
    // src/emitter/cuda/low_rank.rs:69-76): workgroup p runs record tile_list[p] =
    // {tile row, tile column, first k, end k, role}; tiles without a record are not
    // touched.  tile_slice, if given, names the row block of the fp32 workspace that
    // receives this record's partial product (records that share a tile).
    const unsigned *rec = args.tile_records + 5u * args.tile_list[blockIdx.x];
    tile_m = (int)rec[0];
    tile_n = (int)rec[1];
    kb = (int)rec[2];
    K = min(args.K, (int)rec[3]);
    zrow = args.tile_slice != nullptr ? (long long)args.tile_slice[blockIdx.x] * M : 0ll;
  } else {
    tile_coordinates(args, tile_m, tile_n);
  }
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  // ---- per-thread source coordinates of the pieces this thread moves ----
  const int pc = tid % CH;      // 16-byte column of every A piece of this thread
  const int prow = tid / CH;    // first tile row; piece i is prow + i*(NT/CH)
  constexpr int PR_STEP = NT / CH;
  // PIPE 2 moves tiles with loads that write LDS directly: a wave instruction
  // fills 1024 contiguous bytes, lane l at byte 16*l, so the LDS position of a
  // piece is fixed (row tid/CH + i*PR_STEP, 16-byte column tid%CH) and the
  // swizzle is applied to the GLOBAL column instead.  PR_STEP is a multiple of
  // RP*CH, hence the swizzle term is the same for all pieces of a thread.
  static_assert(PIPE < 2 || PR_STEP % (RP * CH) == 0, "bad shape for direct-to-LDS loads");
  static_assert(PIPE == 3 ? NS >= 3 : NS == 2, "stage count does not fit the pipeline mode");
  const int gpc = PIPE >= 2 ? (pc ^ ((prow / RP) & (CH - 1))) : pc;

  const unsigned short *Ag = (const unsigned short *)args.A;
  const unsigned short *Bg = (const unsigned short *)args.B;
  // all phases of a transposed convolution in one launch: blockIdx.z names the phase
  int pad_h = args.pad_h, pad_w = args.pad_w, o_a = args.o_a, o_b = args.o_b;
  if constexpr (CONV) {
    if (args.phases > 1) {
      const int z = (int)blockIdx.z;
      o_a = z / args.o_sw;
      o_b = z - o_a * args.o_sw;
      // selects, not an index: a run-time index into the kernel arguments can move them to scratch memory
      pad_h = o_a == 0 ? args.phase_pad_h[0] : o_a == 1 ? args.phase_pad_h[1] : o_a == 2 ? args.phase_pad_h[2] : args.phase_pad_h[3];
      pad_w = o_b == 0 ? args.phase_pad_w[0] : o_b == 1 ? args.phase_pad_w[1] : o_b == 2 ? args.phase_pad_w[2] : args.phase_pad_w[3];
      Bg += (long long)z * args.phase_b_stride;
    }
  }

  long long a_off[NA];              // GEMM: element offset of the row start (+ piece column)
  int a_hb[CONV ? NA : 1], a_wb[CONV ? NA : 1];  // conv: ho*stride-pad, wo*stride-pad
#pragma unroll
  for (int i = 0; i < NA; ++i) {
    int m = m0 + prow + i * PR_STEP;
    m = m < M ? m : M - 1;
    if constexpr (CONV) {
      int bn, rem, ho, wo;
      fast_divmod(m, args.hw_m, args.hw_s, args.h_out * args.w_out, bn, rem);
      fast_divmod(rem, args.w_m, args.w_s, args.w_out, ho, wo);
      a_off[i] = (long long)bn * args.h_in * args.w_in * args.c_in;
      a_hb[i] = ho * args.stride_h - pad_h;
      a_wb[i] = wo * args.stride_w - pad_w;
    } else {
      a_off[i] = (long long)m * args.lda;
    }
  }

  long long b_off[NB];
  if constexpr (!B_NCONTIG) {
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      int n = n0 + prow + i * PR_STEP;
      n = n < N ? n : N - 1;
      b_off[i] = (long long)n * args.ldb;
    }
  }
  // N-contiguous B: piece q covers k row q / (BN/8), channels (q % (BN/8))*8..+7
  constexpr int NCH = BN / 8;

  // B tile of the direct-to-LDS N-contiguous path: row pitch and pieces per k row.  One
  // transposing read (below) takes 64 B from each of 4 consecutive k rows per half-wave; the
  // 16-byte column is XORed with a function of the row so that those four land in the four
  // different 64-byte bank groups.
  constexpr int NB_ROWB = BN * 2, NB_CH = BN / 8;
  // (16x16x32: the two 16-lane groups of a half-wave read k rows 8 apart at the same channels; the second
  // XOR moves one of them to the other 32 bytes of the bank group)
  auto nb_swz = [](int krow) -> int {
    return (NB_ROWB >= 256 ? ((krow & 3) << 2) : (((krow >> 1) & 1) << 2)) ^ (MS == 16 ? ((krow >> 3) & 1) << 1 : 0);
  };

  u32x4 ra[NA], rb[NB];

  // The chain as the epilogue needs it, and the choice of its row body, are worked
  // out here: their scalar loads complete under the main loop instead of after it.
  // (On the specialised path the output type is the operand type or fp32.)
  const ChainPlan plan = chain_plan(args.epi);
  // (fp32 output takes it only where a wave holds at most 8 accumulator blocks: with 16,
  // a second copy of the row body costs the compiler its register allocation.)
  constexpr bool F32_SIMPLE = FM * FN <= 8;
  const bool out_f32 = F32_SIMPLE && args.out_dtype == DT_F32;
  const bool simple = chain_is_simple(plan, args, n0, BN) && (args.out_dtype == DT || out_f32);

  // This thread's entries of the epilogue operand table (see chain_table_value):
  // requested here so that they arrive under the main loop.
  constexpr int TAB_ENTRIES = TRACEA_MAX_EPILOGUE_OPS * 2 * BN;
  constexpr int TPT = (TAB_ENTRIES + NT - 1) / NT;
  // (An empty chain branches round all of it: the entries are some 1600 instructions with scalar loads
  // between them, 4000 cycles in front of the first tile request of a launch that needs none of them.)
  // (The convolutions with direct-to-LDS tile loads work the entries out behind the first tile requests instead of
  // in front of them: the requests need nothing of this, and their round trip to memory covers it.  Not the GEMMs:
  // with the code in that place the 256x256 kernel of the 4096^3 product took 125 us instead of 101, empty chain
  // and all.)
  float tabr[TPT];
#pragma unroll
  for (int i = 0; i < TPT; ++i) tabr[i] = 0.0f;
#define TRACEA_REQUEST_TABLE()                                                                                                  \
  if (plan.n_ops > 0) {                                                                                                         \
    _Pragma("unroll") for (int i = 0; i < TPT; ++i) {                                                                           \
      const int idx = tid + i * NT;                                                                                             \
      tabr[i] = idx < TAB_ENTRIES ? chain_table_value(args.epi, idx / (2 * BN), (idx / BN) & 1, n0 + idx % BN, N) : 0.0f;       \
    }                                                                                                                           \
  }
  if constexpr (PIPE != 2 || !CONV) {
    TRACEA_REQUEST_TABLE()
  }

  // Every load is issued unconditionally from an address that is always
  // inside the tensor (the real one, or the tensor base when the piece lies in
  // padding or beyond K); pieces that must read as zero are recorded in a bit
  // mask and cleared only when the registers are written to LDS, after the
  // MFMAs of the current K tile.  No branch and no use of the loaded value
  // separates the loads from those MFMAs, so their latency is hidden.
  const u32x4 zero4 = {0u, 0u, 0u, 0u};
  unsigned a_ok = 0, b_ok = 0;  // bit i: piece i holds real data
  auto fetch = [&](int k0) {
    k0 += kb;
    const int kg = k0 + gpc * 8;
    const bool kvalid = kg < K;
    const int k0c = kvalid ? kg : 0;  // column of this thread's piece, or a safe one
    a_ok = 0;
    b_ok = 0;
    if constexpr (CONV) {
      int rf, rem, sf, ci;
      fast_divmod(kg, args.sc_m, args.sc_s, args.s_sz * args.c_in, rf, rem);
      fast_divmod(rem, args.c_m, args.c_s, args.c_in, sf, ci);
      const int dh = rf * args.dil_h, dw = sf * args.dil_w;
#pragma unroll
      for (int i = 0; i < NA; ++i) {
        const int hi = a_hb[i] + dh, wi = a_wb[i] + dw;
        // (unsigned compares and bitwise &: no short-circuit control flow around the address)
        const bool ok = kvalid & ((unsigned)hi < (unsigned)args.h_in) & ((unsigned)wi < (unsigned)args.w_in);
        const long long off = a_off[i] + ((long long)hi * args.w_in + wi) * args.c_in + ci;
        ra[i] = *(const u32x4 *)(Ag + (ok ? off : 0ll));
        a_ok |= ok ? (1u << i) : 0u;
      }
    } else {
#pragma unroll
      for (int i = 0; i < NA; ++i) ra[i] = *(const u32x4 *)(Ag + a_off[i] + k0c);
      a_ok = kvalid ? 0xffffffffu : 0u;
    }
    if constexpr (!B_NCONTIG) {
#pragma unroll
      for (int i = 0; i < NB; ++i) rb[i] = *(const u32x4 *)(Bg + b_off[i] + k0c);
      b_ok = kvalid ? 0xffffffffu : 0u;
    } else {
#pragma unroll
      for (int i = 0; i < NB; ++i) {
        const int q = tid + i * NT;
        const int kk = q / NCH, nch = q % NCH;
        const int n = n0 + nch * 8;
        const bool ok = k0 + kk < K && n < N;
        rb[i] = *(const u32x4 *)(Bg + (ok ? (long long)(k0 + kk) * args.ldb + n : 0ll));
        b_ok |= ok ? (1u << i) : 0u;
      }
    }
  };

  // Direct-to-LDS tile load (PIPE >= 2) through buffer addressing: the address
  // of a piece is (buffer base) + (per-lane 32-bit byte offset) + (scalar byte
  // offset of the K tile).  For a GEMM the per-lane offsets never change, so a
  // request costs one M0 update and one instruction, no vector ALU work.  A
  // per-lane offset at or beyond the buffer size makes the hardware return
  // zeros: pieces that must read as zero (padding, columns of K beyond the end)
  // get the offset 0x80000000 (the dispatcher only selects these variants for
  // operands smaller than 2 GiB).
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  constexpr unsigned OOB = 0x80000000u;
  __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
      (void *)args.A, 0, (int)args.a_bytes, 0x00020000);
  __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(
      (void *)Bg, 0, (int)args.b_bytes, 0x00020000);
  unsigned a_voff[NA], b_voff[NB];
  if constexpr (PIPE >= 2) {
#pragma unroll
    for (int i = 0; i < NA; ++i)
      a_voff[i] = CONV ? (unsigned)(a_off[i] * 2) : (unsigned)((a_off[i] + gpc * 8) * 2);
    if constexpr (!B_NCONTIG) {
#pragma unroll
      for (int i = 0; i < NB; ++i) b_voff[i] = (unsigned)((b_off[i] + gpc * 8) * 2);
    } else {
      // N-contiguous B: the tile stays as it lies in memory, BK rows of BN channels.  Piece q
      // of the tile (LDS byte 16q) is k row q / NB_CH, 16-byte column q % NB_CH, and holds
      // the channels of global column (q % NB_CH) ^ nb_swz(row) (see nb_swz below).
#pragma unroll
      for (int i = 0; i < NB; ++i) {
        const int q = tid + i * NT;
        const int krow = q / NB_CH;
        const int n = n0 + (((q % NB_CH) ^ nb_swz(krow)) << 3);
        b_voff[i] = n < N ? (unsigned)(((long long)krow * args.ldb + n) * 2) : OOB;
      }
    }
  }
  // Only pieces lo <= index < hi of the thread's list (A pieces first, then B)
  // are requested, so that the requests of one tile can be spread over several
  // k-steps.
  auto dma = [&](unsigned char *sA, unsigned char *sB, int k0, int lo, int hi) {
    constexpr int RPI = 64 / CH;  // tile rows one wave instruction covers
    k0 += kb;
    const int kg = k0 + gpc * 8;
    const bool kvalid = kg < K;
    int dh = 0, dw = 0, ci = 0;
    if constexpr (CONV) {
      int rf, rem, sf;
      fast_divmod(kg, args.sc_m, args.sc_s, args.s_sz * args.c_in, rf, rem);
      fast_divmod(rem, args.c_m, args.c_s, args.c_in, sf, ci);
      dh = rf * args.dil_h;
      dw = sf * args.dil_w;
    }
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      if (i < lo || i >= hi) continue;
      unsigned voff;
      int soff;
      if constexpr (CONV) {
        const int hi_ = a_hb[i] + dh, wi = a_wb[i] + dw;
        // The offset is formed unconditionally and selected afterwards, with unsigned compares
        // joined by bitwise &: written with && and inside the conditional, each piece became a
        // predicated block of its own and the post-barrier share of the requests a chain of
        // branches that no MFMA could be scheduled into.
        const bool ok = kvalid & ((unsigned)hi_ < (unsigned)args.h_in) & ((unsigned)wi < (unsigned)args.w_in);
        const unsigned in_range = a_voff[i] + (unsigned)(((hi_ * args.w_in + wi) * args.c_in + ci) * 2);
        voff = ok ? in_range : OOB;
        soff = 0;
      } else {
        voff = kvalid ? a_voff[i] : OOB;
        soff = k0 * 2;
      }
      unsigned char *dst = sA + (i * PR_STEP + wave_u * RPI) * ROW_BYTES;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (__attribute__((address_space(3))) void *)dst, 16,
                                               (int)voff, soff, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      if (NA + i < lo || NA + i >= hi) continue;
      unsigned char *dst = sB + (i * PR_STEP + wave_u * RPI) * ROW_BYTES;
      if constexpr (!B_NCONTIG) {
        const unsigned voff = kvalid ? b_voff[i] : OOB;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (__attribute__((address_space(3))) void *)dst, 16,
                                                 (int)voff, k0 * 2, 0, 0);
      } else {
        // rows at or beyond K must read as zero; the scalar offset takes no part in the
        // hardware's range check, so the row is tested here
        const unsigned voff = k0 + (tid + i * NT) / NB_CH < K ? b_voff[i] : OOB;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (__attribute__((address_space(3))) void *)dst, 16,
                                                 (int)voff, (int)((long long)k0 * args.ldb * 2), 0, 0);
      }
    }
  };

  // Operand fetch from the [k][n] tile: ds_read_b64_tr_b16 hands lane i of a 16-lane group
  // column i of a 4-row x 16-column block, i.e. 4 consecutive k of one channel; lane r of
  // the group supplies the address of row r/4, columns 4*(r%4).  Lanes 0-31 take k 0-7 of
  // the 16-wide k-step, lanes 32-63 k 8-15, in two reads of 4 rows each, which is the
  // operand layout of the K-contiguous path.
  int tr_off[B_NCONTIG && PIPE >= 2 ? FN : 1];
  if constexpr (B_NCONTIG && PIPE >= 2) {
    const int r = lane & 15;
    const int row = (lane >> 5) * 8 + (r >> 2);
#pragma unroll
    for (int j = 0; j < FN; ++j) {
      const int col = wn * TN + j * 32 + ((lane >> 4) & 1) * 16 + (r & 3) * 4;
      tr_off[j] = row * NB_ROWB + (((col >> 3) ^ nb_swz(row)) << 4) + (col & 7) * 2;
    }
  }
  auto read_b_tr = [&](const unsigned char *sB, int j, int ks) -> u32x4 {
    const unsigned char *p = sB + tr_off[j] + ks * 16 * NB_ROWB;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)p);
    const s16x4 hi =
        __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)(p + 4 * NB_ROWB));
    const u32x2 lo2 = __builtin_bit_cast(u32x2, lo), hi2 = __builtin_bit_cast(u32x2, hi);
    u32x4 v;
    v[0] = lo2[0]; v[1] = lo2[1]; v[2] = hi2[0]; v[3] = hi2[1];
    return v;
  };

  // The same for the 16x16x32 operand (16 channels by 32 k): 16-lane group g takes k 8g .. 8g+7 of the
  // 32-wide k-step for the block's 16 channels.
  int tr_off16[B_NCONTIG && MS == 16 ? 2 * FN : 1];
  if constexpr (B_NCONTIG && MS == 16) {
    const int r = lane & 15;
    const int row = (lane >> 4) * 8 + (r >> 2);
#pragma unroll
    for (int j = 0; j < 2 * FN; ++j) {
      const int col = wn * TN + j * 16 + (r & 3) * 4;
      tr_off16[j] = row * NB_ROWB + (((col >> 3) ^ nb_swz(row)) << 4) + (col & 7) * 2;
    }
  }
  // The two transposing reads are written as instructions.  Through the builtin the compiler puts a
  // vmcnt(0) in front of every one of them that follows a direct-to-LDS tile request (it cannot tell that the
  // request writes the other stage), and the k-step behind the barrier, where requests and reads alternate,
  // took 5600 cycles instead of 1200.  As instructions they are outside its bookkeeping altogether: the
  // fragments are complete only after wait_b_tr below, which the MFMAs depend on through its operands.
  // (The hardware counts them like any LDS read, so the full LDS wait the compiler places in front of a
  // barrier covers them too.)
  auto read_b_tr16 = [&](const unsigned char *sB, int j, int ks) -> u32x4 {
    const unsigned addr = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)(sB + tr_off16[j] + ks * 32 * NB_ROWB);
    u32x2 lo2, hi2;
    asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(lo2) : "v"(addr) : "memory");
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(hi2) : "v"(addr), "i"(4 * NB_ROWB) : "memory");
    u32x4 v;
    v[0] = lo2[0]; v[1] = lo2[1]; v[2] = hi2[0]; v[3] = hi2[1];
    return v;
  };
  constexpr int TR_FRAGS = (MS == 16 ? 2 : 1) * FN;  // B fragments of a k-step
  auto wait_b_tr = [&](u32x4 (&f)[TR_FRAGS]) __attribute__((always_inline)) {
    static_assert(TR_FRAGS == 1 || TR_FRAGS == 2 || TR_FRAGS == 4 || TR_FRAGS == 8, "fragments of a k-step");
    if constexpr (TR_FRAGS == 1)
      asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(f[0]));
    else if constexpr (TR_FRAGS == 2)
      asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(f[0]), "+v"(f[1]));
    else if constexpr (TR_FRAGS == 4)
      asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3]));
    else
      asm volatile("s_waitcnt lgkmcnt(0)"
                   : "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3]), "+v"(f[4]), "+v"(f[5]), "+v"(f[6]), "+v"(f[7]));
  };
  // (the same for the 32x32x16 fragments of the direct-to-LDS loop)
  auto read_b_tr_asm = [&](const unsigned char *sB, int j, int ks) -> u32x4 {
    const unsigned addr = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)(sB + tr_off[j] + ks * 16 * NB_ROWB);
    u32x2 lo2, hi2;
    asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(lo2) : "v"(addr) : "memory");
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(hi2) : "v"(addr), "i"(4 * NB_ROWB) : "memory");
    u32x4 v;
    v[0] = lo2[0]; v[1] = lo2[1]; v[2] = hi2[0]; v[3] = hi2[1];
    return v;
  };

  auto lds_piece = [&](int row, int c) -> int {
    return row * ROW_BYTES + ((c ^ ((row / RP) & (CH - 1))) << 4);
  };

  // Zero-masking of pieces is needed for a convolution (padding, K tail of
  // R*S*C) and for a GEMM whose last K tile is partial.  The pipelined loop must
  // stay free of branches (its instruction interleaving is per basic block), so
  // there the decision is made at compile time: always for a convolution, never
  // for a GEMM, and the dispatcher only picks a pipelined GEMM variant when K is
  // a multiple of BK.
  const bool mask_rt = ((K - kb) % BK) != 0;
  auto stash = [&](unsigned char *sA, unsigned char *sB) {
    const bool mask_a = PIPE != 0 ? CONV : (CONV || mask_rt);
    const bool mask_b = PIPE != 0 ? CONV : (CONV || mask_rt);
    if (mask_a) {
#pragma unroll
      for (int i = 0; i < NA; ++i)
        *(u32x4 *)(sA + lds_piece(prow + i * PR_STEP, pc)) = ((a_ok >> i) & 1u) ? ra[i] : zero4;
    } else {
#pragma unroll
      for (int i = 0; i < NA; ++i) *(u32x4 *)(sA + lds_piece(prow + i * PR_STEP, pc)) = ra[i];
    }
    if constexpr (!B_NCONTIG) {
      if (mask_b) {
#pragma unroll
        for (int i = 0; i < NB; ++i)
          *(u32x4 *)(sB + lds_piece(prow + i * PR_STEP, pc)) = ((b_ok >> i) & 1u) ? rb[i] : zero4;
      } else {
#pragma unroll
        for (int i = 0; i < NB; ++i) *(u32x4 *)(sB + lds_piece(prow + i * PR_STEP, pc)) = rb[i];
      }
    } else {
#pragma unroll
      for (int i = 0; i < NB; ++i) {
        const int q = tid + i * NT;
        const int kk = q / NCH, nch = q % NCH;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int row = nch * 8 + e;
          const unsigned w = ((b_ok >> i) & 1u) ? rb[i][e >> 1] : 0u;
          const unsigned short h = (e & 1) ? (unsigned short)(w >> 16) : (unsigned short)(w & 0xffffu);
          *(unsigned short *)(sB + lds_piece(row, kk >> 3) + (kk & 7) * 2) = h;
        }
      }
    }
  };

  f32x16 acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;
  // (MS == 16: 16x16 blocks, block (i, j) = rows 16 i .., channels 16 j .. of the wave tile; the other set is unused)
  f32x4 acc16[MS == 16 ? 2 * FM : 1][MS == 16 ? 2 * FN : 1];
#pragma unroll
  for (int i = 0; i < (MS == 16 ? 2 * FM : 1); ++i)
#pragma unroll
    for (int j = 0; j < (MS == 16 ? 2 * FN : 1); ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc16[i][j][e] = 0.0f;

  const int lrow = lane & 31;
  const int lhalf = lane >> 5;
  const int lswz = (lrow / RP) & (CH - 1);  // wave tiles start on multiples of 32 rows

  auto multiply = [&](const unsigned char *sA, const unsigned char *sB) {
    const unsigned char *pa = sA + (wm * TM + lrow) * ROW_BYTES;
    const unsigned char *pb = sB + (wn * TN + lrow) * ROW_BYTES;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      const int coff = ((ks * 2 + lhalf) ^ lswz) << 4;
      u32x4 af[FM], bf[FN];
#pragma unroll
      for (int i = 0; i < FM; ++i) af[i] = *(const u32x4 *)(pa + i * 32 * ROW_BYTES + coff);
#pragma unroll
      for (int j = 0; j < FN; ++j) bf[j] = *(const u32x4 *)(pb + j * 32 * ROW_BYTES + coff);
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) acc[i][j] = Mfma32<DT>::run(bf[j], af[i], acc[i][j]);
    }
  };

  // ---- main loop: two LDS stages ----
  static_assert(NA <= 32 && NB <= 32, "piece masks are 32 bits");
  const int nk = (K - kb + BK - 1) / BK;
  if constexpr (PIPE < 2) {
    fetch(0);
    stash(smem, smem + A_STAGE);
    __syncthreads();
  }
  if constexpr (PIPE == 0) {
    // Plain form: operands are read from LDS just before the MFMAs that use them.
    for (int kt = 0; kt + 1 < nk; ++kt) {
      unsigned char *cur = smem + (kt & 1) * STAGE;
      unsigned char *nxt = smem + ((kt + 1) & 1) * STAGE;
      // The scheduling fences keep the compiler from sinking the global loads
      // below the MFMAs (towards their first use in stash), which would expose
      // the whole memory latency once per K tile.
      fetch((kt + 1) * BK);
      __builtin_amdgcn_sched_barrier(0);
      multiply(cur, cur + A_STAGE);
      __builtin_amdgcn_sched_barrier(0);
      stash(nxt, nxt + A_STAGE);
      __syncthreads();
    }
    {
      const unsigned char *cur = smem + ((nk - 1) & 1) * STAGE;
      multiply(cur, cur + A_STAGE);
    }
  } else if constexpr (PIPE == 1) {
    // Software-pipelined form.  The operands of k-step s+1 are read from LDS
    // while the MFMAs of k-step s run; the last k-step of a tile runs AFTER the
    // barrier that publishes the next tile, overlapped with the reads of that
    // tile's first operands, so the matrix pipe does not drain at the barrier.
    // Global loads run a whole tile ahead: they are issued right after the
    // barrier (when the staging registers have just been written to LDS) and
    // consumed by the LDS writes spread over the last k-step before the next
    // barrier.
    constexpr int KS = BK / 16;
    static_assert(KS >= 4 && KS % 2 == 0, "pipelined loop needs an even number (>= 4) of k-steps");
    constexpr int R = FM * FN, D = FM + FN, L = NA + NB;
    u32x4 fa[2][FM], fb[2][FN];
    auto read_operands = [&](int set, const unsigned char *sA, const unsigned char *sB, int ks) {
      const unsigned char *pa = sA + (wm * TM + lrow) * ROW_BYTES;
      const unsigned char *pb = sB + (wn * TN + lrow) * ROW_BYTES;
      const int coff = ((ks * 2 + lhalf) ^ lswz) << 4;
#pragma unroll
      for (int i = 0; i < FM; ++i) fa[set][i] = *(const u32x4 *)(pa + i * 32 * ROW_BYTES + coff);
#pragma unroll
      for (int j = 0; j < FN; ++j) fb[set][j] = *(const u32x4 *)(pb + j * 32 * ROW_BYTES + coff);
    };
    auto mma = [&](int set) {
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) acc[i][j] = Mfma32<DT>::run(fb[set][j], fa[set][i], acc[i][j]);
    };
    read_operands(0, smem, smem + A_STAGE, 0);
    if (nk > 1) fetch(BK);  // tile 1 travels while tile 0 is multiplied
    for (int kt = 0; kt + 1 < nk; ++kt) {
      unsigned char *cur = smem + (kt & 1) * STAGE;
      unsigned char *nxt = smem + ((kt + 1) & 1) * STAGE;
#pragma unroll
      for (int ks = 0; ks + 2 < KS; ++ks) {
        read_operands((ks + 1) & 1, cur, cur + A_STAGE, ks + 1);
        mma(ks & 1);
        Interleave<0, R, 0x100, D, 0x100, 0>::run();
        __builtin_amdgcn_sched_barrier(0);
      }
      // k-step KS-2: operand reads of the last k-step, and the LDS writes that
      // stage the next tile (its global loads were issued a whole tile earlier)
      read_operands((KS - 1) & 1, cur, cur + A_STAGE, KS - 1);
      stash(nxt, nxt + A_STAGE);
      mma((KS - 2) & 1);
      Interleave<0, R, 0x100, D, 0x200, (B_NCONTIG ? NA : L)>::run();
      __builtin_amdgcn_sched_barrier(0);
      __syncthreads();
      // k-step KS-1, after the barrier: first operand reads of the tile just
      // published and the global loads of the tile after it (the staging
      // registers are free again); clamped to the last tile, whose reload is
      // never written to LDS
      fetch((kt + 2 < nk ? kt + 2 : nk - 1) * BK);
      read_operands(0, nxt, nxt + A_STAGE, 0);
      mma((KS - 1) & 1);
      Interleave<0, R, 0x020, L, 0x100, D>::run();
      __builtin_amdgcn_sched_barrier(0);
    }
    {
      const unsigned char *cur = smem + ((nk - 1) & 1) * STAGE;
#pragma unroll
      for (int ks = 0; ks + 1 < KS; ++ks) {
        read_operands((ks + 1) & 1, cur, cur + A_STAGE, ks + 1);
        mma(ks & 1);
        Interleave<0, R, 0x100, D, 0x100, 0>::run();
        __builtin_amdgcn_sched_barrier(0);
      }
      mma((KS - 1) & 1);
    }
  } else if constexpr (PIPE == 2) {
    // Software-pipelined form with direct-to-LDS loads: no staging registers and
    // no LDS write instructions.  A tile is requested right after the barrier
    // that frees its buffer, a whole tile of MFMAs before the barrier that
    // publishes it; the only wait on global memory is the one in front of that
    // barrier.
    // A k-step is one MFMA deep: 16 k with 32-row fragments, 32 k with the 16-row fragments of the
    // 16x16x32 shape (XF fragments per 32 rows; same bytes per fragment, same bytes per K tile).
    constexpr int KSTEP = MS == 16 ? 32 : 16, XF = MS == 16 ? 2 : 1;
    constexpr int KS = BK / KSTEP;
    static_assert(KS >= 2 && KS % 2 == 0, "pipelined loop needs an even number of k-steps");
    constexpr int R = XF * FM * XF * FN, D = XF * FM + (B_NCONTIG ? 2 * XF * FN : XF * FN), L = NA + NB;
    u32x4 fa[2][XF * FM], fb[2][XF * FN];
    // (16-row fragments: row lane & 15, 16-byte piece 4 ks + (lane >> 4); the piece swizzle has a period
    // of 16 rows, so every fragment of the wave sees the same one)
    const int row16 = lane & 15, q16 = lane >> 4;
    const int swz16 = (row16 / RP) & (CH - 1);
    auto read_operands = [&](int set, const unsigned char *sA, const unsigned char *sB, int ks) {
      if constexpr (MS == 16) {
        static_assert(16 % (RP * CH) == 0, "the piece swizzle must repeat every 16 rows");
        const unsigned char *pa = sA + (wm * TM + row16) * ROW_BYTES;
        const unsigned char *pb = sB + (wn * TN + row16) * ROW_BYTES;
        const int coff = ((ks * 4 + q16) ^ swz16) << 4;
#pragma unroll
        for (int i = 0; i < 2 * FM; ++i) fa[set][i] = *(const u32x4 *)(pa + i * 16 * ROW_BYTES + coff);
#pragma unroll
        for (int j = 0; j < 2 * FN; ++j) {
          if constexpr (B_NCONTIG) fb[set][j] = read_b_tr16(sB, j, ks);
          else fb[set][j] = *(const u32x4 *)(pb + j * 16 * ROW_BYTES + coff);
        }
      } else {
        const unsigned char *pa = sA + (wm * TM + lrow) * ROW_BYTES;
        const unsigned char *pb = sB + (wn * TN + lrow) * ROW_BYTES;
        const int coff = ((ks * 2 + lhalf) ^ lswz) << 4;
#pragma unroll
        for (int i = 0; i < FM; ++i) fa[set][i] = *(const u32x4 *)(pa + i * 32 * ROW_BYTES + coff);
#pragma unroll
        for (int j = 0; j < FN; ++j) {
          if constexpr (B_NCONTIG) fb[set][j] = read_b_tr_asm(sB, j, ks);
          else fb[set][j] = *(const u32x4 *)(pb + j * 32 * ROW_BYTES + coff);
        }
      }
    };
    // (16x16x32) fragment u of the k-step: A fragments first, then B
    auto read_one = [&](int set, const unsigned char *sA, const unsigned char *sB, int ks, int u) {
      const int coff = ((ks * 4 + q16) ^ swz16) << 4;
      if (u < 2 * FM) {
        fa[set][u] = *(const u32x4 *)(sA + (wm * TM + row16) * ROW_BYTES + u * 16 * ROW_BYTES + coff);
      } else {
        const int j = u - 2 * FM;
        if constexpr (B_NCONTIG) fb[set][j] = read_b_tr16(sB, j, ks);
        else fb[set][j] = *(const u32x4 *)(sB + (wn * TN + row16) * ROW_BYTES + j * 16 * ROW_BYTES + coff);
      }
    };
    // requests [lo, hi) of a tile and the operand reads of a k-step in alternation, in program order
    auto mixed = [&](unsigned char *dA, unsigned char *dB, int k0, int lo, int hi, int set, const unsigned char *sA,
                     const unsigned char *sB, int ks) {
      constexpr int NR = XF * FM + XF * FN;
#pragma unroll
      for (int u = 0; u < NR; ++u) {
        const int p0 = lo + (u * (hi - lo)) / NR, p1 = lo + ((u + 1) * (hi - lo)) / NR;
        if (p1 > p0) dma(dA, dB, k0, p0, p1);
        read_one(set, sA, sB, ks, u);
      }
    };
    auto mma = [&](int set) {
      if constexpr (B_NCONTIG) wait_b_tr(fb[set]);
      if constexpr (MS == 16) {
#pragma unroll
        for (int i = 0; i < 2 * FM; ++i)
#pragma unroll
          for (int j = 0; j < 2 * FN; ++j) acc16[i][j] = Mfma16<DT>::run(fb[set][j], fa[set][i], acc16[i][j]);
      } else {
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
          for (int j = 0; j < FN; ++j) acc[i][j] = Mfma32<DT>::run(fb[set][j], fa[set][i], acc[i][j]);
      }
    };
    // The L requests of a tile are issued in SPREAD consecutive k-step regions,
    // the first of which is the one right after the barrier that freed the
    // destination buffer; the rest follow at the start of the next tile.
    constexpr int SPREAD = 2;  // three shares measured no better than two, one share worse
    // With the 16x16x32 shape a tile has two k-steps, one on either side of the barrier, and the share
    // requested in front of the barrier has only that one k-step to arrive in: three quarters go out behind
    // the barrier, and in both k-steps the requests are issued ahead of the operand reads.  Measured at
    // 4096^3 on four waves (same box): shares of 8/10/12/14/16 of 16 requests behind the barrier 123 / 107.7 /
    // 108.5 / 127 / 119 us; reads first, halves: 113-116 us.  (With the alternation behind the barrier the
    // shares from 10 to 16 are within a percent of each other.)
    constexpr bool DMA_FIRST = MS == 16;
    constexpr int CUT1 = MS == 16 ? (L * 3) / 4 : L / SPREAD, CUT2 = SPREAD == 3 ? 2 * L / SPREAD : L;
    dma(smem, smem + A_STAGE, 0, 0, L);
    dma(smem + STAGE, smem + STAGE + A_STAGE, nk > 1 ? BK : 0, 0, CUT1);  // first share of tile 1
    if constexpr (CONV) {
      TRACEA_REQUEST_TABLE()
    }
#undef TRACEA_REQUEST_TABLE
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's share of tile 0 is in LDS
    __syncthreads();
    read_operands(0, smem, smem + A_STAGE, 0);
    for (int kt = 0; kt + 1 < nk; ++kt) {
      unsigned char *cur = smem + (kt & 1) * STAGE;
      unsigned char *nxt = smem + ((kt + 1) & 1) * STAGE;
      // k-step 0 carries the second share of tile kt+1 (its first share was
      // requested right after the previous barrier, or in the prologue)
      if constexpr (DMA_FIRST) {
        dma(nxt, nxt + A_STAGE, (kt + 1) * BK, CUT1, CUT2);
        read_operands(1, cur, cur + A_STAGE, 1);
        mma(0);
        Sequenced<0, R, 0x020, CUT2 - CUT1, 0x100, D>::run();
      } else {
        read_operands(1, cur, cur + A_STAGE, 1);
        dma(nxt, nxt + A_STAGE, (kt + 1) * BK, CUT1, CUT2);
        mma(0);
        Sequenced<0, R, 0x100, D, 0x020, CUT2 - CUT1>::run();
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ks = 1; ks + 1 < KS; ++ks) {
        if (ks == 1) dma(nxt, nxt + A_STAGE, (kt + 1) * BK, CUT2, L);  // third share, if any
        read_operands((ks + 1) & 1, cur, cur + A_STAGE, ks + 1);
        mma(ks & 1);
        if (ks == 1) Interleave<0, R, 0x020, L - CUT2, 0x100, D>::run();
        else Interleave<0, R, 0x100, D, 0x100, 0>::run();
        __builtin_amdgcn_sched_barrier(0);
      }
      // vmcnt(0): tile kt+1 has landed.  (With an N-contiguous B also lgkmcnt(0): the transposing reads of `cur`
      // issued in front of this barrier are instructions the compiler does not count, and they must have
      // executed before another wave's requests may overwrite `cur`.)
      __builtin_amdgcn_s_waitcnt(B_NCONTIG ? 0x0070 : 0x0f70);
      __syncthreads();
      // every wave has finished reading `cur`: request the first share of tile
      // kt+2 into it (clamped to the last tile, whose second copy is never read)
      // while the last k-step of tile kt runs from registers
      if constexpr (DMA_FIRST) {
        // (behind the barrier requests and operand reads alternate, one group of either kind per MFMA slot:
        // a block of twelve requests in front of the reads held the MFMAs up, 105.8-106.2 against 103.8-104.7 us;
        // in front of the barrier the same alternation delays the requests and costs 5 %)
        mixed(cur, cur + A_STAGE, (kt + 2 < nk ? kt + 2 : nk - 1) * BK, 0, CUT1, 0, nxt, nxt + A_STAGE, 0);
        mma((KS - 1) & 1);
        Interleave<0, R, 0x120, CUT1 + D, 0x100, 0>::run();
      } else {
        read_operands(0, nxt, nxt + A_STAGE, 0);
        dma(cur, cur + A_STAGE, (kt + 2 < nk ? kt + 2 : nk - 1) * BK, 0, CUT1);
        mma((KS - 1) & 1);
        Sequenced<0, R, 0x100, D, 0x020, CUT1>::run();
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    {
      const unsigned char *cur = smem + ((nk - 1) & 1) * STAGE;
#pragma unroll
      for (int ks = 0; ks + 1 < KS; ++ks) {
        read_operands((ks + 1) & 1, cur, cur + A_STAGE, ks + 1);
        mma(ks & 1);
        Interleave<0, R, 0x100, D, 0x100, 0>::run();
        __builtin_amdgcn_sched_barrier(0);
      }
      mma((KS - 1) & 1);
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);  // the clamped reload must not land on the epilogue staging
  } else {
    // Ring of NS >= 3 LDS stages filled by direct-to-LDS loads.  Global-memory
    // latency on this part is of the order of a whole K tile of a 256x256x64
    // block and of several tiles of a smaller one, so one tile of look-ahead
    // cannot hide it: here tile t+NS-1 is requested while tile t is multiplied
    // (its buffer held tile t-1 and was released by the previous barrier), and
    // waited for NS-2 barriers later.  The requests of a tile are spread evenly
    // over the k-steps of the tile that overlaps them.
    constexpr int KS = BK / 16;
    static_assert(KS >= 2 && KS % 2 == 0, "pipelined loop needs an even number of k-steps");
    constexpr int R = FM * FN, D = FM + (B_NCONTIG ? 2 * FN : FN), L = NA + NB;
    constexpr int LAST_SHARE = L - ((KS - 1) * L) / KS;          // pieces issued after the barrier
    constexpr int IN_FLIGHT = (NS - 3) * L + (L - LAST_SHARE);   // requests newer than tile t+1 at barrier t
    static_assert(IN_FLIGHT <= 63, "vmcnt is a 6-bit counter");
    constexpr int WAIT_TILE = (IN_FLIGHT & 15) | (7 << 4) | (15 << 8) | ((IN_FLIGHT >> 4) << 14);
    constexpr int PRO_FLIGHT = (NS - 2) * L;                     // prologue: all but tile 0 may be in flight
    static_assert(PRO_FLIGHT <= 63, "vmcnt is a 6-bit counter");
    constexpr int WAIT_PRO = (PRO_FLIGHT & 15) | (7 << 4) | (15 << 8) | ((PRO_FLIGHT >> 4) << 14);
    u32x4 fa[2][FM], fb[2][FN];
    auto read_operands = [&](int set, const unsigned char *sA, const unsigned char *sB, int ks) {
      const unsigned char *pa = sA + (wm * TM + lrow) * ROW_BYTES;
      const unsigned char *pb = sB + (wn * TN + lrow) * ROW_BYTES;
      const int coff = ((ks * 2 + lhalf) ^ lswz) << 4;
#pragma unroll
      for (int i = 0; i < FM; ++i) fa[set][i] = *(const u32x4 *)(pa + i * 32 * ROW_BYTES + coff);
#pragma unroll
      for (int j = 0; j < FN; ++j) {
        if constexpr (B_NCONTIG) fb[set][j] = read_b_tr(sB, j, ks);
        else fb[set][j] = *(const u32x4 *)(pb + j * 32 * ROW_BYTES + coff);
      }
    };
    auto mma = [&](int set) {
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) acc[i][j] = Mfma32<DT>::run(fb[set][j], fa[set][i], acc[i][j]);
    };
#pragma unroll
    for (int st = 0; st < NS - 1; ++st) {
      const int tile = st < nk ? st : nk - 1;
      dma(smem + st * STAGE, smem + st * STAGE + A_STAGE, tile * BK, 0, L);
    }
    __builtin_amdgcn_s_waitcnt(WAIT_PRO);  // this wave's share of tile 0 is in LDS
    __syncthreads();
    read_operands(0, smem, smem + A_STAGE, 0);
    int cur_i = 0;          // stage of tile kt
    int fill_i = NS - 1;    // stage released by the previous barrier, receives tile kt+NS-1
    for (int kt = 0; kt + 1 < nk; ++kt) {
      unsigned char *cur = smem + cur_i * STAGE;
      const int nxt_i = cur_i + 1 == NS ? 0 : cur_i + 1;
      unsigned char *nxt = smem + nxt_i * STAGE;
      unsigned char *fill = smem + fill_i * STAGE;
      const int tile_f = kt + NS - 1 < nk ? kt + NS - 1 : nk - 1;  // clamped: a repeat of the last tile is never read
#pragma unroll
      for (int ks = 0; ks + 1 < KS; ++ks) {
        dma(fill, fill + A_STAGE, tile_f * BK, (ks * L) / KS, ((ks + 1) * L) / KS);
        read_operands((ks + 1) & 1, cur, cur + A_STAGE, ks + 1);
        mma(ks & 1);
        Interleave<0, R, 0x020, L / KS, 0x100, D>::run();
        __builtin_amdgcn_sched_barrier(0);
      }
      __builtin_amdgcn_s_waitcnt(WAIT_TILE);  // tile kt+1 has landed; newer requests stay in flight
      // (the barrier alone: with the fences of __syncthreads() the compiler waits for every request in flight)
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      dma(fill, fill + A_STAGE, tile_f * BK, ((KS - 1) * L) / KS, L);
      read_operands(0, nxt, nxt + A_STAGE, 0);
      mma((KS - 1) & 1);
      Interleave<0, R, 0x020, LAST_SHARE, 0x100, D>::run();
      __builtin_amdgcn_sched_barrier(0);
      fill_i = cur_i;
      cur_i = nxt_i;
    }
    {
      const unsigned char *cur = smem + cur_i * STAGE;
#pragma unroll
      for (int ks = 0; ks + 1 < KS; ++ks) {
        read_operands((ks + 1) & 1, cur, cur + A_STAGE, ks + 1);
        mma(ks & 1);
        Interleave<0, R, 0x100, D, 0x100, 0>::run();
        __builtin_amdgcn_sched_barrier(0);
      }
      mma((KS - 1) & 1);
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);  // clamped repeats must not land on the epilogue staging
  }
  __syncthreads();

  // ---- one-launch split: leave the partial product, take a ticket; the tile's last workgroup sums ----
  // Every wave's accumulators go out as they lie in registers (block (i, j), group g: one 16-byte piece per
  // lane, 1 KB per store instruction) and come back the same way, so the layout needs no name.  The K
  // ranges of a tile may run on different XCDs, whose L2 caches do not see each other's lines.  Device-
  // scope fences would settle that (write the L2 back, invalidate it) but cost more than the second kernel
  // they save: several microseconds each, one after the other on an L2.  Instead the partial products
  // travel with device scope themselves: stores that write through to memory, loads that do not trust a
  // line of another L2, and a device-scope counter.  Order of events: the workgroup's stores are
  // acknowledged (vmcnt(0)), barrier, one thread takes the ticket; whoever draws the last ticket of the
  // tile reads every partial product.  Nobody waits for anybody.  The sum runs over the K ranges in order,
  // this workgroup's own included, whichever of them comes last: the result does not depend on the
  // order of arrival and equals that of the two-launch reduction.
  if constexpr (FUSE_OK) {
    if (fused) {
      __shared__ unsigned s_ticket;
      constexpr int DEVICE_SCOPE = 16;  // the sc1 bit of a buffer instruction
      const unsigned splits = gridDim.y;
      constexpr unsigned TILE_BYTES = BM * BN * 4, WAVE_BYTES = TM * TN * 4;
      __amdgpu_buffer_rsrc_t rsrc_ws = __builtin_amdgcn_make_buffer_rsrc((void *)args.fuse_ws, 0, 0x7fffffff, 0x00020000);
      const unsigned first = blockIdx.x * splits * TILE_BYTES + wave * WAVE_BYTES + lane * 16;
      const unsigned mine = first + blockIdx.y * TILE_BYTES;
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const f32x4 v = {acc[i][j][g * 4 + 0], acc[i][j][g * 4 + 1], acc[i][j][g * 4 + 2], acc[i][j][g * 4 + 3]};
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), rsrc_ws, (int)(mine + ((i * FN + j) * 4 + g) * 1024), 0,
                                                   DEVICE_SCOPE);
          }
      __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
      __syncthreads();
      if (tid == 0) s_ticket = __hip_atomic_fetch_add(args.fuse_count + blockIdx.x, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __syncthreads();
      if (s_ticket != splits - 1) return;
      // (back to zero for the next launch on this stream)
      if (tid == 0) __hip_atomic_store(args.fuse_count + blockIdx.x, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
          for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;
      // (one K range at a time: with two in flight the loads' registers cost the 128x128 tile its second wave per SIMD)
#pragma unroll 1
      for (unsigned z = 0; z < splits; ++z) {
        const unsigned src = first + z * TILE_BYTES;
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
          for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
              const f32x4 v = __builtin_bit_cast(
                  f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_ws, (int)(src + ((i * FN + j) * 4 + g) * 1024), 0, DEVICE_SCOPE));
#pragma unroll
              for (int e = 0; e < 4; ++e) acc[i][j][g * 4 + e] += v[e];
            }
      }
    }
  }

  // ---- epilogue ----
  // The MFMA leaves lane l with row (l&31) and channels 8g + 4*(l>>5) + 0..3 of
  // each 32x32 block.  32 rows of the wave tile at a time are written to a
  // wave-private fp32 staging area in LDS (free after the last barrier of the
  // main loop) and read back 8 consecutive channels per lane, so that the
  // operator chain runs on 8-vectors and a row leaves as whole 16-byte stores.
  constexpr int EP_PITCH = TN + 4;                 // floats
  constexpr int LPR = TN / 8;                      // lanes per output row
  constexpr int RPI = 64 / LPR;                    // rows per pass
  constexpr int STAGING_FLOATS = WM * WN * 32 * EP_PITCH;
  static_assert((size_t)(STAGING_FLOATS + TAB_ENTRIES) * 4 <= (size_t)NS * STAGE, "staging and operand table must fit");
  // A 16x16x32 tile with nothing to apply leaves from registers.  A lane holds channels 4q .. 4q+3 (q = lane >> 4)
  // of row lane & 15 of each 16x16 block; one v_permlane16_swap per packed register between two neighbouring
  // blocks gives every lane 8 consecutive channels of its row (the lanes of 16-lane group q end up with
  // channels 0-7, 16-23, 8-15, 24-31 of the 32-column pair), i.e. one 16-byte store, with the same
  // round-to-nearest conversion as the staged rows.  Staging the whole tile in fp32 moves 512 KB through
  // LDS at 128 bytes per clock on a CU that has nothing else to run: 8.1 k cycles from the last barrier to
  // the end of the kernel with the stores taken out, 11.2 k with them.  (Decided per block of 32 rows, inside
  // the loop below: as a path of its own in front of the loop it cost the register allocation a hundred spills.)
  // (four-wave kernels: the eight-wave 256x256 member has 256 registers and spills 16 with this path in it)
  constexpr bool REG_EPILOGUE = MS == 16 && !CONV && WM * WN == 4;
  const bool from_registers = REG_EPILOGUE && simple && plan.n_ops == 0 && args.out_dtype == DT;
  float *stage = (float *)smem + wave * (32 * EP_PITCH);
  float *table = (float *)smem + STAGING_FLOATS;
  const int er = lane / LPR, ec = (lane % LPR) * 8;
#pragma unroll
  for (int i = 0; i < TPT; ++i)
    if (tid + i * NT < TAB_ENTRIES) table[tid + i * NT] = tabr[i];
  __syncthreads();
  const float *tab = table + wn * TN + ec;
  // The row map's parameters as scalars of their own: read through `args` inside the row
  // lambdas below, with more than one 32-row block per wave, they made the compiler keep a copy
  // of the whole argument block in scratch memory (568 bytes per lane, every later argument read
  // a scratch load) and the convolution ran at half speed.
  const bool om_on = CONV && args.out_map != 0;
  const unsigned om_hw_m = args.hw_m, om_hw_s = args.hw_s, om_w_m = args.w_m, om_w_s = args.w_s;
  const int om_hw = args.h_out * args.w_out, om_w = args.w_out, om_sh = args.o_sh, om_sw = args.o_sw, om_wo = args.o_wo;
  const long long om_img = args.o_img;
  static_for<0, FM>([&](auto blk) {
    constexpr int i = decltype(blk)::value;
    if constexpr (REG_EPILOGUE) {
      if (from_registers) {
        const int q = lane >> 4;
        unsigned short *cbase = (unsigned short *)args.C + n0 + wn * TN + (q & 1) * 16 + (q >> 1) * 8;
        auto pack2 = [](float x, float y) __attribute__((always_inline)) -> unsigned {
          if constexpr (DT == DT_F16) {
            const f16x2 h = {(_Float16)x, (_Float16)y};
            return __builtin_bit_cast(unsigned, h);
          } else {
            const bf16x2 h = {(__bf16)x, (__bf16)y};
            return __builtin_bit_cast(unsigned, h);
          }
        };
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int m = m0 + wm * TM + i * 32 + h * 16 + (lane & 15);
          unsigned short *crow = cbase + (zrow + m) * args.ldc;
#pragma unroll
          for (int j = 0; j < FN; ++j) {
            const f32x4 a4 = acc16[2 * i + h][2 * j], b4 = acc16[2 * i + h][2 * j + 1];
            unsigned a_lo = pack2(a4[0], a4[1]), a_hi = pack2(a4[2], a4[3]);
            unsigned b_lo = pack2(b4[0], b4[1]), b_hi = pack2(b4[2], b4[3]);
            // (as instructions: the compiler's builtin for the swap returns its first result twice; the s_nop
            // is the wait the hardware asks for between a vector-ALU write of an operand and the swap)
            asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a_lo), "+v"(b_lo));
            asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a_hi), "+v"(b_hi));
            const u32x4 row8 = {a_lo, a_hi, b_lo, b_hi};
            if (m < M) *(u32x4 *)(crow + j * 32) = row8;
          }
        }
        return;
      }
    }
    static_for<0, FN>([&](auto col) {
      constexpr int j = decltype(col)::value;
      if constexpr (MS == 16) {
        // lane: row lane & 15 of each 16x16 block, channels 4 * (lane >> 4) .. + 3
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int jj = 0; jj < 2; ++jj) {
            const f32x4 a4 = acc16[2 * i + h][2 * j + jj];
            f32x4 v = {a4[0], a4[1], a4[2], a4[3]};
            *(f32x4 *)(stage + ((lane & 15) + 16 * h) * EP_PITCH + j * 32 + jj * 16 + (lane >> 4) * 4) = v;
          }
      } else {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          f32x4 v = {acc[i][j][g * 4 + 0], acc[i][j][g * 4 + 1], acc[i][j][g * 4 + 2],
                     acc[i][j][g * 4 + 3]};
          *(f32x4 *)(stage + lrow * EP_PITCH + j * 32 + g * 8 + lhalf * 4) = v;
        }
      }
    });
    // The staging area is private to the wave and a wave's LDS operations
    // complete in program order: a compiler-level fence is all that is needed
    // between the writes above and the reads below (and before the next pass
    // overwrites what this one reads).
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    // Output row of GEMM row m.  A convolution may scatter its pixels into a larger image: pixel
    // (q, p) of image b goes to row b*o_img + (o_a + o_sh*q)*o_wo + o_b + o_sw*p (one phase of a
    // transposed convolution writing its share of the full output).
    auto out_row = [&](int m) -> long long {
      if constexpr (CONV) {
        if (om_on) {
          int img, rem, q, pcol;
          fast_divmod(m, om_hw_m, om_hw_s, om_hw, img, rem);
          fast_divmod(rem, om_w_m, om_w_s, om_w, q, pcol);
          return (long long)img * om_img + (long long)(o_a + om_sh * q) * om_wo + o_b + om_sw * pcol;
        }
      }
      return zrow + m;
    };
    if (simple) {
      const int mb = m0 + wm * TM + i * 32;
      auto row_of = [&](int r) -> long long { return mb + r < M ? out_row(mb + r) : -1ll; };
      if constexpr (F32_SIMPLE) {
        if (out_f32) simple_rows<DT, TN, true>(stage, lane, n0 + wn * TN + ec, args, plan, tab, BN, row_of);
        else simple_rows<DT, TN, false>(stage, lane, n0 + wn * TN + ec, args, plan, tab, BN, row_of);
      } else {
        simple_rows<DT, TN, false>(stage, lane, n0 + wn * TN + ec, args, plan, tab, BN, row_of);
      }
    } else {
      for (int r = er; r < 32; r += RPI) {
        const int m = m0 + wm * TM + i * 32 + r;
        const int n = n0 + wn * TN + ec;
        if (m < M && n < N) {
          float v[8];
          const f32x4 lo = *(const f32x4 *)(stage + r * EP_PITCH + ec);
          const f32x4 hi = *(const f32x4 *)(stage + r * EP_PITCH + ec + 4);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            v[e] = lo[e];
            v[4 + e] = hi[e];
          }
          const int nvalid = N - n;
          const long long row = out_row(m);
          apply_epilogue_tab(v, row, n, nvalid, args.epi, plan, tab, BN);
          store_from_float<8>(args.C, args.out_dtype, row * args.ldc + n, nvalid, v);
        }
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
  });
}

template <int BM, int BN, int BK, int WM, int WN, int NS, int PIPE, int MS = 32>
int launch_contraction(const ContractionArgs &a, bool conv, int dtype, bool b_ncontig,
                       hipStream_t stream) {
  if (MS == 16 && conv) return (int)hipErrorInvalidValue;  // (the dispatcher sends convolutions to the 32x32x16 twin)
  constexpr size_t lds = (size_t)NS * (BM + BN) * BK * 2;
  const bool listed = !conv && a.tile_list != nullptr;  // one workgroup per record, no split grid
  const dim3 grid((unsigned)(listed ? a.tile_count : a.grid_m * a.grid_n),
                  (unsigned)(!listed && a.k_split > 0 ? (a.K + a.k_split - 1) / a.k_split : 1),
                  (unsigned)(conv && a.phases > 1 ? a.phases : 1)),
      block(WM * WN * 64);
#define TRACEA_LAUNCH(DTV, CONVV, NCV)                                                       \
  do {                                                                                       \
    auto kfn = contraction_kernel<DTV, BM, BN, BK, WM, WN, NS, PIPE, MS, (CONVV) && MS == 32, NCV>; \
    static bool attr_done = false;                                                           \
    if (!attr_done) {                                                                        \
      hipError_t e = hipFuncSetAttribute((const void *)kfn,                                  \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
      if (e != hipSuccess) return (int)e;                                                    \
      attr_done = true;                                                                      \
    }                                                                                        \
    hipLaunchKernelGGL(kfn, grid, block, lds, stream, a);                                    \
    return (int)hipGetLastError();                                                           \
  } while (0)
  if (dtype == DT_F16) {
    if (conv) { if (b_ncontig) TRACEA_LAUNCH(DT_F16, true, true); else TRACEA_LAUNCH(DT_F16, true, false); }
    else      { if (b_ncontig) TRACEA_LAUNCH(DT_F16, false, true); else TRACEA_LAUNCH(DT_F16, false, false); }
  } else {
    if (conv) { if (b_ncontig) TRACEA_LAUNCH(DT_BF16, true, true); else TRACEA_LAUNCH(DT_BF16, true, false); }
    else      { if (b_ncontig) TRACEA_LAUNCH(DT_BF16, false, true); else TRACEA_LAUNCH(DT_BF16, false, false); }
  }
#undef TRACEA_LAUNCH
  return (int)hipErrorInvalidValue;
}

}  // namespace tracea_amd
