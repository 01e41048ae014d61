// FlashAttention-2 forward for gfx950.
//
// Replaces flash_attention_v2_kernel of the reference
// (src/kernels/attention/cuda_emitter.rs:69-238) and fa2_template_kernel
// (src/kernels/gpu/templates_fa2.cu:41-388): O = softmax(scale Q K^T) V with
// an online (running max / running sum) softmax in fp32, one pass over K/V.
// Causal masking follows the reference's intent (keys strictly after the
// query are excluded, cuda_emitter.rs.tmp:217-218); sequence-length bounds
// masking follows templates_fa2.cu:201-206.  Masked scores are -inf instead of
// the reference's -50000 sentinel, and the final division uses the exact l
// (the reference adds 1e-9 / 1e-6): both differences are far below bf16
// resolution.
//
// Work split: a workgroup of 4 waves owns 128 query rows of one (batch, head);
// each wave owns 32 of them.  Per 64-key tile the wave computes the TRANSPOSED
// score block S^T = K Q^T with v_mfma_f32_32x32x16 (A operand = 32 keys from
// LDS, B operand = the wave's 32 queries, resident in registers).  In the
// 32x32 accumulator layout lane l then holds scores of ONE query (l & 31) for
// 32 of the 64 keys; its partner lane l^32 holds the other 32.  Row max and
// row sum are therefore in-register reductions plus a single cross-lane
// exchange per tile, and P^T is already laid out as the B operand of the
// second product O^T += V^T P^T without touching LDS: accumulator registers
// 8h..8h+7 of block b, converted to 16 bit, are exactly the 8 k-slots a lane
// feeds to the MFMA that covers keys 32b+16h..+15, provided the A operand
// (V^T) enumerates the keys in the same order.  That order is
// key(slot j, half g) = 8*(j/4) + 4g + j%4, i.e. two runs of four consecutive
// keys at a fixed head-dim column, which the LDS transpose load
// ds_read_b64_tr_b16 delivers from a row-major [key][d] tile.
// O^T accumulators of a lane all belong to the lane's query, so the online
// rescale is a per-lane scalar multiply.
#include <type_traits>

#include "contraction_kernel.hpp"

namespace tracea_amd {

// Scheduling pipeline of the softmax region: per step one LDS read, one MFMA and
// eight vector-ALU instructions (classes 0x100, 0x008, 0x002 of
// __builtin_amdgcn_sched_group_barrier).
template <int kStep, int kSteps>
struct Interleave3 {
  static __device__ __forceinline__ void run() {
    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    __builtin_amdgcn_sched_group_barrier(0x002, 8, 0);
    if constexpr (kStep + 1 < kSteps) Interleave3<kStep + 1, kSteps>::run();
  }
};

// kMfmas steps of: one MFMA, kValu vector-ALU instructions, and an LDS read in the first kReads steps.
// A wave that has its SIMD to itself must be given this order explicitly: MFMAs issued back to back
// hold the wave's issue slot while each waits for the matrix pipe, and the vector work of the chunk
// then runs behind the last of them instead of under all of them.
template <int kStep, int kMfmas, int kValu, int kReads>
struct MfmaValu {
  static __device__ __forceinline__ void run() {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    if constexpr (kValu > 0) __builtin_amdgcn_sched_group_barrier(0x002, kValu, 0);
    if constexpr (kStep < kReads) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    if constexpr (kStep + 1 < kMfmas) MfmaValu<kStep + 1, kMfmas, kValu, kReads>::run();
  }
};

typedef short s16x4 __attribute__((ext_vector_type(4)));

// max(x, x of lane l ^ 32) without a trip through LDS: v_permlane32_swap exchanges the upper half of its
// first operand with the lower half of its second; given the same value twice, the two results are a
// lane's own value and its partner's, in one order or the other.  (Written as an instruction: the
// compiler's builtin for the swap hands back its first result twice, and the maximum of the two would be
// folded away.  The s_nop covers the wait the hardware asks for between a vector-ALU write of an operand
// and the swap, which the compiler cannot see to insert.)
__device__ __forceinline__ float max_with_lane_xor32(float x) {
  float a0 = x, a1 = x;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a0), "+v"(a1));
  return fmaxf(a0, a1);
}

template <int DT>
__device__ __forceinline__ u32x4 pack8(const float (&p)[8]) {
  if constexpr (DT == DT_F16) {
    f16x8 h = {(_Float16)p[0], (_Float16)p[1], (_Float16)p[2], (_Float16)p[3],
               (_Float16)p[4], (_Float16)p[5], (_Float16)p[6], (_Float16)p[7]};
    return __builtin_bit_cast(u32x4, h);
  } else {
    bf16x8 h = {(__bf16)p[0], (__bf16)p[1], (__bf16)p[2], (__bf16)p[3],
                (__bf16)p[4], (__bf16)p[5], (__bf16)p[6], (__bf16)p[7]};
    return __builtin_bit_cast(u32x4, h);
  }
}

// The running maximum follows the scores lazily: it moves (and O and the row sum are rescaled) only when a
// tile's maximum exceeds it by more than FA_RESCALE_TAU in the exponent's log2 units.  Softmax needs ONE
// reference value per query for all its keys, not the true maximum: with a reference up to TAU below it the
// probabilities of a tile reach 2^TAU instead of 1, far inside the range of fp32 sums and 16-bit operands,
// and the final division by the row sum takes the factor out again.  With the exact maximum a wave of 32
// queries rescales in about 54 of the 64 tiles of a 4096-key sequence (some query's maximum moves in a tile
// with probability min(1, 32/t)), 64 multiplies each on a vector ALU that is the busiest unit of the kernel;
// lazily it rescales once or twice.  (A dominant key still moves the reference at once.)
constexpr float FA_RESCALE_TAU = 8.0f;
__device__ __forceinline__ bool lazy_running_max(float &m_run, float candidate, float &alpha) {
  const bool moved = candidate > m_run + FA_RESCALE_TAU;
  const float m_new = moved ? candidate : m_run;
  alpha = __builtin_amdgcn_exp2f(m_run - m_new);  // exactly 1 where the reference stays
  m_run = m_new;
  return moved;
}

constexpr int FA_BQ = 128;   // query rows per workgroup
constexpr int FA_BKV = 64;   // keys per tile
constexpr int FA_WAVES = 4;

// V_TR: fetch the V^T operand with the LDS transpose load (fast); otherwise
// with eight 16-bit LDS reads per operand (slow, instruction-for-instruction
// obvious; kept as the cross-check of the transpose path).
template <int DT, int D, bool V_TR>
__global__ void __launch_bounds__(FA_WAVES * 64) __attribute__((amdgpu_waves_per_eu(2, 2)))
fa2_fwd_kernel(const AttentionArgs a) {
  constexpr int NT = FA_WAVES * 64;
  constexpr int ROW_BYTES = D * 2;
  constexpr int CH = D / 8;                      // 16-byte pieces per row
  constexpr int TILE_BYTES = FA_BKV * ROW_BYTES; // one K or V tile
  constexpr int STAGE = 2 * TILE_BYTES;          // K + V
  constexpr int NP = FA_BKV * CH / NT;           // pieces per thread per tensor per tile
  constexpr int KS = D / 16;                     // k steps of the score product
  constexpr int DB = D / 32;                     // 32-wide head-dim blocks of O^T
  static_assert(D % 32 == 0 && (FA_BKV * CH) % NT == 0, "unsupported head dim");

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lrow = lane & 31, g = lane >> 5;

  // workgroup -> (batch*head, query block); consecutive ids land on different
  // XCDs, so regroup them to keep one head's K/V in one L2, and walk the query
  // blocks from the last (most keys under a causal mask) to the first.
  const int nqb = (a.S + FA_BQ - 1) / FA_BQ;
  const int total = nqb * a.B * a.H;
  int vid = blockIdx.x;
  if ((total & 7) == 0) vid = (vid & 7) * (total >> 3) + (vid >> 3);
  const int bh = vid / nqb;
  const int qb = nqb - 1 - (vid - bh * nqb);
  const int b = bh / a.H, h = bh - b * a.H;
  const int q0 = qb * FA_BQ;
  const int S = a.S;

  const unsigned short *Qg = (const unsigned short *)a.Q + (long long)b * a.q_sb + (long long)h * a.q_sh;
  const unsigned short *Kg = (const unsigned short *)a.K + (long long)b * a.k_sb + (long long)h * a.k_sh;
  const unsigned short *Vg = (const unsigned short *)a.V + (long long)b * a.v_sb + (long long)h * a.v_sh;
  unsigned short *Og = (unsigned short *)a.O + (long long)b * a.o_sb + (long long)h * a.o_sh;

  // ---- this wave's 32 queries, B operand of S^T: lane (q = lrow, g) holds
  //      Q[q][16*ks + 8*g .. +7] for every k step ----
  const int q_wave0 = q0 + wave * 32;
  const int q_mine = q_wave0 + lrow;
  u32x4 qf[KS];
  {
    const int qr = q_mine < S ? q_mine : S - 1;
    const unsigned short *qp = Qg + (long long)qr * a.q_ss + g * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = *(const u32x4 *)(qp + ks * 16);
  }

  // ---- key/value tile movement: piece p -> row p / CH, 16-byte column p % CH.
  //      K rows are swizzled for 32 lanes reading the same column of 32 rows;
  //      V rows are swizzled at 64-byte granularity for the transpose load,
  //      whose 32 lanes read a 64-byte window of 4 consecutive rows. ----
  constexpr int RP = 256 / ROW_BYTES > 0 ? 256 / ROW_BYTES : 1;  // rows per 256 bytes of LDS
  constexpr int WIN = ROW_BYTES / 64;                            // 64-byte windows per row
  auto k_piece = [&](int row, int c) -> int {
    return row * ROW_BYTES + ((c ^ ((row / RP) & (CH - 1))) << 4);
  };
  auto v_piece = [&](int row, int c) -> int {
    return row * ROW_BYTES + ((c ^ (((row / RP) % WIN) << 2)) << 4);
  };

  const int ntiles_all = (S + FA_BKV - 1) / FA_BKV;
  int ntiles = ntiles_all;
  if (a.causal) {
    const int last_q = (q0 + FA_BQ - 1 < S ? q0 + FA_BQ - 1 : S - 1);
    const int need = last_q / FA_BKV + 1;
    ntiles = need < ntiles ? need : ntiles;
  }

  u32x4 rk[NP], rv[NP];
  auto fetch = [&](int t) {
    const int kv0 = t * FA_BKV;
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      const int p = tid + i * NT;
      int row = kv0 + p / CH;
      row = row < S ? row : S - 1;  // rows beyond S are masked in the scores
      const int c = p % CH;
      rk[i] = *(const u32x4 *)(Kg + (long long)row * a.k_ss + c * 8);
      rv[i] = *(const u32x4 *)(Vg + (long long)row * a.v_ss + c * 8);
    }
  };
  auto stash = [&](unsigned char *sK, unsigned char *sV) {
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      const int p = tid + i * NT;
      const int row = p / CH, c = p % CH;
      *(u32x4 *)(sK + k_piece(row, c)) = rk[i];
      *(u32x4 *)(sV + v_piece(row, c)) = rv[i];
    }
  };

  f32x16 o[DB];
#pragma unroll
  for (int d = 0; d < DB; ++d)
#pragma unroll
    for (int e = 0; e < 16; ++e) o[d][e] = 0.0f;
  float m_run = -1.0e30f;  // running max, log2 domain, finite so that exp2(m-m) is 1
  float l_run = 0.0f;      // this lane's share of the running sum

  fetch(0);
  stash(smem, smem + TILE_BYTES);
  __syncthreads();

  for (int t = 0; t < ntiles; ++t) {
    const unsigned char *sK = smem + (t & 1) * STAGE;
    const unsigned char *sV = sK + TILE_BYTES;
    unsigned char *nK = smem + ((t + 1) & 1) * STAGE;
    const bool more = t + 1 < ntiles;
    fetch(more ? t + 1 : t);
    __builtin_amdgcn_sched_barrier(0);

    const int kv0 = t * FA_BKV;
    // a wave whose every query precedes every key of the tile has nothing to add
    const bool wave_active = !(a.causal && kv0 > q_wave0 + 31);
    if (wave_active) {
      // ---- S^T = K Q^T : two 32-key blocks ----
      f32x16 s[2];
#pragma unroll
      for (int blk = 0; blk < 2; ++blk)
#pragma unroll
        for (int e = 0; e < 16; ++e) s[blk][e] = 0.0f;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
          const u32x4 kf = *(const u32x4 *)(sK + k_piece(blk * 32 + lrow, ks * 2 + g));
          s[blk] = Mfma32<DT>::run(kf, qf[ks], s[blk]);
        }
      }

      // ---- scale to the log2 domain, mask, running max ----
      const bool edge = (kv0 + FA_BKV > S) || (a.causal && kv0 + FA_BKV - 1 > q_wave0);
      float mx = -INFINITY;
#pragma unroll
      for (int blk = 0; blk < 2; ++blk)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          float x = s[blk][e] * a.scale_log2;
          if (edge) {
            const int kv = kv0 + blk * 32 + (e >> 2) * 8 + g * 4 + (e & 3);
            if (kv >= S || (a.causal && kv > q_mine)) x = -INFINITY;
          }
          s[blk][e] = x;
          mx = fmaxf(mx, x);
        }
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = fmaxf(m_run, mx);
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
      m_run = m_new;

      // ---- P = exp2(S - m), row-sum share, B operands of the second product ----
      float lsum = 0.0f;
      u32x4 pf[4];
#pragma unroll
      for (int blk = 0; blk < 2; ++blk)
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
          float p[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            p[j] = exp2f(s[blk][hh * 8 + j] - m_new);
            lsum += p[j];
          }
          pf[blk * 2 + hh] = pack8<DT>(p);
        }
      l_run = l_run * alpha + lsum;
#pragma unroll
      for (int d = 0; d < DB; ++d)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[d][e] *= alpha;

      // ---- O^T += V^T P^T : 4 key groups of 16 x DB head-dim blocks ----
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
#pragma unroll
        for (int d = 0; d < DB; ++d) {
          u32x4 vf;
          if constexpr (V_TR) {
            // 16-lane group: lane r supplies row (base + r/4), 4 columns at
            // 4*(r%4) of its 16-column window; lane n receives column n of the
            // 4 rows.
            const int r = lane & 15;
            const int col = d * 32 + ((lane >> 4) & 1) * 16 + (r & 3) * 4;
            const int row_lo = kk * 16 + g * 4 + (r >> 2);
            const int row_hi = row_lo + 8;
            const unsigned char *p_lo = sV + v_piece(row_lo, col >> 3) + (col & 7) * 2;
            const unsigned char *p_hi = sV + v_piece(row_hi, col >> 3) + (col & 7) * 2;
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (__attribute__((address_space(3))) s16x4 *)(p_lo));
            const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (__attribute__((address_space(3))) s16x4 *)(p_hi));
            const u32x2 lo2 = __builtin_bit_cast(u32x2, lo), hi2 = __builtin_bit_cast(u32x2, hi);
            vf[0] = lo2[0]; vf[1] = lo2[1]; vf[2] = hi2[0]; vf[3] = hi2[1];
          } else {
            const int col = d * 32 + lrow;
            unsigned short hv[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              const int row = kk * 16 + (j >> 2) * 8 + g * 4 + (j & 3);
              hv[j] = *(const unsigned short *)(sV + v_piece(row, col >> 3) + (col & 7) * 2);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) vf[j] = (unsigned)hv[2 * j] | ((unsigned)hv[2 * j + 1] << 16);
          }
          o[d] = Mfma32<DT>::run(vf, pf[kk], o[d]);
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    if (more) stash(nK, nK + TILE_BYTES);
    __syncthreads();
  }

  // ---- normalise, regroup through LDS, store 16 bytes per lane ----
  const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
  const float inv_l = 1.0f / l_tot;
  unsigned char *so = smem + wave * (32 * ROW_BYTES);  // [32 queries][D] of the output type
#pragma unroll
  for (int d = 0; d < DB; ++d)
#pragma unroll
    for (int v4 = 0; v4 < 4; ++v4) {
      float x[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) x[e] = o[d][v4 * 4 + e] * inv_l;
      u32x2 w;
      if constexpr (DT == DT_F16) {
        f16x4 hq = {(_Float16)x[0], (_Float16)x[1], (_Float16)x[2], (_Float16)x[3]};
        w = __builtin_bit_cast(u32x2, hq);
      } else {
        bf16x4 hq = {(__bf16)x[0], (__bf16)x[1], (__bf16)x[2], (__bf16)x[3]};
        w = __builtin_bit_cast(u32x2, hq);
      }
      *(u32x2 *)(so + lrow * ROW_BYTES + (d * 32 + v4 * 8 + g * 4) * 2) = w;
    }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 32 * CH / 64; ++i) {
    const int p = lane + i * 64;
    const int row = p / CH, c = p % CH;
    const int q = q_wave0 + row;
    if (q < S)
      *(u32x4 *)(Og + (long long)q * a.o_ss + c * 8) = *(const u32x4 *)(so + row * ROW_BYTES + c * 16);
  }
}

// ---------------------------------------------------------------------------
// Pipelined form.  Same arithmetic and register layouts as fa2_fwd_kernel, but
//   * K and V tiles travel with direct-to-LDS buffer loads (no staging
//     registers, no LDS write instructions; rows at or beyond S are outside the
//     buffer and read as zeros),
//   * K runs one tile ahead of V: the score product of tile t+1 is issued
//     before the softmax of tile t, so the matrix pipe works on S^T(t+1) while
//     the vector ALU does the exponentials of tile t, and
//   * the rescale of O is skipped while no running maximum of the wave moves.
// LDS: two K stages and two V stages.  Iteration t starts with one barrier
// that publishes K(t+1) and V(t) and retires K(t) and V(t-1); K(t+2) and
// V(t+1) are then requested into the retired stages, a whole iteration before
// they are needed.
//
// EARLY_MAX: an iteration of the form above has three phases -- running maximum
// of tile t (vector ALU only), score product of t+1 with the exponentials of t
// (both pipes), P.V of t (matrix pipe only).  The maximum of tile t+1 depends
// only on S(t+1), which is complete after the second phase, so with EARLY_MAX it
// is computed under the P.V MFMAs of tile t (whose operand reads then run one
// step ahead): two phases, both pipes busy in each.  Only the rescale of O,
// which needs P.V(t) finished, stays between iterations.  The last iteration
// takes the maximum of a tile past the end, all of whose scores are masked:
// nothing moves.
// ---------------------------------------------------------------------------
// WAVES: waves of 32 queries per workgroup (4 or 8: 128 or 256 queries share every K/V tile);
// NSTG: LDS stages per K and per V ring (2: tiles requested one iteration ahead, 3: two).
// ITEMS: query blocks a workgroup takes one after the other (1 or 2; the reference's fusion_count,
// src/optimizer/benchmark.rs:131-132).  With 2 the K/V rings run on across the two: the look-ahead requests
// of the first block's last iterations fetch the second block's first tiles, its queries are fetched together
// with the first block's, and O leaves from registers (the staging area in LDS would lie under those tiles)
// -- the second block starts without a load to wait for.  Under a causal mask the pair is block j and block
// nqb-1-j: every workgroup then has the same number of tiles.  Same bits as one block per workgroup.
// Measured at B4 H32 S4096 D128 (replayed graphs, one box): dense 1002 -> 980 us on 8 waves, causal 585 -> 553
// on 4.  (Four blocks per workgroup: the third set of queries in flight spills at head dimension 128, and the
// coarser units balance worse: 999 and 572 us.)
//
// SHIFT: the softmax shift rides the score product.  The queries are multiplied by scale * log2(e) when they
// are loaded (rounded once more to the operand type: a relative 2^-9 on q, about as much on a probability),
// and the first MFMA of every S^T block accumulates onto a register block holding -m, the query's reference
// maximum, instead of zero: the product comes out as z = s * scale * log2(e) - m and a probability is one
// v_exp_f32 of it, without the multiply-add per score that the vector ALU, the busiest unit of this kernel,
// spent on the shift.  The maximum of a tile is taken of z: while it stays below FA_RESCALE_TAU the reference
// stays; when it moves, the tile's z are lowered by the step and O and the row sum rescaled.  Costs 16
// registers per query block (the -m block), which the paired members at head dimension 128 do not have.
constexpr bool fa2_pipe_parks_queries(int d, int qb, int items, bool shift) { return items > 1 && shift && d == 128 && qb == 1; }
//
// PP: the two waves of a SIMD half an iteration apart.  Phase A of an iteration (exponentials of tile t under
// the score product of tile t+1) is mostly vector ALU, phase B (P.V of tile t under the maximum of tile t+1)
// mostly matrix pipe; with one barrier per tile every wave of the workgroup enters phase A together, the two
// waves of a SIMD contend for the vector ALU while the matrix pipe idles, and then the other way round.  Here
// the barrier comes twice per tile, between the phases, and waves 4-7 run one phase behind waves 0-3 (they
// sit out the first slot, waves 0-3 the last): in every slot a SIMD holds one wave in phase A and one in
// phase B.  K(u+2) is requested by every wave at the barrier that opens slot 2u, V(u+1) at the one that opens
// slot 2u+1; a request has two slots to land, and a barrier waits for the one before last.  Eight waves, one
// query block per workgroup, two-stage rings, no causal mask (waves would differ in their number of tiles).
template <int DT, int D, bool EARLY_MAX, int WAVES, int NSTG, int QB, int ITEMS = 1, bool SHIFT = false, bool PP = false>
__global__ void __launch_bounds__(WAVES * 64) __attribute__((amdgpu_waves_per_eu(QB == 1 ? 2 : 1, QB == 1 ? 2 : 1)))
fa2_fwd_pipe_kernel(const AttentionArgs a) {
  static_assert(!PP || (EARLY_MAX && WAVES == 8 && NSTG == 2 && QB == 1 && ITEMS == 1), "the half-iteration offset exists for eight waves, one block, two stages");
  static_assert(!SHIFT || EARLY_MAX, "the shifted score product exists in the two-phase form only");
  constexpr bool PARK = fa2_pipe_parks_queries(D, QB, ITEMS, SHIFT);
  static_assert(QB == 1 || (QB == 2 && EARLY_MAX), "two query blocks per wave exist in the two-phase form only");
  static_assert(ITEMS == 1 || (ITEMS == 2 && EARLY_MAX), "pairs of query blocks exist in the two-phase form only");
  constexpr int WQ = 32 * QB;  // queries per wave
  constexpr int BQ = WQ * WAVES;
  constexpr int ROW_BYTES = D * 2;
  constexpr int CH = D / 8;
  constexpr int TILE_BYTES = FA_BKV * ROW_BYTES;
  constexpr int KS = D / 16;
  constexpr int DB = D / 32;
  constexpr int RPI = 64 / CH;                 // tile rows per wave-wide load instruction
  constexpr int NI = FA_BKV / (RPI * WAVES); // load instructions per wave per tensor per tile
  constexpr int RP = 256 / ROW_BYTES > 0 ? 256 / ROW_BYTES : 1;
  constexpr int WIN = ROW_BYTES / 64;
  static_assert(D % 32 == 0 && FA_BKV % (RPI * WAVES) == 0, "unsupported head dim");

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  static_assert(NSTG == 2 || NSTG == 3 || NSTG == 4, "ring depth");
  // Four stages: one barrier for every TWO tiles.  The barrier in front of tiles (t, t+1), t even, publishes
  // K(t+1), K(t+2), V(t), V(t+1), requested at the barrier before, and the stages of the pair before receive
  // K(t+3), K(t+4), V(t+2), V(t+3): half the barriers and waits per key, and a request has two tiles to land.
  constexpr bool PAIR_SYNC = NSTG == 4;
  static_assert(!PAIR_SYNC || (EARLY_MAX && ITEMS == 1 && !PP), "the two-tile barrier exists for one query block per workgroup");
  unsigned char *const sKbase = smem;                      // NSTG stages
  unsigned char *const sVbase = smem + NSTG * TILE_BYTES;  // NSTG stages

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int lrow = lane & 31, g = lane >> 5;
  const int grp = wave_u >> 2;  // (PP) 0: waves 0-3, 1: waves 4-7, one phase behind

  const int nqb = (a.S + BQ - 1) / BQ;
  const int per_bh = nqb / ITEMS;  // workgroups per (batch, head); the host launches pairs for an even nqb only
  const int total = per_bh * a.B * a.H;
  int vid = blockIdx.x;
  if ((total & 7) == 0) vid = (vid & 7) * (total >> 3) + (vid >> 3);
  const int bh = vid / per_bh;
  const int slot = vid - bh * per_bh;
  // the query block of item i: alone, from the last block to the first; in pairs, a heavy and a light one
  // under a causal mask and two neighbours otherwise
  auto item_block = [&](int i) __attribute__((always_inline)) -> int {
    if constexpr (ITEMS == 1) return nqb - 1 - slot;
    else return a.causal ? (i == 0 ? nqb - 1 - slot : slot) : 2 * slot + i;
  };
  const int b = bh / a.H, h = bh - b * a.H;
  int q0 = item_block(0) * BQ;
  const int S = a.S;

  const unsigned short *Qg = (const unsigned short *)a.Q + (long long)b * a.q_sb + (long long)h * a.q_sh;
  const unsigned short *Kg = (const unsigned short *)a.K + (long long)b * a.k_sb + (long long)h * a.k_sh;
  const unsigned short *Vg = (const unsigned short *)a.V + (long long)b * a.v_sb + (long long)h * a.v_sh;
  unsigned short *Og = (unsigned short *)a.O + (long long)b * a.o_sb + (long long)h * a.o_sh;

  int q_wave0 = q0 + wave * WQ;
  int q_mine[QB];  // this lane's query in each of the wave's blocks of 32
  // The last key this lane's scores may keep (the query itself under a causal mask, else the end of the
  // sequence), less the lane half's offset inside a group of 8 keys: an edge tile then masks element e with one
  // comparison of a constant against last_key - kv0 (two comparisons, index arithmetic and their scalar
  // combination per element cost an edge tile 1.55 times the vector instructions of an interior one).
  int last_key[QB];
  int wave_last_key;  // (wave-uniform) the last key any query of the wave may keep
  u32x4 qf[QB][KS];
  // (SHIFT) a fragment of queries times scale * log2(e), rounded to the operand type
  auto prescale = [&](u32x4 raw) __attribute__((always_inline)) -> u32x4 {
    if constexpr (!SHIFT) return raw;
    float qs[8];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if constexpr (DT == DT_F16) {
        qs[2 * e] = (float)__builtin_bit_cast(_Float16, (unsigned short)(raw[e] & 0xffffu)) * a.scale_log2;
        qs[2 * e + 1] = (float)__builtin_bit_cast(_Float16, (unsigned short)(raw[e] >> 16)) * a.scale_log2;
      } else {
        qs[2 * e] = __builtin_bit_cast(float, raw[e] << 16) * a.scale_log2;
        qs[2 * e + 1] = __builtin_bit_cast(float, raw[e] & 0xffff0000u) * a.scale_log2;
      }
    }
    return pack8<DT>(qs);
  };
  // the first NK k-step fragments of the queries of the block that starts at first_query
  auto load_q = [&](int first_query, auto &dst, auto nk_tag) __attribute__((always_inline)) {
    constexpr int NK = decltype(nk_tag)::value;
#pragma unroll
    for (int qi = 0; qi < QB; ++qi) {
      const int mine = first_query + wave * WQ + qi * 32 + lrow;
      const int qr = mine < S ? mine : S - 1;
      const unsigned short *qp = Qg + (long long)qr * a.q_ss + g * 8;
#pragma unroll
      for (int ks = 0; ks < NK; ++ks) dst[qi][ks] = prescale(*(const u32x4 *)(qp + ks * 16));
    }
  };
#pragma unroll
  for (int qi = 0; qi < QB; ++qi) {
    q_mine[qi] = q_wave0 + qi * 32 + lrow;
    last_key[qi] = (a.causal && q_mine[qi] < S - 1 ? q_mine[qi] : S - 1) - g * 4;
  }
  wave_last_key = a.causal && q0 + (wave_u + 1) * WQ - 1 < S - 1 ? q0 + (wave_u + 1) * WQ - 1 : S - 1;
  // (the queries are fetched behind the first tile requests, below: the scaling of a fragment waits for its load,
  // and in front of the requests that wait was a round trip to memory of its own at the start of every workgroup)

  auto k_piece = [&](int row, int c) __attribute__((always_inline)) -> int {
    return row * ROW_BYTES + ((c ^ ((row / RP) & (CH - 1))) << 4);
  };
  auto v_piece = [&](int row, int c) __attribute__((always_inline)) -> int {
    return row * ROW_BYTES + ((c ^ (((row / RP) % WIN) << 2)) << 4);
  };

  // Buffer views of this (batch, head) slice: rows 0..S-1; anything beyond reads as zero.
  __amdgpu_buffer_rsrc_t rsrc_k = __builtin_amdgcn_make_buffer_rsrc(
      (void *)Kg, 0, (int)(((long long)(S - 1) * a.k_ss + D) * 2), 0x00020000);
  __amdgpu_buffer_rsrc_t rsrc_v = __builtin_amdgcn_make_buffer_rsrc(
      (void *)Vg, 0, (int)(((long long)(S - 1) * a.v_ss + D) * 2), 0x00020000);
  // Load instruction i of this wave covers tile rows (i*WAVES + wave)*RPI + lane/CH; the lane's
  // LDS slot is 16-byte column lane%CH of that row, so it fetches the global column that the
  // swizzle of the tensor maps there.
  unsigned k_voff[NI], v_voff[NI];
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int row = (i * WAVES + wave) * RPI + lane / CH;
    const int p = lane % CH;
    k_voff[i] = (unsigned)(row * (int)a.k_ss * 2 + ((p ^ ((row / RP) & (CH - 1))) << 4));
    v_voff[i] = (unsigned)(row * (int)a.v_ss * 2 + ((p ^ (((row / RP) % WIN) << 2)) << 4));
  }
  auto load_k = [&](int t, unsigned char *dst) __attribute__((always_inline)) {
    const unsigned adv = (unsigned)t * (unsigned)(FA_BKV * 2) * (unsigned)a.k_ss;
#pragma unroll
    for (int i = 0; i < NI; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          rsrc_k, (__attribute__((address_space(3))) void *)(dst + (i * WAVES + wave_u) * RPI * ROW_BYTES),
          16, (int)(k_voff[i] + adv), 0, 0, 0);
  };
  auto load_v = [&](int t, unsigned char *dst) __attribute__((always_inline)) {
    const unsigned adv = (unsigned)t * (unsigned)(FA_BKV * 2) * (unsigned)a.v_ss;
#pragma unroll
    for (int i = 0; i < NI; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          rsrc_v, (__attribute__((address_space(3))) void *)(dst + (i * WAVES + wave_u) * RPI * ROW_BYTES),
          16, (int)(v_voff[i] + adv), 0, 0, 0);
  };

  auto tiles_of = [&](int first_query) __attribute__((always_inline)) -> int {
    int n = (S + FA_BKV - 1) / FA_BKV;
    if (a.causal) {
      const int last_q = (first_query + BQ - 1 < S ? first_query + BQ - 1 : S - 1);
      const int need = last_q / FA_BKV + 1;
      n = need < n ? need : n;
    }
    return n;
  };
  int ntiles = tiles_of(q0);
  // tb: K/V tiles of the items before the current one.  Tile t of an item lives in ring stage (tb + t) % NSTG,
  // and a look-ahead request past the item's last tile fetches the next item's tiles (same batch and head).
  int tb = 0, item = 0;
  auto ahead = [&](int f) __attribute__((always_inline)) -> int {
    if constexpr (ITEMS == 1) return f;
    else return (f >= ntiles && item + 1 < ITEMS) ? f - ntiles : f;
  };

  // (a key fragment read from LDS serves all QB query blocks of the wave: with one block every MFMA
  // needs 1 KB of LDS, which is all that LDS delivers while the four matrix pipes of the CU run)
  auto scores = [&](const unsigned char *sK, f32x16 (&s)[QB][2]) {
#pragma unroll
    for (int qi = 0; qi < QB; ++qi)
#pragma unroll
      for (int blk = 0; blk < 2; ++blk)
#pragma unroll
        for (int e = 0; e < 16; ++e) s[qi][blk][e] = 0.0f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int blk = 0; blk < 2; ++blk) {
        const u32x4 kf = *(const u32x4 *)(sK + k_piece(blk * 32 + lrow, ks * 2 + g));
#pragma unroll
        for (int qi = 0; qi < QB; ++qi) s[qi][blk] = Mfma32<DT>::run(kf, qf[qi][ks], s[qi][blk]);
      }
  };

  f32x16 o[QB][DB];
  float m_run[QB], l_run[QB];

  // tiles at or beyond the end of the sequence lie outside the buffers and load as zeros
  // requests of a wave that may stay in flight where an iteration waits for its tiles: those of the
  // iteration before (NSTG = 3), none (NSTG = 2)
  constexpr int FLIGHT = PAIR_SYNC ? 0 : (NSTG - 2) * 2 * NI;
  constexpr int WAIT_TILES = (FLIGHT & 15) | (7 << 4) | (15 << 8) | ((FLIGHT >> 4) << 14);
  load_k(0, sKbase);
  load_v(0, sVbase);
  load_k(1, sKbase + TILE_BYTES);
  if constexpr (PAIR_SYNC) {
    load_k(2, sKbase + 2 * TILE_BYTES);
    load_v(1, sVbase + TILE_BYTES);
  }
  if constexpr (NSTG == 3) {
    load_v(1, sVbase + TILE_BYTES);
    load_k(2, sKbase + 2 * TILE_BYTES);
  }
  __builtin_amdgcn_sched_barrier(0);
  load_q(q0, qf, std::integral_constant<int, KS>{});
  // The second item's queries travel with the first tiles.  PARK: the upper half of their k-steps waits in LDS
  // behind the rings (fetched there directly, each lane's fragment in a slot of its own) instead of in
  // registers: the 16 registers that the -m block of SHIFT needs at head dimension 128.
  constexpr int KQN = PARK ? KS / 2 : KS;  // k-step fragments of the next item's queries kept in registers
  unsigned char *const sPark = smem + 2 * NSTG * TILE_BYTES;
  u32x4 qf_next[ITEMS > 1 ? QB : 1][KQN];
  if constexpr (ITEMS > 1) {
    load_q(item_block(1) * BQ, qf_next, std::integral_constant<int, KQN>{});
    if constexpr (PARK) {
      const int mine = item_block(1) * BQ + wave * WQ + lrow;
      const int qr = mine < S ? mine : S - 1;
      __amdgpu_buffer_rsrc_t rsrc_q = __builtin_amdgcn_make_buffer_rsrc(
          (void *)Qg, 0, (int)(((long long)(S - 1) * a.q_ss + D) * 2), 0x00020000);
      const unsigned q_voff = (unsigned)(qr * (int)a.q_ss * 2 + g * 16);
#pragma unroll
      for (int ks = KQN; ks < KS; ++ks)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rsrc_q, (__attribute__((address_space(3))) void *)(sPark + ((wave_u * (KS - KQN) + ks - KQN) * 64) * 16), 16,
            (int)(q_voff + ks * 32), 0, 0, 0);
    }
  }
  f32x16 s_cur[QB][2], s_nxt[QB][2];

  // Masks tile `tile`'s scores in s (EDGE only) and folds them into the running
  // maximum.  The maximum is taken over the raw scores (the scale is positive);
  // the scale is folded into the exponent's multiply-add.  Leaves the rescale
  // factor of the earlier tiles in `alpha` (exactly 1 where the maximum did not
  // move) and returns whether this lane's maximum moved.
  float alpha[QB];
#pragma unroll
  for (int qi = 0; qi < QB; ++qi) alpha[qi] = 1.0f;
  f32x16 negm[SHIFT ? QB : 1];  // SHIFT: -m_run in every element, where the score product of a tile starts
  // SHIFT: folds the maxima mx of a tile's z (scores relative to the reference) into the reference.  It moves by
  // the whole excess once that exceeds TAU (`force`: by whatever it is -- the first tile's case, whose reference
  // is the arbitrary 0); the tile's z follow, O is rescaled at once, and alpha is the factor the row sum of the
  // earlier tiles takes with the next tile's sum (exactly 1 where nothing moved).  One branch for all of it.
  auto fold_shift = [&](const float (&mx)[QB], f32x16 (&z)[QB][2], bool force) __attribute__((always_inline)) {
    bool moved = false;
    float step[QB];
#pragma unroll
    for (int qi = 0; qi < QB; ++qi) {
      const float mw = max_with_lane_xor32(mx[qi]);
      const bool mv = (force & (mw > -INFINITY)) | (mw > FA_RESCALE_TAU);
      step[qi] = mv ? mw : 0.0f;
      alpha[qi] = __builtin_amdgcn_exp2f(-step[qi]);
      m_run[qi] += step[qi];
      moved |= mv;
    }
    if (__any(moved)) {
#pragma unroll
      for (int qi = 0; qi < QB; ++qi) {
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
#pragma unroll
          for (int e = 0; e < 16; ++e) z[qi][blk][e] -= step[qi];
#pragma unroll
        for (int e = 0; e < 16; ++e) negm[SHIFT ? qi : 0][e] = -m_run[qi];
#pragma unroll
        for (int d = 0; d < DB; ++d)
#pragma unroll
          for (int e = 0; e < 16; ++e) o[qi][d][e] *= alpha[qi];
      }
    }
  };
  auto take_max = [&](int tile, auto edge_tag, f32x16 (&s)[QB][2]) -> bool {
    constexpr bool EDGE = decltype(edge_tag)::value;
    const int kv0 = tile * FA_BKV;
    bool moved = false;
    float mxs[QB];
#pragma unroll
    for (int qi = 0; qi < QB; ++qi) {
      float mx = -INFINITY;
#pragma unroll
      for (int blk = 0; blk < 2; ++blk)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          if constexpr (EDGE) s[qi][blk][e] = blk * 32 + (e >> 2) * 8 + (e & 3) > last_key[qi] - kv0 ? -INFINITY : s[qi][blk][e];
          mx = fmaxf(mx, s[qi][blk][e]);
        }
      mxs[qi] = mx;
      if constexpr (!SHIFT) {
        mx = max_with_lane_xor32(mx);
        moved |= lazy_running_max(m_run[qi], mx * a.scale_log2, alpha[qi]);
      }
    }
    if constexpr (SHIFT) {  // (tile 0 of a block: O and the row sum are still zero, the factor stays 1)
      fold_shift(mxs, s, true);
#pragma unroll
      for (int qi = 0; qi < QB; ++qi) alpha[qi] = 1.0f;
    }
    return moved;
  };
  // alpha is exactly 1 for every lane whose maximum did not move: the 16*DB
  // multiplies are skipped unless some lane of the wave needs them
  auto rescale = [&](bool moved) __attribute__((always_inline)) {
    if (__any(moved)) {
#pragma unroll
      for (int qi = 0; qi < QB; ++qi)
#pragma unroll
        for (int d = 0; d < DB; ++d)
#pragma unroll
          for (int e = 0; e < 16; ++e) o[qi][d][e] *= alpha[qi];
    }
  };
  // One scheduling region: the score product of tile t+1 on the matrix pipe, the
  // exponentials and row sums of tile t (maximum m_run, rescale factor alpha) on
  // the vector ALU.
  u32x4 pf[QB][4];
  auto softmax_and_next_scores = [&](int t) __attribute__((always_inline)) {  // (one query block per wave)
    const unsigned char *sKn = sKbase + ((tb + t + 1) % NSTG) * TILE_BYTES;
#pragma unroll
    for (int blk = 0; blk < 2; ++blk)
#pragma unroll
      for (int e = 0; e < 16; ++e) s_nxt[0][blk][e] = 0.0f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int blk = 0; blk < 2; ++blk) {
        const u32x4 kf = *(const u32x4 *)(sKn + k_piece(blk * 32 + lrow, ks * 2 + g));
        s_nxt[0][blk] = Mfma32<DT>::run(kf, qf[0][ks], s_nxt[0][blk]);
      }
    float lsum = 0.0f;
#pragma unroll
    for (int blk = 0; blk < 2; ++blk)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        float p[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          p[j] = __builtin_amdgcn_exp2f(fmaf(s_cur[0][blk][hh * 8 + j], a.scale_log2, -m_run[0]));
          lsum += p[j];
        }
        pf[0][blk * 2 + hh] = pack8<DT>(p);
      }
    l_run[0] = l_run[0] * alpha[0] + lsum;
    Interleave3<0, 2 * KS>::run();
    __builtin_amdgcn_sched_barrier(0);
  };
  // The transposed V operand of P.V step (kk, d): V rows kk*16.., head-dim block d.  The two transposing reads
  // of a fragment are written as instructions: through the builtin the compiler puts a vmcnt(0) in front of the
  // first of them that follows a tile request (it cannot tell that the request writes another stage), and every
  // iteration then waited in its middle for the K and V tiles it had asked for at its head.  As instructions they
  // are outside its bookkeeping; v_landed, on the fragment, is the wait (LDS answers in order: lgkmcnt(N) says
  // "all but the latest N").  v_lane[d]: the lane's part of the address, first row g*4 + (r>>2) of key block 0;
  // the piece swizzle has a period of RP * WIN = 4 rows, so key block kk and the fragment's second half (8 rows
  // on) are immediates.
  static_assert(8 % (RP * WIN) == 0, "the V piece swizzle must repeat every 8 rows");
  unsigned v_lane[DB];
  {
    const int r = lane & 15;
#pragma unroll
    for (int d = 0; d < DB; ++d) {
      const int col = d * 32 + ((lane >> 4) & 1) * 16 + (r & 3) * 4;
      v_lane[d] = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)sVbase +
                  (unsigned)(v_piece(g * 4 + (r >> 2), col >> 3) + (col & 7) * 2);
    }
  }
  // (va: v_lane plus whatever of the stage's offset is not in the immediate OFF)
  auto issue_v = [&](const unsigned (&va)[DB], auto off_tag, int kk, int d, u32x4 &vf) __attribute__((always_inline)) {
    constexpr int OFF = decltype(off_tag)::value;
    u32x2 lo2, hi2;
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(lo2) : "v"(va[d]), "i"(OFF + kk * 16 * ROW_BYTES));
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(hi2) : "v"(va[d]), "i"(OFF + kk * 16 * ROW_BYTES + 8 * ROW_BYTES));
    vf[0] = lo2[0]; vf[1] = lo2[1]; vf[2] = hi2[0]; vf[3] = hi2[1];
  };
  auto v_landed = [&](auto newer_tag, u32x4 &vf) __attribute__((always_inline)) {
    constexpr int NEWER = decltype(newer_tag)::value;  // LDS instructions issued behind the fragment's two
    static_assert(NEWER == 0 || NEWER == 2, "fragments in flight");
    if constexpr (NEWER == 0) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(vf));
    else asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(vf));
  };
  // a stage's offset as an immediate where the stage is a constant of the loop's copy and the offsets fit 16 bits
  auto v_stage = [&](auto stage_tag, int stage, unsigned (&va)[DB]) __attribute__((always_inline)) {
    constexpr int STG = decltype(stage_tag)::value;
    constexpr bool IMM = STG >= 0 && STG * TILE_BYTES + 56 * ROW_BYTES < 65536;
#pragma unroll
    for (int d = 0; d < DB; ++d) va[d] = IMM ? v_lane[d] : v_lane[d] + (unsigned)(stage * TILE_BYTES);
    return std::integral_constant<int, IMM ? STG * TILE_BYTES : 0>{};
  };

  // The barrier at the head of iteration t publishes K(t+1) and V(t) and retires K(t) and V(t-1),
  // whose stages then receive K(t+NSTG) and V(t+NSTG-1).  PP: the barrier that opens the slot of this wave's
  // phase A of tile tt (head_of) or phase B (mid_of), with the slot's share of requests (see the kernel's head).
  constexpr int WAIT_ONE_BATCH = (NI & 15) | (7 << 4) | (15 << 8) | ((NI >> 4) << 14);  // all but the latest NI requests
  // (PP) what a wave requests at the barrier in front of its phase A (h) and of its phase B (m), by group, as
  // data: a branch on the group inside the iteration cost the register allocation 64 bytes of scratch
  const bool odd_grp = PP && grp != 0;
  const __amdgpu_buffer_rsrc_t rsrc_h = odd_grp ? rsrc_v : rsrc_k, rsrc_m = odd_grp ? rsrc_k : rsrc_v;
  unsigned char *const base_h = odd_grp ? sVbase : sKbase, *const base_m = odd_grp ? sKbase : sVbase;
  const unsigned adv_h = (unsigned)(FA_BKV * 2) * (unsigned)(odd_grp ? a.v_ss : a.k_ss);
  const unsigned adv_m = (unsigned)(FA_BKV * 2) * (unsigned)(odd_grp ? a.k_ss : a.v_ss);
  unsigned voff_h[NI], voff_m[NI];
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    voff_h[i] = odd_grp ? v_voff[i] : k_voff[i];
    voff_m[i] = odd_grp ? k_voff[i] : v_voff[i];
  }
  auto slot_load = [&](__amdgpu_buffer_rsrc_t rsrc, const unsigned (&voff)[NI], unsigned adv, unsigned char *dst) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < NI; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          rsrc, (__attribute__((address_space(3))) void *)(dst + (i * WAVES + wave_u) * RPI * ROW_BYTES), 16,
          (int)(voff[i] + adv), 0, 0, 0);
  };
  auto head_of = [&](int tt) __attribute__((always_inline)) {
    if constexpr (PP) {
      __builtin_amdgcn_s_waitcnt(WAIT_ONE_BATCH);
      __builtin_amdgcn_s_barrier();
      // waves 0-3: K(tt+2) into stage tt % 2; waves 4-7: V(tt+1) into stage (tt+1) % 2
      slot_load(rsrc_h, voff_h, (unsigned)(tt + 2 - grp) * adv_h, base_h + ((tt + grp) % NSTG) * TILE_BYTES);
    } else if constexpr (PAIR_SYNC) {
      if ((tt & 1) == 0) {
        __builtin_amdgcn_s_waitcnt(WAIT_TILES);
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        load_k(tt + 3, sKbase + ((tt + 3) % NSTG) * TILE_BYTES);
        load_v(tt + 2, sVbase + ((tt + 2) % NSTG) * TILE_BYTES);
        load_k(tt + 4, sKbase + ((tt + 4) % NSTG) * TILE_BYTES);
        load_v(tt + 3, sVbase + ((tt + 3) % NSTG) * TILE_BYTES);
      }
    } else {
      __builtin_amdgcn_s_waitcnt(WAIT_TILES);  // K(tt+1) and V(tt), requested NSTG-1 iterations ago
      // (the barrier alone: with the fences of __syncthreads() the compiler waits for every request in flight,
      // and a ring of three or four stages is no deeper than two)
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      load_k(ahead(tt + NSTG), sKbase + ((tb + tt) % NSTG) * TILE_BYTES);
      load_v(ahead(tt + NSTG - 1), sVbase + ((tb + tt + NSTG - 1) % NSTG) * TILE_BYTES);
    }
  };
  auto mid_of = [&](int tt) __attribute__((always_inline)) {
    if constexpr (PP) {
      __builtin_amdgcn_s_waitcnt(WAIT_ONE_BATCH);
      __builtin_amdgcn_s_barrier();
      // waves 0-3: V(tt+1) into stage (tt+1) % 2; waves 4-7: K(tt+3) into stage (tt+1) % 2
      slot_load(rsrc_m, voff_m, (unsigned)(tt + 1 + 2 * grp) * adv_m, base_m + ((tt + 1) % NSTG) * TILE_BYTES);
    }
  };

  // DEFER: the requests of an iteration are not issued in a block behind its barrier, where they hold every wave
  // of the workgroup at once (a request holds its wave for some 130 cycles, and the matrix pipes stand still),
  // but one by one behind the MFMAs of the first k-steps of phase A.
  constexpr bool DEFER = EARLY_MAX && !PP && !PAIR_SYNC;
  auto head_wait = [&](int tt) __attribute__((always_inline)) {
    if constexpr (DEFER) {
      __builtin_amdgcn_s_waitcnt(WAIT_TILES);
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
    } else {
      head_of(tt);
    }
  };
  // request r of iteration tt: r < NI a piece of K(tt+NSTG), else a piece of V(tt+NSTG-1)
  auto request_nth = [&](int tt, int r) __attribute__((always_inline)) {
    if (r < NI) {
      const unsigned adv = (unsigned)ahead(tt + NSTG) * (unsigned)(FA_BKV * 2) * (unsigned)a.k_ss;
      unsigned char *dst = sKbase + ((tb + tt) % NSTG) * TILE_BYTES;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          rsrc_k, (__attribute__((address_space(3))) void *)(dst + (r * WAVES + wave_u) * RPI * ROW_BYTES), 16, (int)(k_voff[r] + adv), 0, 0, 0);
    } else {
      const unsigned adv = (unsigned)ahead(tt + NSTG - 1) * (unsigned)(FA_BKV * 2) * (unsigned)a.v_ss;
      unsigned char *dst = sVbase + ((tb + tt + NSTG - 1) % NSTG) * TILE_BYTES;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          rsrc_v, (__attribute__((address_space(3))) void *)(dst + ((r - NI) * WAVES + wave_u) * RPI * ROW_BYTES), 16,
          (int)(v_voff[r - NI] + adv), 0, 0, 0);
    }
  };

  // One iteration, compiled twice: EDGE tiles (sequence end or causal diagonal)
  // mask scores with selects, interior tiles do not test at all.  Either body is
  // branch-free up to the optional rescale, so MFMAs and vector-ALU work can be
  // interleaved instruction by instruction.  For EARLY_MAX the tag describes
  // tile t+1, the one whose maximum the iteration takes.
  // cur / nxt: the score arrays of tile t (read) and tile t+1 (written); with copy_tag the new scores are
  // moved into cur at the end, without it the caller swaps the roles of the two arrays for the next tile
  // (the interior loop does, two tiles per trip: the move is 16 of a tile's 165 vector instructions).
  // stage_tag: the ring stage of tile t where the caller knows it at compile time (the interior loop, which
  // starts its pairs on stage 0 of a two-stage ring), else -1: with a constant stage the LDS addresses of the
  // K and V fragments are loop invariants plus immediates instead of an addition per read group.
  auto iteration_on = [&](int t, auto edge_tag, f32x16 (&cur)[QB][2], f32x16 (&nxt)[QB][2], auto copy_tag, auto stage_tag) __attribute__((always_inline)) {
    constexpr int STG = decltype(stage_tag)::value;
    unsigned va[DB];
    const auto v_off = v_stage(stage_tag, STG >= 0 ? STG : (tb + t) % NSTG, va);
    if constexpr (!EARLY_MAX) {
      const bool moved = take_max(t, edge_tag, s_cur);
      rescale(moved);
      __builtin_amdgcn_sched_barrier(0);
      softmax_and_next_scores(t);
#pragma unroll
      for (int kk = 0; kk < 4; ++kk)
#pragma unroll
        for (int d = 0; d < DB; ++d) {
          u32x4 vf;
          issue_v(va, v_off, kk, d, vf);
          v_landed(std::integral_constant<int, 0>{}, vf);
          o[0][d] = Mfma32<DT>::run(vf, pf[0][kk], o[0][d]);
        }
    } else {
      // Both phases are written as short chunks -- a few MFMAs and their share of
      // the vector-ALU work -- each closed by a full scheduling fence: MFMA issue
      // is asynchronous, so the vector instructions of a chunk execute while the
      // matrix pipe works on its MFMAs, whatever order the compiler gives them
      // inside the chunk.
      constexpr bool EDGE = decltype(edge_tag)::value;
      const unsigned char *sKn = sKbase + (STG >= 0 ? (STG + 1) % NSTG : (tb + t + 1) % NSTG) * TILE_BYTES;
      // ---- phase A: S^T(t+1) = K(t+1) Q^T  with  P(t) = exp2(S(t)*scale - m), row sums ----
      // chunk ks: the 2*QB MFMAs of k-step ks (operands read one chunk ahead) and
      // 32*QB/KS of the 32*QB exponentials
      constexpr int EPC = 32 * QB / KS;  // exponentials per chunk
      static_assert((32 * QB) % KS == 0 && (EPC == 4 || EPC == 8 || EPC == 16), "exponentials must divide over the k-steps");
      __builtin_amdgcn_sched_barrier(0);
      // The wave runs this phase at raised priority: a SIMD holds two waves (of two workgroups, or of one
      // eight-wave workgroup) that are not in step, and the one inside its exponentials -- the vector ALU's
      // longest stretch of a tile -- is served first, so that it reaches phase B, where the matrix pipe and LDS
      // latency dominate, while its neighbour takes the vector ALU in turn (measured on one device: dense
      // 944 -> 929 us, causal pairs 528 -> 509 us; the same priority on phase B instead changed nothing).
      __builtin_amdgcn_s_setprio(1);
      u32x4 kf0 = *(const u32x4 *)(sKn + k_piece(lrow, g));
      u32x4 kf1 = *(const u32x4 *)(sKn + k_piece(32 + lrow, g));
      float lsum[QB];
#pragma unroll
      for (int qi = 0; qi < QB; ++qi) lsum[qi] = 0.0f;
      float p[8];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        u32x4 kn0 = kf0, kn1 = kf1;
        if (ks + 1 < KS) {
          kn0 = *(const u32x4 *)(sKn + k_piece(lrow, (ks + 1) * 2 + g));
          kn1 = *(const u32x4 *)(sKn + k_piece(32 + lrow, (ks + 1) * 2 + g));
        }
#pragma unroll
        for (int qi = 0; qi < QB; ++qi) {
          // (the first k-step starts from the MFMA's constant zero: no 32 registers to clear per tile)
          const f32x16 zero16 = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
          // (SHIFT: from -m, and the shift of the whole block costs no instruction)
          nxt[qi][0] = Mfma32<DT>::run(kf0, qf[qi][ks], ks == 0 ? (SHIFT ? negm[SHIFT ? qi : 0] : zero16) : nxt[qi][0]);
          nxt[qi][1] = Mfma32<DT>::run(kf1, qf[qi][ks], ks == 0 ? (SHIFT ? negm[SHIFT ? qi : 0] : zero16) : nxt[qi][1]);
        }
        if constexpr (DEFER) {
          constexpr int PER_CHUNK = (2 * NI + KS - 1) / KS;
#pragma unroll
          for (int x = 0; x < PER_CHUNK; ++x)
            if (ks * PER_CHUNK + x < 2 * NI) request_nth(t, ks * PER_CHUNK + x);
        }
#pragma unroll
        for (int j = 0; j < EPC; ++j) {
          const int idx = ks * EPC + j;  // 0..32*QB-1 over (query block, blk, element): block idx/32, blk (idx%32)/16
          const int qi = idx >> 5, w = idx & 31;
          const float x = SHIFT ? __builtin_amdgcn_exp2f(cur[qi][w >> 4][w & 15])
                                : __builtin_amdgcn_exp2f(fmaf(cur[qi][w >> 4][w & 15], a.scale_log2, -m_run[qi]));
          p[idx & 7] = x;
          lsum[qi] += x;
          if ((idx & 7) == 7) pf[qi][w >> 3] = pack8<DT>(p);
        }
        // The row sum is not needed before the next iteration, and the compiler would sink
        // its additions, one dependent chain, out of the chunks into the tail of the loop
        // body, behind every MFMA: pinning the partial sum at the end of each chunk keeps
        // the additions where the matrix pipe hides them.
#pragma unroll
        for (int qi = 0; qi < QB; ++qi) asm volatile("" : "+v"(lsum[qi]));
        kf0 = kn0;
        kf1 = kn1;
        if constexpr (QB > 1) MfmaValu<0, 2 * QB, (EPC * 7 / 2 + 2 * QB - 1) / (2 * QB), 2>::run();
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int qi = 0; qi < QB; ++qi) l_run[qi] = l_run[qi] * alpha[qi] + lsum[qi];
      __builtin_amdgcn_s_setprio(0);
      mid_of(t);

      // ---- phase B: O^T += V^T(t) P^T(t)  with  the running maximum of tile t+1 ----
      // chunk kk: the DB*QB MFMAs of key block kk (operand reads one fragment ahead) and
      // the maximum over 8 of the 32 scores of S(t+1) of each query block
      const int kv0n = (t + 1) * FA_BKV;
      float mx[QB];
#pragma unroll
      for (int qi = 0; qi < QB; ++qi) mx[qi] = -INFINITY;
      u32x4 vr[2];  // the fragment being multiplied and the one on its way
      issue_v(va, v_off, 0, 0, vr[0]);
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
#pragma unroll
        for (int d = 0; d < DB; ++d) {
          const int idx = kk * DB + d;
          if (idx + 1 < 4 * DB) {
            issue_v(va, v_off, (idx + 1) / DB, (idx + 1) % DB, vr[(idx + 1) & 1]);
            v_landed(std::integral_constant<int, 2>{}, vr[idx & 1]);
          } else {
            v_landed(std::integral_constant<int, 0>{}, vr[idx & 1]);
          }
#pragma unroll
          for (int qi = 0; qi < QB; ++qi) o[qi][d] = Mfma32<DT>::run(vr[idx & 1], pf[qi][kk], o[qi][d]);
        }
#pragma unroll
        for (int qi = 0; qi < QB; ++qi)
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const int idx = kk * 8 + j, blk = idx >> 4, e = idx & 15;
            if constexpr (EDGE) nxt[qi][blk][e] = blk * 32 + (e >> 2) * 8 + (e & 3) > last_key[qi] - kv0n ? -INFINITY : nxt[qi][blk][e];
            mx[qi] = fmaxf(mx[qi], nxt[qi][blk][e]);
          }
        if constexpr (QB > 1) MfmaValu<0, DB * QB, (8 * QB * (EDGE ? 4 : 1) + DB * QB - 1) / (DB * QB), 2 * DB>::run();
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (SHIFT) {
        fold_shift(mx, nxt, false);
      } else {
        bool moved = false;
#pragma unroll
        for (int qi = 0; qi < QB; ++qi) {
          const float mw = max_with_lane_xor32(mx[qi]);
          moved |= lazy_running_max(m_run[qi], mw * a.scale_log2, alpha[qi]);
        }
        rescale(moved);
      }
    }
    if constexpr (decltype(copy_tag)::value) {
#pragma unroll
      for (int qi = 0; qi < QB; ++qi)
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) cur[qi][blk] = nxt[qi][blk];
    }
  };
  // (the form every caller but the interior loop uses: scores of tile t in s_cur on entry, of tile t+1 on exit)
  auto iteration = [&](int t, auto edge_tag) __attribute__((always_inline)) {
    iteration_on(t, edge_tag, s_cur, s_nxt, std::true_type{}, std::integral_constant<int, -1>{});
  };

  // The iteration of the last tile any query of the wave may keep: its exponentials and its P.V product.
  // The tile after it has no key for this wave: no score product and no maximum.
  auto last_live_iteration = [&](int t) __attribute__((always_inline)) {
    unsigned va[DB];
    const auto v_off = v_stage(std::integral_constant<int, -1>{}, (tb + t) % NSTG, va);
#pragma unroll
    for (int qi = 0; qi < QB; ++qi) {
      float lsum = 0.0f;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        float p[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          p[j] = SHIFT ? __builtin_amdgcn_exp2f(s_cur[qi][w >> 1][(w & 1) * 8 + j])
                       : __builtin_amdgcn_exp2f(fmaf(s_cur[qi][w >> 1][(w & 1) * 8 + j], a.scale_log2, -m_run[qi]));
          lsum += p[j];
        }
        pf[qi][w] = pack8<DT>(p);
      }
      l_run[qi] = l_run[qi] * alpha[qi] + lsum;
    }
    mid_of(t);
#pragma unroll
    for (int kk = 0; kk < 4; ++kk)
#pragma unroll
      for (int d = 0; d < DB; ++d) {
        u32x4 vf;
        issue_v(va, v_off, kk, d, vf);
        v_landed(std::integral_constant<int, 0>{}, vf);
#pragma unroll
        for (int qi = 0; qi < QB; ++qi) o[qi][d] = Mfma32<DT>::run(vf, pf[qi][kk], o[qi][d]);
      }
  };
#pragma unroll 1
  for (item = 0; item < ITEMS; ++item) {
  if constexpr (ITEMS > 1) {
    if (item > 0) {
      q0 = item_block(item) * BQ;
      q_wave0 = q0 + wave * WQ;
      wave_last_key = a.causal && q0 + (wave_u + 1) * WQ - 1 < S - 1 ? q0 + (wave_u + 1) * WQ - 1 : S - 1;
      ntiles = tiles_of(q0);
#pragma unroll
      for (int qi = 0; qi < QB; ++qi) {
        q_mine[qi] = q_wave0 + qi * 32 + lrow;
        last_key[qi] = (a.causal && q_mine[qi] < S - 1 ? q_mine[qi] : S - 1) - g * 4;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          if (ks < KQN) qf[qi][ks] = qf_next[qi][ks < KQN ? ks : 0];
          else qf[qi][ks] = prescale(*(const u32x4 *)(sPark + ((wave * (KS - KQN) + ks - KQN) * 64 + lane) * 16));
        }
      }
    }
  }
#pragma unroll
  for (int qi = 0; qi < QB; ++qi) {
#pragma unroll
    for (int d = 0; d < DB; ++d)
#pragma unroll
      for (int e = 0; e < 16; ++e) o[qi][d][e] = 0.0f;
    m_run[qi] = SHIFT ? 0.0f : -1.0e30f;
    l_run[qi] = 0.0f;
    alpha[qi] = 1.0f;
    if constexpr (SHIFT) {
#pragma unroll
      for (int e = 0; e < 16; ++e) negm[qi][e] = 0.0f;
    }
  }
  // (a later item finds its first tiles requested by the item before it, and published by that item's last barrier)
  __builtin_amdgcn_s_waitcnt(WAIT_TILES);
  __syncthreads();
  scores(sKbase + (tb % NSTG) * TILE_BYTES, s_cur);

  // Interior tiles first, then the edge tiles (they are the last ones: the tail of
  // the sequence and, under a causal mask, the tiles that reach the diagonal of
  // this wave's queries), each in a loop of its own with a single body.
  int first_edge = ntiles;
  if (ntiles * FA_BKV > S) first_edge = ntiles - 1;
  if (a.causal) {
    const int fe = (q_wave0 + 1) / FA_BKV;  // first tile with kv0 + 63 > q_wave0
    first_edge = fe < first_edge ? fe : first_edge;
  }
  first_edge = __builtin_amdgcn_readfirstlane(first_edge);
  if constexpr (EARLY_MAX) {
    // the maximum of tile 0 has no P.V to hide under; O is still zero, no rescale
    if (first_edge == 0) (void)take_max(0, std::true_type{}, s_cur);
    else (void)take_max(0, std::false_type{}, s_cur);
  }
  // iteration t handles tile t, and with EARLY_MAX the maximum of tile t+1: its
  // body is the interior one while that tile is interior
  const int interior_end = EARLY_MAX ? first_edge - 1 : first_edge;
  int t = 0;
  // (PP) waves 4-7 sit out the first slot
  if constexpr (PP) {
    if (grp == 1) {
      __builtin_amdgcn_s_waitcnt(WAIT_ONE_BATCH);
      __builtin_amdgcn_s_barrier();
      load_k(2, sKbase);
    }
  }
  if constexpr (EARLY_MAX && QB == 1) {
    // Two tiles per trip with the score arrays changing roles, and (two-stage rings) the pairs starting on
    // ring stage 0: a single tile in front if the first one lies on stage 1, a single one behind if one is left.
    // (One query block per wave: with two the kernel has no register to spare and spills.)
    // (one-block members only: the four-wave paired kernel at head dimension 128 spills four registers with
    // the hoisted addresses, and the eight-wave paired kernels measured level with and without)
    constexpr bool CONST_STAGES = NSTG == 2 && ITEMS == 1;
    constexpr int S0 = CONST_STAGES ? 0 : -1, S1 = CONST_STAGES ? 1 : -1;
    if (CONST_STAGES && t < interior_end && ((tb + t) & 1)) {
      head_wait(t);
      iteration(t, std::false_type{});
      ++t;
    }
    for (; t + 1 < interior_end; t += 2) {
      head_wait(t);
      iteration_on(t, std::false_type{}, s_cur, s_nxt, std::false_type{}, std::integral_constant<int, S0>{});
      head_wait(t + 1);
      iteration_on(t + 1, std::false_type{}, s_nxt, s_cur, std::false_type{}, std::integral_constant<int, S1>{});
    }
    if (t < interior_end) {
      head_wait(t);
      iteration(t, std::false_type{});
      ++t;
    }
  } else {
    for (; t < interior_end; ++t) {
      head_wait(t);
      iteration(t, std::false_type{});
    }
  }
  if constexpr (EARLY_MAX) {
    // A tile none of whose keys any query of this wave may keep -- the one after the last, and under a causal
    // mask the tiles past the wave's diagonal -- gets no score product, no maximum, no exponentials and no P.V
    // product: full iterations while tile t+1 has a key for the wave, the softmax and P.V of the last such
    // tile, and then only the workgroup's barriers and tile requests.  (Per block of 128 queries under a
    // causal mask that is one and a half iterations of two of the four waves and half an iteration of the others.)
    const int last_live = wave_last_key / FA_BKV;
    for (; t < last_live; ++t) {
      head_wait(t);
      iteration(t, std::true_type{});
    }
    head_of(t);
    last_live_iteration(t);
    for (++t; t < ntiles; ++t) {
      head_of(t);
      mid_of(t);
    }
    // (PP) waves 0-3 sit out the last slot
    if constexpr (PP) {
      if (grp == 0) {
        __builtin_amdgcn_s_waitcnt(WAIT_ONE_BATCH);
        __builtin_amdgcn_s_barrier();
      }
    }
  } else {
    for (; t < ntiles; ++t) {
      __builtin_amdgcn_s_waitcnt(WAIT_TILES);
      __syncthreads();
      load_k(ahead(t + NSTG), sKbase + ((tb + t) % NSTG) * TILE_BYTES);
      load_v(ahead(t + NSTG - 1), sVbase + ((tb + t + NSTG - 1) % NSTG) * TILE_BYTES);
      iteration(t, std::true_type{});
    }
  }
  {
    // O from registers: the lanes of the two halves of the wave hold head-dim values 0..3 and 4..7 of a group
    // of 8; one swap per register between the halves gives every lane 16 bytes of one row.  (No staging in
    // LDS: it would lie under the tiles a later item has in flight, it cost a wait, two barriers and the bank
    // conflicts of 8-byte writes at a row pitch -- 10 to 18 % of the kernel's LDS cycles -- per block.)
#pragma unroll
    for (int qi = 0; qi < QB; ++qi) {
      const float l_tot = l_run[qi] + __shfl_xor(l_run[qi], 32, 64);
      const float inv_l = 1.0f / l_tot;
      unsigned short *orow = Og + (long long)q_mine[qi] * a.o_ss;
#pragma unroll
      for (int d = 0; d < DB; ++d)
#pragma unroll
        for (int vp = 0; vp < 2; ++vp) {
          u32x2 w[2];
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            float x[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) x[e] = o[qi][d][(vp * 2 + half) * 4 + e] * inv_l;
            if constexpr (DT == DT_F16) {
              f16x4 hq = {(_Float16)x[0], (_Float16)x[1], (_Float16)x[2], (_Float16)x[3]};
              w[half] = __builtin_bit_cast(u32x2, hq);
            } else {
              bf16x4 hq = {(__bf16)x[0], (__bf16)x[1], (__bf16)x[2], (__bf16)x[3]};
              w[half] = __builtin_bit_cast(u32x2, hq);
            }
          }
          unsigned e0 = w[0][0], e1 = w[0][1], o0 = w[1][0], o1 = w[1][1];
          asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(e0), "+v"(o0));
          asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(e1), "+v"(o1));
          const u32x4 row16 = {e0, e1, o0, o1};
          if (q_mine[qi] < S) *(u32x4 *)(orow + d * 32 + (vp * 2 + g) * 8) = row16;
        }
    }
    tb += ntiles;
  }
  }  // items
  // (the last item's look-ahead requests write LDS: they must have landed before the workgroup gives it up)
  __builtin_amdgcn_s_waitcnt(0x0f70);
}

template <int D, bool EARLY_MAX, int WAVES, int NSTG, int QB = 1, int ITEMS = 1, bool SHIFT = false, bool PP = false>
static int launch_fa2_pipe(const AttentionArgs &a, int dtype, hipStream_t stream) {
  if (PP && a.causal) return (int)hipErrorInvalidValue;  // (its feasibility test keeps such a call away)
  // the K and V rings (O leaves from registers), and where they are parked half of the next block's queries
  constexpr size_t lds = 2 * (size_t)NSTG * FA_BKV * D * 2 +
                         (fa2_pipe_parks_queries(D, QB, ITEMS, SHIFT) ? (size_t)WAVES * (D / 32) * 1024 : 0);
  const int nqb = (a.S + 32 * QB * WAVES - 1) / (32 * QB * WAVES);
  if (nqb % ITEMS != 0) return (int)hipErrorInvalidValue;  // (feasible_pairs keeps such a call away)
  const dim3 grid((unsigned)(nqb / ITEMS * a.B * a.H)), block(WAVES * 64);
#define TRACEA_FA_LAUNCH(DTV)                                                                  \
  do {                                                                                         \
    auto kfn = fa2_fwd_pipe_kernel<DTV, D, EARLY_MAX, WAVES, NSTG, QB, ITEMS, SHIFT, PP>;      \
    static bool attr_done = false;                                                             \
    if (!attr_done) {                                                                          \
      hipError_t e = hipFuncSetAttribute((const void *)kfn,                                    \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
      if (e != hipSuccess) return (int)e;                                                      \
      attr_done = true;                                                                        \
    }                                                                                          \
    hipLaunchKernelGGL(kfn, grid, block, lds, stream, a);                                      \
    return (int)hipGetLastError();                                                             \
  } while (0)
  if (dtype == DT_F16) TRACEA_FA_LAUNCH(DT_F16);
  else TRACEA_FA_LAUNCH(DT_BF16);
#undef TRACEA_FA_LAUNCH
}

}  // namespace tracea_amd
#include "attention_m16_kernel.hpp"
namespace tracea_amd {

// The buffer loads address a (batch, head) slice with 32-bit byte offsets.
static bool slice_fits(const AttentionArgs &a) {
  const long long k_ext = ((long long)(a.S - 1 + 4 * FA_BKV) * a.k_ss + a.D) * 2;  // (tiles up to 3 past the end are requested)
  const long long v_ext = ((long long)(a.S - 1 + 4 * FA_BKV) * a.v_ss + a.D) * 2;
  return k_ext < (1ll << 31) && v_ext < (1ll << 31);
}
// (the running maximum is taken over raw scores, which needs a positive scale)
static bool feasible_pipe_d128(const AttentionArgs &a) { return a.D == 128 && a.scale_log2 > 0.0f && slice_fits(a); }
static bool feasible_pipe_d64(const AttentionArgs &a) { return a.D == 64 && a.scale_log2 > 0.0f && slice_fits(a); }
// (the members whose wave groups run half an iteration apart: no causal mask)
static bool feasible_dense_d128(const AttentionArgs &a) { return !a.causal && feasible_pipe_d128(a); }
static bool feasible_dense_d64(const AttentionArgs &a) { return !a.causal && feasible_pipe_d64(a); }
// Two query blocks per workgroup: an even number of blocks, and at least two K/V tiles in the lightest one.
template <int D, int BQ>
static bool feasible_pairs(const AttentionArgs &a) {
  const int nqb = (a.S + BQ - 1) / BQ;
  return a.D == D && a.scale_log2 > 0.0f && slice_fits(a) && nqb % 2 == 0 && a.S >= 2 * FA_BKV;
}

template <int D, bool V_TR>
static int launch_fa2(const AttentionArgs &a, int dtype, hipStream_t stream) {
  constexpr size_t lds = 2 * 2 * (size_t)FA_BKV * D * 2;
  const int nqb = (a.S + FA_BQ - 1) / FA_BQ;
  const dim3 grid((unsigned)(nqb * a.B * a.H)), block(FA_WAVES * 64);
#define TRACEA_FA_LAUNCH(DTV)                                                                  \
  do {                                                                                         \
    auto kfn = fa2_fwd_kernel<DTV, D, V_TR>;                                                   \
    static bool attr_done = false;                                                             \
    if (!attr_done) {                                                                          \
      hipError_t e = hipFuncSetAttribute((const void *)kfn,                                    \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
      if (e != hipSuccess) return (int)e;                                                      \
      attr_done = true;                                                                        \
    }                                                                                          \
    hipLaunchKernelGGL(kfn, grid, block, lds, stream, a);                                      \
    return (int)hipGetLastError();                                                             \
  } while (0)
  if (dtype == DT_F16) TRACEA_FA_LAUNCH(DT_F16);
  else TRACEA_FA_LAUNCH(DT_BF16);
#undef TRACEA_FA_LAUNCH
}

static bool feasible_d128(const AttentionArgs &a) { return a.D == 128; }
static bool feasible_d64(const AttentionArgs &a) { return a.D == 64; }

// The kernel family: MFMA shape (m16: v_mfma_f32_16x16x32, attention_m16_kernel.hpp; the others 32x32x16),
// queries per workgroup (32 per wave, 4 or 8 waves), K/V ring depth (2 or 3 stages per
// tensor), head dimension, and the three kernel forms (pipe2 / pipe: direct-to-LDS tiles, maximum taken
// under the P.V MFMAs or in a phase of its own; tr / u16: the register-staged cross-check).  The tuner
// measures every feasible member (tracea_tune_fa2); the first feasible entry is the default.  (The m16
// members need 13 % more cycles than pipe2 and get a higher clock from the power limit: at B4 H32 S4096 D128
// 1055-1062 us against 1070 dense, 629-639 against 625 causal, so they are not the default.)  (Head
// dimension 128 has no 3-stage member: the third set of per-lane tile addresses does not fit the 256
// registers of two waves per SIMD and the kernel spills.)
static const AttentionVariant kAttentionVariants[] = {
    {"fa2_q128_kv64_d128_pipe2", 128, FA_BKV, 4, 2, &launch_fa2_pipe<128, true, 4, 2, 1, 1, true>, &feasible_pipe_d128, 32, 1},
    {"fa2_q128_kv64_d64_pipe2", 128, FA_BKV, 4, 2, &launch_fa2_pipe<64, true, 4, 2, 1, 1, true>, &feasible_pipe_d64, 32, 1},
    {"fa2_q128_kv64_d128_m16", 128, FA_BKV, 4, 2, &launch_fa2_m16<128, 4>, &feasible_pipe_d128, 16, 1},
    {"fa2_q128_kv64_d64_m16", 128, FA_BKV, 4, 2, &launch_fa2_m16<64, 4>, &feasible_pipe_d64, 16, 1},
    {"fa2_q256_kv64_d128_s2_m16", 256, FA_BKV, 8, 2, &launch_fa2_m16<128, 8>, &feasible_pipe_d128, 16, 1},
    {"fa2_q256_kv64_d64_s2_m16", 256, FA_BKV, 8, 2, &launch_fa2_m16<64, 8>, &feasible_pipe_d64, 16, 1},
    {"fa2_q128_kv64_d128_pipe2_x2", 128, FA_BKV, 4, 2, &launch_fa2_pipe<128, true, 4, 2, 1, 2, true>, &feasible_pairs<128, 128>, 32, 2},
    {"fa2_q128_kv64_d64_pipe2_x2", 128, FA_BKV, 4, 2, &launch_fa2_pipe<64, true, 4, 2, 1, 2, true>, &feasible_pairs<64, 128>, 32, 2},
    {"fa2_q256_kv64_d128_s2_pipe2_x2", 256, FA_BKV, 8, 2, &launch_fa2_pipe<128, true, 8, 2, 1, 2, true>, &feasible_pairs<128, 256>, 32, 2},
    {"fa2_q256_kv64_d64_s2_pipe2_x2", 256, FA_BKV, 8, 2, &launch_fa2_pipe<64, true, 8, 2, 1, 2, true>, &feasible_pairs<64, 256>, 32, 2},
    {"fa2_q256_kv64_d128_w4_pipe2", 256, FA_BKV, 4, 2, &launch_fa2_pipe<128, true, 4, 2, 2>, &feasible_pipe_d128, 32, 1},
    {"fa2_q256_kv64_d64_w4_pipe2", 256, FA_BKV, 4, 2, &launch_fa2_pipe<64, true, 4, 2, 2>, &feasible_pipe_d64, 32, 1},
    {"fa2_q256_kv64_d128_s2_pipe2", 256, FA_BKV, 8, 2, &launch_fa2_pipe<128, true, 8, 2, 1, 1, true>, &feasible_pipe_d128, 32, 1},
    {"fa2_q256_kv64_d64_s2_pipe2", 256, FA_BKV, 8, 2, &launch_fa2_pipe<64, true, 8, 2, 1, 1, true>, &feasible_pipe_d64, 32, 1},
    {"fa2_q256_kv64_d128_s4_pipe2", 256, FA_BKV, 8, 4, &launch_fa2_pipe<128, true, 8, 4, 1, 1, true>, &feasible_pipe_d128, 32, 1},
    {"fa2_q256_kv64_d64_s4_pipe2", 256, FA_BKV, 8, 4, &launch_fa2_pipe<64, true, 8, 4, 1, 1, true>, &feasible_pipe_d64, 32, 1},
    {"fa2_q128_kv64_d64_s4_pipe2", 128, FA_BKV, 4, 4, &launch_fa2_pipe<64, true, 4, 4, 1, 1, true>, &feasible_pipe_d64, 32, 1},
    {"fa2_q256_kv64_d128_s2_pp", 256, FA_BKV, 8, 2, &launch_fa2_pipe<128, true, 8, 2, 1, 1, true, true>, &feasible_dense_d128, 32, 1, 1},
    {"fa2_q256_kv64_d64_s2_pp", 256, FA_BKV, 8, 2, &launch_fa2_pipe<64, true, 8, 2, 1, 1, true, true>, &feasible_dense_d64, 32, 1, 1},
    {"fa2_q256_kv64_d64_s3_pipe2", 256, FA_BKV, 8, 3, &launch_fa2_pipe<64, true, 8, 3, 1, 1, true>, &feasible_pipe_d64, 32, 1},
    {"fa2_q128_kv64_d64_s3_pipe2", 128, FA_BKV, 4, 3, &launch_fa2_pipe<64, true, 4, 3, 1, 1, true>, &feasible_pipe_d64, 32, 1},
    {"fa2_q128_kv64_d128_pipe", 128, FA_BKV, 4, 2, &launch_fa2_pipe<128, false, 4, 2>, &feasible_pipe_d128, 32, 1},
    {"fa2_q128_kv64_d64_pipe", 128, FA_BKV, 4, 2, &launch_fa2_pipe<64, false, 4, 2>, &feasible_pipe_d64, 32, 1},
    {"fa2_q128_kv64_d128_tr", FA_BQ, FA_BKV, FA_WAVES, 2, &launch_fa2<128, true>, &feasible_d128, 32, 1},
    {"fa2_q128_kv64_d128_u16", FA_BQ, FA_BKV, FA_WAVES, 2, &launch_fa2<128, false>, &feasible_d128, 32, 1},
    {"fa2_q128_kv64_d64_tr", FA_BQ, FA_BKV, FA_WAVES, 2, &launch_fa2<64, true>, &feasible_d64, 32, 1},
    {"fa2_q128_kv64_d64_u16", FA_BQ, FA_BKV, FA_WAVES, 2, &launch_fa2<64, false>, &feasible_d64, 32, 1},
};

int attention_variant_count() { return (int)(sizeof(kAttentionVariants) / sizeof(kAttentionVariants[0])); }
const AttentionVariant &attention_variant(int i) { return kAttentionVariants[i]; }

}  // namespace tracea_amd
