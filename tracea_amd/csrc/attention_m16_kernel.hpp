// FlashAttention-2 forward on v_mfma_f32_16x16x32: the two-phase pipelined form of fa2_fwd_pipe_kernel
// (K/V tiles by direct-to-LDS loads, K one tile ahead of V, score product of tile t+1 under the
// exponentials of tile t, P.V of tile t under the running maximum of tile t+1) with the other MFMA shape.
// Same math (src/kernels/attention/cuda_emitter.rs:126-237 of the reference), same tiles, same LDS traffic;
// what changes is the register side: a 16x16x32 MFMA carries 32 k per pass over its accumulators where
// 32x32x16 carries 16, half the accumulator traffic per flop, and on a device that is power-limited under
// this kernel the clock rises with the energy saved.
//
// Layouts.  A wave owns 32 queries as two blocks of 16.  S^T block (kb, qb) = K[16 keys] Q^T[16 queries]:
// lane l holds query l & 15 of block qb and keys 16 kb + 4 (l >> 4) + e, e = 0..3.  A query's 64 scores of a
// tile are spread over the four 16-lane groups: maximum and sum take two cross-lane exchanges.  P^T for the
// 32-key step s of O^T += V^T P^T is the pair of blocks kb = 2s, 2s+1 of the lane, converted to 16 bit: slots
// 0-3 are keys 32 s + 4 g + e, slots 4-7 keys 32 s + 16 + 4 g + e (g = l >> 4), and the V^T operand
// enumerates the keys in that order: two transposing reads of four consecutive key rows each.
// O^T block (db, qb): lane l holds query l & 15, head-dim 16 db + 4 g + e.
//
// The softmax shift rides the score product.  The queries are multiplied by scale * log2(e) when they are
// loaded (rounded once more to the operand type: a relative 2^-9 on q, about 2^-9 on a probability), and
// the first MFMA of every S^T block accumulates onto a register block holding -m, the query's running
// reference maximum, instead of zero: the product comes out as z = s * scale * log2(e) - m and a
// probability is one v_exp_f32 of it, without the multiply-add per score that the vector ALU, the busiest
// unit of this kernel, spent on the shift.  The maximum of a tile is taken of z: while it stays below
// FA_RESCALE_TAU the reference stays (the lazy running maximum of fa2_fwd_pipe_kernel); when it moves, the
// tile's z are lowered by the step and O and the row sum rescaled.
#pragma once

namespace tracea_amd {

template <int DT, int D, int WAVES>
__global__ void __launch_bounds__(WAVES * 64) __attribute__((amdgpu_waves_per_eu(2, 2)))
fa2_fwd_m16_kernel(const AttentionArgs a) {
  constexpr int NSTG = 2;
  constexpr int WQ = 32, BQ = WQ * WAVES;
  constexpr int ROW_BYTES = D * 2;
  constexpr int CH = D / 8;
  constexpr int TILE_BYTES = FA_BKV * ROW_BYTES;
  constexpr int KS = D / 32;        // k-steps of the score product
  constexpr int DB = D / 16;        // head-dim blocks of O^T
  constexpr int KB = FA_BKV / 16;   // key blocks of a tile
  constexpr int PS = FA_BKV / 32;   // key steps of P.V
  constexpr int RPI = 64 / CH;
  constexpr int NI = FA_BKV / (RPI * WAVES);
  constexpr int RP = 256 / ROW_BYTES > 0 ? 256 / ROW_BYTES : 1;
  constexpr int WIN = ROW_BYTES / 64;
  static_assert(D % 32 == 0 && FA_BKV % (RPI * WAVES) == 0 && KB == 4 && PS == 2, "unsupported shape");

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  unsigned char *const sKbase = smem;
  unsigned char *const sVbase = smem + NSTG * TILE_BYTES;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int r16 = lane & 15, g4 = lane >> 4;

  const int nqb = (a.S + BQ - 1) / BQ;
  const int total = nqb * a.B * a.H;
  int vid = blockIdx.x;
  if ((total & 7) == 0) vid = (vid & 7) * (total >> 3) + (vid >> 3);
  const int bh = vid / nqb;
  const int qblk = nqb - 1 - (vid - bh * nqb);  // heavy query blocks (most keys under a causal mask) first
  const int b = bh / a.H, h = bh - b * a.H;
  const int q0 = qblk * BQ;
  const int S = a.S;

  const unsigned short *Qg = (const unsigned short *)a.Q + (long long)b * a.q_sb + (long long)h * a.q_sh;
  const unsigned short *Kg = (const unsigned short *)a.K + (long long)b * a.k_sb + (long long)h * a.k_sh;
  const unsigned short *Vg = (const unsigned short *)a.V + (long long)b * a.v_sb + (long long)h * a.v_sh;
  unsigned short *Og = (unsigned short *)a.O + (long long)b * a.o_sb + (long long)h * a.o_sh;

  const int q_wave0 = q0 + wave * WQ;
  int q_mine[2];
  u32x4 qf[2][KS];
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    q_mine[qb] = q_wave0 + qb * 16 + r16;
    const int qr = q_mine[qb] < S ? q_mine[qb] : S - 1;
    const unsigned short *qp = Qg + (long long)qr * a.q_ss + g4 * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const u32x4 raw = *(const u32x4 *)(qp + ks * 32);
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
      qf[qb][ks] = pack8<DT>(qs);
    }
  }

  // K tile: 16-byte column XOR row (conflict-free for 16 rows x one column group per 16 lanes).  V tile: the
  // four key rows of a transposing read go to the four 64-byte windows of a 256-byte span, and the two
  // 16-lane groups of a half-wave (key rows 4 apart) to different halves of a window.
  auto k_piece = [&](int row, int c) __attribute__((always_inline)) -> int {
    return row * ROW_BYTES + ((c ^ ((row / RP) & (CH - 1))) << 4);
  };
  auto v_swz = [](int row) -> int { return (((row / RP) % WIN) << 2) ^ (((row >> 2) & 1) << 1); };
  auto v_piece = [&](int row, int c) __attribute__((always_inline)) -> int { return row * ROW_BYTES + ((c ^ v_swz(row)) << 4); };

  __amdgpu_buffer_rsrc_t rsrc_k = __builtin_amdgcn_make_buffer_rsrc(
      (void *)Kg, 0, (int)(((long long)(S - 1) * a.k_ss + D) * 2), 0x00020000);
  __amdgpu_buffer_rsrc_t rsrc_v = __builtin_amdgcn_make_buffer_rsrc(
      (void *)Vg, 0, (int)(((long long)(S - 1) * a.v_ss + D) * 2), 0x00020000);
  unsigned k_voff[NI], v_voff[NI];
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int row = (i * WAVES + wave) * RPI + lane / CH;
    const int p = lane % CH;
    k_voff[i] = (unsigned)(row * (int)a.k_ss * 2 + ((p ^ ((row / RP) & (CH - 1))) << 4));
    v_voff[i] = (unsigned)(row * (int)a.v_ss * 2 + ((p ^ v_swz(row)) << 4));
  }
  auto load_k = [&](int t, unsigned char *dst) __attribute__((always_inline)) {
    const unsigned adv = (unsigned)t * (unsigned)(FA_BKV * 2) * (unsigned)a.k_ss;
#pragma unroll
    for (int i = 0; i < NI; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          rsrc_k, (__attribute__((address_space(3))) void *)(dst + (i * WAVES + wave_u) * RPI * ROW_BYTES), 16,
          (int)(k_voff[i] + adv), 0, 0, 0);
  };
  auto load_v = [&](int t, unsigned char *dst) __attribute__((always_inline)) {
    const unsigned adv = (unsigned)t * (unsigned)(FA_BKV * 2) * (unsigned)a.v_ss;
#pragma unroll
    for (int i = 0; i < NI; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          rsrc_v, (__attribute__((address_space(3))) void *)(dst + (i * WAVES + wave_u) * RPI * ROW_BYTES), 16,
          (int)(v_voff[i] + adv), 0, 0, 0);
  };

  int ntiles = (S + FA_BKV - 1) / FA_BKV;
  if (a.causal) {
    const int last_q = (q0 + BQ - 1 < S ? q0 + BQ - 1 : S - 1);
    const int need = last_q / FA_BKV + 1;
    ntiles = need < ntiles ? need : ntiles;
  }

  // (per-lane byte offsets of the K fragments, worked out once: the swizzle of row 16 kb + r16 is r16's, so a
  // fragment's offset is that of k-step ks in key block 0 plus a constant)
  static_assert(16 % (RP * CH) == 0 || (RP * CH) % 16 == 0, "K swizzle period");
  int k_off[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) k_off[ks] = k_piece(r16, ks * 4 + g4);
  auto read_k = [&](const unsigned char *sK, int kb, int ks) __attribute__((always_inline)) -> u32x4 {
    if constexpr (16 % (RP * CH) == 0) return *(const u32x4 *)(sK + k_off[ks] + kb * 16 * ROW_BYTES);
    else return *(const u32x4 *)(sK + k_piece(kb * 16 + r16, ks * 4 + g4));
  };
  // V^T operand of P.V step (s, db): head-dim block db, keys 32 s + 4 g + 0..3 and 32 s + 16 + 4 g + 0..3
  auto read_v = [&](const unsigned char *sV, int s, int db) __attribute__((always_inline)) -> u32x4 {
    const int col = db * 16 + (r16 & 3) * 4;
    const int row_lo = s * 32 + g4 * 4 + (r16 >> 2);
    const int row_hi = row_lo + 16;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (__attribute__((address_space(3))) s16x4 *)(sV + v_piece(row_lo, col >> 3) + (col & 7) * 2));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (__attribute__((address_space(3))) s16x4 *)(sV + v_piece(row_hi, col >> 3) + (col & 7) * 2));
    const u32x2 lo2 = __builtin_bit_cast(u32x2, lo), hi2 = __builtin_bit_cast(u32x2, hi);
    u32x4 vf;
    vf[0] = lo2[0]; vf[1] = lo2[1]; vf[2] = hi2[0]; vf[3] = hi2[1];
    return vf;
  };

  f32x4 o[2][DB];
#pragma unroll
  for (int qb = 0; qb < 2; ++qb)
#pragma unroll
    for (int d = 0; d < DB; ++d)
#pragma unroll
      for (int e = 0; e < 4; ++e) o[qb][d][e] = 0.0f;
  float m_run[2] = {0.0f, 0.0f}, l_run[2] = {0.0f, 0.0f}, alpha[2] = {1.0f, 1.0f};
  f32x4 negm[2];  // -m_run in every element: where the score product of a tile starts

  load_k(0, sKbase);
  load_v(0, sVbase);
  load_k(1, sKbase + TILE_BYTES);
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
  __syncthreads();

  f32x4 s_a[2][KB], s_b[2][KB];  // z of two consecutive tiles; which is which alternates
#pragma unroll
  for (int qb = 0; qb < 2; ++qb)
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int e = 0; e < 4; ++e) s_a[qb][kb][e] = 0.0f;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      const u32x4 kf = read_k(sKbase, kb, ks);
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) s_a[qb][kb] = Mfma16<DT>::run(kf, qf[qb][ks], s_a[qb][kb]);
    }

  // the maximum of a query's 64 scores: in-lane over 16, then across the four 16-lane groups
  // (v_permlane16_swap exchanges the odd 16-lane rows of its first operand with the even rows of its second,
  // v_permlane32_swap the upper half of the first with the lower half of the second: given the same value
  // twice, the two results hold a lane's own value and its partner's, in one order or the other.  Vector-ALU
  // instructions: a __shfl_xor goes through LDS and the wave would wait out two round trips per tile.)
  auto row_max = [&](float mx) __attribute__((always_inline)) -> float {
    // (written as instructions: the compiler's builtin for these swaps hands back its first result twice, and
    // the maximum of the two would be folded away.  The s_nop covers the wait the hardware asks for between
    // a vector-ALU write of an operand and the swap, which the compiler cannot see to insert.)
    float a0 = mx, a1 = mx;
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a0), "+v"(a1));
    float b0 = fmaxf(a0, a1), b1 = b0;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(b0), "+v"(b1));
    return fmaxf(b0, b1);
  };
  auto mask_tile = [&](int tile, f32x4 (&z)[2][KB]) __attribute__((always_inline)) {
    const int kv0 = tile * FA_BKV;
#pragma unroll
    for (int qb = 0; qb < 2; ++qb)
#pragma unroll
      for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int kv = kv0 + kb * 16 + g4 * 4 + e;
          const bool dead = (kv >= S) | ((a.causal != 0) & (kv > q_mine[qb]));
          z[qb][kb][e] = dead ? -INFINITY : z[qb][kb][e];
        }
  };
  // Folds the maxima mx (of z, i.e. relative to the reference) of a tile into the reference: it moves by the
  // whole excess once that exceeds TAU (`force`: by whatever it is, the first tile's case, whose reference
  // is the arbitrary 0), the tile's z follow, O is rescaled at once and alpha is the factor the row sum of the
  // earlier tiles takes with the next tile's sum (exactly 1 where nothing moved).
  auto fold_max = [&](const float (&mx)[2], f32x4 (&z)[2][KB], bool force) __attribute__((always_inline)) {
    bool moved = false;
    float step[2];
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      const float mw = row_max(mx[qb]);
      const bool mv = (force & (mw > -INFINITY)) | (mw > FA_RESCALE_TAU);
      step[qb] = mv ? mw : 0.0f;
      alpha[qb] = __builtin_amdgcn_exp2f(-step[qb]);
      m_run[qb] += step[qb];
      moved |= mv;
    }
    // (one branch for everything a moving reference touches: the multiplies are skipped unless some lane of
    // the wave needs them, alpha being exactly 1 and the step 0 for every other lane)
    if (__any(moved)) {
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) {
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
#pragma unroll
          for (int e = 0; e < 4; ++e) z[qb][kb][e] -= step[qb];
        negm[qb] = f32x4{-m_run[qb], -m_run[qb], -m_run[qb], -m_run[qb]};
#pragma unroll
        for (int d = 0; d < DB; ++d)
#pragma unroll
          for (int e = 0; e < 4; ++e) o[qb][d][e] *= alpha[qb];
      }
    }
  };

  u32x4 pf[2][PS];
  // One iteration, compiled for both roles of the score arrays and twice more for EDGE (the tile whose
  // maximum the iteration takes, t+1, reaches the end of the sequence or the causal diagonal).  Both phases
  // are short chunks of MFMAs and their share of the vector work, each closed by a scheduling fence.
  auto iteration = [&](int t, auto edge_tag, f32x4 (&s_cur)[2][KB], f32x4 (&s_nxt)[2][KB]) __attribute__((always_inline)) {
    constexpr bool EDGE = decltype(edge_tag)::value;
    const unsigned char *sV = sVbase + (t % NSTG) * TILE_BYTES;
    const unsigned char *sKn = sKbase + ((t + 1) % NSTG) * TILE_BYTES;
    // ---- phase A: z(t+1) = K(t+1) Q'^T - m  with  P(t) = exp2(z(t)) and its row sums ----
    constexpr int EPC = 32 / KS;  // exponentials per chunk (of the lane's 32 scores)
    static_assert(EPC == 8 || EPC == 16, "exponentials must come in groups of eight");
    __builtin_amdgcn_sched_barrier(0);
    u32x4 kf[KB];
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) kf[kb] = read_k(sKn, kb, 0);
    float lsum[2] = {0.0f, 0.0f};
    float p[8];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      u32x4 kn[KB];
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) kn[kb] = ks + 1 < KS ? read_k(sKn, kb, ks + 1) : kf[kb];
#pragma unroll
      for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)  // (the first k-step starts from -m: the shift costs no instruction)
          s_nxt[qb][kb] = Mfma16<DT>::run(kf[kb], qf[qb][ks], ks == 0 ? negm[qb] : s_nxt[qb][kb]);
#pragma unroll
      for (int j = 0; j < EPC; ++j) {
        const int idx = ks * EPC + j;  // over (query block, key block, element): 16 per query block
        const int qb = idx >> 4, kb = (idx & 15) >> 2, e = idx & 3;
        const float x = __builtin_amdgcn_exp2f(s_cur[qb][kb][e]);
        p[idx & 7] = x;
        lsum[qb] += x;
        if ((idx & 7) == 7) pf[qb][kb >> 1] = pack8<DT>(p);
      }
      // (pinned: left alone, the compiler sinks the sums' additions behind every MFMA of the loop body)
      asm volatile("" : "+v"(lsum[0]), "+v"(lsum[1]));
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) kf[kb] = kn[kb];
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) l_run[qb] = l_run[qb] * alpha[qb] + lsum[qb];

    // ---- phase B: O^T += V^T(t) P^T(t)  with  the maximum of tile t+1 ----
    // chunk c: key step c / 2, head-dim blocks (c % 2) * DB/2 .. + DB/2, and the maximum over 8 of the 32
    // scores of z(t+1)
    const int kv0n = (t + 1) * FA_BKV;
    float mx[2] = {-INFINITY, -INFINITY};
    constexpr int HB = DB / 2;
    u32x4 vf = read_v(sV, 0, 0);
#pragma unroll
    for (int c = 0; c < 2 * PS; ++c) {
      const int s = c >> 1;
#pragma unroll
      for (int dd = 0; dd < HB; ++dd) {
        const int d = (c & 1) * HB + dd;
        const int nxt = c * HB + dd + 1;  // (s, d) in issue order
        const u32x4 vn = nxt < PS * DB ? read_v(sV, nxt / DB, nxt % DB) : vf;
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) o[qb][d] = Mfma16<DT>::run(vf, pf[qb][s], o[qb][d]);
        vf = vn;
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int idx = c * 8 + j;
        const int qb = idx >> 4, kb = (idx & 15) >> 2, e = idx & 3;
        if constexpr (EDGE) {
          const int kv = kv0n + kb * 16 + g4 * 4 + e;
          const bool dead = (kv >= S) | ((a.causal != 0) & (kv > q_mine[qb]));
          s_nxt[qb][kb][e] = dead ? -INFINITY : s_nxt[qb][kb][e];
        }
        mx[qb] = fmaxf(mx[qb], s_nxt[qb][kb][e]);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    fold_max(mx, s_nxt, false);
  };

  // interior tiles first, then the edge tiles (the tail of the sequence and, under a causal mask, the
  // tiles that reach the diagonal of this wave's queries)
  int first_edge = ntiles;
  if (ntiles * FA_BKV > S) first_edge = ntiles - 1;
  if (a.causal) {
    const int fe = (q_wave0 + 1) / FA_BKV;
    first_edge = fe < first_edge ? fe : first_edge;
  }
  first_edge = __builtin_amdgcn_readfirstlane(first_edge);
  {  // tile 0: its maximum becomes the reference, whatever it is
    if (first_edge == 0) mask_tile(0, s_a);
    float mx[2] = {-INFINITY, -INFINITY};
#pragma unroll
    for (int qb = 0; qb < 2; ++qb)
#pragma unroll
      for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int e = 0; e < 4; ++e) mx[qb] = fmaxf(mx[qb], s_a[qb][kb][e]);
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) negm[qb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    fold_max(mx, s_a, true);
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) alpha[qb] = 1.0f;
  }
  const int interior_end = first_edge - 1;
  auto step = [&](int t, auto edge_tag, f32x4 (&s_cur)[2][KB], f32x4 (&s_nxt)[2][KB]) __attribute__((always_inline)) {
    __builtin_amdgcn_s_waitcnt(0x0f70);  // K(t+1) and V(t)
    __syncthreads();
    load_k(t + NSTG, sKbase + (t % NSTG) * TILE_BYTES);
    load_v(t + NSTG - 1, sVbase + ((t + NSTG - 1) % NSTG) * TILE_BYTES);
    iteration(t, edge_tag, s_cur, s_nxt);
  };
  // D = 64: interior tiles in pairs whose second step has the arrays in the other roles (an odd tile first,
  // with a copy); the few edge tiles copy.  D = 128 has no registers for the doubled loop body (150-200 bytes
  // of scratch per lane) and copies every tile's z into place.
  constexpr bool SWAP = D <= 64;
  auto copy_back = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int qb = 0; qb < 2; ++qb)
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) s_a[qb][kb] = s_b[qb][kb];
  };
  int t = 0;
  const int n_int = interior_end > 0 ? interior_end : 0;
  if constexpr (SWAP) {
    if (n_int & 1) {
      step(0, std::false_type{}, s_a, s_b);
      copy_back();
      t = 1;
    }
    for (; t < n_int; t += 2) {
      step(t, std::false_type{}, s_a, s_b);
      step(t + 1, std::false_type{}, s_b, s_a);
    }
  } else {
    for (; t < n_int; ++t) {
      step(t, std::false_type{}, s_a, s_b);
      copy_back();
    }
  }
  for (; t < ntiles; ++t) {
    step(t, std::true_type{}, s_a, s_b);
    copy_back();
  }
  __builtin_amdgcn_s_waitcnt(0x0f70);  // look-ahead loads must not land on the output staging
  __syncthreads();

  // ---- normalise, regroup through LDS, store 16 bytes per lane ----
  unsigned char *so = smem + wave * (WQ * ROW_BYTES);
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    float l_tot = l_run[qb] + __shfl_xor(l_run[qb], 16, 64);
    l_tot += __shfl_xor(l_tot, 32, 64);
    const float inv_l = 1.0f / l_tot;
#pragma unroll
    for (int d = 0; d < DB; ++d) {
      float x[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) x[e] = o[qb][d][e] * inv_l;
      u32x2 w;
      if constexpr (DT == DT_F16) {
        f16x4 hq = {(_Float16)x[0], (_Float16)x[1], (_Float16)x[2], (_Float16)x[3]};
        w = __builtin_bit_cast(u32x2, hq);
      } else {
        bf16x4 hq = {(__bf16)x[0], (__bf16)x[1], (__bf16)x[2], (__bf16)x[3]};
        w = __builtin_bit_cast(u32x2, hq);
      }
      *(u32x2 *)(so + (qb * 16 + r16) * ROW_BYTES + (d * 16 + g4 * 4) * 2) = w;
    }
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < WQ * CH / 64; ++i) {
    const int pidx = lane + i * 64;
    const int row = pidx / CH, c = pidx % CH;
    const int q = q_wave0 + row;
    if (q < S) *(u32x4 *)(Og + (long long)q * a.o_ss + c * 8) = *(const u32x4 *)(so + row * ROW_BYTES + c * 16);
  }
}

template <int D, int WAVES>
static int launch_fa2_m16(const AttentionArgs &a, int dtype, hipStream_t stream) {
  constexpr size_t ring = 2 * 2 * (size_t)FA_BKV * D * 2, staging = (size_t)WAVES * 32 * D * 2;
  constexpr size_t lds = ring > staging ? ring : staging;
  const int nqb = (a.S + 32 * WAVES - 1) / (32 * WAVES);
  const dim3 grid((unsigned)(nqb * a.B * a.H)), block(WAVES * 64);
#define TRACEA_FA_LAUNCH(DTV)                                                                  \
  do {                                                                                         \
    auto kfn = fa2_fwd_m16_kernel<DTV, D, WAVES>;                                              \
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
