// Convolution with the input patch resident in LDS (gfx950).
//
// The implicit-GEMM kernel gathers every input pixel once per filter tap, R*S
// times in all, through the L2.  Here a workgroup owns TM consecutive output
// pixels of one image and first copies the part of the (zero-padded) input
// those pixels touch into LDS, once; the A operand of every tap is then read
// from that patch at a tap-dependent byte offset.  Only the filter bank still
// streams, K tile by K tile, through a ring of LDS stages.
//
// Same arithmetic as the reference's kernel_main (src/emitter/cuda/conv.rs:153-331):
// out[n,ho,wo,k] = epilogue(sum_{r,s,c} x[n, ho*sh-ph+r*dh, wo*sw-pw+s*dw, c] * w[k,r,s,c]),
// fp32 accumulation in ascending (r,s,c) order per 16-wide k-step, zero padding.
//
// Patch addressing.  Padded coordinates hp = hi + pad_h, wp = wi + pad_w and
// PW = W + 2 pad_w give every padded input pixel the linear index
// q = hp * PW + wp.  Output pixel (ho,wo) under tap (r,s) reads
// q = (ho*sh*PW + wo*sw) + (r*dh*PW + s*dw): a per-pixel base plus a per-tap
// constant.  The patch is the contiguous q range [qmin, qmax] of the tile, one
// pixel every `cpp` 16-byte chunks (C/8 data chunks, padded to an odd count so
// that 8 consecutive pixels fall in 8 different bank groups).
#pragma once
#include "contraction_kernel.hpp"

namespace tracea_amd {

template <int DT, int TM, int BN, int WM, int WN, int NSB, bool FULL>
__global__ void __launch_bounds__(WM *WN * 64) conv_patch_kernel(const ContractionArgs args) {
  constexpr int NT = WM * WN * 64;
  constexpr int BK = 64, CH = 8, ROW_BYTES = 128, RP = 2;  // filter tile: BN rows x 64 k, XOR-swizzled
  constexpr int TMW = TM / WM, TN = BN / WN, FM = TMW / 32, FN = TN / 32;
  constexpr int B_STAGE = BN * ROW_BYTES;
  constexpr int NB = BN * CH / NT;  // filter pieces per thread per K tile
  constexpr int KS = BK / 16;
  static_assert(TM % (WM * 32) == 0 && BN % (WN * 32) == 0, "wave tile must be 32-aligned");
  static_assert((BN * CH) % NT == 0 && NB >= 1, "filter pieces must divide over threads");
  static_assert(NSB >= 3, "the filter ring needs three stages");
  constexpr int FLIGHT = (NSB - 2) * NB;  // requests that may stay in flight at the per-tile wait
  static_assert(FLIGHT <= 63, "vmcnt is a 6-bit counter");
  constexpr int WAIT_TILE = (FLIGHT & 15) | (7 << 4) | (15 << 8) | ((FLIGHT >> 4) << 14);

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave_u = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave_u % WM, wn = wave_u / WM;
  const int lrow = lane & 31, lhalf = lane >> 5;

  // ---- which tile ----
  int bid = blockIdx.x;
  const int total = gridDim.x;
  if ((total & 7) == 0) bid = (bid & 7) * (total >> 3) + (bid >> 3);  // contiguous run per XCD
  const int tile_n = bid % args.grid_n;
  const int tm = bid / args.grid_n;
  const int img = tm / args.p_tiles;
  const int p0 = (tm - img * args.p_tiles) * TM;  // first output pixel of the tile, within the image
  const int hw = args.h_out * args.w_out;
  const int npix = min(TM, hw - p0);
  const int n0 = tile_n * BN;
  const int N = args.N, K = args.K, C = args.c_in;
  const int PW = args.p_pw, cpp = args.p_cpp;
  const int pitch = cpp * 16;

  int ho_f, wo_f, ho_l, wo_l;
  fast_divmod(p0, args.w_m, args.w_s, args.w_out, ho_f, wo_f);
  fast_divmod(p0 + npix - 1, args.w_m, args.w_s, args.w_out, ho_l, wo_l);
  const int qmin = ho_f * args.stride_h * PW + wo_f * args.stride_w;
  const int r_sz = args.r_sz, s_sz = args.s_sz;
  const int tap_h = args.dil_h * PW;  // q step of one filter row
  const int qmax = ho_l * args.stride_h * PW + wo_l * args.stride_w + (r_sz - 1) * tap_h + (s_sz - 1) * args.dil_w;
  const int np = qmax - qmin + 1;  // the plan's LDS reservation covers the worst tile

  unsigned char *patch = smem;
  unsigned char *ring = smem + args.p_np_bytes;

  constexpr unsigned OOB = 0x80000000u;  // beyond every buffer: the load returns zeros
  const long long img_elems = (long long)args.h_in * args.w_in * C;
  __amdgpu_buffer_rsrc_t rsrc_x = __builtin_amdgcn_make_buffer_rsrc(
      (void *)((const unsigned short *)args.A + (long long)img * img_elems), 0, (int)(img_elems * 2), 0x00020000);
  __amdgpu_buffer_rsrc_t rsrc_w =
      __builtin_amdgcn_make_buffer_rsrc((void *)args.B, 0, (int)args.b_bytes, 0x00020000);

  // ---- patch: chunk c of the patch is padded pixel qmin + c / cpp, 16-byte part c % cpp ----
  const int cdata = C >> 3;
  for (int it = 0; it < args.p_iters; ++it) {
    const int chunk = it * NT + tid;
    int qrel, part, hp, wp;
    fast_divmod(chunk, args.p_cpp_m, args.p_cpp_s, cpp, qrel, part);
    fast_divmod(qmin + qrel, args.p_pw_m, args.p_pw_s, PW, hp, wp);
    const int hi = hp - args.pad_h, wi = wp - args.pad_w;
    const bool ok = (qrel < np) & (part < cdata) & ((unsigned)hi < (unsigned)args.h_in) &
                    ((unsigned)wi < (unsigned)args.w_in);  // bitwise: no control flow around the address
    const unsigned in_range = (unsigned)(((hi * args.w_in + wi) * C + part * 8) * 2);
    const unsigned voff = ok ? in_range : OOB;
    unsigned char *dst = patch + (it * NT + wave_u * 64) * 16;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_x, (__attribute__((address_space(3))) void *)dst, 16, (int)voff,
                                             0, 0, 0);
  }

  // ---- filter tiles: piece (row, 16-byte column pc) sits at row*128 + (pc ^ swizzle(row))*16 ----
  const int pc = tid % CH, prow = tid / CH;
  constexpr int PR_STEP = NT / CH;
  static_assert(PR_STEP % (RP * CH) == 0, "swizzle must be the same for all pieces of a thread");
  const int gpc = pc ^ ((prow / RP) & (CH - 1));
  unsigned b_voff[NB];
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    const int n = n0 + prow + i * PR_STEP;
    b_voff[i] = n < N ? (unsigned)(((long long)n * args.ldb + gpc * 8) * 2) : OOB;
  }
  auto dma_b = [&](int stage, int k0) {
    unsigned char *sB = ring + stage * B_STAGE;
    // columns of the last tile past K read as zero (and are not fetched: the scalar offset
    // takes no part in the hardware's range check, so they would lie past the row's end)
    const bool inside = FULL || k0 + gpc * 8 < K;
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      unsigned char *dst = sB + (i * PR_STEP + wave_u * (64 / CH)) * ROW_BYTES;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w, (__attribute__((address_space(3))) void *)dst, 16,
                                               (int)(inside ? b_voff[i] : OOB), k0 * 2, 0, 0);
    }
  };
  // K is a multiple of 16 (C is); when it is not a multiple of BK (FULL false) the last
  // filter tile holds fewer than KS k-steps: its missing k-steps are multiplied all the same,
  // with zero operands, so that the loop below has no conditions
  const int nk = (K + BK - 1) / BK;
  const int ksteps = K >> 4;
#pragma unroll
  for (int st = 0; st < NSB - 1; ++st) dma_b(st, (st < nk ? st : nk - 1) * BK);

  // chain description and choice of the row body: read here, under the main loop
  const ChainPlan plan = chain_plan(args.epi);
  const bool simple = chain_is_simple(plan, args, n0, BN) && args.out_dtype == DT;

  // this thread's entries of the epilogue operand table, requested under the main loop
  constexpr int TAB_ENTRIES = TRACEA_MAX_EPILOGUE_OPS * 2 * BN;
  constexpr int TPT = (TAB_ENTRIES + NT - 1) / NT;
  float tabr[TPT];
#pragma unroll
  for (int i = 0; i < TPT; ++i) {
    const int idx = tid + i * NT;
    tabr[i] = idx < TAB_ENTRIES ? chain_table_value(args.epi, idx / (2 * BN), (idx / BN) & 1, n0 + idx % BN, N) : 0.0f;
  }

  // ---- per-lane operand addresses ----
  // A: the lane's pixel of each 32-row block (rows past the tile re-read its last pixel)
  int a_base[FM];
#pragma unroll
  for (int i = 0; i < FM; ++i) {
    int pr = wm * TMW + i * 32 + lrow;
    pr = pr < npix ? pr : npix - 1;
    int ho, wo;
    fast_divmod(p0 + pr, args.w_m, args.w_s, args.w_out, ho, wo);
    a_base[i] = (ho * args.stride_h * PW + wo * args.stride_w - qmin) * pitch + lhalf * 16;
  }
  const int lswz = (lrow / RP) & (CH - 1);
  const int b_row = (wn * TN + lrow) * ROW_BYTES;

  f32x16 acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  // Tap state of the next k-step to be read: filter row r, column s, first channel c0.
  int tap_q = 0, tap_s = 0, tap_c = 0;  // q offset of (r, s=0); s; c0
  auto tap_offset = [&]() { return (tap_q + tap_s * args.dil_w) * pitch + tap_c * 2; };
  // (selects, not branches: the main loop must stay one basic block, see below)
  auto tap_advance = [&]() {
    tap_c += 16;
    const bool wrap_c = tap_c == C;
    tap_c = wrap_c ? 0 : tap_c;
    tap_s += wrap_c ? 1 : 0;
    const bool wrap_s = tap_s == s_sz;
    tap_s = wrap_s ? 0 : tap_s;
    tap_q += wrap_s ? tap_h : 0;
  };

  u32x4 fa[2][FM], fb[2][FN];
  int next_step = 0;  // k-steps read so far (FULL false only)
  auto read_operands = [&](int set, const unsigned char *sB, int ks) {
    const bool live = FULL || next_step < ksteps;
    next_step += 1;
    const int toff = live ? tap_offset() : 0;  // past the last tap the patch is not addressed
    tap_advance();
    const int coff = ((ks * 2 + lhalf) ^ lswz) << 4;
    const u32x4 zero4 = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      const u32x4 v = *(const u32x4 *)(patch + a_base[i] + toff);
      fa[set][i] = live ? v : zero4;
    }
#pragma unroll
    for (int j = 0; j < FN; ++j) fb[set][j] = *(const u32x4 *)(sB + b_row + j * 32 * ROW_BYTES + coff);
  };
  auto mma = [&](int set) {
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j) acc[i][j] = Mfma32<DT>::run(fb[set][j], fa[set][i], acc[i][j]);
  };

  __builtin_amdgcn_s_waitcnt(WAIT_TILE);  // patch and filter tile 0 of this wave have landed
  __syncthreads();
  read_operands(0, ring, 0);
  {
    // The loop body is free of branches (the last tile is peeled off, a partial last tile is
    // padded with zero operands), which matters beyond the branches themselves: with the
    // k-steps of a partial tile behind conditions the accumulators were live across several
    // paths and the compiler reconciled its register choices at the loop head with a copy of
    // all of them -- 64 v_accvgpr_mov per K tile and wave, as long as the 16 MFMAs of the tile.
    int cur_i = 0, fill_i = NSB - 1;
    for (int kt = 0; kt + 1 < nk; ++kt) {
      const unsigned char *cur = ring + cur_i * B_STAGE;
      const int nxt_i = cur_i + 1 == NSB ? 0 : cur_i + 1;
      // the stage released by the previous barrier receives tile kt+NSB-1 (clamped:
      // a repeat of the last tile lands in a stage that is not read again)
      const int tf = kt + NSB - 1 < nk ? kt + NSB - 1 : nk - 1;
      dma_b(fill_i, tf * BK);
#pragma unroll
      for (int ks = 0; ks + 1 < KS; ++ks) {
        read_operands((ks + 1) & 1, cur, ks + 1);
        mma(ks & 1);
      }
      __builtin_amdgcn_s_waitcnt(WAIT_TILE);  // tile kt+1 has landed; newer requests stay in flight
      // (the barrier alone: with the fences of __syncthreads() the compiler waits for every request in flight,
      // and the ring is no deeper than one tile)
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      // the last k-step of the tile runs behind the barrier, together with the first
      // operand reads of the next tile
      read_operands(0, ring + nxt_i * B_STAGE, 0);
      mma((KS - 1) & 1);
      fill_i = cur_i;
      cur_i = nxt_i;
    }
    {
      const unsigned char *cur = ring + cur_i * B_STAGE;
#pragma unroll
      for (int ks = 0; ks + 1 < KS; ++ks) {
        read_operands((ks + 1) & 1, cur, ks + 1);
        mma(ks & 1);
      }
      mma((KS - 1) & 1);
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0f70);  // no request may still land on the epilogue staging
  __syncthreads();

  // ---- epilogue: as in contraction_kernel (32 rows of the wave tile at a time through
  // a wave-private fp32 staging area, 8 consecutive channels per lane) ----
  constexpr int EP_PITCH = TN + 4;
  constexpr int LPR = TN / 8;
  constexpr int RPI = 64 / LPR;
  constexpr int STAGING_FLOATS = WM * WN * 32 * EP_PITCH;
  float *stage = (float *)smem + wave_u * (32 * EP_PITCH);
  float *table = (float *)smem + STAGING_FLOATS;
  const int er = lane / LPR, ec = (lane % LPR) * 8;
  const long long m_img = (long long)img * hw + p0;
#pragma unroll
  for (int i = 0; i < TPT; ++i)
    if (tid + i * NT < TAB_ENTRIES) table[tid + i * NT] = tabr[i];
  __syncthreads();
  const float *tab = table + wn * TN + ec;
  static_for<0, FM>([&](auto blk) {
    constexpr int i = decltype(blk)::value;
    static_for<0, FN>([&](auto col) {
      constexpr int j = decltype(col)::value;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        f32x4 v = {acc[i][j][g * 4 + 0], acc[i][j][g * 4 + 1], acc[i][j][g * 4 + 2], acc[i][j][g * 4 + 3]};
        *(f32x4 *)(stage + lrow * EP_PITCH + j * 32 + g * 8 + lhalf * 4) = v;
      }
    });
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    if (simple) {
      const int pb = wm * TMW + i * 32;
      simple_rows<DT, TN>(stage, lane, n0 + wn * TN + ec, args, plan, tab, BN,
                          [&](int r) -> long long { return pb + r < npix ? m_img + pb + r : -1ll; });
    } else {
      for (int r = er; r < 32; r += RPI) {
        const int pr = wm * TMW + i * 32 + r;
        const int n = n0 + wn * TN + ec;
        if (pr < npix && n < N) {
          float v[8];
          const f32x4 lo = *(const f32x4 *)(stage + r * EP_PITCH + ec);
          const f32x4 hi = *(const f32x4 *)(stage + r * EP_PITCH + ec + 4);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            v[e] = lo[e];
            v[4 + e] = hi[e];
          }
          const int nvalid = N - n;
          const long long m = m_img + pr;
          apply_epilogue_tab(v, m, n, nvalid, args.epi, plan, tab, BN);
          store_from_float<8>(args.C, args.out_dtype, m * args.ldc + n, nvalid, v);
        }
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
  });
}

// LDS bytes of one filter stage and of the epilogue staging, for the host-side plan.
template <int TM, int BN, int WM, int WN, int NSB>
int launch_conv_patch(const ContractionArgs &a, bool conv, int dtype, bool b_ncontig, hipStream_t stream) {
  if (!conv || b_ncontig || a.p_np_bytes <= 0) return (int)hipErrorInvalidValue;
  // epilogue: wave-private staging areas followed by the operand table
  const size_t staging = ((size_t)WM * WN * 32 * (BN / WN + 4) + (size_t)TRACEA_MAX_EPILOGUE_OPS * 2 * BN) * 4;
  size_t lds = (size_t)a.p_np_bytes + (size_t)NSB * BN * 128;
  if (lds < staging) lds = staging;
  const dim3 grid((unsigned)(a.grid_m * a.grid_n)), block(WM * WN * 64);
#define TRACEA_LAUNCH_PATCH(DTV, FULLV)                                                             \
  do {                                                                                              \
    auto kfn = conv_patch_kernel<DTV, TM, BN, WM, WN, NSB, FULLV>;                                  \
    static bool attr_done = false;                                                                  \
    if (!attr_done) {                                                                               \
      hipError_t e = hipFuncSetAttribute((const void *)kfn, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                         160 * 1024);                                               \
      if (e != hipSuccess) return (int)e;                                                           \
      attr_done = true;                                                                             \
    }                                                                                               \
    hipLaunchKernelGGL(kfn, grid, block, lds, stream, a);                                           \
    return (int)hipGetLastError();                                                                  \
  } while (0)
  const bool full = a.K % 64 == 0;  // every filter tile holds all of its k-steps
  if (dtype == DT_F16) { if (full) TRACEA_LAUNCH_PATCH(DT_F16, true); else TRACEA_LAUNCH_PATCH(DT_F16, false); }
  else { if (full) TRACEA_LAUNCH_PATCH(DT_BF16, true); else TRACEA_LAUNCH_PATCH(DT_BF16, false); }
#undef TRACEA_LAUNCH_PATCH
  return (int)hipErrorInvalidValue;
}

}  // namespace tracea_amd
