// Convolution on 16x16x32 MFMAs with the input patch resident in LDS and the filter slab either
// resident beside it or streamed through a ring of one filter tap per stage (gfx950).
//
// Same arithmetic as the reference's kernel_main (src/emitter/cuda/conv.rs:153-331):
// out[n,ho,wo,k] = epilogue(sum_{r,s,c} x[n, ho*sh-ph+r*dh, wo*sw-pw+s*dw, c] * w[k,r,s,c]),
// fp32 accumulation in ascending (r,s,c) order, 32 channels per MFMA, zero padding.
//
// Work split.  A workgroup owns p_tm <= 16 * (4 * PBW + 1) consecutive output pixels of one image and
// 64 filters; the host picks p_tm so that the launch is one balanced round over the CUs.  Pixels are cut
// into blocks of 16, filters into 4 blocks of 16, and the unit of work is one pixel block x one filter
// block = one v_mfma_f32_16x16x32 per 32-wide k-step.  Four multiplying waves, one per SIMD: wave w takes
// the PBW consecutive pixel blocks w*PBW .. with all four filter blocks, and filter block w of the one
// pixel block 4*PBW that is left over (392 pixels = 24.5 blocks: 6 whole blocks per wave and a quarter of
// the 25th; with 32-pixel blocks the same tile was 28 units of which 24.5 held pixels).  A wave reads
// PBW + 1 pixel fragments and 4 filter fragments of 1 KB per k-step for 4*PBW + 1 MFMAs of 16 cycles;
// PBW = 6 is 0.44 KB of LDS reads per MFMA, PBW = 3 0.62.  Four more waves only move data; or (WK = 8) all
// eight multiply, three blocks each: the two waves of a SIMD do not multiply faster than one (468 MFMAs in
// 9.1 k cycles against 450 in 8.5 k: eight waves read 64 KB of fragments per k-step, more than LDS delivers in
// the 416 cycles of their MFMAs), but the store phase is shared by twice the waves (10.7-11.3 us against
// 11.3-11.9 for N32 56x56 64->64).
//
// A wave's pixels are consecutive, its results leave from registers (below), and nothing after the
// operand wait is shared between the multiplying waves: each runs on its own.
//
// LDS layouts.  Patch: whole padded rows, pixel (hp, wp) at ((hp - hp0) * PW + wp) * cpp 16-byte chunks,
// cpp = C/8 rounded up to odd, so that the 16 pixels of a fragment start in 16 different bank groups.
// Filters, resident (C = 64): tap t of the 64 filters at t * 8 KB, row n at n * 128 bytes, its 16-byte part p at
// position p ^ ((n >> 1) & 7); requested tap by tap behind the patch, and a 3x3 layer starts multiplying when
// the patch and taps 0 to 2 have landed (a second barrier, behind the other six, stands at the end of tap 1).
// Filters, ring: stage t % RING holds tap t of the 64 filters, row n at n * (C/8 | 1) chunks.
//
// Epilogue.  The filter fragment is the first MFMA operand, so a lane ends with 4 consecutive output
// channels (4q .. 4q+3 of a filter block, q = lane >> 4) of pixel lane & 15 of a pixel block.  For the
// chains of the form [affine] [ReLU] [residual] [ReLU] everything happens in registers: per pair of filter
// blocks one v_permlane16_swap per packed register gives every lane 8 consecutive channels of its pixel,
// one 16-byte store; a residual is fetched in that layout, 16 bytes per lane, and taken back to the
// accumulators' layout by the same swap.  Any other chain goes through LDS and the general operator loop.
#pragma once
#include "conv_epilogue16.hpp"

namespace tracea_amd {

constexpr int CW_THREADS = 512;
constexpr int CW_TABLE_BYTES = TRACEA_MAX_EPILOGUE_OPS * 2 * 64 * 4;
// bytes of the filter area: whole load iterations of the eight waves (resident) or RING stages of 64 rows
constexpr int cw_ring_cpb(int cin) { return (cin / 8) | 1; }
// (a stage is whole load instructions of the four helper waves: the lanes past its 64 rows write zeros)
constexpr int cw_ring_iters(int cin) { return (64 * cw_ring_cpb(cin) + 255) / 256; }
constexpr int cw_ring_stage_bytes(int cin) { return cw_ring_iters(cin) * 256 * 16; }
// (the resident slab: tap t of the 64 filters at t * 64 * 2 * CIN bytes, without padding)
inline int cw_resident_filter_bytes(int k) { return 64 * k * 2; }

template <int DT, int CIN, int PBW, int RING, int WK = 4>
__global__ void __launch_bounds__(CW_THREADS) conv_wave16_kernel(const ContractionArgs args) {
  static_assert(WK == 4 || (WK == 8 && RING == 0), "eight multiplying waves only with the resident filter slab");
  static_assert(RING != 0 || CIN == 64, "the resident slab's layout: one load instruction per thread and tap");
  constexpr int NT = CW_THREADS, BN = 64, NW = NT / 64;
  constexpr int KPT = CIN / 32;   // 32-wide k-steps per filter tap
  constexpr int TAPB = CIN * 2;   // bytes of one tap in a filter row
  constexpr int NPF = PBW + 1;    // pixel fragments per k-step
  static_assert(KPT >= 2 && KPT % 2 == 0, "the two operand sets alternate with the k-steps of a tap");
  static_assert(RING == 0 || RING >= 3, "the ring keeps two taps readable and at least one in flight");
  constexpr int RCPB = cw_ring_cpb(CIN), RSTAGE = cw_ring_stage_bytes(CIN);
  constexpr int RIT = cw_ring_iters(CIN);  // load instructions per helper wave and tap

  // Everything the prologue reads from the kernel arguments, asked for here in one batch of scalar loads
  // (left alone the compiler loads each field where it is first used, one round trip after the other).
  asm volatile("" ::"s"(args.A), "s"(args.B), "s"(args.N), "s"(args.K), "s"(args.ldb), "s"(args.b_bytes), "s"(args.grid_n),
               "s"(args.h_in), "s"(args.w_in), "s"(args.h_out), "s"(args.w_out), "s"(args.s_sz), "s"(args.r_sz));
  asm volatile("" ::"s"(args.stride_h), "s"(args.stride_w), "s"(args.pad_h), "s"(args.pad_w), "s"(args.dil_h), "s"(args.dil_w),
               "s"(args.w_m), "s"(args.w_s), "s"(args.p_tiles), "s"(args.p_pw), "s"(args.p_cpp), "s"(args.p_np_bytes),
               "s"(args.p_tm), "s"(args.p_seg), "s"(args.p_ppi), "s"(args.p_cpp_m), "s"(args.p_cpp_s), "s"(args.p_pw_m),
               "s"(args.p_pw_s), "s"(args.gn_m), "s"(args.gn_s), "s"(args.pt_m), "s"(args.pt_s));
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  unsigned char *patch = smem;
  unsigned char *filt = smem + args.p_np_bytes;
  const int taps = args.r_sz * args.s_sz;
  constexpr int CPB = RCPB;        // (ring) 16-byte chunks per filter row of a stage
  constexpr int TAPS = 64 * TAPB;  // (resident slab) bytes of one tap of the 64 filters
  const int filt_bytes = RING ? RING * RSTAGE : taps * TAPS;
  // (the operand table lies behind the operands or, if that is more, behind the general epilogue's staging)
  const int operand_bytes = args.p_np_bytes + filt_bytes, staging_bytes = args.p_tm * (BN + 4) * 4;
  float *table = (float *)(smem + (operand_bytes > staging_bytes ? operand_bytes : staging_bytes));

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave_u = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int w = wave_u & 3;          // SIMD; the filter block a multiplying wave starts with
  const int ww = wave_u & (WK - 1);  // the multiplying wave's index: its pixel blocks are ww*PBW .. + PBW-1
  const bool worker = wave_u < WK;
  const int l15 = lane & 15, q = lane >> 4;

  // ---- which tile ----
  int bid = blockIdx.x;
  const int total = gridDim.x;
  if ((total & 7) == 0) bid = (bid & 7) * (total >> 3) + (bid >> 3);  // contiguous run per XCD
  int tile_n, tm, img, tim;
  fast_divmod(bid, args.gn_m, args.gn_s, args.grid_n, tm, tile_n);
  fast_divmod(tm, args.pt_m, args.pt_s, args.p_tiles, img, tim);
  const int TM = args.p_tm;
  const int p0 = tim * TM;
  const int hw = args.h_out * args.w_out;
  const int npix = min(TM, hw - p0);
  const int n0 = tile_n * BN;
  const int N = args.N, C = CIN;
  const int PW = args.p_pw, cpp = args.p_cpp;
  const int pitch = cpp * 16;

  constexpr unsigned OOB = 0x80000000u;  // beyond every buffer: the load returns zeros
  const long long img_elems = (long long)args.h_in * args.w_in * C;
  __amdgpu_buffer_rsrc_t rsrc_x = __builtin_amdgcn_make_buffer_rsrc(
      (void *)((const unsigned short *)args.A + (long long)img * img_elems), 0, (int)(img_elems * 2), 0x00020000);
  __amdgpu_buffer_rsrc_t rsrc_w =
      __builtin_amdgcn_make_buffer_rsrc((void *)args.B, 0, (int)args.b_bytes, 0x00020000);

  // ---- epilogue form ----
  // sig >= 0: the chain reads [affine] [ReLU] [residual] [ReLU] (bit 0 affine, 1 first ReLU, 2 residual,
  // 3 second ReLU), affine = v*a + b per channel; table [0..63] = a, [64..127] = b.  sig < 0: any other
  // chain, table in the layout of chain_table_value.
  const int sig = args.fe.sig;
  // the resident slab's nine taps are awaited in two groups (the general chain's table takes the old road)
  const bool prog = RING == 0 && taps == 9 && sig >= 0;

  // ---- filters ----
  // resident: tap t of the 64 filters at t * TAPS, row r at r * TAPB, its 16-byte part p at position
  // p ^ ((r >> 1) & 7) (the 16 rows of a fragment then read 16 different bank groups); one load instruction per
  // thread and tap, taps in ascending order behind the patch: the first taps are multiplied while the others travel
  // ring: the helper waves bring tap t into stage t % RING: chunk c is row c / RCPB, part c % RCPB of the tap
  unsigned ring_voff[RIT];
  const int htid = tid - 256;
  const bool ring_wave = RING != 0 && !worker;
  auto ring_issue = [&](int t) __attribute__((always_inline)) {
    unsigned char *sb = filt + (t % RING) * RSTAGE;
#pragma unroll
    for (int it = 0; it < RIT; ++it) {
      unsigned char *dst = sb + (it * 256 + (wave_u - 4) * 64) * 16;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w, (__attribute__((address_space(3))) void *)dst, 16,
                                               (int)ring_voff[it], t * TAPB, 0, 0);
    }
  };
  if constexpr (RING != 0) {
#pragma unroll
    for (int it = 0; it < RIT; ++it) {
      const int chunk = it * 256 + htid;
      const int row = chunk / RCPB, part = chunk - row * RCPB;
      const bool ok = (htid >= 0) & (part < CIN / 8) & (row < BN) & (n0 + row < N);
      ring_voff[it] = ok ? (unsigned)(((n0 + row) * (int)args.ldb + part * 8) * 2) : OOB;
    }
  }

  // ---- patch, by columns of load instructions ----
  // One load instruction moves the PPI = 64 / cpp pixels wp0 .. wp0 + PPI - 1 of one padded row (lane l:
  // pixel l / cpp, 16-byte part l % cpp; the part past the channels is padding and is written as zeros).
  // A wave takes segment j = wave, wave + 8, ... of EVERY row: what depends on the lane is then fixed per
  // segment.  Padding pixels and rows get an out-of-range offset and are written as zeros; lanes past the
  // row's end are switched off (they would land on the next row's pixels).
  int ho_f, wo_f, ho_l, wo_l;
  fast_divmod(p0, args.w_m, args.w_s, args.w_out, ho_f, wo_f);
  fast_divmod(p0 + npix - 1, args.w_m, args.w_s, args.w_out, ho_l, wo_l);
  const int hp0 = ho_f * args.stride_h;
  const int tap_h = args.dil_h * PW;  // pixel index step of one filter row
  const int n_rows = ho_l * args.stride_h + (args.r_sz - 1) * args.dil_h - hp0 + 1;
  const int SEG = args.p_seg, PPI = args.p_ppi;
  constexpr int cdata = CIN >> 3;
  int ldl, lpart;
  fast_divmod(lane, args.p_cpp_m, args.p_cpp_s, cpp, ldl, lpart);
  const int lane_off = (ldl - args.pad_w) * C * 2 + lpart * 16;
  const int row_bytes = args.w_in * C * 2, row_pitch = PW * pitch;
  for (int j = wave_u; j < SEG; j += NW) {
    const int wp = j * PPI + ldl;
    const bool lane_ok = ((unsigned)(wp - args.pad_w) < (unsigned)args.w_in) & (lpart < cdata);
    const unsigned v_seg = lane_ok ? (unsigned)(lane_off + j * PPI * C * 2) : OOB;
    if (wp < PW) {
      int hi = hp0 - args.pad_h;
      unsigned char *dst = patch + j * PPI * pitch;
      for (int r = 0; r < n_rows; ++r) {
        const bool row_ok = (unsigned)hi < (unsigned)args.h_in;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_x, (__attribute__((address_space(3))) void *)dst, 16,
                                                 (int)(row_ok ? v_seg : OOB), row_ok ? hi * row_bytes : 0, 0, 0);
        hi += 1;
        dst += row_pitch;
      }
    }
  }
  // ---- per-lane operand addresses (worked out between the requests for the patch and those for the filters:
  // the requests queue in front of the memory pipe, and what a wave computes behind its last request is time it
  // stands between the operands' arrival and the first MFMA) ----
  __builtin_amdgcn_sched_barrier(0);
  // pixel fragment i < PBW: block w*PBW + i; fragment PBW: the shared block 4*PBW
  int a_base[NPF];
#pragma unroll
  for (int i = 0; i < NPF; ++i) {
    const int blk = i < PBW ? ww * PBW + i : WK * PBW;
    const int pr = blk * 16 + l15;
    const int prc = pr < npix ? pr : npix - 1;
    int ho, wo;
    fast_divmod(p0 + prc, args.w_m, args.w_s, args.w_out, ho, wo);
    a_base[i] = ((ho * args.stride_h - hp0) * PW + wo * args.stride_w) * pitch + q * 16;
  }
  // filter fragment i: filter block w ^ i (fragment 0 is the wave's own block, which the shared pixel block
  // multiplies; fragments 2j and 2j+1 are neighbours in the channel order): row (w ^ i)*16 + l15, 16-byte part q
  // (resident slab: the address of the tap's first k-step; the second one is 64 bytes up or down, by the row)
  int f_base[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = (w ^ i) * 16 + l15;
    f_base[i] = RING ? (row * CPB + q) * 16 : row * TAPB + ((q ^ ((row >> 1) & 7)) << 4);
  }
  int step_s = args.dil_w * pitch;
  int step_r = tap_h * pitch - (args.s_sz - 1) * step_s;
  int off_last = ((args.r_sz - 1) * tap_h + (args.s_sz - 1) * args.dil_w) * pitch;
  int s_size = args.s_sz;
#pragma unroll
  for (int i = 0; i < NPF; ++i) asm volatile("" : "+v"(a_base[i]));
#pragma unroll
  for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(f_base[i]));
  asm volatile("" : "+s"(step_s), "+s"(step_r), "+s"(off_last), "+s"(s_size));
  __builtin_amdgcn_sched_barrier(0);

  // (the patch first: every tap needs it; its rows come from memory, the filters from the L2 every workgroup shares)
  if constexpr (RING == 0) {
    const int row = tid >> 3, pos = tid & 7;
    const unsigned voff = n0 + row < N ? (unsigned)(((n0 + row) * (int)args.ldb + ((pos ^ ((row >> 1) & 7)) << 3)) * 2) : OOB;
    unsigned char *dst = filt + wave_u * 1024;
    for (int t = 0; t < taps; ++t) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w, (__attribute__((address_space(3))) void *)dst, 16, (int)voff,
                                               t * TAPB, 0, 0);
      dst += TAPS;
    }
  }
  // ring: the first RING taps follow the patch, one per stage
  if constexpr (RING != 0) {
    if (ring_wave) {
#pragma unroll
      for (int t = 0; t < RING; ++t)
        if (t < taps) ring_issue(t);
    }
  }

  // ---- this thread's entry of the operand table (requested behind the operands, worked out where the table is
  // published: in front of the first barrier, or -- prog -- of the second, when everything has landed anyway) ----
  // Waves 0 and 1 (threads 0..127: a of channel n0 + tid, b of channel n0 + tid - 64) request the raw vector
  // entries, every lane and the same number per wave, so that the waits for the taps can count them: 1 (bias,
  // scale and shift) or 4 (BatchNorm: gamma, variance, beta, mean).
  constexpr int TPT = CW_TABLE_BYTES / 4 / NT;
  float tabg[TPT];
  // (two sets of registers, one per road: a set that both roads touched would be copied where they meet, and a
  // copy reads the registers -- it waits for the requests)
  unsigned traw_now[4] = {0u, 0u, 0u, 0u}, traw_late[4] = {0u, 0u, 0u, 0u};
  const int tab_loads = (sig >= 0 && (sig & 1) && wave_u < 2) ? (args.fe.aff_kind == TRACEA_EPI_OP_BATCHNORM ? 4 : 1) : 0;
  if (sig < 0) {
#pragma unroll
    for (int i = 0; i < TPT; ++i) {
      const int e = tid + i * NT;
      tabg[i] = chain_table_value(args.epi, e / (2 * BN), (e / BN) & 1, n0 + e % BN, N);
    }
  } else if (tab_loads != 0) {
    auto request = [&](unsigned (&r)[4]) __attribute__((always_inline)) {
      const int which = tid / BN;
      const int n = min(n0 + (tid & (BN - 1)), N - 1);
      if (args.fe.aff_kind == TRACEA_EPI_OP_BIAS_ADD) {
        r[0] = args.fe.aff_dtype == DT_F32 ? ((const unsigned *)args.fe.p0)[n] : (unsigned)((const unsigned short *)args.fe.p0)[n];
      } else if (args.fe.aff_kind == TRACEA_EPI_OP_SCALE_SHIFT) {
        r[0] = ((const unsigned *)(which == 0 ? args.fe.p0 : args.fe.p1))[n];
      } else {
        r[0] = ((const unsigned *)args.fe.p0)[n];
        r[1] = ((const unsigned *)args.fe.p3)[n];
        r[2] = ((const unsigned *)args.fe.p1)[n];
        r[3] = ((const unsigned *)args.fe.p2)[n];
      }
    };
    if (prog) request(traw_late);
    else request(traw_now);
  }
  // (called by every thread, between a wait that covers the requests above and a barrier)
  auto publish_table = [&](unsigned (&rv)[4]) __attribute__((always_inline)) {
#pragma unroll
    for (int e = 0; e < 4; ++e) asm volatile("" : "+v"(rv[e]));  // (nothing of this moves in front of the wait)
    if (sig < 0) {
#pragma unroll
      for (int i = 0; i < TPT; ++i) table[tid + i * NT] = tabg[i];
    } else if (tab_loads != 0) {
      const int which = tid / BN;
      float t;
      if (args.fe.aff_kind == TRACEA_EPI_OP_BIAS_ADD) {
        const float bv = args.fe.aff_dtype == DT_F32   ? __builtin_bit_cast(float, rv[0])
                         : args.fe.aff_dtype == DT_F16 ? (float)__builtin_bit_cast(_Float16, (unsigned short)rv[0])
                                                       : __builtin_bit_cast(float, rv[0] << 16);
        t = which == 0 ? 1.0f : bv;
      } else if (args.fe.aff_kind == TRACEA_EPI_OP_SCALE_SHIFT) {
        t = __builtin_bit_cast(float, rv[0]);
      } else {  // BatchNorm folded: a = gamma / sqrt(var + eps), b = beta - mean * a
        const float scale = __builtin_bit_cast(float, rv[0]) * (1.0f / sqrtf(__builtin_bit_cast(float, rv[1]) + args.fe.epsilon));
        t = which == 0 ? scale : __builtin_bit_cast(float, rv[2]) - __builtin_bit_cast(float, rv[3]) * scale;
      }
      table[tid] = t;
    }
  };
  // vmcnt(LEFT + this wave's table requests): all but the last LEFT taps of the resident slab have landed
  auto wait_taps = [&](auto left_tag) __attribute__((always_inline)) {
    constexpr int L = decltype(left_tag)::value;
    if (tab_loads == 0) __builtin_amdgcn_s_waitcnt(0x0f70 | L);
    else if (tab_loads == 1) __builtin_amdgcn_s_waitcnt(0x0f70 | (L + 1));
    else __builtin_amdgcn_s_waitcnt(0x0f70 | (L + 4));
  };

  // A bias that opens a chain of the fast form is where the accumulators start (one fp32 rounding apart from
  // adding it last, and a hundred additions less in the epilogue of a wave that has nobody to share them with).
  // (Not with the taps awaited in groups: the accumulators would wait for the last request of the wave.)
  const bool bias_init = !prog && sig >= 0 && (sig & 1) && args.fe.aff_kind == TRACEA_EPI_OP_BIAS_ADD;
  const int form_sig = bias_init ? (sig & ~1) : sig;

  f32x4 acc[PBW][4], acc_x;
  if (bias_init) {  // (a branch of its own: the wait for these loads must not stand on the other road)
    f32x4 start[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float b4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
      load_as_float<4>(args.fe.p0, args.fe.aff_dtype, n0 + (w ^ i) * 16 + q * 4, 4, b4);
      start[i] = f32x4{b4[0], b4[1], b4[2], b4[3]};
    }
#pragma unroll
    for (int p = 0; p < PBW; ++p)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[p][i] = start[i];
    acc_x = start[0];
#pragma unroll
    for (int p = 0; p < PBW; ++p)
#pragma unroll
      for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(acc[p][i]));
    asm volatile("" : "+v"(acc_x));
  } else {
    const f32x4 zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int p = 0; p < PBW; ++p)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[p][i] = zero4;
    acc_x = zero4;
#pragma unroll
    for (int p = 0; p < PBW; ++p)
#pragma unroll
      for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(acc[p][i]));
    asm volatile("" : "+v"(acc_x));
  }

  // ring: taps 0 and 1 must have landed; the RING - 2 later taps may stay in flight
  if constexpr (RING != 0) {
    constexpr int fl = RIT * (RING - 2);
    static_assert(fl <= 63, "vmcnt is a 6-bit counter");
    if (ring_wave && taps >= RING) __builtin_amdgcn_s_waitcnt(0x0f70 | (fl & 15) | ((fl >> 4) << 14));
    else __builtin_amdgcn_s_waitcnt(0x0f70);
  } else {
    // resident slab of nine taps: the patch and taps 0 to 2 must have landed (a wave's requests complete in
    // order, the taps are the last nine operand requests); the other six are awaited at the end of tap 1, where
    // the second barrier stands.  Any other number of taps: everything here.
    if (prog) wait_taps(std::integral_constant<int, 6>{});
    else __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
  }
  if (!prog) {
    publish_table(traw_now);
    __syncthreads();
  } else {
    // (the bare barrier: the fence of __syncthreads would wait for the table requests, the last of the wave)
    __builtin_amdgcn_s_barrier();
  }

  // ---- the residual of this wave's pixels, asked for now: fetched in the epilogue it is a round trip to memory
  // with nothing left to hide it (28x28 128->128 with a residual 11.4 us against 9.9 without).  Where the kernel
  // has the registers (three pixel blocks per wave: 26 of them). ----
  constexpr bool PRE_RES = PBW <= 3;
  const long long m_img = (long long)img * hw + p0;
  __amdgpu_buffer_rsrc_t rsrc_r = __builtin_amdgcn_make_buffer_rsrc(
      (void *)((const unsigned short *)args.fe.res + ((sig >= 0 && (sig & 4)) ? m_img * args.fe.res_ld + n0 : 0ll)), 0,
      (sig >= 0 && (sig & 4)) ? (int)((long long)npix * args.fe.res_ld * 2) : 0, 0x00020000);
  const int row_r = (int)args.fe.res_ld * 2;
  u32x4 resv[PRE_RES ? PBW : 1][2] = {};
  u32x2 resx = {0u, 0u};
  if constexpr (PRE_RES) {
    if (worker && sig >= 0 && (sig & 4)) {
      using E0 = Epilogue16<DT, 4>;
#pragma unroll
      for (int p = 0; p < PBW; ++p) {
        const int pr = (ww * PBW + p) * 16 + l15;
#pragma unroll
        for (int j = 0; j < 2; ++j)
          resv[p][j] = E0::fetch_pair_residual(w ^ (2 * j), w ^ (2 * j + 1), pr < npix ? pr : -1, q, rsrc_r, row_r);
      }
      const int prx = WK * PBW * 16 + l15;
      resx = E0::fetch_single_residual(w * 16 + q * 4, (prx < npix && wave_u < 4) ? prx : -1, rsrc_r, row_r);
    }
  }

  if constexpr (RING == 0) {
    if (!worker && prog) {  // (four multiplying waves) the other waves' share of the second barrier
      __builtin_amdgcn_s_waitcnt(0x0f70);
      publish_table(traw_late);
      __syncthreads();
    }
  }
  if constexpr (RING != 0) {
    if (!worker) {
      // helper waves: taps t .. t + RING - 1 occupy the stages; before barrier t tap t + 2 has landed (the
      // RING - 3 after it may be in flight); behind it stage t % RING is free and receives tap t + RING.
      // (No barrier where neither matters any more: t >= taps - 2.)
      for (int t = 0; t + 2 < taps; ++t) {
        if (t + RING - 1 < taps) {
          constexpr int fl = RIT * (RING - 3);
          __builtin_amdgcn_s_waitcnt(0x0f70 | (fl & 15) | ((fl >> 4) << 14));
        } else {
          __builtin_amdgcn_s_waitcnt(0x0f70);
        }
        __builtin_amdgcn_s_barrier();
        if (ring_wave && t + RING < taps) ring_issue(t + RING);
      }
      __builtin_amdgcn_s_waitcnt(0x0f70);
    }
  }

  if (worker) {
    u32x4 xa[2][NPF], xb[2][4];
    int ts = 0, off = 0;
    auto next_tap = [&]() {
      ts += 1;
      const bool wrap_s = ts == s_size;
      ts = wrap_s ? 0 : ts;
      off += wrap_s ? step_r : step_s;
      off = off < off_last ? off : off_last;
    };
    // operand addresses of "the tap whose first k-step was read last": one set, moved on to the next tap in
    // front of the read of its first k-step
    // (fq: resident slab, the tap's second k-step, 64 bytes up or down from the first by the row's swizzle; kept
    // beside fp where registers allow, else worked out per read -- the kernel with six pixel blocks per wave
    // has none to spare)
    constexpr bool FQ = RING == 0 && PBW <= 3;
    const unsigned char *pp[NPF], *fp[4], *fq[FQ ? 4 : 1];
#pragma unroll
    for (int i = 0; i < NPF; ++i) pp[i] = patch + a_base[i];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      fp[i] = filt + f_base[i];
      if constexpr (FQ) fq[i] = filt + (f_base[i] ^ 64);
    }
    auto read = [&](auto setc, auto kc) __attribute__((always_inline)) {
      constexpr int set = decltype(setc)::value, k = decltype(kc)::value;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if constexpr (FQ) xb[set][i] = *(const u32x4 *)(k == 0 ? fp[i] : fq[i]);
        else if constexpr (RING == 0) xb[set][i] = *(const u32x4 *)(smem + ((unsigned)(fp[i] - smem) ^ (k * 64u)));
        else xb[set][i] = *(const u32x4 *)(fp[i] + k * 64);
      }
#pragma unroll
      for (int i = 0; i < NPF; ++i) xa[set][i] = *(const u32x4 *)(pp[i] + k * 64);
    };
    auto mma = [&](auto setc) __attribute__((always_inline)) {
      constexpr int s = decltype(setc)::value;
#pragma unroll
      for (int p = 0; p < PBW; ++p)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[p][i] = Mfma16<DT>::run(xb[s][i], xa[s][p], acc[p][i]);
      acc_x = Mfma16<DT>::run(xb[s][0], xa[s][PBW], acc_x);
      Interleave<0, 4 * PBW + 1, 0x100, NPF + 4, 0x100, 0>::run();
      __builtin_amdgcn_sched_barrier(0);
    };
    using std::integral_constant;
    read(integral_constant<int, 0>{}, integral_constant<int, 0>{});
    __builtin_amdgcn_sched_barrier(0);
    int t_now = 0;
    auto tap = [&]() __attribute__((always_inline)) {
      static_for<0, KPT>([&](auto kc) {
        constexpr int k = decltype(kc)::value;
        if constexpr (k + 1 < KPT) {
          read(integral_constant<int, (k + 1) & 1>{}, integral_constant<int, k + 1>{});
        } else {
          // on to the next tap (worked out HERE, in front of the tap's last MFMAs: behind them it is a dozen
          // instructions during which a lone wave's matrix pipe idles); past the last tap the addresses stay
          // (the last tap is read again, unused)
          next_tap();
          const bool more = t_now + 1 < taps;
#pragma unroll
          for (int i = 0; i < NPF; ++i) pp[i] = patch + a_base[i] + off;
          if constexpr (RING == 0) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              fp[i] += more ? TAPS : 0;
              if constexpr (FQ) fq[i] += more ? TAPS : 0;
            }
          } else {
            const int st = more ? (t_now + 1) % RING : t_now % RING;
#pragma unroll
            for (int i = 0; i < 4; ++i) fp[i] = filt + f_base[i] + st * RSTAGE;
          }
          read(integral_constant<int, 0>{}, integral_constant<int, 0>{});
        }
        mma(integral_constant<int, k & 1>{});
      });
      if constexpr (RING != 0) {
        // barrier t: taps up to t + 2 are readable behind it (see the helper waves' loop)
        if (t_now + 2 < taps) __builtin_amdgcn_s_barrier();
      } else if (prog) {
        // (tap 1's last k-step was issued behind the read of tap 2's first: taps 0 to 2 stand behind the first
        // barrier, the others behind this one)
        if (t_now == 1) {
          __builtin_amdgcn_s_waitcnt(0x0f70);
          publish_table(traw_late);
          __syncthreads();
        }
      }
      t_now += 1;
    };
    if constexpr (RING == 0) {
      // several taps per trip: a taken branch costs a lone wave more than a hundred cycles of idle matrix pipe
      const int trips = taps / 3;
#pragma unroll 1
      for (int t = 0; t < trips; ++t) {
        tap();
        tap();
        tap();
      }
#pragma unroll 1
      for (int t = trips * 3; t < taps; ++t) tap();
    } else {
#pragma unroll 1
      for (int t = 0; t < taps; ++t) tap();
    }
  }

  if (sig >= 0) {
    if (!worker) return;
    // ---- epilogue from registers ----
    __amdgpu_buffer_rsrc_t rsrc_c = __builtin_amdgcn_make_buffer_rsrc(
        (void *)((unsigned short *)args.C + m_img * args.ldc + n0), 0, (int)((long long)npix * args.ldc * 2), 0x00020000);
    const int row_c = (int)args.ldc * 2;
    int fb[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) fb[i] = w ^ i;
    auto run_form = [&](auto form) __attribute__((always_inline)) {
      using E = Epilogue16<DT, decltype(form)::value>;
      f32x4 ta[4] = {}, tb[4] = {};
      if constexpr (E::AFF) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          ta[i] = *(const f32x4 *)(table + fb[i] * 16 + q * 4);
          tb[i] = *(const f32x4 *)(table + BN + fb[i] * 16 + q * 4);
        }
      }
      static_for<0, PBW>([&](auto pc) {
        constexpr int p = decltype(pc)::value;
        const int pr = (ww * PBW + p) * 16 + l15;
        if constexpr (PRE_RES) E::pixel_block_with(acc[p], fb, ta, tb, pr < npix ? pr : -1, q, rsrc_c, row_c, resv[p]);
        else E::pixel_block(acc[p], fb, ta, tb, pr < npix ? pr : -1, q, rsrc_c, rsrc_r, row_c, row_r);
      });
      {  // the shared block: filter block w only
        // (with eight multiplying waves the shared block is computed by waves w and w + 4 alike: one stores)
        const int pr = WK * PBW * 16 + l15;
        if constexpr (PRE_RES) E::single_block_with(acc_x, ta[0], tb[0], w * 16 + q * 4, (pr < npix && wave_u < 4) ? pr : -1, rsrc_c, row_c, resx);
        else E::single_block(acc_x, ta[0], tb[0], w * 16 + q * 4, (pr < npix && wave_u < 4) ? pr : -1, rsrc_c, rsrc_r, row_c, row_r);
      }
    };
#define TRACEA_CW_FORM(F) run_form(std::integral_constant<int, F>{})
    TRACEA_EPILOGUE16_FORMS(form_sig, TRACEA_CW_FORM)
#undef TRACEA_CW_FORM
    return;
  }

  // ---- any other chain: accumulators through LDS, then the general operator loop over whole pixels ----
  constexpr int SP = BN + 4;  // floats per staged pixel
  float *stage = (float *)smem;
  __syncthreads();  // every wave has left the main loop: patch and filters may be overwritten
  if (worker) {
    static_for<0, PBW>([&](auto pc) {
      constexpr int p = decltype(pc)::value;
      const int pr = (ww * PBW + p) * 16 + l15;
      if (pr < npix) {
#pragma unroll
        for (int i = 0; i < 4; ++i) *(f32x4 *)(stage + pr * SP + (w ^ i) * 16 + q * 4) = acc[p][i];
      }
    });
    const int pr = WK * PBW * 16 + l15;
    if (pr < npix && wave_u < 4) *(f32x4 *)(stage + pr * SP + w * 16 + q * 4) = acc_x;
  }
  __syncthreads();
  const int ec = (tid & 7) * 8;
  const ChainPlan plan = chain_plan(args.epi);
  for (int idx = tid; idx < npix * (BN / 8); idx += NT) {
    const int pr = idx >> 3;
    const int n = n0 + ec;
    if (n < N) {
      float v[8];
      const f32x4 lo = *(const f32x4 *)(stage + pr * SP + ec);
      const f32x4 hi = *(const f32x4 *)(stage + pr * SP + ec + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        v[e] = lo[e];
        v[4 + e] = hi[e];
      }
      const int nvalid = N - n;
      const long long m = m_img + pr;
      apply_epilogue_tab(v, m, n, nvalid, args.epi, plan, table + ec, BN);
      store_from_float<8>(args.C, args.out_dtype, m * args.ldc + n, nvalid, v);
    }
  }
}

// bm = 16 * (4 * PBW + 1) pixels at most per workgroup; CIN input channels exactly; RING = 0: the whole
// filter slab (64 x K) resident beside the patch, else a ring of RING one-tap stages.
template <int CIN, int PBW, int RING, int WK = 4>
int launch_conv_wave16(const ContractionArgs &a, bool conv, int dtype, bool b_ncontig, hipStream_t stream) {
  if (!conv || b_ncontig || a.c_in != CIN || a.K != a.r_sz * a.s_sz * CIN || a.p_tm <= 0 || a.p_tm > 16 * (WK * PBW + 1) ||
      a.p_np_bytes <= 0)
    return (int)hipErrorInvalidValue;
  const size_t filt = RING ? (size_t)RING * cw_ring_stage_bytes(CIN) : (size_t)cw_resident_filter_bytes(a.K);
  size_t lds = (size_t)a.p_np_bytes + filt + CW_TABLE_BYTES;
  // the general epilogue stages p_tm x 68 floats in front of the table
  if ((size_t)a.p_tm * 68 * 4 > lds - CW_TABLE_BYTES) lds = (size_t)a.p_tm * 68 * 4 + CW_TABLE_BYTES;
  if (lds > 160 * 1024) return (int)hipErrorInvalidValue;
  const dim3 grid((unsigned)(a.grid_m * a.grid_n)), block(CW_THREADS);
#define TRACEA_LAUNCH_CW(DTV)                                                                        \
  do {                                                                                               \
    auto kfn = conv_wave16_kernel<DTV, CIN, PBW, RING, WK>;                                               \
    static bool attr_done = false;                                                                   \
    if (!attr_done) {                                                                                \
      hipError_t e = hipFuncSetAttribute((const void *)kfn, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                         160 * 1024);                                                \
      if (e != hipSuccess) return (int)e;                                                            \
      attr_done = true;                                                                              \
    }                                                                                                \
    hipLaunchKernelGGL(kfn, grid, block, lds, stream, a);                                            \
    return (int)hipGetLastError();                                                                   \
  } while (0)
  if (dtype == DT_F16) TRACEA_LAUNCH_CW(DT_F16);
  else TRACEA_LAUNCH_CW(DT_BF16);
#undef TRACEA_LAUNCH_CW
  return (int)hipErrorInvalidValue;
}

}  // namespace tracea_amd
