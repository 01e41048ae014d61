// Convolution with the input patch AND the whole filter bank resident in LDS (gfx950).
//
// For layers with few, short filters (64 filters of 3x3x64: 72 KB) both operands of the
// implicit GEMM of one output tile fit LDS together.  A workgroup copies the padded input rows
// its pixels touch and the 64 filters of its slab into LDS once, waits once, and then
// multiplies with no barrier, no ring of stages and no wait on global memory in the loop: a
// k-step of a wave is six 16-byte LDS reads (four pixel fragments, two filter fragments)
// feeding seven MFMAs.
//
// Same arithmetic as the reference's kernel_main (src/emitter/cuda/conv.rs:153-331):
// out[n,ho,wo,k] = epilogue(sum_{r,s,c} x[n, ho*sh-ph+r*dh, wo*sw-pw+s*dw, c] * w[k,r,s,c]),
// fp32 accumulation in ascending (r,s,c) order, 16 channels per MFMA, zero padding.
//
// Work split.  A workgroup owns `p_tm` <= 448 consecutive output pixels of one image (the host
// picks p_tm so that the launch is one balanced round over the CUs) and 64 filters.  The
// pixels are cut into 14 blocks of 32 and the unit of work is one block x 32 filters (one
// v_mfma_f32_32x32x16 per 16-wide k-step; the 16x16x32 shape, which would halve the pixel
// granularity, sustains two thirds of this one's rate here): 28 units, 7 per SIMD.  Four
// waves, one per SIMD; wave s runs blocks s, s+4 and s+8 with both filter halves (6 units)
// and filters (s&1)*32.. of block 12 + (s>>1).  LDS delivers 128 bytes per clock to the CU,
// which is 1 KB per MFMA when all four matrix pipes run: a wave's reads per MFMA decide
// whether the loop runs at the MFMA rate or at the LDS rate.  Seven units on one wave take
// 6 reads per 7 MFMAs; the same units on two waves per SIMD (2 x 2 and 2 x 2 - 1 units,
// 4 reads per 4 and per 3 MFMAs) ran at the LDS rate, 9400 cycles for the 8064 of the MFMAs.
// Blocks past the tile repeat its last pixel and are not stored.  The filter fragment is the
// first MFMA operand, so a lane ends with 4 consecutive output channels of one pixel per
// (unit, 8-channel group).
//
// LDS layouts.  Patch: whole padded rows, pixel (hp, wp) at ((hp - hp0) * PW + wp) * cpp
// 16-byte chunks, cpp = C/8 rounded up to odd so that 16 consecutive pixels start in 16
// different bank groups.  Filters: row n at n * (K/8 | 1) chunks, for the same reason.
//
// An earlier form kept the filter bank in registers (one wave per SIMD, 288 registers of
// filters per lane): its main loop ran at 88 % of the MFMA rate, but everything around it --
// issuing the loads, moving the filters to registers, the epilogue -- is a single instruction
// stream per SIMD with nothing to overlap it and took twice as long as the loop.
#pragma once
#include "contraction_kernel.hpp"

namespace tracea_amd {

// LDS layout (bytes): [patch: p_np_bytes][filters: 64 rows x rs_cpb chunks, rounded to whole load
// iterations][epilogue operand table].
constexpr int rs_cpb(int ks) { return (ks * 2) | 1; }                                 // 16-byte chunks per filter row (odd)
constexpr int RS_THREADS = 512;  // four waves multiply; four more help to load the operands and to store the tile
constexpr int rs_filter_iters(int ks) { return (64 * rs_cpb(ks) + RS_THREADS - 1) / RS_THREADS; }  // one 16-byte chunk per thread
constexpr int rs_filter_bytes(int ks) { return rs_filter_iters(ks) * RS_THREADS * 16; }
constexpr int RS_TABLE_BYTES = TRACEA_MAX_EPILOGUE_OPS * 2 * 64 * 4;

// KS: 16-wide k-steps (K / 16); KPT: k-steps per filter tap (C / 16).
template <int DT, int KS, int KPT>
__global__ void __launch_bounds__(RS_THREADS) conv_resident_kernel(const ContractionArgs args) {
  constexpr int NT = RS_THREADS, BN = 64, NW = NT / 64;
  constexpr int CPB = rs_cpb(KS), FIT = rs_filter_iters(KS);

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  unsigned char *patch = smem;
  unsigned char *filt = smem + args.p_np_bytes;
  float *table = (float *)(filt + rs_filter_bytes(KS));

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave_u = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int simd = wave_u & 3;                       // (waves w and w + 4 share a SIMD)
  const bool worker = wave_u < 4;                    // waves 4-7 only move data: they sit at the barriers during the main loop
  const int lrow = lane & 31, lhalf = lane >> 5;     // operand row (pixel or filter) and 8-wide k group of the lane

  // ---- which tile ----
  int bid = blockIdx.x;
  const int total = gridDim.x;
  if ((total & 7) == 0) bid = (bid & 7) * (total >> 3) + (bid >> 3);  // contiguous run per XCD
  const int tile_n = bid % args.grid_n;
  const int tm = bid / args.grid_n;
  const int img = tm / args.p_tiles;
  const int TM = args.p_tm;
  const int p0 = (tm - img * args.p_tiles) * TM;  // first output pixel of the tile, within the image
  const int hw = args.h_out * args.w_out;
  const int npix = min(TM, hw - p0);
  const int n0 = tile_n * BN;
  const int N = args.N, C = args.c_in;
  const int PW = args.p_pw, cpp = args.p_cpp;
  const int pitch = cpp * 16;

  constexpr unsigned OOB = 0x80000000u;  // beyond every buffer: the load returns zeros
  const long long img_elems = (long long)args.h_in * args.w_in * C;
  __amdgpu_buffer_rsrc_t rsrc_x = __builtin_amdgcn_make_buffer_rsrc(
      (void *)((const unsigned short *)args.A + (long long)img * img_elems), 0, (int)(img_elems * 2), 0x00020000);
  __amdgpu_buffer_rsrc_t rsrc_w =
      __builtin_amdgcn_make_buffer_rsrc((void *)args.B, 0, (int)args.b_bytes, 0x00020000);

  // ---- filter bank -> LDS: chunk c is filter row c / CPB, 16-byte part c % CPB (the last part is padding) ----
#pragma unroll
  for (int it = 0; it < FIT; ++it) {
    const int chunk = it * NT + tid;
    const int row = chunk / CPB, part = chunk - row * CPB;
    const bool ok = (part < KS * 2) & (row < BN) & (n0 + row < N);
    const unsigned voff = ok ? (unsigned)(((n0 + row) * (int)args.ldb + part * 8) * 2) : OOB;
    unsigned char *dst = filt + (it * NT + wave_u * 64) * 16;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w, (__attribute__((address_space(3))) void *)dst, 16, (int)voff, 0, 0,
                                             0);
  }

  // ---- patch, by columns of load instructions ----
  // One load instruction moves the PPI = 64 / cpp pixels wp0 .. wp0 + PPI - 1 of one padded row (lane l:
  // pixel l / cpp, 16-byte part l % cpp; the part past the channels is padding and is written as zeros;
  // a last lane, if any, repeats the first part of the next pixel).  A wave takes segment j = wave,
  // wave + 8, ... of EVERY row: what depends on the lane (its pixel's column, whether that is padding)
  // is then fixed per segment and worked out once, and a load costs fourteen instructions with its loop --
  // row test, two selects, address updates -- where a mapping by instruction number, with the lane tests
  // redone for every load, cost thirty-six: with 160 loads per tile that was a seventh of the kernel's time.
  // Padding pixels and rows get an out-of-range offset and are written as zeros; lanes past the row's
  // end are switched off (they would land on the next row's pixels).
  int ho_f, wo_f, ho_l, wo_l;
  fast_divmod(p0, args.w_m, args.w_s, args.w_out, ho_f, wo_f);
  fast_divmod(p0 + npix - 1, args.w_m, args.w_s, args.w_out, ho_l, wo_l);
  const int hp0 = ho_f * args.stride_h;
  const int tap_h = args.dil_h * PW;  // pixel index step of one filter row
  const int n_rows = ho_l * args.stride_h + (args.r_sz - 1) * args.dil_h - hp0 + 1;
  const int SEG = args.p_seg, PPI = args.p_ppi;
  const int cdata = C >> 3;  // 16-byte parts of a pixel that hold channels
  int ldl, lpart;
  fast_divmod(lane, args.p_cpp_m, args.p_cpp_s, cpp, ldl, lpart);
  const int lane_off = (ldl - args.pad_w) * C * 2 + lpart * 16;  // byte offset from the row's first real pixel
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

  // ---- epilogue form and this thread's entry of the operand table (requested now, read after the wait) ----
  // Fast form (worked out by the host, args.fe): the chain reads [affine] [ReLU] [residual] [ReLU], each
  // part at most once and in this order, where affine is a bias, a scale-shift or a BatchNorm (all three
  // become v*a + b with per-channel a, b: a bias is a = 1); every channel of every tile exists, rows are
  // 8-byte aligned, output and residual have the operand type.  sig says which parts are present (bit 0
  // affine, 1 first ReLU, 2 residual, 3 second ReLU) and selects one of 16 straight-line epilogues; sig < 0:
  // any other chain, the general path.  Table: fast form entries [0..63] = a, [64..127] = b; general path
  // the layout of chain_table_value.
  const int sig = args.fe.sig;
  constexpr int TPT = RS_TABLE_BYTES / 4 / NT;  // table entries per thread on the general path
  float tabr = 0.0f, tabg[TPT];
  if (sig < 0) {
#pragma unroll
    for (int i = 0; i < TPT; ++i) {
      const int e = tid + i * NT;
      tabg[i] = chain_table_value(args.epi, e / (2 * BN), (e / BN) & 1, n0 + e % BN, N);
    }
  } else if ((sig & 1) && tid < 2 * BN) {
    const int which = tid / BN, n = n0 + tid % BN;
    if (args.fe.aff_kind == TRACEA_EPI_OP_BIAS_ADD) {
      float one[1] = {1.0f};
      if (which == 1) load_as_float<1>(args.fe.p0, args.fe.aff_dtype, n, 1, one);
      tabr = one[0];
    } else if (args.fe.aff_kind == TRACEA_EPI_OP_SCALE_SHIFT) {
      tabr = ((const float *)(which == 0 ? args.fe.p0 : args.fe.p1))[n];
    } else {  // BatchNorm folded: a = gamma / sqrt(var + eps), b = beta - mean * a
      const float scale = ((const float *)args.fe.p0)[n] * (1.0f / sqrtf(((const float *)args.fe.p3)[n] + args.fe.epsilon));
      tabr = which == 0 ? scale : ((const float *)args.fe.p1)[n] - ((const float *)args.fe.p2)[n] * scale;
    }
  }

  // ---- per-lane operand addresses ----
  // pixel blocks of this wave: slots 0-2 with both filter halves, slot 3 with the half hA
  const int hA = simd & 1;
  int a_base[4];
  int pix[4];  // pixel within the tile, -1 past its end
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int blk = i < 3 ? simd + 4 * i : 12 + (simd >> 1);
    const int pr = blk * 32 + lrow;
    pix[i] = pr < npix ? pr : -1;
    const int prc = pr < npix ? pr : npix - 1;
    int ho, wo;
    fast_divmod(p0 + prc, args.w_m, args.w_s, args.w_out, ho, wo);
    a_base[i] = ((ho * args.stride_h - hp0) * PW + wo * args.stride_w) * pitch + lhalf * 16;
  }
  // filter fragment (ks, h): filter h*32 + lrow, k = ks*16 + lhalf*8 .. +7, at ((h*32 + lrow)*CPB + lhalf)*16
  // + ks*32 bytes.  b_base[0] is the half hA (the one unit of the shared block uses it), b_base[1] the
  // other: the loop needs no select between the two fragments.
  const unsigned char *b_base[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) b_base[h] = filt + (((h == 0 ? hA : 1 - hA) * 32 + lrow) * CPB + lhalf) * 16;
  // tap offsets of the main loop (see there)
  int step_s = args.dil_w * pitch;
  int step_r = tap_h * pitch - (args.s_sz - 1) * step_s;
  int off_last = ((args.r_sz - 1) * tap_h + (args.s_sz - 1) * args.dil_w) * pitch;
  int s_size = args.s_sz;
  // (all of this is worked out HERE, while the operands travel: only the multiplying waves use it, and
  // the compiler would otherwise move it into their branch behind the barrier, 700 cycles of divisions
  // and argument loads in front of the first MFMA)
#pragma unroll
  for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(a_base[i]));
  asm volatile("" : "+s"(step_s), "+s"(step_r), "+s"(off_last), "+s"(s_size));

  f32x16 acc[7];  // units (slot i, half hA) = 2i, (slot i, half 1-hA) = 2i+1 for i < 3; (slot 3, half hA) = 6
#pragma unroll
  for (int u = 0; u < 7; ++u)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[u][e] = 0.0f;
  // (pinned here, in front of the wait for the operands: left alone the compiler clears the 112
  // registers right in front of the loop, 600 cycles after the operands have arrived)
#pragma unroll
  for (int u = 0; u < 7; ++u) asm volatile("" : "+a"(acc[u]));

  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): the table entry and this wave's shares of filters and patch are here
  if (sig < 0) {
#pragma unroll
    for (int i = 0; i < TPT; ++i) table[tid + i * NT] = tabg[i];
  } else if (tid < 2 * BN) {
    table[tid] = tabr;
  }
  __syncthreads();

  // ---- main loop: one filter tap (KPT k-steps) per iteration, operands read two k-steps ahead ----
  // An LDS read takes about 150 cycles to return and the wave has nobody to hide that behind, hence
  // the two k-steps of look-ahead (four operand sets in rotation: with KPT = 4 the set of a k-step is
  // the same in every iteration).  The loop is rolled over the taps on purpose: written as one
  // straight line of K/16 k-steps it ran at 39 cycles per MFMA instead of 33, every instruction being
  // fetched exactly once and never found in the instruction cache.
  static_assert(KPT == 4, "the operand sets rotate with the four k-steps of a tap");
  constexpr int TAPS = KS / KPT;
  // a wave whose first block lies past the tile has no pixels at all (its other blocks come later still)
  const bool active = worker && simd * 32 < npix;
  if (active) {
    u32x4 xa[4][4], xb[4][2];
    // byte offset of the tap being read: a step along the filter row adds step_s, the step to the next
    // row step_r; kept by additions and clamped to the last tap (the two look-ahead reads past the end of
    // K are never used, they only have to stay inside the patch), so that the loop's tail is a handful of
    // scalar instructions without a branch: the matrix pipe idles while a lone wave executes them
    int ts = 0, off = 0;
    auto next_tap = [&]() {
      ts += 1;
      const bool wrap_s = ts == s_size;
      ts = wrap_s ? 0 : ts;
      off += wrap_s ? step_r : step_s;
      off = off < off_last ? off : off_last;
    };
    const unsigned char *pa[4], *pn[4];  // the wave's pixel fragments under the current and the next tap
    const unsigned char *pb[2] = {b_base[0], b_base[1]};
#pragma unroll
    for (int i = 0; i < 4; ++i) pa[i] = patch + a_base[i];
    next_tap();
#pragma unroll
    for (int i = 0; i < 4; ++i) pn[i] = patch + a_base[i] + off;
    // set: operand set written; src: fragments of the current (false) or next (true) tap; k: k-step within that tap
    auto read = [&](auto setc, auto nextc, auto kc) __attribute__((always_inline)) {
      constexpr int set = decltype(setc)::value, k = decltype(kc)::value;
      constexpr bool nx = decltype(nextc)::value;
      xb[set][0] = *(const u32x4 *)(pb[0] + (nx ? KPT * 32 : 0) + k * 32);
      xa[set][0] = *(const u32x4 *)((nx ? pn[0] : pa[0]) + k * 32);
      xb[set][1] = *(const u32x4 *)(pb[1] + (nx ? KPT * 32 : 0) + k * 32);
      xa[set][1] = *(const u32x4 *)((nx ? pn[1] : pa[1]) + k * 32);
      xa[set][2] = *(const u32x4 *)((nx ? pn[2] : pa[2]) + k * 32);
      xa[set][3] = *(const u32x4 *)((nx ? pn[3] : pa[3]) + k * 32);
    };
    auto mma = [&](auto setc) __attribute__((always_inline)) {
      constexpr int s = decltype(setc)::value;
      acc[0] = Mfma32<DT>::run(xb[s][0], xa[s][0], acc[0]);
      acc[1] = Mfma32<DT>::run(xb[s][1], xa[s][0], acc[1]);
      acc[2] = Mfma32<DT>::run(xb[s][0], xa[s][1], acc[2]);
      acc[3] = Mfma32<DT>::run(xb[s][1], xa[s][1], acc[3]);
      acc[4] = Mfma32<DT>::run(xb[s][0], xa[s][2], acc[4]);
      acc[5] = Mfma32<DT>::run(xb[s][1], xa[s][2], acc[5]);
      acc[6] = Mfma32<DT>::run(xb[s][0], xa[s][3], acc[6]);
      Interleave<0, 7, 0x100, 6, 0x100, 0>::run();
      __builtin_amdgcn_sched_barrier(0);
    };
    using std::integral_constant;
    using std::false_type;
    using std::true_type;
    read(integral_constant<int, 0>{}, false_type{}, integral_constant<int, 0>{});
    read(integral_constant<int, 1>{}, false_type{}, integral_constant<int, 1>{});
    __builtin_amdgcn_sched_barrier(0);
    auto tap = [&]() __attribute__((always_inline)) {
      read(integral_constant<int, 2>{}, false_type{}, integral_constant<int, 2>{});
      mma(integral_constant<int, 0>{});
      read(integral_constant<int, 3>{}, false_type{}, integral_constant<int, 3>{});
      mma(integral_constant<int, 1>{});
      // (after the last tap these two read the last tap again: in range, never used)
      read(integral_constant<int, 0>{}, true_type{}, integral_constant<int, 0>{});
      mma(integral_constant<int, 2>{});
      read(integral_constant<int, 1>{}, true_type{}, integral_constant<int, 1>{});
      mma(integral_constant<int, 3>{});
      next_tap();
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        pa[i] = pn[i];
        pn[i] = patch + a_base[i] + off;
      }
      pb[0] += KPT * 32;  // (the reads past the last tap run into the row's padding and the next row)
      pb[1] += KPT * 32;
    };
    // TPI taps per trip: a taken branch costs a lone wave more than a hundred cycles of idle matrix
    // pipe, code that is executed for the first time about five cycles per MFMA
    constexpr int TPI = TAPS % 3 == 0 ? 3 : 1;
#pragma unroll 1
    for (int t = 0; t < TAPS; t += TPI) {
#pragma unroll
      for (int j = 0; j < TPI; ++j) tap();
    }
  }

  // ---- epilogue ----
  // lane: pixel lrow of each block; accumulator element 4g + r of a unit with filter half h is channel
  // n0 + h*32 + 8g + 4*lhalf + r.  The accumulators go through LDS (patch and filters are dead once every
  // wave has left the main loop): a pixel's 64 channels become one contiguous row, and a rolled loop
  // takes them from there, 8 channels of one pixel per thread and step, so that a pixel leaves as one
  // whole 128-byte row written by 8 neighbouring lanes.  Storing straight from the MFMA layout (a lane
  // holds 4 channels of a pixel: 8-byte pieces, 32 different rows per store instruction) kept the
  // write path busy with four times the requests and took three times as long; and code that runs once
  // per wave, as one straight line per unit does, is fetched at about a third of a cycle per byte here,
  // nothing of a launch being in the instruction cache when it starts.
  const long long m_img = (long long)img * hw + p0;
  constexpr int SP = BN + 4;  // floats per staged pixel
  float *stage = (float *)smem;
  __syncthreads();  // every wave has left the main loop: the patch may be overwritten
  // (only pixels of the tile are staged: the area reserved for staging is p_tm pixels, and the operand
  // table lies behind it)
  auto stage_unit = [&](const f32x16 &a, int blk, int h) __attribute__((always_inline)) {
    if (blk * 32 + lrow < npix) {
      static_for<0, 4>([&](auto gc) {
        constexpr int g = decltype(gc)::value;
        const f32x4 v = {a[g * 4 + 0], a[g * 4 + 1], a[g * 4 + 2], a[g * 4 + 3]};
        *(f32x4 *)(stage + (blk * 32 + lrow) * SP + h * 32 + g * 8 + lhalf * 4) = v;
      });
    }
  };
  if (active) {
    stage_unit(acc[0], simd, hA);
    stage_unit(acc[1], simd, 1 - hA);
    stage_unit(acc[2], simd + 4, hA);
    stage_unit(acc[3], simd + 4, 1 - hA);
    stage_unit(acc[4], simd + 8, hA);
    stage_unit(acc[5], simd + 8, 1 - hA);
    stage_unit(acc[6], 12 + (simd >> 1), hA);
  }
  __syncthreads();
  const int ec = (tid & 7) * 8;  // this thread's 8 channels, the same in every step
  if (sig >= 0) {
    // Stores and residual loads go through buffer addressing: base = first row of the tile, 32-bit
    // per-lane byte offset, which for a pixel past the tile is out of range (the store is dropped, the
    // load returns zero).  One loop per form, the form a compile-time constant: with the parts behind
    // run-time tests every value ended in a wait for the previous store.
    __amdgpu_buffer_rsrc_t rsrc_c = __builtin_amdgcn_make_buffer_rsrc(
        (void *)((unsigned short *)args.C + m_img * args.ldc + n0), 0, (int)((long long)npix * args.ldc * 2), 0x00020000);
    __amdgpu_buffer_rsrc_t rsrc_r = __builtin_amdgcn_make_buffer_rsrc(
        (void *)((const unsigned short *)args.fe.res + ((sig & 4) ? m_img * args.fe.res_ld + n0 : 0ll)), 0,
        (sig & 4) ? (int)((long long)npix * args.fe.res_ld * 2) : 0, 0x00020000);
    const int row_c = (int)args.ldc * 2, row_r = (int)args.fe.res_ld * 2;
    auto run_form = [&](auto form) __attribute__((always_inline)) {
      constexpr int F = decltype(form)::value;
      constexpr bool AFF = (F & 1) != 0, RELU1 = (F & 2) != 0, RES = (F & 4) != 0, RELU2 = (F & 8) != 0;
      float ta[8], tb[8];
      if constexpr (AFF) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          ta[e] = table[ec + e];
          tb[e] = table[BN + ec + e];
        }
      }
      constexpr int PPS = NT / 8;  // pixels per step of the workgroup
      constexpr int UN = 4;        // steps in flight: their LDS reads and residual loads are issued together
      for (int pr0 = tid >> 3; pr0 < npix; pr0 += UN * PPS) {
        f32x4 lo[UN], hi[UN];
        u32x4 raw[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
          const int pr = pr0 + u * PPS;
          const int prc = pr < npix ? pr : npix - 1;
          lo[u] = *(const f32x4 *)(stage + prc * SP + ec);
          hi[u] = *(const f32x4 *)(stage + prc * SP + ec + 4);
          if constexpr (RES)
            raw[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(
                         rsrc_r, pr < npix ? pr * row_r + ec * 2 : (int)OOB, 0, 0));
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
          const int pr = pr0 + u * PPS;
          float v[8] = {lo[u][0], lo[u][1], lo[u][2], lo[u][3], hi[u][0], hi[u][1], hi[u][2], hi[u][3]};
          if constexpr (AFF) {
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = v[e] * ta[e] + tb[e];
          }
          if constexpr (RELU1) {
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = fmaxf(0.0f, v[e]);
          }
          if constexpr (RES) {  // (the fast form requires the residual in the operand type)
            if constexpr (DT == DT_F16) {
              const f16x8 hv = __builtin_bit_cast(f16x8, raw[u]);
#pragma unroll
              for (int e = 0; e < 8; ++e) v[e] = v[e] + (float)hv[e];
            } else {
              const bf16x8 hv = __builtin_bit_cast(bf16x8, raw[u]);
#pragma unroll
              for (int e = 0; e < 8; ++e) v[e] = v[e] + (float)hv[e];
            }
          }
          if constexpr (RELU2) {
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = fmaxf(0.0f, v[e]);
          }
          u32x4 out;
          if constexpr (DT == DT_F16) {
            const f16x8 hv = {(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3],
                              (_Float16)v[4], (_Float16)v[5], (_Float16)v[6], (_Float16)v[7]};
            out = __builtin_bit_cast(u32x4, hv);
          } else {
            const bf16x8 hv = {(__bf16)v[0], (__bf16)v[1], (__bf16)v[2], (__bf16)v[3],
                               (__bf16)v[4], (__bf16)v[5], (__bf16)v[6], (__bf16)v[7]};
            out = __builtin_bit_cast(u32x4, hv);
          }
          __builtin_amdgcn_raw_buffer_store_b128(out, rsrc_c, pr < npix ? pr * row_c + ec * 2 : (int)OOB, 0, 0);
        }
      }
    };
    switch (sig) {
#define TRACEA_RS_FORM(F) case F: run_form(std::integral_constant<int, F>{}); break;
      TRACEA_RS_FORM(0) TRACEA_RS_FORM(1) TRACEA_RS_FORM(2) TRACEA_RS_FORM(3) TRACEA_RS_FORM(4) TRACEA_RS_FORM(5)
      TRACEA_RS_FORM(6) TRACEA_RS_FORM(7) TRACEA_RS_FORM(8) TRACEA_RS_FORM(9) TRACEA_RS_FORM(10) TRACEA_RS_FORM(11)
      TRACEA_RS_FORM(12) TRACEA_RS_FORM(13) TRACEA_RS_FORM(14) TRACEA_RS_FORM(15)
#undef TRACEA_RS_FORM
      default: break;
    }
  } else {
    // every other case (partial channel groups, unaligned rows, fp32 output, GELU / SiLU, further
    // residuals): the general operator chain on the staged values
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
}

template <int KS, int KPT>
int launch_conv_resident(const ContractionArgs &a, bool conv, int dtype, bool b_ncontig, hipStream_t stream) {
  if (!conv || b_ncontig || a.K != KS * 16 || a.c_in != KPT * 16 || a.p_tm <= 0 || a.p_tm > 448 || a.p_np_bytes <= 0) return (int)hipErrorInvalidValue;
  const size_t lds = (size_t)a.p_np_bytes + (size_t)rs_filter_bytes(KS) + RS_TABLE_BYTES;
  // the general epilogue stages p_tm x 68 floats in front of the table
  if (lds > 160 * 1024 || (size_t)a.p_tm * 68 * 4 > lds - RS_TABLE_BYTES) return (int)hipErrorInvalidValue;
  const dim3 grid((unsigned)(a.grid_m * a.grid_n)), block(RS_THREADS);
#define TRACEA_LAUNCH_RS(DTV)                                                                        \
  do {                                                                                               \
    auto kfn = conv_resident_kernel<DTV, KS, KPT>;                                                    \
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
  if (dtype == DT_F16) TRACEA_LAUNCH_RS(DT_F16);
  else TRACEA_LAUNCH_RS(DT_BF16);
#undef TRACEA_LAUNCH_RS
  return (int)hipErrorInvalidValue;
}

}  // namespace tracea_amd
