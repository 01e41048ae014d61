// Convolution with the input patch AND the whole filter bank resident in LDS (gfx950).
//
// For layers with few, short filters (64 filters of 3x3x64: 72 KB) both operands of the
// implicit GEMM of one output tile fit LDS together.  A workgroup copies the padded input rows
// its pixels touch and the 64 filters of its slab into LDS once, waits once, and then
// multiplies with no barrier, no ring of stages and no wait on global memory in the loop: a
// k-step of a wave is four 16-byte LDS reads (two pixel fragments, two filter fragments)
// feeding four MFMAs.
//
// Same arithmetic as the reference's kernel_main (src/emitter/cuda/conv.rs:153-331):
// out[n,ho,wo,k] = epilogue(sum_{r,s,c} x[n, ho*sh-ph+r*dh, wo*sw-pw+s*dw, c] * w[k,r,s,c]),
// fp32 accumulation in ascending (r,s,c) order, 16 channels per MFMA, zero padding.
//
// Work split.  A workgroup owns `p_tm` <= 448 consecutive output pixels of one image (the host
// picks p_tm so that the launch is one balanced round over the CUs) and 64 filters.  The
// pixels are cut into 14 blocks of 32 and the unit of work is one block x 32 filters (one
// v_mfma_f32_32x32x16 per 16-wide k-step; the 16x16x32 shape, which would halve the pixel
// granularity, sustains two thirds of this one's rate here): 28 units, 7 per SIMD.  Eight
// waves, two per SIMD; on SIMD s the first wave runs blocks 3s and 3s+1 with both filter
// halves (4 units), the second block 3s+2 with both halves and filters (s&1)*32.. of block
// 12 + (s>>1) (3 units).  Blocks past the tile repeat its last pixel and are not stored.  The
// filter fragment is the first MFMA operand, so a lane ends with 4 consecutive output
// channels of one pixel per (unit, 8-channel group) and stores them as 8 bytes, straight from
// registers.
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
constexpr int rs_filter_iters(int ks) { return (64 * rs_cpb(ks) + 511) / 512; }       // 512 threads x 16 bytes
constexpr int rs_filter_bytes(int ks) { return rs_filter_iters(ks) * 512 * 16; }
constexpr int RS_TABLE_BYTES = TRACEA_MAX_EPILOGUE_OPS * 2 * 64 * 4;

// KS: 16-wide k-steps (K / 16); KPT: k-steps per filter tap (C / 16).
template <int DT, int KS, int KPT>
__global__ void __launch_bounds__(512) conv_resident_kernel(const ContractionArgs args) {
  constexpr int NT = 512, BN = 64;
  constexpr int CPB = rs_cpb(KS), FIT = rs_filter_iters(KS);

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  unsigned char *patch = smem;
  unsigned char *filt = smem + args.p_np_bytes;
  float *table = (float *)(filt + rs_filter_bytes(KS));

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave_u = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int simd = wave_u & 3, wtype = wave_u >> 2;  // (waves w and w+4 of a workgroup share a SIMD)
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
  for (int j = wave_u; j < SEG; j += 8) {
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
  float tabr = 0.0f;
  if (sig < 0) {
    tabr = chain_table_value(args.epi, tid / (2 * BN), (tid / BN) & 1, n0 + tid % BN, N);
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
  // pixel blocks of this wave: slot 0 and slot 1 (see the work split above)
  const int xh = simd & 1;  // filter half a second wave computes of its shared block
  int a_base[2];
  int pix[2];  // pixel within the tile, -1 past its end
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int blk = wtype == 0 ? 3 * simd + i : (i == 0 ? 3 * simd + 2 : 12 + (simd >> 1));
    const int pr = blk * 32 + lrow;
    pix[i] = pr < npix ? pr : -1;
    const int prc = pr < npix ? pr : npix - 1;
    int ho, wo;
    fast_divmod(p0 + prc, args.w_m, args.w_s, args.w_out, ho, wo);
    a_base[i] = ((ho * args.stride_h - hp0) * PW + wo * args.stride_w) * pitch + lhalf * 16;
  }
  // filter fragment (ks, h): filter h*32 + lrow, k = ks*16 + lhalf*8 .. +7, at b_base[h] + ks*32 bytes
  const unsigned char *b_base[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) b_base[h] = filt + ((h * 32 + lrow) * CPB + lhalf) * 16;

  // byte offset into the patch of filter tap t (uniform values); the KPT k-steps of a tap are 32 bytes apart
  constexpr int TAPS = KS / KPT;
  int tapoff[TAPS];
  {
    int tq = 0, ts = 0;  // pixel offset of (r, s=0); s
#pragma unroll
    for (int t = 0; t < TAPS; ++t) {
      tapoff[t] = (tq + ts * args.dil_w) * pitch;
      ts += 1;
      const bool wrap_s = ts == args.s_sz;
      ts = wrap_s ? 0 : ts;
      tq += wrap_s ? tap_h : 0;
    }
  }

  f32x16 acc[4];  // units (slot 0, half 0), (slot 0, half 1), (slot 1, half 0 or xh), (slot 1, half 1)
#pragma unroll
  for (int u = 0; u < 4; ++u)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[u][e] = 0.0f;

  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): the table entry and this wave's shares of filters and patch are here
  table[tid] = tabr;
  __syncthreads();

  // ---- main loop: operands of k-step ks+1 are read while k-step ks is multiplied ----
  auto main_loop = [&](auto full) __attribute__((always_inline)) {
    constexpr bool FULL = decltype(full)::value;  // 4 units; else 3: (slot 1) has the one half xh
    u32x4 xa[2][2], xb[2][2];
    const unsigned char *ap[2] = {patch, patch};  // the wave's two pixel fragments under the current tap
    auto read = [&](int set, int ks) __attribute__((always_inline)) {
      if (ks % KPT == 0) {
        ap[0] = patch + a_base[0] + tapoff[ks / KPT];
        ap[1] = patch + a_base[1] + tapoff[ks / KPT];
      }
      xa[set][0] = *(const u32x4 *)(ap[0] + (ks % KPT) * 32);
      xa[set][1] = *(const u32x4 *)(ap[1] + (ks % KPT) * 32);
      xb[set][0] = *(const u32x4 *)(b_base[0] + ks * 32);
      xb[set][1] = *(const u32x4 *)(b_base[1] + ks * 32);
    };
    read(0, 0);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (ks + 1 < KS) read((ks + 1) & 1, ks + 1);
      const int s = ks & 1;
      acc[0] = Mfma32<DT>::run(xb[s][0], xa[s][0], acc[0]);
      acc[1] = Mfma32<DT>::run(xb[s][1], xa[s][0], acc[1]);
      if constexpr (FULL) {
        acc[2] = Mfma32<DT>::run(xb[s][0], xa[s][1], acc[2]);
        acc[3] = Mfma32<DT>::run(xb[s][1], xa[s][1], acc[3]);
      } else {
        acc[2] = Mfma32<DT>::run(xh ? xb[s][1] : xb[s][0], xa[s][1], acc[2]);
      }
      if (ks + 1 < KS) Interleave<0, FULL ? 4 : 3, 0x100, 4, 0x100, 0>::run();
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // a wave whose first block lies past the tile has no pixels at all (its second block comes later still)
  const bool active = (wtype == 0 ? 3 * simd : 3 * simd + 2) * 32 < npix;
  if (active) {
    if (wtype == 0) main_loop(std::true_type{});
    else main_loop(std::false_type{});
  }

  // ---- epilogue ----
  // lane: pixel lrow of each block; accumulator element 4g + r of a unit with filter half h is channel
  // n0 + h*32 + 8g + 4*lhalf + r
  const long long m_img = (long long)img * hw + p0;
  if (sig >= 0) {
    // Stores and residual loads go through buffer addressing: base = first row of the tile, 32-bit
    // per-lane byte offset, which for a pixel past the tile is out of range (the store is dropped, the
    // load returns zero): no branches, no 64-bit address arithmetic.  The code of a unit is a straight
    // line for each of the 16 forms: with the parts behind run-time tests every group of four values
    // ended in a wait for the previous group's store.
    __amdgpu_buffer_rsrc_t rsrc_c = __builtin_amdgcn_make_buffer_rsrc(
        (void *)((unsigned short *)args.C + m_img * args.ldc + n0), 0, (int)((long long)npix * args.ldc * 2), 0x00020000);
    __amdgpu_buffer_rsrc_t rsrc_r = __builtin_amdgcn_make_buffer_rsrc(
        (void *)((const unsigned short *)args.fe.res + ((sig & 4) ? m_img * args.fe.res_ld + n0 : 0ll)), 0,
        (sig & 4) ? (int)((long long)npix * args.fe.res_ld * 2) : 0, 0x00020000);
    unsigned c_off[2], r_off[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      c_off[i] = pix[i] >= 0 ? (unsigned)(pix[i] * (int)args.ldc * 2 + lhalf * 8) : OOB;
      r_off[i] = pix[i] >= 0 ? (unsigned)(pix[i] * (int)args.fe.res_ld * 2 + lhalf * 8) : OOB;
    }
    // filter half of the unit in accumulator 2: 0 for a first wave, xh for a second
    const int h2 = wtype == 0 ? 0 : xh;
    auto run_form = [&](auto form) __attribute__((always_inline)) {
      constexpr int F = decltype(form)::value;
      constexpr bool AFF = (F & 1) != 0, RELU1 = (F & 2) != 0, RES = (F & 4) != 0, RELU2 = (F & 8) != 0;
      // one unit: 4 groups of 4 consecutive channels of pixel slot i, filter half h (a uniform run-time value
      // for accumulator 2: it only enters addresses)
      auto finish = [&](const f32x16 &a, auto ic, int h) __attribute__((always_inline)) {
        constexpr int i = decltype(ic)::value;
        u32x2 raw[4];
        f32x4 ta[4], tb[4];
        if constexpr (RES) {
#pragma unroll
          for (int g = 0; g < 4; ++g)
            raw[g] = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(rsrc_r, (int)r_off[i], (h * 32 + g * 8) * 2, 0));
        }
        if constexpr (AFF) {
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const int ch = h * 32 + g * 8 + lhalf * 4;  // first of this lane's 4 channels in group g
            ta[g] = *(const f32x4 *)(table + ch);
            tb[g] = *(const f32x4 *)(table + BN + ch);
          }
        }
        static_for<0, 4>([&](auto gc) {
          constexpr int g = decltype(gc)::value;
          float v[4] = {a[g * 4 + 0], a[g * 4 + 1], a[g * 4 + 2], a[g * 4 + 3]};
          if constexpr (AFF) {
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = v[e] * ta[g][e] + tb[g][e];
          }
          if constexpr (RELU1) {
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = fmaxf(0.0f, v[e]);
          }
          if constexpr (RES) {  // (the fast form requires the residual in the operand type)
            if constexpr (DT == DT_F16) {
              const f16x4 hv = __builtin_bit_cast(f16x4, raw[g]);
#pragma unroll
              for (int e = 0; e < 4; ++e) v[e] = v[e] + (float)hv[e];
            } else {
              const bf16x4 hv = __builtin_bit_cast(bf16x4, raw[g]);
#pragma unroll
              for (int e = 0; e < 4; ++e) v[e] = v[e] + (float)hv[e];
            }
          }
          if constexpr (RELU2) {
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = fmaxf(0.0f, v[e]);
          }
          u32x2 out;
          if constexpr (DT == DT_F16) {
            const f16x4 hv = {(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
            out = __builtin_bit_cast(u32x2, hv);
          } else {
            const bf16x4 hv = {(__bf16)v[0], (__bf16)v[1], (__bf16)v[2], (__bf16)v[3]};
            out = __builtin_bit_cast(u32x2, hv);
          }
          __builtin_amdgcn_raw_buffer_store_b64(out, rsrc_c, (int)c_off[i], (h * 32 + g * 8) * 2, 0);
        });
      };
      using std::integral_constant;
      finish(acc[0], integral_constant<int, 0>{}, 0);
      finish(acc[1], integral_constant<int, 0>{}, 1);
      finish(acc[2], integral_constant<int, 1>{}, h2);
      if (wtype == 0) finish(acc[3], integral_constant<int, 1>{}, 1);
    };
    switch (active ? sig : -1) {
#define TRACEA_RS_FORM(F) case F: run_form(std::integral_constant<int, F>{}); break;
      TRACEA_RS_FORM(0) TRACEA_RS_FORM(1) TRACEA_RS_FORM(2) TRACEA_RS_FORM(3) TRACEA_RS_FORM(4) TRACEA_RS_FORM(5)
      TRACEA_RS_FORM(6) TRACEA_RS_FORM(7) TRACEA_RS_FORM(8) TRACEA_RS_FORM(9) TRACEA_RS_FORM(10) TRACEA_RS_FORM(11)
      TRACEA_RS_FORM(12) TRACEA_RS_FORM(13) TRACEA_RS_FORM(14) TRACEA_RS_FORM(15)
#undef TRACEA_RS_FORM
      default: break;
    }
  } else {
    // every other case (partial channel groups, unaligned rows, fp32 output, GELU / SiLU, further
    // residuals): the accumulators go through LDS (the patch and the filter area are free now) and a
    // rolled loop takes them from there, 8 channels of one pixel per thread and step
    constexpr int SP = BN + 4;  // floats per staged pixel
    float *stage = (float *)smem;
    const ChainPlan plan = chain_plan(args.epi);
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
    const int blk0 = wtype == 0 ? 3 * simd : 3 * simd + 2, blk1 = wtype == 0 ? 3 * simd + 1 : 12 + (simd >> 1);
    stage_unit(acc[0], blk0, 0);
    stage_unit(acc[1], blk0, 1);
    stage_unit(acc[2], blk1, wtype == 0 ? 0 : xh);
    if (wtype == 0) stage_unit(acc[3], blk1, 1);
    __syncthreads();
    for (int idx = tid; idx < npix * (BN / 8); idx += NT) {
      const int pr = idx >> 3, ec = (idx & 7) * 8;
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
  const dim3 grid((unsigned)(a.grid_m * a.grid_n)), block(512);
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
