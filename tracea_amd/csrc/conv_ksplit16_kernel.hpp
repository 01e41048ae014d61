// Convolution on 16x16x32 MFMAs for layers with few pixels per image and many channels (the 14x14x256 and
// 7x7x512 stages of a ResNet): the input patch resident in LDS, the filter slab streamed through a ring of
// 128-channel stages, and the K axis split over the four multiplying waves of the workgroup (gfx950).
//
// Same arithmetic as the reference's kernel_main (src/emitter/cuda/conv.rs:153-331):
// out[n,ho,wo,k] = epilogue(sum_{r,s,c} x[n, ho*sh-ph+r*dh, wo*sw-pw+s*dw, c] * w[k,r,s,c]), fp32 accumulation,
// zero padding; the sum over (r,s,c) is formed as four partial sums (one per wave: the 32-channel quarter
// c % 128 / 32 of every tap) that are added in wave order at the end.
//
// Why the split.  For one balanced round over 256 CUs these layers leave a workgroup 98 or 49 pixels by 64
// filters.  Cut by pixels over four waves, a wave would multiply 2 pixel blocks by 4 filter blocks per
// k-step and read 6 KB of LDS for 8 MFMAs, 1.5 times what LDS delivers while the matrix pipes run.  Cut by
// K, every wave multiplies ALL the tile's pixel blocks by all four filter blocks (NPB + 4 fragments of 1 KB
// for 4 NPB MFMAs: 0.39 KB per MFMA at NPB = 7) on its own quarter of the channels of each stage, and the
// four partial tiles meet once, through LDS: each wave keeps the pixel blocks p with p % 4 == wave and
// writes the others out for their owners (3/4 of 4 NPB KB per wave, once per tile).
//
// LDS layouts.  Patch: whole padded rows, pixel (hp, wp) at ((hp - hp0) * PW + wp) * cpp 16-byte chunks,
// cpp = C/8 rounded up to odd (the 16 pixels of a fragment start in 16 different bank groups); fetched as a
// flat run of chunks per row, so any channel count fits the 64-lane load.  Ring: stage s % RING holds
// channels 128 (s % (C/128)) .. + 127 of tap s / (C/128) for the 64 filters, row n at n * 256 bytes with its
// 16-byte column XOR (n & 7): a wave's fragment (16 filters x its 32 channels) reads conflict-free and a load
// instruction fills four whole rows.
//
// Epilogue: from registers, by the owner of each pixel block (conv_epilogue16.hpp); any other chain goes
// through LDS and the general operator loop.
#pragma once
#include "conv_epilogue16.hpp"

namespace tracea_amd {

constexpr int CK_THREADS = 512;
constexpr int CK_TABLE_BYTES = TRACEA_MAX_EPILOGUE_OPS * 2 * 64 * 4;
constexpr int CK_STAGE_BYTES = 64 * 256;  // 64 filters x 128 channels

template <int DT, int CIN, int NPB, int RING>
__global__ void __launch_bounds__(CK_THREADS) conv_ksplit16_kernel(const ContractionArgs args) {
  constexpr int NT = CK_THREADS, BN = 64, NW = NT / 64;
  constexpr int CPT = CIN / 128;  // stages (128-channel chunks) per filter tap
  static_assert(CIN % 256 == 0 && RING >= 3 && NPB >= 1 && NPB <= 8, "unsupported shape");
  constexpr int RIT = CK_STAGE_BYTES / 1024 / 4;  // load instructions per helper wave and stage
  constexpr int OWN = (NPB + 3) / 4;              // pixel blocks a wave finishes at most

  asm volatile("" ::"s"(args.A), "s"(args.B), "s"(args.N), "s"(args.K), "s"(args.ldb), "s"(args.b_bytes), "s"(args.grid_n),
               "s"(args.h_in), "s"(args.w_in), "s"(args.h_out), "s"(args.w_out), "s"(args.s_sz), "s"(args.r_sz));
  asm volatile("" ::"s"(args.stride_h), "s"(args.stride_w), "s"(args.pad_h), "s"(args.pad_w), "s"(args.dil_h), "s"(args.dil_w),
               "s"(args.w_m), "s"(args.w_s), "s"(args.p_tiles), "s"(args.p_pw), "s"(args.p_cpp), "s"(args.p_np_bytes),
               "s"(args.p_tm), "s"(args.p_seg), "s"(args.p_cpp_m), "s"(args.p_cpp_s), "s"(args.gn_m), "s"(args.gn_s),
               "s"(args.pt_m), "s"(args.pt_s));
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  unsigned char *patch = smem;
  unsigned char *ring = smem + args.p_np_bytes;
  const int stages = args.r_sz * args.s_sz * CPT;
  // (the operand table lies behind the operands or, if that is more, behind what the end of the kernel stages)
  const int operand_bytes = args.p_np_bytes + RING * CK_STAGE_BYTES;
  constexpr int REDUCE_BYTES = 4 * NPB * 4 * 1024;  // [unit][wave][lane] float4
  const int general_bytes = args.p_tm * (BN + 4) * 4;
  const int staging_bytes = REDUCE_BYTES > general_bytes ? REDUCE_BYTES : general_bytes;
  float *table = (float *)(smem + (operand_bytes > staging_bytes ? operand_bytes : staging_bytes));

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave_u = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int w = wave_u & 3;
  const bool worker = wave_u < 4;
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
  const int N = args.N;
  const int PW = args.p_pw, cpp = args.p_cpp;
  const int pitch = cpp * 16;

  constexpr unsigned OOB = 0x80000000u;  // beyond every buffer: the load returns zeros
  const long long img_elems = (long long)args.h_in * args.w_in * CIN;
  __amdgpu_buffer_rsrc_t rsrc_x = __builtin_amdgcn_make_buffer_rsrc(
      (void *)((const unsigned short *)args.A + (long long)img * img_elems), 0, (int)(img_elems * 2), 0x00020000);
  __amdgpu_buffer_rsrc_t rsrc_w =
      __builtin_amdgcn_make_buffer_rsrc((void *)args.B, 0, (int)args.b_bytes, 0x00020000);

  // ---- ring: helper wave h, load instruction it, fills rows (it*4 + h)*4 .. + 3 of a stage; lane l is row
  // l / 16 of them, 16-byte slot l % 16, and fetches the column that the row's swizzle maps there ----
  unsigned ring_voff[RIT];
#pragma unroll
  for (int it = 0; it < RIT; ++it) {
    const int row = (it * 4 + (wave_u & 3)) * 4 + (lane >> 4);
    const int col = (lane & 15) ^ (row & 7);
    ring_voff[it] = n0 + row < N ? (unsigned)(((n0 + row) * (int)args.ldb + col * 8) * 2) : OOB;
  }
  auto ring_issue = [&](int s) __attribute__((always_inline)) {
    unsigned char *sb = ring + (s % RING) * CK_STAGE_BYTES;
    const int tap = s / CPT, chunk = s - tap * CPT;
    const int koff = (tap * CIN + chunk * 128) * 2;
#pragma unroll
    for (int it = 0; it < RIT; ++it) {
      unsigned char *dst = sb + (it * 4 + (wave_u & 3)) * 1024;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w, (__attribute__((address_space(3))) void *)dst, 16,
                                               (int)ring_voff[it], koff, 0, 0);
    }
  };

  // ---- patch: every padded row as a flat run of PW * cpp chunks; load instruction j of a row covers chunks
  // 64 j .. 64 j + 63, lane l chunk 64 j + l = pixel c / cpp, part c % cpp (the part past the channels is
  // padding and is written as zeros, as are padding pixels and rows); wave v takes instructions v, v + 8, ...
  // of EVERY row, so what depends on the lane is worked out once per instruction ----
  int ho_f, wo_f, ho_l, wo_l;
  fast_divmod(p0, args.w_m, args.w_s, args.w_out, ho_f, wo_f);
  fast_divmod(p0 + npix - 1, args.w_m, args.w_s, args.w_out, ho_l, wo_l);
  const int hp0 = ho_f * args.stride_h;
  const int tap_h = args.dil_h * PW;
  const int n_rows = ho_l * args.stride_h + (args.r_sz - 1) * args.dil_h - hp0 + 1;
  const int row_chunks = PW * cpp;
  const int SEG = args.p_seg;  // load instructions per row: ceil(row_chunks / 64)
  const int row_bytes = args.w_in * CIN * 2, row_pitch = row_chunks * 16;
  for (int j = wave_u; j < SEG; j += NW) {
    const int c = j * 64 + lane;
    int wp, part;
    fast_divmod(c, args.p_cpp_m, args.p_cpp_s, cpp, wp, part);
    const bool lane_ok = ((unsigned)(wp - args.pad_w) < (unsigned)args.w_in) & (part < CIN / 8);
    const unsigned v_seg = lane_ok ? (unsigned)((wp - args.pad_w) * CIN * 2 + part * 16) : OOB;
    if (c < row_chunks) {
      int hi = hp0 - args.pad_h;
      unsigned char *dst = patch + j * 1024;
      for (int r = 0; r < n_rows; ++r) {
        const bool row_ok = (unsigned)hi < (unsigned)args.h_in;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_x, (__attribute__((address_space(3))) void *)dst, 16,
                                                 (int)(row_ok ? v_seg : OOB), row_ok ? hi * row_bytes : 0, 0, 0);
        hi += 1;
        dst += row_pitch;
      }
    }
  }
  // the first RING stages follow the patch, one per ring slot (helper waves only)
  if (!worker) {
#pragma unroll
    for (int s = 0; s < RING; ++s)
      if (s < stages) ring_issue(s);
  }

  // ---- epilogue form and this thread's entry of the operand table ----
  const int sig = args.fe.sig;
  constexpr int TPT = CK_TABLE_BYTES / 4 / NT;
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
  // pixel fragment p: block p of the tile, this wave's 32 channels (w) of a 128-channel chunk, part q of them
  int a_base[NPB];
#pragma unroll
  for (int p = 0; p < NPB; ++p) {
    const int pr = p * 16 + l15;
    const int prc = pr < npix ? pr : npix - 1;
    int ho, wo;
    fast_divmod(p0 + prc, args.w_m, args.w_s, args.w_out, ho, wo);
    a_base[p] = ((ho * args.stride_h - hp0) * PW + wo * args.stride_w) * pitch + w * 64 + q * 16;
  }
  // filter fragment i: rows i*16 + l15 of a stage, the wave's columns 4w + q under the row's swizzle
  int f_base[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) f_base[i] = (i * 16 + l15) * 256 + (((4 * w + q) ^ (l15 & 7)) << 4);
  int step_s = args.dil_w * pitch;
  int step_r = tap_h * pitch - (args.s_sz - 1) * step_s;
  int s_size = args.s_sz;
#pragma unroll
  for (int p = 0; p < NPB; ++p) asm volatile("" : "+v"(a_base[p]));
#pragma unroll
  for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(f_base[i]));
  asm volatile("" : "+s"(step_s), "+s"(step_r), "+s"(s_size));

  // stages 0 and 1 must have landed; the RING - 2 later ones may stay in flight
  {
    constexpr int fl = RIT * (RING - 2);
    static_assert(fl <= 63, "vmcnt is a 6-bit counter");
    if (!worker && stages >= RING) __builtin_amdgcn_s_waitcnt(0x0f70 | (fl & 15) | ((fl >> 4) << 14));
    else __builtin_amdgcn_s_waitcnt(0x0f70);
  }
  if (sig < 0) {
#pragma unroll
    for (int i = 0; i < TPT; ++i) table[tid + i * NT] = tabg[i];
  } else if (tid < 2 * BN) {
    table[tid] = tabr;
  }
  __syncthreads();

  const long long m_img = (long long)img * hw + p0;
  constexpr int SP = BN + 4;      // floats per pixel staged for the general operator loop
  float *stage = (float *)smem;   // (over the operands, once they are used up)
  float4 *red = (float4 *)smem;   // partial sums [unit = p*4 + i][wave][lane] (likewise)

  if (!worker) {
    // helper waves: stages s .. s + RING - 1 occupy the ring; before barrier s stage s + 2 has landed (the
    // RING - 3 after it may be in flight); behind it slot s % RING is free and receives stage s + RING.
    // (No barrier where neither matters any more: s >= stages - 2.)
    for (int s = 0; s + 2 < stages; ++s) {
      if (s + RING - 1 < stages) {
        constexpr int fl = RIT * (RING - 3);
        __builtin_amdgcn_s_waitcnt(0x0f70 | (fl & 15) | ((fl >> 4) << 14));
      } else {
        __builtin_amdgcn_s_waitcnt(0x0f70);
      }
      __builtin_amdgcn_s_barrier();
      if (s + RING < stages) ring_issue(s + RING);
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);
    // the multiplying waves' barriers around the exchange of partial sums (and around the staging)
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_s_barrier();
    if (sig >= 0) return;
    __builtin_amdgcn_s_barrier();
    __syncthreads();
  } else {
    f32x4 acc[NPB][4];
#pragma unroll
    for (int p = 0; p < NPB; ++p)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[p][i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int p = 0; p < NPB; ++p)
#pragma unroll
      for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(acc[p][i]));

    // ---- the residual of the pixel blocks this wave finishes (w, w + 4), asked for now: fetched in the epilogue
    // it is a round trip to memory with nothing left to hide it ----
    __amdgpu_buffer_rsrc_t rsrc_r = __builtin_amdgcn_make_buffer_rsrc(
        (void *)((const unsigned short *)args.fe.res + ((sig >= 0 && (sig & 4)) ? m_img * args.fe.res_ld + n0 : 0ll)), 0,
        (sig >= 0 && (sig & 4)) ? (int)((long long)npix * args.fe.res_ld * 2) : 0, 0x00020000);
    const int row_r = (int)args.fe.res_ld * 2;
    u32x4 resv[OWN][2] = {};
    if (sig >= 0 && (sig & 4)) {
      using E0 = Epilogue16<DT, 4>;
#pragma unroll
      for (int o = 0; o < OWN; ++o) {
        const int p = w + 4 * o;
        const int pr = p * 16 + l15;
#pragma unroll
        for (int j = 0; j < 2; ++j)
          resv[o][j] = E0::fetch_pair_residual(2 * j, 2 * j + 1, (p < NPB && pr < npix) ? pr : -1, q, rsrc_r, row_r);
      }
    }

    // ---- main loop: one stage (this wave's 32 channels of it) per step, operands read one step ahead ----
    u32x4 xa[2][NPB], xb[2][4];
    int ts = 0, chunk = 0, s_now = 0;
    const unsigned char *pp[NPB], *fp[4];
#pragma unroll
    for (int p = 0; p < NPB; ++p) pp[p] = patch + a_base[p];
#pragma unroll
    for (int i = 0; i < 4; ++i) fp[i] = ring + f_base[i];
    // (in the order the MFMAs want them: the first pixel block's fragment right behind the first filter block's)
    auto read = [&](auto setc) __attribute__((always_inline)) {
      constexpr int set = decltype(setc)::value;
      xb[set][0] = *(const u32x4 *)fp[0];
      xa[set][0] = *(const u32x4 *)pp[0];
#pragma unroll
      for (int i = 1; i < 4; ++i) xb[set][i] = *(const u32x4 *)fp[i];
#pragma unroll
      for (int p = 1; p < NPB; ++p) xa[set][p] = *(const u32x4 *)pp[p];
    };
    // on to the next stage: the next 128 channels of the tap, or the next tap; the ring slot after this one
    // (past the last stage the addresses stay: the last stage is read again, unused)
    auto advance = [&]() __attribute__((always_inline)) {
      const bool more = s_now + 1 < stages;
      chunk += 1;
      const bool wrap_c = chunk == CPT;
      chunk = wrap_c ? 0 : chunk;
      ts += wrap_c ? 1 : 0;
      const bool wrap_s = ts == s_size;
      ts = wrap_s ? 0 : ts;
      const int tap_step = wrap_c ? (wrap_s ? step_r : step_s) - (CPT - 1) * 256 : 256;
      const int p_step = more ? tap_step : 0;
      const int f_step = !more ? 0 : ((s_now + 1) % RING == 0 ? -(RING - 1) * CK_STAGE_BYTES : CK_STAGE_BYTES);
      fp[0] += f_step;
      pp[0] += p_step;
#pragma unroll
      for (int i = 1; i < 4; ++i) fp[i] += f_step;
#pragma unroll
      for (int p = 1; p < NPB; ++p) pp[p] += p_step;
    };
    auto mma = [&](auto setc) __attribute__((always_inline)) {
      constexpr int s = decltype(setc)::value;
#pragma unroll
      for (int p = 0; p < NPB; ++p)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[p][i] = Mfma16<DT>::run(xb[s][i], xa[s][p], acc[p][i]);
      // per MFMA its share of the address updates and, behind them, of the reads they feed
      Interleave<0, 4 * NPB, 0x002, NPB + 4, 0x100, NPB + 4>::run();
      __builtin_amdgcn_sched_barrier(0);
    };
    using std::integral_constant;
    read(integral_constant<int, 0>{});
    __builtin_amdgcn_sched_barrier(0);
    auto stage_step = [&](auto setc) __attribute__((always_inline)) {
      constexpr int set = decltype(setc)::value;
      advance();
      read(integral_constant<int, set ^ 1>{});
      mma(integral_constant<int, set>{});
      // barrier s: stages up to s + 2 are readable behind it (see the helper waves' loop)
      if (s_now + 2 < stages) __builtin_amdgcn_s_barrier();
      s_now += 1;
    };
    // (stages is even and at least 2: a tap is a whole number of pairs of stages)
    const int pairs = stages / 2;
    int t = 0;
#pragma unroll 1
    do {
      stage_step(integral_constant<int, 0>{});
      stage_step(integral_constant<int, 1>{});
    } while (++t < pairs);

    // ---- the four partial tiles meet: wave w finishes the pixel blocks p with p % 4 == w ----
    __syncthreads();  // every wave has left the main loop: patch and ring may be overwritten
    static_for<0, NPB>([&](auto pc) {
      constexpr int p = decltype(pc)::value;
      if ((p & 3) != w) {
#pragma unroll
        for (int i = 0; i < 4; ++i) *(f32x4 *)(red + ((p * 4 + i) * 4 + w) * 64 + lane) = acc[p][i];
      }
    });
    __syncthreads();
    f32x4 fin[OWN][4];  // the finished sums of the wave's pixel blocks w, w + 4
    static_for<0, OWN>([&](auto oc) {
      constexpr int o = decltype(oc)::value;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        // (the wave's own partial: picked by constants, the wave index deciding)
        f32x4 mine = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        static_for<0, 4>([&](auto wc) {
          constexpr int ww = decltype(wc)::value;
          if constexpr (ww + 4 * o < NPB) mine = w == ww ? acc[ww + 4 * o][i] : mine;
        });
        fin[o][i] = mine;
      }
      const int p = w + 4 * o;
      if (p < NPB) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          // in wave order 0, 1, 2, 3, the wave's own partial in its place
          f32x4 sum = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
          for (int v = 0; v < 4; ++v)
            sum += v == w ? fin[o][i] : *(const f32x4 *)(red + ((p * 4 + i) * 4 + v) * 64 + lane);
          fin[o][i] = sum;
        }
      }
    });

    if (sig >= 0) {
      // ---- epilogue from registers ----
      __amdgpu_buffer_rsrc_t rsrc_c = __builtin_amdgcn_make_buffer_rsrc(
          (void *)((unsigned short *)args.C + m_img * args.ldc + n0), 0, (int)((long long)npix * args.ldc * 2), 0x00020000);
      const int row_c = (int)args.ldc * 2;
      const int fb[4] = {0, 1, 2, 3};
      auto run_form = [&](auto form) __attribute__((always_inline)) {
        using E = Epilogue16<DT, decltype(form)::value>;
        f32x4 ta[4] = {}, tb[4] = {};
        if constexpr (E::AFF) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            ta[i] = *(const f32x4 *)(table + i * 16 + q * 4);
            tb[i] = *(const f32x4 *)(table + BN + i * 16 + q * 4);
          }
        }
        static_for<0, OWN>([&](auto oc) {
          constexpr int o = decltype(oc)::value;
          const int p = w + 4 * o;
          const int pr = p * 16 + l15;
          E::pixel_block_with(fin[o], fb, ta, tb, (p < NPB && pr < npix) ? pr : -1, q, rsrc_c, row_c, resv[o]);
        });
      };
#define TRACEA_CK_FORM(F) run_form(std::integral_constant<int, F>{})
      TRACEA_EPILOGUE16_FORMS(sig, TRACEA_CK_FORM)
#undef TRACEA_CK_FORM
      return;
    }

    // ---- any other chain: the finished sums through LDS ----
    __syncthreads();  // the partial sums have been read
    static_for<0, OWN>([&](auto oc) {
      constexpr int o = decltype(oc)::value;
      const int p = w + 4 * o;
      const int pr = p * 16 + l15;
      if (p < NPB && pr < npix) {
#pragma unroll
        for (int i = 0; i < 4; ++i) *(f32x4 *)(stage + pr * SP + i * 16 + q * 4) = fin[o][i];
      }
    });
    __syncthreads();
  }

  // ---- the general operator loop over whole pixels, all waves ----
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

// bm = 16 * NPB pixels at most per workgroup; CIN input channels exactly (a multiple of 256); a ring of RING
// stages of 64 filters x 128 channels.
template <int CIN, int NPB, int RING>
int launch_conv_ksplit16(const ContractionArgs &a, bool conv, int dtype, bool b_ncontig, hipStream_t stream) {
  if (!conv || b_ncontig || a.c_in != CIN || a.K != a.r_sz * a.s_sz * CIN || a.p_tm <= 0 || a.p_tm > 16 * NPB ||
      a.p_np_bytes <= 0)
    return (int)hipErrorInvalidValue;
  const size_t operands = (size_t)a.p_np_bytes + (size_t)RING * CK_STAGE_BYTES;
  size_t staging = (size_t)4 * NPB * 4 * 1024;
  if ((size_t)a.p_tm * 68 * 4 > staging) staging = (size_t)a.p_tm * 68 * 4;
  const size_t lds = (operands > staging ? operands : staging) + CK_TABLE_BYTES;
  if (lds > 160 * 1024) return (int)hipErrorInvalidValue;
  const dim3 grid((unsigned)(a.grid_m * a.grid_n)), block(CK_THREADS);
#define TRACEA_LAUNCH_CK(DTV)                                                                        \
  do {                                                                                               \
    auto kfn = conv_ksplit16_kernel<DTV, CIN, NPB, RING>;                                             \
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
  if (dtype == DT_F16) TRACEA_LAUNCH_CK(DT_F16);
  else TRACEA_LAUNCH_CK(DT_BF16);
#undef TRACEA_LAUNCH_CK
  return (int)hipErrorInvalidValue;
}

}  // namespace tracea_amd
