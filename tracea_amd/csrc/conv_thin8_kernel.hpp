// Convolution of an image with 8 channels (a network's first layer: 3 real channels padded to one 16-byte
// group) on 16x16x32 MFMAs: the input patch in LDS, the whole filter bank of the workgroup's 64 filters in
// registers (gfx950).
//
// Same arithmetic as the reference's kernel_main (src/emitter/cuda/conv.rs:153-331):
// out[n,ho,wo,k] = epilogue(sum_{r,s,c} x[n, ho*sh-ph+r*dh, wo*sw-pw+s, c] * w[k,r,s,c]), fp32 accumulation,
// zero padding; filter dilation along W must be 1.
//
// Why its own kernel.  As an implicit GEMM this layer has K = R*S*8 (392 for 7x7) gathered from 16-byte
// pixels, and a 64-filter tile re-reads every pixel R*S times from L2; the streamed kernels spend 19 us on
// the 7x7 stride-4 layer of a 224x224 batch of 32 whose memory traffic is worth 5.  Here a filter row (one r,
// S <= 8 taps of 8 channels) is two k-steps of 32: for output pixel (ho, wo) the operand of k-step (r, h) is
// the 64 contiguous bytes of pixels wo*sw + 4h .. + 3 of input row ho*sh + r*dh, straight from the resident
// patch (taps s >= S meet zero filter values).  The 2 R filter fragments of a wave's two filter blocks stay in
// registers for the whole tile (16 R registers), so LDS serves only the patch: 4 fragments per 8 MFMAs.
//
// Work split: a workgroup owns 64 filters and walks over tiles of p_tm <= 128 consecutive output pixels (whole
// output rows where they fit) of the images, tile after tile with a stride of the workgroups that share its
// filters: the filter bank is fetched once per workgroup, and the patch of the next tile travels while the
// current one is multiplied (two patch buffers, one barrier per tile).  Wave (fh, ph) of eight multiplies
// pixel blocks 2 ph, 2 ph + 1 by filter blocks 2 fh, 2 fh + 1: two multiplying waves per SIMD.
//
// Patch layout: whole padded input rows, RP 16-byte pixels per row (a multiple of 8), pixel x at position
// x ^ ((x >> 3) & 3) of its row: the 8 lanes that read together are 4 or 2 pixels apart (stride 4 or 2) and
// land in 8 different 16-byte bank groups.
//
// LDS: patch buffer 0 | patch buffer 1 | staging | operand table.  The filter fragments pass through LDS once
// on their way to the registers (over buffer 1 and the staging area, before either is used): fetched as one
// copy per workgroup instead of one per wave.
//
// Epilogue: from registers (conv_epilogue16.hpp), or through the staging area and the general operator loop.
#pragma once
#include "conv_epilogue16.hpp"

namespace tracea_amd {

constexpr int CT_THREADS = 512;
constexpr int CT_TABLE_BYTES = TRACEA_MAX_EPILOGUE_OPS * 2 * 64 * 4;
// bytes between the two patch buffers and the operand table: the general epilogue's staging (68 floats per
// pixel), and room for the filter fragments (2 R x 4 KB) to lie over buffer 1 and this area
__host__ __device__ constexpr int ct_aux_bytes(int r, int p_tm, int patch_bytes) {
  const int staging = p_tm * 68 * 4, spill = r * 8 * 1024 - patch_bytes;
  return staging > spill ? staging : spill;
}

template <int DT, int R>
__global__ void __launch_bounds__(CT_THREADS) conv_thin8_kernel(const ContractionArgs args) {
  constexpr int NT = CT_THREADS, BN = 64, NW = NT / 64, C = 8, PBW = 2, STEPS = 2 * R;
  asm volatile("" ::"s"(args.A), "s"(args.B), "s"(args.N), "s"(args.ldb), "s"(args.b_bytes), "s"(args.grid_n), "s"(args.h_in),
               "s"(args.w_in), "s"(args.h_out), "s"(args.w_out), "s"(args.s_sz), "s"(args.stride_h), "s"(args.stride_w));
  asm volatile("" ::"s"(args.pad_h), "s"(args.pad_w), "s"(args.dil_h), "s"(args.w_m), "s"(args.w_s), "s"(args.p_tiles),
               "s"(args.p_pw), "s"(args.p_np_bytes), "s"(args.p_tm), "s"(args.p_seg), "s"(args.gn_m), "s"(args.gn_s),
               "s"(args.pt_m), "s"(args.pt_s), "s"(args.grid_m));
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int PB = args.p_np_bytes;
  unsigned char *frag = smem + PB;
  float *stage = (float *)(smem + 2 * PB);
  float *table = (float *)(smem + 2 * PB + ct_aux_bytes(R, args.p_tm, PB));

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave_u = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int fh = wave_u & 1, ph = wave_u >> 1;
  const int l15 = lane & 15, q = lane >> 4;

  // ---- which filters, which tiles: workgroup (slot, tile_n) walks tiles slot, slot + nslots, ... ----
  int bid = blockIdx.x;
  const int total = gridDim.x;
  if ((total & 7) == 0) bid = (bid & 7) * (total >> 3) + (bid >> 3);  // contiguous run per XCD
  int tile_n, slot;
  fast_divmod(bid, args.gn_m, args.gn_s, args.grid_n, slot, tile_n);
  const int nslots = total / args.grid_n;
  const int TM = args.p_tm;
  const int hw = args.h_out * args.w_out;
  const int n0 = tile_n * BN;
  const int N = args.N;
  const int RP = args.p_pw;  // 16-byte pixels per patch row

  constexpr unsigned OOB = 0x80000000u;  // beyond every buffer: the load returns zeros
  const long long img_elems = (long long)args.h_in * args.w_in * C;
  __amdgpu_buffer_rsrc_t rsrc_w =
      __builtin_amdgcn_make_buffer_rsrc((void *)args.B, 0, (int)args.b_bytes, 0x00020000);

  // ---- patch of tile mt into buffer buf: load instruction j of a row fills positions 64 j .. 64 j + 63 of
  // it; lane l brings the pixel that lives at position 64 j + l (the swizzle is its own inverse); padding
  // pixels and rows are zeros.  The (row, j) pairs go round the waves. ----
  const int SEG = args.p_seg;  // load instructions per row: ceil(RP / 64)
  const int row_bytes = args.w_in * C * 2, row_pitch = RP * 16;
  auto issue_patch = [&](int mt, int buf) __attribute__((always_inline)) {
    int img, tim;
    fast_divmod(mt, args.pt_m, args.pt_s, args.p_tiles, img, tim);
    const int p0 = tim * TM;
    const int npix = min(TM, hw - p0);
    int ho_f, wo_f, ho_l, wo_l;
    fast_divmod(p0, args.w_m, args.w_s, args.w_out, ho_f, wo_f);
    fast_divmod(p0 + npix - 1, args.w_m, args.w_s, args.w_out, ho_l, wo_l);
    const int hp0 = ho_f * args.stride_h;
    const int n_rows = ho_l * args.stride_h + (R - 1) * args.dil_h - hp0 + 1;
    __amdgpu_buffer_rsrc_t rsrc_x = __builtin_amdgcn_make_buffer_rsrc(
        (void *)((const unsigned short *)args.A + (long long)img * img_elems), 0, (int)(img_elems * 2), 0x00020000);
    unsigned char *base = smem + buf * PB;
    int j = wave_u, r = 0;
    while (j >= SEG) {
      j -= SEG;
      r += 1;
    }
    while (r < n_rows) {
      const int pos = j * 64 + lane;
      const int xi = (pos ^ ((pos >> 3) & 3)) - args.pad_w;
      const int hi = hp0 - args.pad_h + r;
      const bool row_ok = (unsigned)hi < (unsigned)args.h_in;  // (the same for every lane)
      const bool ok = ((unsigned)xi < (unsigned)args.w_in) & row_ok;
      if (pos < RP)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_x, (__attribute__((address_space(3))) void *)(base + r * row_pitch + j * 1024),
                                                 16, (int)(ok ? (unsigned)(xi * C * 2) : OOB), row_ok ? hi * row_bytes : 0, 0, 0);
      j += NW;
      while (j >= SEG) {
        j -= SEG;
        r += 1;
      }
    }
  };

  int mt = slot;
  issue_patch(mt, 0);

  // ---- filters: fragment (r, h, fb) = filter block fb, taps 4h .. 4h + 3 of filter row r; lane (l15, q):
  // filter 16 fb + l15, tap 4h + q, its 8 channels; taps past S and filters past N: zeros.  One load
  // instruction per fragment, through LDS ----
  for (int fi = wave_u; fi < STEPS * 4; fi += NW) {
    const int fb = fi & 3, h = (fi >> 2) & 1, r = fi >> 3;
    const int n = n0 + fb * 16 + l15, s = 4 * h + q;
    const unsigned voff = (n < N) & (s < args.s_sz) ? (unsigned)((n * (int)args.ldb + s * C) * 2) : OOB;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w, (__attribute__((address_space(3))) void *)(frag + fi * 1024), 16, (int)voff,
                                             r * args.s_sz * C * 2, 0, 0);
  }

  // ---- epilogue form and this thread's entry of the operand table ----
  const int sig = args.fe.sig;
  float tabr = 0.0f, tabg[2];
  const bool tab_general = sig < 0 && tid * 2 < CT_TABLE_BYTES / 4;
  if (tab_general) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int e = tid * 2 + i;
      tabg[i] = chain_table_value(args.epi, e / (2 * BN), (e / BN) & 1, n0 + e % BN, N);
    }
  } else if (sig >= 0 && (sig & 1) && tid < 2 * BN) {
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
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): first patch, filters, table values
  if (tab_general) {
    table[tid * 2] = tabg[0];
    table[tid * 2 + 1] = tabg[1];
  } else if (sig >= 0 && tid < 2 * BN) {
    table[tid] = tabr;
  }
  __syncthreads();
  u32x4 bw[R][2][2];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int f = 0; f < 2; ++f) bw[r][h][f] = *(const u32x4 *)(frag + (((r * 2 + h) * 4) + 2 * fh + f) * 1024 + lane * 16);
  f32x4 ta[2] = {}, tb[2] = {};
  if (sig >= 0 && (sig & 1)) {
#pragma unroll
    for (int f = 0; f < 2; ++f) {
      ta[f] = *(const f32x4 *)(table + (2 * fh + f) * 16 + q * 4);
      tb[f] = *(const f32x4 *)(table + BN + (2 * fh + f) * 16 + q * 4);
    }
  }
  __syncthreads();  // the fragments are in registers: buffer 1 and the staging area are free

  const int r_step = args.dil_h * RP * 16;
  const ChainPlan plan = chain_plan(args.epi);
  int buf = 0;
  while (true) {
    const int next = mt + nslots;
    const bool has_next = next < args.grid_m;
    if (has_next) issue_patch(next, buf ^ 1);

    int img, tim;
    fast_divmod(mt, args.pt_m, args.pt_s, args.p_tiles, img, tim);
    const int p0 = tim * TM;
    const int npix = min(TM, hw - p0);
    int ho_f, wo_f;
    fast_divmod(p0, args.w_m, args.w_s, args.w_out, ho_f, wo_f);
    const int hp0 = ho_f * args.stride_h;
    const unsigned char *patch = smem + buf * PB;

    // per-lane patch addresses: pixel block b of the wave (block 2 ph + b of the tile), half h of a filter row
    const unsigned char *pa[PBW][2];
#pragma unroll
    for (int b = 0; b < PBW; ++b) {
      const int pr = (ph * PBW + b) * 16 + l15;
      const int prc = pr < npix ? pr : npix - 1;
      int ho, wo;
      fast_divmod(p0 + prc, args.w_m, args.w_s, args.w_out, ho, wo);
      const int row = (ho * args.stride_h - hp0) * RP;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int x = wo * args.stride_w + 4 * h + q;
        pa[b][h] = patch + (row + (x ^ ((x >> 3) & 3))) * 16;
      }
    }

    // main loop: 2 R k-steps, patch fragments read one step ahead
    f32x4 acc[PBW][2];
#pragma unroll
    for (int b = 0; b < PBW; ++b)
#pragma unroll
      for (int f = 0; f < 2; ++f) acc[b][f] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    if (ph * PBW * 16 < npix) {  // (a wave whose pixel blocks lie past the tile's end has nothing to multiply)
      // patch fragments read two steps ahead (a step is four MFMAs, shorter than an LDS round trip); the
      // scheduling fences keep the reads of step t + 2 in front of the MFMAs of step t
      u32x4 xa[3][PBW];
      auto read = [&](auto tc) __attribute__((always_inline)) {
        constexpr int t = decltype(tc)::value, r = t >> 1, h = t & 1;
#pragma unroll
        for (int b = 0; b < PBW; ++b) xa[t % 3][b] = *(const u32x4 *)(pa[b][h] + r * r_step);
      };
      read(std::integral_constant<int, 0>{});
      read(std::integral_constant<int, 1>{});
      __builtin_amdgcn_sched_barrier(0);
      static_for<0, STEPS>([&](auto tc) {
        constexpr int t = decltype(tc)::value, r = t >> 1, h = t & 1;
        if constexpr (t + 2 < STEPS) read(std::integral_constant<int, t + 2>{});
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int b = 0; b < PBW; ++b)
#pragma unroll
          for (int f = 0; f < 2; ++f) acc[b][f] = Mfma16<DT>::run(bw[r][h][f], xa[t % 3][b], acc[b][f]);
        __builtin_amdgcn_sched_barrier(0);
      });
    }

    const long long m_img = (long long)img * hw + p0;
    if (sig >= 0) {
      // epilogue from registers
      __amdgpu_buffer_rsrc_t rsrc_c = __builtin_amdgcn_make_buffer_rsrc(
          (void *)((unsigned short *)args.C + m_img * args.ldc + n0), 0, (int)((long long)npix * args.ldc * 2), 0x00020000);
      __amdgpu_buffer_rsrc_t rsrc_r = __builtin_amdgcn_make_buffer_rsrc(
          (void *)((const unsigned short *)args.fe.res + ((sig & 4) ? m_img * args.fe.res_ld + n0 : 0ll)), 0,
          (sig & 4) ? (int)((long long)npix * args.fe.res_ld * 2) : 0, 0x00020000);
      const int row_c = (int)args.ldc * 2, row_r = (int)args.fe.res_ld * 2;
      auto run_form = [&](auto form) __attribute__((always_inline)) {
        using E = Epilogue16<DT, decltype(form)::value>;
#pragma unroll
        for (int b = 0; b < PBW; ++b) {
          const int pr = (ph * PBW + b) * 16 + l15;
          E::pair_block(acc[b][0], acc[b][1], 2 * fh, 2 * fh + 1, ta[0], tb[0], ta[1], tb[1], pr < npix ? pr : -1, q, rsrc_c,
                        rsrc_r, row_c, row_r);
        }
      };
#define TRACEA_CT_FORM(F) run_form(std::integral_constant<int, F>{})
      TRACEA_EPILOGUE16_FORMS(sig, TRACEA_CT_FORM)
#undef TRACEA_CT_FORM
    } else {
      // any other chain: accumulators through the staging area, then the general operator loop over whole pixels
      constexpr int SP = BN + 4;  // floats per staged pixel
#pragma unroll
      for (int b = 0; b < PBW; ++b) {
        const int pr = (ph * PBW + b) * 16 + l15;
        if (pr < npix) {
#pragma unroll
          for (int f = 0; f < 2; ++f) *(f32x4 *)(stage + pr * SP + (2 * fh + f) * 16 + q * 4) = acc[b][f];
        }
      }
      __syncthreads();
      const int ec = (tid & 7) * 8;
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
    if (!has_next) break;
    // the next patch has landed, and every wave is done with this one (and with the staging area)
    __builtin_amdgcn_s_waitcnt(0x0f70);
    __syncthreads();
    mt = next;
    buf ^= 1;
  }
}

// Tiles of at most 128 pixels; 8 input channels exactly, R filter rows exactly, up to 8 taps per row, no
// dilation along W; p_iters workgroups per filter slab walk the grid_m tiles.
template <int R>
int launch_conv_thin8(const ContractionArgs &a, bool conv, int dtype, bool b_ncontig, hipStream_t stream) {
  if (!conv || b_ncontig || a.c_in != 8 || a.r_sz != R || a.s_sz > 8 || a.dil_w != 1 || a.K != R * a.s_sz * 8 || a.p_tm <= 0 ||
      a.p_tm > 128 || a.p_np_bytes <= 0 || a.p_np_bytes % 1024 != 0 || a.p_pw % 8 != 0 || a.p_iters < 1 || a.p_iters > a.grid_m)
    return (int)hipErrorInvalidValue;
  const size_t lds = (size_t)2 * a.p_np_bytes + ct_aux_bytes(R, a.p_tm, a.p_np_bytes) + CT_TABLE_BYTES;
  if (lds > 160 * 1024) return (int)hipErrorInvalidValue;
  const dim3 grid((unsigned)(a.p_iters * a.grid_n)), block(CT_THREADS);
#define TRACEA_LAUNCH_CT(DTV)                                                                        \
  do {                                                                                               \
    auto kfn = conv_thin8_kernel<DTV, R>;                                                            \
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
  if (dtype == DT_F16) TRACEA_LAUNCH_CT(DT_F16);
  else TRACEA_LAUNCH_CT(DT_BF16);
#undef TRACEA_LAUNCH_CT
  return (int)hipErrorInvalidValue;
}

}  // namespace tracea_amd
