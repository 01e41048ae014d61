// Transposed convolution, second stage.
//
// The reference computes y[b,ho,wo,k] = sum over (c,r,s) of
// x[b,(ho+pad-r)/stride,(wo+pad-s)/stride,c] * w[c,r,s,k] where both divisions
// are exact (src/emitter/conv_transpose.rs:207-225), as one implicit GEMM whose
// K axis runs over every tap, so stride^2 - 1 of every stride^2 products are
// zeros.  Here the sum is split: a plain GEMM cols[(b,hi,wi),(r,s,k)] =
// x[(b,hi,wi),c] . w[c,(r,s,k)] does exactly the non-zero products on the matrix
// cores (NHWC activations are already the row-major left matrix; the filter bank
// is first copied into the K-contiguous order the fast GEMM kernels read, a few
// megabytes), and the gather kernel adds, for each output
// pixel, the ceil(R/stride_h) * ceil(S/stride_w) entries of cols that land on
// it, runs the operator chain and stores.  It reads cols once and writes the
// output once: bound by HBM.
#include "contraction_kernel.hpp"

namespace tracea_amd {

// One thread per output pixel and V consecutive channels (V = 4 when channels
// are the contiguous column index of cols, else 1).  Consecutive threads take
// consecutive channel groups, so a wave reads whole rows of cols.
template <int V>
__global__ void __launch_bounds__(256) col2im_epilogue_kernel(const Col2imArgs a) {
  const unsigned groups = (unsigned)(a.k_out + V - 1) / V;
  const unsigned idx = blockIdx.x * 256u + threadIdx.x;
  const unsigned total = (unsigned)a.nb * a.h_out * a.w_out * groups;  // < 2^31, checked by the host
  if (idx >= total) return;
  const unsigned g = idx % groups, p = idx / groups;
  const unsigned ow = p % (unsigned)a.w_out, q = p / (unsigned)a.w_out;
  const unsigned oh = q % (unsigned)a.h_out, bl = q / (unsigned)a.h_out;
  const int n = (int)g * V;
  const int nvalid = a.k_out - n;

  float acc[V];
#pragma unroll
  for (int e = 0; e < V; ++e) acc[e] = 0.0f;
  // taps r with (oh + pad_h - r) divisible by stride_h: r = r0, r0 + stride_h, ...
  // and the input row falls by one per step
  const int th = (int)oh + a.pad_h, tw = (int)ow + a.pad_w;
  const int r0 = th % a.stride_h, s0 = tw % a.stride_w;
  const int hi0 = th / a.stride_h, wi0 = tw / a.stride_w;
  const float *img = a.cols + (long long)bl * a.h_in * a.w_in * a.ld_cols + (long long)n * a.st_k;
  for (int r = r0, hi = hi0; r < a.r_sz && hi >= 0; r += a.stride_h, --hi) {
    if (hi >= a.h_in) continue;
    for (int s = s0, wi = wi0; s < a.s_sz && wi >= 0; s += a.stride_w, --wi) {
      if (wi >= a.w_in) continue;
      const float *src = img + ((long long)hi * a.w_in + wi) * a.ld_cols + r * a.st_r + s * a.st_s;
      if constexpr (V == 4) {
        const f32x4 t = *(const f32x4 *)src;
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] += t[e];
      } else {
        acc[0] += src[0];
      }
    }
  }
  const long long m = ((long long)(a.b0 + (int)bl) * a.h_out + oh) * a.w_out + ow;
  apply_epilogue<V>(acc, m, n, nvalid, a.epi);
  store_from_float<V>(a.out, a.out_dtype, m * a.ldc + n, nvalid, acc);
}

int launch_col2im_epilogue(const Col2imArgs &a, hipStream_t stream) {
  const bool vec = a.st_k == 1 && a.k_out % 4 == 0 && a.ld_cols % 4 == 0 && a.st_r % 4 == 0 && a.st_s % 4 == 0 &&
                   (((uintptr_t)a.cols) & 15) == 0;
  const long long groups = vec ? a.k_out / 4 : a.k_out;
  const long long total = (long long)a.nb * a.h_out * a.w_out * groups;
  if (total <= 0) return 0;
  if (total >= (1ll << 31)) return (int)hipErrorInvalidValue;
  const dim3 grid((unsigned)((total + 255) / 256)), block(256);
  if (vec) hipLaunchKernelGGL(col2im_epilogue_kernel<4>, grid, block, 0, stream, a);
  else hipLaunchKernelGGL(col2im_epilogue_kernel<1>, grid, block, 0, stream, a);
  return (int)hipGetLastError();
}

// Filter repack: a 64 (c) x 64 (k) tile per workgroup and tap, transposed through
// LDS so that the side with the smaller source stride is read along the lanes and
// the destination is written along its contiguous side.
template <typename T>
__global__ void __launch_bounds__(256) filter_repack_kernel(const FilterRepackArgs a) {
  __shared__ T tile[64][65];
  const int c0 = blockIdx.x * 64, k0 = blockIdx.y * 64;
  const int r = blockIdx.z / a.S, s = blockIdx.z % a.S;
  const int fast = threadIdx.x & 63, slow = threadIdx.x >> 6;
  const bool k_fast = a.sk <= a.sc;
  const T *src = (const T *)a.w + (long long)r * a.sr + (long long)s * a.ss;
  for (int i = 0; i < 16; ++i) {
    const int kk = k_fast ? fast : slow + i * 4, cc = k_fast ? slow + i * 4 : fast;
    const int k = k0 + kk, c = c0 + cc;
    if (k < a.K && c < a.C) tile[cc][kk] = src[(long long)k * a.sk + (long long)c * a.sc];
  }
  __syncthreads();
  if (a.c_inner) {
    T *dst = (T *)a.out + (long long)blockIdx.z * a.K * a.C;
    for (int i = 0; i < 16; ++i) {
      const int kk = slow + i * 4, k = k0 + kk, c = c0 + fast;
      if (k < a.K && c < a.C) dst[(long long)k * a.C + c] = tile[fast][kk];
    }
  } else {
    T *dst = (T *)a.out + (long long)blockIdx.z * a.K;
    const long long row = (long long)a.R * a.S * a.K;
    for (int i = 0; i < 16; ++i) {
      const int cc = slow + i * 4, c = c0 + cc, k = k0 + fast;
      if (k < a.K && c < a.C) dst[(long long)c * row + k] = tile[cc][fast];
    }
  }
}

int launch_filter_repack(const FilterRepackArgs &a, hipStream_t stream) {
  const dim3 grid((unsigned)((a.C + 63) / 64), (unsigned)((a.K + 63) / 64), (unsigned)(a.R * a.S)), block(256);
  if (grid.y > 65535 || grid.z > 65535) return (int)hipErrorInvalidValue;
  if (a.elem_bytes == 4) hipLaunchKernelGGL(filter_repack_kernel<unsigned>, grid, block, 0, stream, a);
  else hipLaunchKernelGGL(filter_repack_kernel<unsigned short>, grid, block, 0, stream, a);
  return (int)hipGetLastError();
}

// One workgroup per (64 input channels, 64 filters, tap): a 64x64 tile goes through LDS so that
// both the reads (whichever of c and k is the faster axis of w) and the writes (c fastest) are
// coalesced.
__global__ void __launch_bounds__(256) phase_filter_kernel(const PhaseFilterArgs a) {
  __shared__ unsigned short tile[64][65];
  const int c0 = blockIdx.x * 64, k0 = blockIdx.y * 64;
  const int z = blockIdx.z, r = z / a.S, s = z % a.S;
  const int fast = threadIdx.x & 63, slow = threadIdx.x >> 6;
  const bool k_fast = a.sk <= a.sc;
  const unsigned short *src = (const unsigned short *)a.w + (long long)r * a.sr + (long long)s * a.ss;
  // all sixteen loads in flight before the first LDS write (a rolled loop waits for each in turn)
  unsigned short v[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int kk = k_fast ? fast : slow + i * 4, cc = k_fast ? slow + i * 4 : fast;
    const int k = k0 + kk, c = c0 + cc;
    v[i] = (k < a.K && c < a.C) ? src[(long long)k * a.sk + (long long)c * a.sc] : (unsigned short)0;
  }
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int kk = k_fast ? fast : slow + i * 4, cc = k_fast ? slow + i * 4 : fast;
    tile[cc][kk] = v[i];
  }
  __syncthreads();
  // two channels per store (C is a multiple of 8 on this path, every destination 4-byte aligned)
  unsigned short *dst = (unsigned short *)a.out + a.tap_base[z];
  const long long kstride = a.tap_kstride[z];
  const int pair = threadIdx.x & 31, krow = threadIdx.x >> 5;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int kk = krow + i * 8, k = k0 + kk, c = c0 + pair * 2;
    if (k < a.K && c < a.C)
      *(unsigned *)(dst + k * kstride + c) = (unsigned)tile[pair * 2][kk] | ((unsigned)tile[pair * 2 + 1][kk] << 16);
  }
}

int launch_phase_filters(const PhaseFilterArgs &a, hipStream_t stream) {
  if (a.R * a.S > 64 || a.R * a.S <= 0) return (int)hipErrorInvalidValue;
  const dim3 grid((unsigned)((a.C + 63) / 64), (unsigned)((a.K + 63) / 64), (unsigned)(a.R * a.S));
  if (grid.y > 65535) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(phase_filter_kernel, grid, dim3(256), 0, stream, a);
  return (int)hipGetLastError();
}

}  // namespace tracea_amd
