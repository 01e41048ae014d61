// Kernels for graph nodes that are not contractions: operator chains over an
// existing tensor, global average pooling, row softmax.  All are bound by HBM;
// they exist so that a whole network graph runs without leaving the library
// (the reference's counterparts: src/emitter/cuda/nn.rs:3-103, elementwise.rs).
#include "contraction_kernel.hpp"

namespace tracea_amd {

// One thread per row and 8 consecutive channels (1 when channels % 8 != 0).
template <int V>
__global__ void __launch_bounds__(256) chain_apply_kernel(const ChainApplyArgs a) {
  const long long groups = (a.channels + V - 1) / V;
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= a.rows * groups) return;
  const long long m = idx / groups;
  const int n = (int)(idx % groups) * V;
  const int nvalid = a.channels - n;
  float v[V];
  load_as_float<V>(a.x, a.x_dtype, m * a.channels + n, nvalid, v);
  apply_epilogue<V>(v, m, n, nvalid, a.epi);
  store_from_float<V>(a.out, a.out_dtype, m * a.channels + n, nvalid, v);
}

int launch_chain_apply(const ChainApplyArgs &a, hipStream_t stream) {
  if (a.rows <= 0 || a.channels <= 0) return 0;
  const bool vec = a.channels % 8 == 0 && (((uintptr_t)a.x) & 15) == 0 && (((uintptr_t)a.out) & 15) == 0;
  const long long groups = vec ? a.channels / 8 : a.channels;
  const long long blocks = (a.rows * groups + 255) / 256;
  if (blocks >= (1ll << 31)) return (int)hipErrorInvalidValue;
  if (vec) hipLaunchKernelGGL(chain_apply_kernel<8>, dim3((unsigned)blocks), dim3(256), 0, stream, a);
  else hipLaunchKernelGGL(chain_apply_kernel<1>, dim3((unsigned)blocks), dim3(256), 0, stream, a);
  return (int)hipGetLastError();
}

// One workgroup per image and 64 channels: 4 waves split the pixels, consecutive
// lanes read consecutive channels, partial sums meet in LDS.
__global__ void __launch_bounds__(256) global_avg_pool_kernel(const void *x, void *out, int dtype, int out_dtype,
                                                              int hw, int channels) {
  __shared__ float part[4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = blockIdx.x * 64 + lane;
  const long long base = (long long)blockIdx.y * hw * channels;
  float sum = 0.0f;
  if (c < channels) {
    for (int p = wave; p < hw; p += 4) {
      float t[1];
      load_as_float<1>(x, dtype, base + (long long)p * channels + c, 1, t);
      sum += t[0];
    }
  }
  part[wave][lane] = sum;
  __syncthreads();
  if (wave == 0 && c < channels) {
    float v[1] = {(part[0][lane] + part[1][lane] + part[2][lane] + part[3][lane]) / (float)hw};
    store_from_float<1>(out, out_dtype, (long long)blockIdx.y * channels + c, 1, v);
  }
}

int launch_global_avg_pool(const void *x, void *out, int dtype, int out_dtype, int batch, int hw, int channels,
                           hipStream_t stream) {
  if (batch <= 0 || channels <= 0 || hw <= 0) return 0;
  if (batch > 65535) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(global_avg_pool_kernel, dim3((unsigned)((channels + 63) / 64), (unsigned)batch), dim3(256), 0,
                     stream, x, out, dtype, out_dtype, hw, channels);
  return (int)hipGetLastError();
}

// One wave per row: maximum, sum of exponentials and the normalised values, with
// the row kept in registers when it has at most 64*16 entries and re-read otherwise.
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}

__global__ void __launch_bounds__(256) softmax_rows_kernel(const void *x, void *out, int dtype, int out_dtype,
                                                           long long rows, int cols) {
  const int lane = threadIdx.x & 63;
  const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const long long base = row * cols;
  float mx = -INFINITY;
  for (int c = lane; c < cols; c += 64) {
    float t[1];
    load_as_float<1>(x, dtype, base + c, 1, t);
    mx = fmaxf(mx, t[0]);
  }
  mx = wave_max(mx);
  float sum = 0.0f;
  for (int c = lane; c < cols; c += 64) {
    float t[1];
    load_as_float<1>(x, dtype, base + c, 1, t);
    sum += __expf(t[0] - mx);
  }
  sum = wave_sum(sum);
  const float inv = 1.0f / sum;
  for (int c = lane; c < cols; c += 64) {
    float t[1];
    load_as_float<1>(x, dtype, base + c, 1, t);
    t[0] = __expf(t[0] - mx) * inv;
    store_from_float<1>(out, out_dtype, base + c, 1, t);
  }
}

int launch_softmax_rows(const void *x, void *out, int dtype, int out_dtype, long long rows, int cols,
                        hipStream_t stream) {
  if (rows <= 0 || cols <= 0) return 0;
  const long long blocks = (rows + 3) / 4;
  if (blocks >= (1ll << 31)) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(softmax_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, x, out, dtype, out_dtype,
                     rows, cols);
  return (int)hipGetLastError();
}

}  // namespace tracea_amd
