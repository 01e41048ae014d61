// Kernels for graph nodes that are not contractions: operator chains over an
// existing tensor, global average pooling, row softmax.  All are bound by HBM;
// they exist so that a whole network graph runs without leaving the library
// (the reference's counterparts: src/emitter/cuda/nn.rs:3-103, elementwise.rs).
#include "contraction_kernel.hpp"
#include "conv_epilogue16.hpp"

namespace tracea_amd {

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

// v as the element type `dtype` holds it (round to nearest even), back in fp32
__device__ __forceinline__ float round_through(float v, int dtype) {
  if (dtype == DT_F16) return (float)(_Float16)v;
  if (dtype == DT_BF16) return (float)(__bf16)v;
  return v;
}

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

// Global average pooling and the linear layer that reads it, in one launch (a network's classifier head:
// each of the two alone is a few microseconds of launch for a few hundred kilobytes).
// Workgroup (slab, image): the channel means of the image (fp32 sums, rounded through `dtype` as the
// pooling node stores them; slab 0 also stores them, so the pooling node's output exists), then the
// slab's outputs out[image, j] = chain(sum_k mean[k] * w[k, j]), fp32 accumulation.
// KCONTIG: w[k, j] at j * w_ld + k (a wave per output, lanes over k); else at k * w_ld + j (a thread per
// output, consecutive threads consecutive j).
template <bool KCONTIG>
__global__ void __launch_bounds__(256) pool_linear_kernel(const PoolLinearArgs a) {
  extern __shared__ float pl_smem[];  // [channels] means, then [4][channels] partial sums (at least 2048 floats)
  float *mean = pl_smem, *part = pl_smem + a.channels;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int img = blockIdx.y;
  const long long base = (long long)img * a.hw * a.channels;
  const int groups = (a.channels + 7) / 8;
  for (int g = lane; g < groups; g += 64) {
    float sum[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    const int nvalid = a.channels - g * 8;
#pragma unroll 4
    for (int p = wave; p < a.hw; p += 4) {
      float t[8];
      load_as_float<8>(a.x, a.dtype, base + (long long)p * a.channels + g * 8, nvalid, t);
#pragma unroll
      for (int e = 0; e < 8; ++e) sum[e] += t[e];
    }
#pragma unroll
    for (int e = 0; e < 8; ++e)
      if (e < nvalid) part[wave * a.channels + g * 8 + e] = sum[e];
  }
  __syncthreads();
  for (int c = tid; c < a.channels; c += 256) {
    float v[1] = {(part[c] + part[a.channels + c] + part[2 * a.channels + c] + part[3 * a.channels + c]) / (float)a.hw};
    v[0] = round_through(v[0], a.dtype);
    mean[c] = v[0];
    if (blockIdx.x == 0 && a.pooled != nullptr) store_from_float<1>(a.pooled, a.dtype, (long long)img * a.channels + c, 1, v);
  }
  __syncthreads();
  const int per = (a.n_out + (int)gridDim.x - 1) / (int)gridDim.x;
  const int j0 = blockIdx.x * per, j1 = min(a.n_out, j0 + per);
  if constexpr (KCONTIG) {
    // four outputs per wave and trip: their rows are requested together
    for (int jb = j0 + wave * 4; jb < j1; jb += 16) {
      float acc[4] = {0, 0, 0, 0};
      for (int g = lane; g < groups; g += 64) {
        float t[4][8];
#pragma unroll
        for (int u = 0; u < 4; ++u)
          load_as_float<8>(a.w, a.dtype, (long long)min(jb + u, j1 - 1) * a.w_ld + g * 8, a.channels - g * 8, t[u]);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float mk = g * 8 + e < a.channels ? mean[g * 8 + e] : 0.0f;
#pragma unroll
          for (int u = 0; u < 4; ++u) acc[u] += mk * t[u][e];
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) acc[u] = wave_sum(acc[u]);
      if (lane < 4 && jb + lane < j1) {
        float v[1] = {lane == 0 ? acc[0] : lane == 1 ? acc[1] : lane == 2 ? acc[2] : acc[3]};
        apply_epilogue<1>(v, img, jb + lane, 1, a.epi);
        store_from_float<1>(a.out, a.out_dtype, (long long)img * a.n_out + jb + lane, 1, v);
      }
    }
  } else {
    // thread (kg, jl): rows kg, kg + 16, ... of w, outputs 8 jl .. 8 jl + 7 of a run of 128; the 16 partial
    // sums of an output meet in LDS (over the pixel sums, which are used up)
    const int kg = tid >> 4, jl = tid & 15;
    for (int jb = j0; jb < j1; jb += 128) {
      const int j = jb + jl * 8;
      const int nvalid = j1 - j;  // (<= 0: nothing to do for this thread)
      float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
      if (nvalid > 0) {
#pragma unroll 8
        for (int k = kg; k < a.channels; k += 16) {
          float t[8];
          load_as_float<8>(a.w, a.dtype, (long long)k * a.w_ld + j, nvalid, t);
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[e] += mean[k] * t[e];
        }
      }
      __syncthreads();  // (the partial sums of the previous run have been read)
#pragma unroll
      for (int e = 0; e < 8; ++e) part[kg * 128 + jl * 8 + e] = acc[e];
      __syncthreads();
      if (tid < 128 && jb + tid < j1) {
        float v[1] = {0.0f};
#pragma unroll
        for (int q = 0; q < 16; ++q) v[0] += part[q * 128 + tid];
        apply_epilogue<1>(v, img, jb + tid, 1, a.epi);
        store_from_float<1>(a.out, a.out_dtype, (long long)img * a.n_out + jb + tid, 1, v);
      }
    }
  }
}

// The same for the common case, with every load requested before the first is used (the kernel is a chain
// of memory round trips otherwise): w stored [K, N], half or bfloat16 operands, channels a multiple of 8 and
// at most 512, n_out a multiple of 8, at most 64 pixels per image, slabs of at most 128 outputs, 16-byte
// aligned rows.  Same sums in the same order as the kernel above.
template <int DT>
__global__ void __launch_bounds__(256) pool_linear_kn_kernel(const PoolLinearArgs a) {
  extern __shared__ float pl_smem[];
  float *mean = pl_smem, *part = pl_smem + a.channels;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int img = blockIdx.y;
  const int per = ((a.n_out + (int)gridDim.x - 1) / (int)gridDim.x + 7) & ~7;
  const int j0 = blockIdx.x * per, j1 = min(a.n_out, j0 + per);
  constexpr unsigned OOB = 0x80000000u;
  __amdgpu_buffer_rsrc_t rsrc_w = __builtin_amdgcn_make_buffer_rsrc((void *)a.w, 0, (int)((long long)a.channels * a.w_ld * 2), 0x00020000);
  __amdgpu_buffer_rsrc_t rsrc_x = __builtin_amdgcn_make_buffer_rsrc(
      (void *)((const unsigned short *)a.x + (long long)img * a.hw * a.channels), 0, a.hw * a.channels * 2, 0x00020000);
  // rows kg, kg + 16, ... of w, outputs j .. j + 7
  const int kg = tid >> 4, jl = tid & 15;
  const int j = j0 + jl * 8;
  u32x4 wr[32];
#pragma unroll
  for (int i = 0; i < 32; ++i) {
    const int k = kg + 16 * i;
    wr[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(
                                          rsrc_w, (k < a.channels) & (j < j1) ? (int)((k * a.w_ld + j) * 2) : (int)OOB, 0, 0));
  }
  // pixels wave, wave + 4, ... of the image, channels 8 lane .. 8 lane + 7
  u32x4 xr[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int p = wave + 4 * i;
    xr[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(
                                          rsrc_x, (p < a.hw) & (lane * 8 < a.channels) ? (p * a.channels + lane * 8) * 2 : (int)OOB, 0, 0));
  }
  using U = Epilogue16<DT, 0>;
  {
    float sum[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      if (wave + 4 * i < a.hw) {  // (the same for the whole wave)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float lo, hi;
          U::unpack2(xr[i][e], lo, hi);
          sum[2 * e] += lo;
          sum[2 * e + 1] += hi;
        }
      }
    }
    if (lane * 8 < a.channels) {
#pragma unroll
      for (int e = 0; e < 8; ++e) part[wave * a.channels + lane * 8 + e] = sum[e];
    }
  }
  __syncthreads();
  for (int c = tid; c < a.channels; c += 256) {
    float v[1] = {(part[c] + part[a.channels + c] + part[2 * a.channels + c] + part[3 * a.channels + c]) / (float)a.hw};
    v[0] = round_through(v[0], a.dtype);
    mean[c] = v[0];
    if (blockIdx.x == 0 && a.pooled != nullptr) store_from_float<1>(a.pooled, a.dtype, (long long)img * a.channels + c, 1, v);
  }
  __syncthreads();
  float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
  for (int i = 0; i < 32; ++i) {
    const int k = kg + 16 * i;
    const float mk = k < a.channels ? mean[k] : 0.0f;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float lo, hi;
      U::unpack2(wr[i][e], lo, hi);
      acc[2 * e] += mk * lo;
      acc[2 * e + 1] += mk * hi;
    }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) part[kg * 128 + jl * 8 + e] = acc[e];
  __syncthreads();
  if (tid < 128 && j0 + tid < j1) {
    float v[1] = {0.0f};
#pragma unroll
    for (int q = 0; q < 16; ++q) v[0] += part[q * 128 + tid];
    apply_epilogue<1>(v, img, j0 + tid, 1, a.epi);
    store_from_float<1>(a.out, a.out_dtype, (long long)img * a.n_out + j0 + tid, 1, v);
  }
}

int launch_pool_linear(const PoolLinearArgs &a, bool k_contiguous, hipStream_t stream) {
  if (a.batch <= 0 || a.channels <= 0 || a.hw <= 0 || a.n_out <= 0) return 0;
  if (a.batch > 65535 || a.channels > 8192) return (int)hipErrorInvalidValue;
  // about one workgroup per CU and more, slabs of at least 32 outputs
  int slabs = (256 + a.batch - 1) / a.batch;
  if (slabs > (a.n_out + 31) / 32) slabs = (a.n_out + 31) / 32;
  if (slabs < 1) slabs = 1;
  // means, then the four partial pixel sums or (later, over them) 16 x 128 partial outputs
  const size_t lds = ((size_t)a.channels + (4 * (size_t)a.channels > 2048 ? 4 * (size_t)a.channels : 2048)) * sizeof(float);
  const bool half_type = a.dtype == DT_F16 || a.dtype == DT_BF16;
  if (!k_contiguous && half_type && a.channels % 8 == 0 && a.channels <= 512 && a.n_out % 8 == 0 && a.hw <= 64 && a.w_ld % 8 == 0 &&
      (((uintptr_t)a.x | (uintptr_t)a.w) & 15) == 0 && (long long)a.channels * a.w_ld * 2 < (1ll << 31)) {
    if (slabs < (a.n_out + 127) / 128) slabs = (a.n_out + 127) / 128;  // slabs of at most 128 outputs
    if (a.dtype == DT_F16)
      hipLaunchKernelGGL(pool_linear_kn_kernel<DT_F16>, dim3((unsigned)slabs, (unsigned)a.batch), dim3(256), lds, stream, a);
    else
      hipLaunchKernelGGL(pool_linear_kn_kernel<DT_BF16>, dim3((unsigned)slabs, (unsigned)a.batch), dim3(256), lds, stream, a);
    return (int)hipGetLastError();
  }
  if (k_contiguous)
    hipLaunchKernelGGL(pool_linear_kernel<true>, dim3((unsigned)slabs, (unsigned)a.batch), dim3(256), lds, stream, a);
  else
    hipLaunchKernelGGL(pool_linear_kernel<false>, dim3((unsigned)slabs, (unsigned)a.batch), dim3(256), lds, stream, a);
  return (int)hipGetLastError();
}

// One wave per row: maximum, sum of exponentials and the normalised values, with
// the row kept in registers when it has at most 64*16 entries and re-read otherwise.

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
