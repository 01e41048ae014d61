// Calibration probe for the matrix-pipe roofline: sustained MFMA throughput of the whole
// device from registers only (no LDS, no global traffic inside the loop), for all-zero and
// for normally distributed fp16 operands, and for the two fp16 MFMA shapes of gfx950.
// What it measures is the ceiling a GEMM can approach on this part with the operands the
// benchmark prescribes: the published peak assumes the maximum clock, which the power limit
// does not allow once the operands toggle.  Two workgroups of four waves per CU (two waves
// per SIMD, as the 256x256 GEMM tiles run), eight independent accumulator blocks per wave.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <vector>

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef float float4v __attribute__((ext_vector_type(4)));

#define CHECK(x)                                                                       \
  do {                                                                                 \
    hipError_t e_ = (x);                                                               \
    if (e_ != hipSuccess) {                                                            \
      std::fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));                     \
      return 1;                                                                        \
    }                                                                                  \
  } while (0)

// SHAPE 32: 8 x v_mfma_f32_32x32x16_f16 per iteration (4 A fragments x 2 B fragments, the
// operand pattern of a 128x64 wave tile); SHAPE 16: 32 x v_mfma_f32_16x16x32_f16, twice the flops.
template <int SHAPE>
__global__ void __launch_bounds__(256) mfma_loop(const half8 *src, float *sink, int iters) {
  const int tid = blockIdx.x * 256 + threadIdx.x;
  half8 a[4], b[2];
  for (int i = 0; i < 4; ++i) a[i] = src[(tid * 6 + i) & 0xfffff];
  for (int i = 0; i < 2; ++i) b[i] = src[(tid * 6 + 4 + i) & 0xfffff];
  float s = 0.f;
  if constexpr (SHAPE == 32) {
    float16v acc[4][2];
    for (int i = 0; i < 4; ++i)
      for (int j = 0; j < 2; ++j)
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b[j], a[i], acc[i][j], 0, 0, 0);
    }
    for (int i = 0; i < 4; ++i)
      for (int j = 0; j < 2; ++j)
        for (int e = 0; e < 16; ++e) s += acc[i][j][e];
  } else {
    float4v acc[8][4];
    for (int i = 0; i < 8; ++i)
      for (int j = 0; j < 4; ++j)
        for (int e = 0; e < 4; ++e) acc[i][j][e] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b[j & 1], a[i & 3], acc[i][j], 0, 0, 0);
    }
    for (int i = 0; i < 8; ++i)
      for (int j = 0; j < 4; ++j)
        for (int e = 0; e < 4; ++e) s += acc[i][j][e];
  }
  if (s == 12345.678f) sink[tid] = s;  // keeps the accumulators alive; practically never true
}

// The same 8 MFMAs per iteration with the data movement of a GEMM main loop around them: R operand
// fragments read from LDS (ds_read_b128 per lane) and G direct-to-LDS tile requests of 16 bytes per
// lane.  The 256x256x64 tile with 128x64 wave tiles has R = 6, G = 2 per 8 MFMAs; 128x128 wave tiles R = 4.
template <int R, int G>
__global__ void __launch_bounds__(256) mfma_mix_loop(const half8 *src, float *sink, int iters) {
  __shared__ half8 lds[4096];  // 64 KB
  const int tid = blockIdx.x * 256 + threadIdx.x, t = threadIdx.x;
  for (int i = t; i < 4096; i += 256) lds[i] = src[(blockIdx.x * 4096 + i) & 0xfffff];
  __syncthreads();
  half8 f[6];
  for (int i = 0; i < 6; ++i) f[i] = src[(tid * 6 + i) & 0xfffff];
  float16v acc[4][2];
  for (int i = 0; i < 4; ++i)
    for (int j = 0; j < 2; ++j)
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)src, 0, 1 << 24, 0x00020000);
  int off = t;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int r = 0; r < R; ++r) f[r % 6] = lds[(off + r * 256) & 4095];
    off += 67;
    if constexpr (G > 0) {
#pragma unroll
      for (int g = 0; g < G; ++g)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rs, (__attribute__((address_space(3))) void *)(lds + ((g * 256 + (t & ~63)) & 4095)), 16,
            ((it * 8 + g) * 4096 + tid * 16) & 0xffffff, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f[4 + j], f[i], acc[i][j], 0, 0, 0);
    if constexpr (G > 0) {
      if ((it & 7) == 7) __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): bounds the requests in flight
    }
  }
  float s = 0.f;
  for (int i = 0; i < 4; ++i)
    for (int j = 0; j < 2; ++j)
      for (int e = 0; e < 16; ++e) s += acc[i][j][e];
  if (s == 12345.678f) sink[tid] = s;
}

// The same with v_mfma_f32_16x16x32_f16: 32 MFMAs per iteration (8 A fragments x 4 B fragments of a
// 128x64 wave tile over 32 k: twice the flops of the loop above), hence R = 12 reads and G = 4 requests
// for the same bytes per flop.
template <int R, int G>
__global__ void __launch_bounds__(256) mfma_mix_loop16(const half8 *src, float *sink, int iters) {
  __shared__ half8 lds[4096];  // 64 KB
  const int tid = blockIdx.x * 256 + threadIdx.x, t = threadIdx.x;
  for (int i = t; i < 4096; i += 256) lds[i] = src[(blockIdx.x * 4096 + i) & 0xfffff];
  __syncthreads();
  half8 f[12];
  for (int i = 0; i < 12; ++i) f[i] = src[(tid * 12 + i) & 0xfffff];
  float4v acc[8][4];
  for (int i = 0; i < 8; ++i)
    for (int j = 0; j < 4; ++j)
      for (int e = 0; e < 4; ++e) acc[i][j][e] = 0.f;
  __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)src, 0, 1 << 24, 0x00020000);
  int off = t;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int r = 0; r < R; ++r) f[r % 12] = lds[(off + r * 256) & 4095];
    off += 67;
    if constexpr (G > 0) {
#pragma unroll
      for (int g = 0; g < G; ++g)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rs, (__attribute__((address_space(3))) void *)(lds + ((g * 256 + (t & ~63)) & 4095)), 16,
            ((it * 8 + g) * 4096 + tid * 16) & 0xffffff, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(f[8 + j], f[i], acc[i][j], 0, 0, 0);
    if constexpr (G > 0) {
      if ((it & 3) == 3) __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): bounds the requests in flight
    }
  }
  float s = 0.f;
  for (int i = 0; i < 8; ++i)
    for (int j = 0; j < 4; ++j)
      for (int e = 0; e < 4; ++e) s += acc[i][j][e];
  if (s == 12345.678f) sink[tid] = s;
}

template <int R, int G>
static int run_mix16(const half8 *src, float *sink, int blocks, int iters, int launches, const char *what) {
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  float ms = 0.f;
  for (int rep = 0; rep < 2; ++rep) {
    CHECK(hipEventRecord(e0));
    for (int q = 0; q < launches; ++q) hipLaunchKernelGGL((mfma_mix_loop16<R, G>), dim3(blocks), dim3(256), 0, 0, src, sink, iters);
    CHECK(hipGetLastError());
    CHECK(hipEventRecord(e1));
    CHECK(hipEventSynchronize(e1));
    CHECK(hipEventElapsedTime(&ms, e0, e1));
  }
  std::printf("16x16x32, %-44s %7.2f ms, %6.0f TFLOP/s\n", what, ms,
              (double)launches * blocks * 4.0 * iters * 32.0 * 16384.0 / ms / 1e9);
  return 0;
}

template <int R, int G>
static int run_mix(const half8 *src, float *sink, int blocks, int iters, int launches, const char *what) {
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  float ms = 0.f;
  for (int rep = 0; rep < 2; ++rep) {
    CHECK(hipEventRecord(e0));
    for (int q = 0; q < launches; ++q) hipLaunchKernelGGL((mfma_mix_loop<R, G>), dim3(blocks), dim3(256), 0, 0, src, sink, iters);
    CHECK(hipGetLastError());
    CHECK(hipEventRecord(e1));
    CHECK(hipEventSynchronize(e1));
    CHECK(hipEventElapsedTime(&ms, e0, e1));
  }
  std::printf("32x32x16, %-44s %7.2f ms, %6.0f TFLOP/s\n", what, ms,
              (double)launches * blocks * 4.0 * iters * 8.0 * 32768.0 / ms / 1e9);
  return 0;
}

int main() {
  const int iters = 4000, launches = 5;
  const size_t n = 1 << 20;
  std::vector<_Float16> host(n * 8);
  half8 *src = nullptr;
  float *sink = nullptr;
  CHECK(hipMalloc((void **)&src, n * 16));
  CHECK(hipMalloc((void **)&sink, 1 << 24));
  hipDeviceProp_t prop;
  CHECK(hipGetDeviceProperties(&prop, 0));
  const int blocks = prop.multiProcessorCount * 2;
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  std::printf("%s, %d CUs, %d workgroups of 256 threads, %d launches of %d iterations\n", prop.gcnArchName,
              prop.multiProcessorCount, blocks, launches, iters);
  for (int mode = 0; mode < 2; ++mode) {
    std::srand(1);
    for (size_t i = 0; i < n * 8; ++i) {
      const float u1 = (std::rand() + 1.0f) / ((float)RAND_MAX + 2.0f), u2 = std::rand() / (float)RAND_MAX;
      const float g = std::sqrt(-2.f * std::log(u1)) * std::cos(6.2831853f * u2);
      host[i] = (_Float16)(mode == 0 ? 0.f : g / 64.f);  // N(0,1)/sqrt(K) at K = 4096
    }
    CHECK(hipMemcpy(src, host.data(), n * 16, hipMemcpyHostToDevice));
    for (int shape : {32, 16}) {
      float ms = 0.f;
      for (int rep = 0; rep < 2; ++rep) {  // the second repetition is reported: clocks have settled
        CHECK(hipEventRecord(e0));
        for (int k = 0; k < launches; ++k) {
          if (shape == 32) hipLaunchKernelGGL(mfma_loop<32>, dim3(blocks), dim3(256), 0, 0, src, sink, iters);
          else hipLaunchKernelGGL(mfma_loop<16>, dim3(blocks), dim3(256), 0, 0, src, sink, iters);
        }
        CHECK(hipGetLastError());
        CHECK(hipEventRecord(e1));
        CHECK(hipEventSynchronize(e1));
        CHECK(hipEventElapsedTime(&ms, e0, e1));
      }
      // per wave and iteration: 8 x 32768 flop, or 32 x 16384 flop
      const double flop = (double)launches * blocks * 4.0 * iters * (shape == 32 ? 8.0 * 32768.0 : 32.0 * 16384.0);
      std::printf("operands %-10s v_mfma_f32_%s_f16: %7.2f ms, %6.0f TFLOP/s\n", mode == 0 ? "zero" : "N(0,1)/64",
                  shape == 32 ? "32x32x16" : "16x16x32", ms, flop / ms / 1e9);
    }
    // the data-movement mixes, on all-zero operands first (no power limit: what is lost is issue slots), then on N(0,1)/64
    std::printf("-- mixes on %s operands --\n", mode == 0 ? "all-zero" : "N(0,1)/64");
    if (run_mix<0, 0>(src, sink, blocks, iters, launches, "no data movement")) return 1;
    if (run_mix<4, 0>(src, sink, blocks, iters, launches, "4 LDS reads per 8 MFMAs")) return 1;
    if (run_mix<6, 0>(src, sink, blocks, iters, launches, "6 LDS reads per 8 MFMAs")) return 1;
    if (run_mix<0, 2>(src, sink, blocks, iters, launches, "2 tile requests per 8 MFMAs")) return 1;
    if (run_mix<4, 2>(src, sink, blocks, iters, launches, "4 LDS reads + 2 tile requests per 8 MFMAs")) return 1;
    if (run_mix<6, 2>(src, sink, blocks, iters, launches, "6 LDS reads + 2 tile requests per 8 MFMAs")) return 1;
    if (run_mix16<0, 0>(src, sink, blocks, iters / 2, launches, "no data movement")) return 1;
    if (run_mix16<12, 0>(src, sink, blocks, iters / 2, launches, "12 LDS reads per 32 MFMAs")) return 1;
    if (run_mix16<0, 4>(src, sink, blocks, iters / 2, launches, "4 tile requests per 32 MFMAs")) return 1;
    if (run_mix16<12, 4>(src, sink, blocks, iters / 2, launches, "12 LDS reads + 4 tile requests per 32 MFMAs")) return 1;
    if (run_mix16<8, 4>(src, sink, blocks, iters / 2, launches, "8 LDS reads + 4 tile requests per 32 MFMAs")) return 1;
  }
  return 0;
}
