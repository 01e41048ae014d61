// Kernels around the half-precision MFMA family: the fp32 GEMM, the
// any-layout fallback GEMM and the coordinate-table dump of the convolution.
#include <mutex>

#include "contraction_kernel.hpp"

namespace tracea_amd {

// ---------------------------------------------------------------------------
// fp32 GEMM on the fp32 matrix cores (v_mfma_f32_32x32x2_f32).
// C[M,N] = epilogue(A[M,K] . B[K,N]), all row-major.  This is the device
// counterpart of the reference's only executable CPU path, gemm_cpu_packed
// (src/kernels/cpu/gemm.rs:241-298), except that C is overwritten, as in the
// reference's GPU GEMM (src/emitter/cuda/gemm.rs:179-205), not accumulated.
// Tile 128x128x16, 4 waves (2x2), wave tile 64x64.  A is staged k-major in LDS
// so that a wave's operand fetch reads 32 consecutive floats.
// Requires K % 4 == 0, N % 4 == 0, lda % 4 == 0, ldb % 4 == 0 and 16-byte
// aligned bases (checked by the dispatcher).
// ---------------------------------------------------------------------------
constexpr int F32_BM = 128, F32_BN = 128, F32_BK = 16, F32_PITCH = 132;

// Epilogue of the fp32 tile kernels.  Operands were swapped in the MFMAs: a lane owns row
// (lane&31), channels 8g + 4*(lane>>5) + 0..3 of each 32x32 block of its wave's 32FM x 32FN tile.
// The accumulators go through LDS, ROWS rows at a time (`stage` is ROWS x 32FN floats private to
// the wave), and a rolled loop takes them from there row by row.  Applying the operator chain
// to the accumulators in place needs compile-time indices, i.e. sixteen copies of the chain
// code, and with them the compiler copied the chain description from the kernel arguments to
// scratch memory (488 bytes per lane) and kept 192 registers: 1024^3 took 46.6 us that way and
// 32.9 us this way (128x128 tiles), 4096^3 1194 -> 979 us.
template <int ROWS, int FM, int FN>
__device__ __forceinline__ void f32_tile_epilogue(const f32x16 (&acc)[FM][FN], float *stage, const ContractionArgs &args,
                                                  int m_wave, int n_wave, long long zrow, int lane) {
  static_assert(ROWS == 32 || ROWS == 16, "a 32-row block is staged whole or in two halves");
  constexpr int W = 32 * FN, CH = 8 * FN;  // floats and 16-byte chunks per staged row
  const int lrow = lane & 31, lhalf = lane >> 5;
  const int er = lane / CH, lc = lane % CH;  // reader: 64/CH rows per step, CH lanes x 4 channels per row
  const int M = args.M, N = args.N;
  static_for<0, FM * (32 / ROWS)>([&](auto blk) {
    constexpr int i = decltype(blk)::value / (32 / ROWS), part = decltype(blk)::value % (32 / ROWS);
    if (ROWS == 32 || (lrow / ROWS) == part) {
      const int srow = lrow % ROWS;
#pragma unroll
      for (int jj = 0; jj < FN; ++jj)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const f32x4 v = {acc[i][jj][g * 4 + 0], acc[i][jj][g * 4 + 1], acc[i][jj][g * 4 + 2], acc[i][jj][g * 4 + 3]};
          const int chunk = jj * 8 + g * 2 + lhalf;  // 16-byte chunk of the row, XOR-ed with the row against bank conflicts
          *(f32x4 *)(stage + srow * W + ((chunk ^ (srow & (CH - 1))) << 2)) = v;
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma nounroll
    for (int r = er; r < ROWS; r += 64 / CH) {
      const int m = m_wave + i * 32 + part * ROWS + r;
      const int n = n_wave + lc * 4;
      if (m < M && n < N) {
        const f32x4 t = *(const f32x4 *)(stage + r * W + ((lc ^ (r & (CH - 1))) << 2));
        float v[4] = {t[0], t[1], t[2], t[3]};
        apply_epilogue<4>(v, zrow + m, n, N - n, args.epi);
        store_from_float<4>(args.C, args.out_dtype, (zrow + m) * args.ldc + n, N - n, v);
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
  });
}

__global__ void __launch_bounds__(256) gemm_f32_kernel(const ContractionArgs args) {
  __shared__ float As[F32_BK][F32_PITCH];
  __shared__ float Bs[F32_BK][F32_PITCH];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;
  int tile_m, tile_n;
  tile_coordinates(args, tile_m, tile_n);
  const int m0 = tile_m * F32_BM, n0 = tile_n * F32_BN;
  const int M = args.M, N = args.N;
  // split-K as in the half-precision kernels: K range [kb, K) of this workgroup, partial
  // product to rows zrow.. of the workspace
  const int kb = args.k_split > 0 ? (int)blockIdx.y * args.k_split : 0;
  const int K = args.k_split > 0 ? min(args.K, kb + args.k_split) : args.K;
  const long long zrow = args.k_split > 0 ? (long long)blockIdx.y * M : 0ll;
  const float *A = (const float *)args.A;
  const float *B = (const float *)args.B;

  // A tile: 128 rows x 16 k = 512 float4 pieces, 2 per thread (row = q/4, kq = q%4)
  // B tile: 16 k x 128 n   = 512 float4 pieces, 2 per thread (k = q/32, nq = q%32)
  f32x4 ra[2], rb[2];
  auto fetch = [&](int k0) {
    k0 += kb;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int q = tid + i * 256;
      int m = m0 + q / 4;
      m = m < M ? m : M - 1;
      const int k = k0 + (q % 4) * 4;
      const bool ok = k < K;
      const f32x4 v = *(const f32x4 *)(A + (long long)m * args.lda + (ok ? k : 0));
      const f32x4 z = {0.f, 0.f, 0.f, 0.f};
      ra[i] = ok ? v : z;
      const int krow = k0 + q / 32;
      const int n = n0 + (q % 32) * 4;
      const bool okb = krow < K && n < N;
      const f32x4 w = *(const f32x4 *)(B + (okb ? (long long)krow * args.ldb + n : 0ll));
      rb[i] = okb ? w : z;
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int q = tid + i * 256;
      const int row = q / 4, kq = (q % 4) * 4;
#pragma unroll
      for (int e = 0; e < 4; ++e) As[kq + e][row] = ra[i][e];
      *(f32x4 *)&Bs[q / 32][(q % 32) * 4] = rb[i];
    }
  };

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  const int lrow = lane & 31, lhalf = lane >> 5;
  const int nk = (K - kb + F32_BK - 1) / F32_BK;
  fetch(0);
  for (int kt = 0; kt < nk; ++kt) {
    stash();
    __syncthreads();
    if (kt + 1 < nk) fetch((kt + 1) * F32_BK);
#pragma unroll
    for (int ks = 0; ks < F32_BK / 2; ++ks) {
      const int k = ks * 2 + lhalf;
      float af[2], bf[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) af[i] = As[k][wm * 64 + i * 32 + lrow];
#pragma unroll
      for (int j = 0; j < 2; ++j) bf[j] = Bs[k][wn * 64 + j * 32 + lrow];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bf[j], af[i], acc[i][j], 0, 0, 0);
    }
    __syncthreads();
  }

  // the tile buffers are too small to stage 32 rows per wave: 16 rows at a time in a buffer of their own
  __shared__ __attribute__((aligned(16))) float stage_mem[4 * 16 * 64];
  f32_tile_epilogue<16, 2, 2>(acc, stage_mem + (tid >> 6) * (16 * 64), args, m0 + wm * 64, n0 + wn * 64, zrow, lane);
}


// ---------------------------------------------------------------------------
// fp32 GEMM, direct-to-LDS form.  Same product as gemm_f32_kernel, for operands
// below 2 GiB (32-bit buffer offsets).  Tile 64T x 64T x 16 (T = 2 or 1), 4 waves
// (2x2), wave tile 32T x 32T = TxT blocks of v_mfma_f32_32x32x2_f32.  Both operand
// tiles are requested with buffer loads that write LDS directly into one of
// STAGES stages while an earlier one is multiplied: one barrier per K tile, no
// staging registers, no LDS write instructions.
//   A tile [64T rows][16 k], 64-byte rows; piece q (16 bytes at LDS byte 16q) is
//     row q/4, column q%4, and holds global column (q%4) ^ ((row/4)&3): the
//     16-byte operand reads of 16 consecutive rows then fall in 16 different
//     bank groups.
//   B tile [16 k][64T n], 256T-byte rows; piece q is k row q/16T, column q%16T, and
//     holds global column (q%16T) ^ (8*(row/8)): lanes 0-31 read k rows 0-7, lanes
//     32-63 rows 8-15 of the same 32 channels, which the XOR moves to the other
//     half of the banks.
// An MFMA sums over two k; lane half h supplies k = 8h + t to the t-th MFMA of a
// K tile for A and B alike, so A's operands are two 16-byte reads per row block
// and B's are eight 4-byte reads per channel block.
// The 128x128 tile multiplies a K tile for 2048 cycles and runs two stages; the
// 64x64 tile, for problems with fewer than a CU's worth of large tiles each, has
// 512 cycles per K tile and keeps three tiles in flight (four stages) to cover
// the latency of a request (two sub-tiles of 16 k per stage and barrier, KSUB = 2,
// gained 3 % at 1024^3 and lost 7 % at 2048^3, where the 64 KB of LDS leave two
// workgroups per CU instead of five; a third stage for the 128x128 tile lost 2-6 %).
// Past the end of K the requests are still issued,
// out of range (they write zeros to a stage nobody multiplies), so that the
// count of outstanding requests a wave waits on is the same in every iteration.
// ---------------------------------------------------------------------------
template <int TM, int TN, int STAGES, int KSUB, int FIRST_T = 1>
__global__ void __launch_bounds__(256) gemm_f32_dma_kernel(const ContractionArgs args) {
  constexpr int BM = 64 * TM, BN = 64 * TN, BK = F32_BK * KSUB;  // a stage holds KSUB sub-tiles of 16 k, each [A][B]
  constexpr int A_STAGE = BM * F32_BK * 4, B_STAGE = F32_BK * BN * 4, SUB = A_STAGE + B_STAGE, STAGE = KSUB * SUB;
  constexpr int B_PITCH = BN * 4, B_PIECES = BN / 4;  // bytes and 16-byte pieces per k row of B
  static_assert(STAGES * STAGE >= 4 * 32 * 32 * TN * 4, "the epilogue stages 32 rows per wave in the tile buffers");
  static_assert((STAGES - 1) * (TM + TN) * KSUB < 64, "outstanding requests must fit the 6-bit wait count");
  __shared__ __attribute__((aligned(16))) unsigned char smem[STAGES * STAGE];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int wm = wave & 1, wn = wave >> 1;
  int tile_m, tile_n;
  tile_coordinates(args, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int M = args.M, N = args.N;
  const int kb = args.k_split > 0 ? (int)blockIdx.y * args.k_split : 0;
  const int K = args.k_split > 0 ? min(args.K, kb + args.k_split) : args.K;
  // one-launch split: see the block in front of the epilogue
  const bool fused = args.k_split > 0 && args.fuse_ws != nullptr;
  const long long zrow = args.k_split > 0 && !fused ? (long long)blockIdx.y * M : 0ll;

  constexpr unsigned OOB = 0x80000000u;
  __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc((void *)args.A, 0, (int)args.a_bytes, 0x00020000);
  __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc((void *)args.B, 0, (int)args.b_bytes, 0x00020000);
  // TM pieces of A and TN of B per thread and K tile
  unsigned a_voff[TM], b_voff[TN];
  int a_kcol[TM], b_krow[TN];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int q = tid + i * 256;
    const int row = q >> 2;
    int m = m0 + row;
    m = m < M ? m : M - 1;  // rows past the end re-read the last row; their results are never stored
    a_kcol[i] = ((q & 3) ^ ((row >> 2) & 3)) * 4;
    a_voff[i] = (unsigned)(((long long)m * args.lda + a_kcol[i]) * 4);
  }
#pragma unroll
  for (int i = 0; i < TN; ++i) {
    const int q = tid + i * 256;
    b_krow[i] = q / B_PIECES;
    const int n = n0 + (((q % B_PIECES) ^ ((b_krow[i] >> 3) << 3)) << 2);
    b_voff[i] = n < N ? (unsigned)(((long long)b_krow[i] * args.ldb + n) * 4) : OOB;
  }
  // request r of a K tile: sub-tile r / (TM + TN), then TM pieces of A and TN of B
  auto dma_nth = [&](unsigned char *stage, int k0, int r) __attribute__((always_inline)) {
    const int u = r / (TM + TN), w = r % (TM + TN);
    stage += u * SUB;
    k0 += kb + u * F32_BK;
    const bool any = k0 < K;  // uniform: a tile wholly past K asks for nothing but zeros
    if (w < TM) {
      unsigned char *dst = stage + (w * 256 + wave_u * 64) * 16;
      const unsigned va = k0 + a_kcol[w] < K ? a_voff[w] : OOB;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (__attribute__((address_space(3))) void *)dst, 16, (int)va,
                                               any ? k0 * 4 : 0, 0, 0);
    } else {
      unsigned char *dst = stage + A_STAGE + ((w - TM) * 256 + wave_u * 64) * 16;
      const unsigned vb = k0 + b_krow[w - TM] < K ? b_voff[w - TM] : OOB;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (__attribute__((address_space(3))) void *)dst, 16, (int)vb,
                                               any ? (int)((long long)k0 * args.ldb * 4) : 0, 0, 0);
    }
  };
  constexpr int REQS = (TM + TN) * KSUB;  // requests per thread and K tile
  auto dma = [&](unsigned char *stage, int k0) {
#pragma unroll
    for (int r = 0; r < REQS; ++r) dma_nth(stage, k0, r);
  };

  constexpr bool ONE = TM * TN == 1;
  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  // With one 32x32 block per wave (TM = TN = 1) every MFMA would wait for the one before it, the same accumulator
  // being its input: the odd k pairs of a tile go to a second accumulator, added in once at the end, and
  // the matrix pipe always has an independent MFMA to start.
  f32x16 acc_odd;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc_odd[e] = 0.0f;

  const int lrow = lane & 31, lhalf = lane >> 5;
  // A: row wm*32TM + i*32 + lrow, 16-byte columns 2h and 2h+1 (k = 8h .. 8h+7)
  int a_off[TM][2];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int row = wm * (32 * TM) + i * 32 + lrow;
#pragma unroll
    for (int c = 0; c < 2; ++c) a_off[i][c] = row * 64 + (((2 * lhalf + c) ^ ((row >> 2) & 3)) << 4);
  }
  // B: k row 8h + t, channel wn*32TN + j*32 + lrow
  int b_off[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int n = wn * (32 * TN) + j * 32 + lrow;
    b_off[j] = A_STAGE + (8 * lhalf) * B_PITCH + ((((n >> 2) ^ (lhalf << 3)) << 2) + (n & 3)) * 4;
  }

  // Operands of tile kt+1 are read from LDS while tile kt is multiplied from registers (with one
  // wave per SIMD nothing else would cover the latency of those reads).  Stage kt%STAGES is free
  // once every wave has its operands of tile kt, so tile kt+STAGES is requested into it: after the
  // prologue STAGES-1 tiles are in flight or landed beyond the one being read.
  constexpr int PER = REQS;
  constexpr auto vmcnt = [](int n) constexpr { return 0x0f70 | (n & 15) | ((n >> 4) << 14); };  // the count's bits 5:4 sit in 15:14
  constexpr int WAIT_FIRST = vmcnt((STAGES - 1) * PER), WAIT_NEXT = vmcnt((STAGES - 2) * PER);
  // The operand reads are written as instructions.  Through a pointer the compiler puts a vmcnt(0) in front
  // of the first of them that follows a tile request (it cannot tell that the request writes another stage),
  // so every K tile waited out the request issued a few instructions earlier and no number of stages covered
  // anything.  As instructions they are outside its bookkeeping: operands_landed, in front of the MFMAs that
  // take them, is the wait.
  constexpr int READS_SUB = 2 * TM + 8 * TN, READS = KSUB * READS_SUB;  // operand reads per sub-tile and per K tile
  auto read_nth = [&](unsigned base, f32x4 (&af)[KSUB][TM][2], float (&bf)[KSUB][TN][8], int r) __attribute__((always_inline)) {
    const int u = r / READS_SUB, w = r % READS_SUB;
    if (w < 2 * TM)
      asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(af[u][w >> 1][w & 1]) : "v"(base + a_off[w >> 1][w & 1]), "i"(u * SUB));
    else
      asm volatile("ds_read_b32 %0, %1 offset:%2"
                   : "=v"(bf[u][(w - 2 * TM) >> 3][(w - 2 * TM) & 7])
                   : "v"(base + b_off[(w - 2 * TM) >> 3]), "i"(u * SUB + ((w - 2 * TM) & 7) * B_PITCH));
  };
  auto read_operands = [&](const unsigned char *cur, f32x4 (&af)[KSUB][TM][2], float (&bf)[KSUB][TN][8]) {
    const unsigned base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)cur;
#pragma unroll
    for (int r = 0; r < READS; ++r) read_nth(base, af, bf, r);
  };
  auto operands_landed = [&](f32x4 (&af)[KSUB][TM][2], float (&bf)[KSUB][TN][8]) {
    asm volatile("s_waitcnt lgkmcnt(0)");
#pragma unroll
    for (int u = 0; u < KSUB; ++u) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int c = 0; c < 2; ++c) asm volatile("" : "+v"(af[u][i][c]));
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int t = 0; t < 8; ++t) asm volatile("" : "+v"(bf[u][j][t]));
    }
  };
  auto step = [&](int kt, f32x4 (&af)[KSUB][TM][2], float (&bf)[KSUB][TN][8], f32x4 (&af_next)[KSUB][TM][2],
                  float (&bf_next)[KSUB][TN][8]) {
    operands_landed(af, bf);
    // A few of tile kt's MFMAs, then the barrier, then the rest with the requests of tile kt+STAGES and the
    // operand reads of tile kt+1 between them: with one wave per SIMD whatever is issued without an MFMA in
    // flight is time the matrix pipe stands still.  A request holds the wave for about 64 cycles (measured:
    // two behind one MFMA cost the pipe 65 cycles, four behind two 220), so each goes behind an MFMA of its
    // own; the reads, about 8 cycles each, follow at an even rate and leave the last MFMAs for their
    // latency.  (The order is held with scheduling barriers: left alone the compiler puts every MFMA
    // behind the barrier and the requests, and the matrix pipe drains while the workgroup gathers.)
    auto mfma_nth = [&](int q) __attribute__((always_inline)) {
      const int j = q % TN, i = (q / TN) % TM, t = (q / (TN * TM)) % 8, u = q / (TN * TM * 8);
      if constexpr (ONE) {
        if (t & 1) acc_odd = __builtin_amdgcn_mfma_f32_32x32x2f32(bf[u][0][t], af[u][0][t >> 2][t & 3], acc_odd, 0, 0, 0);
        else acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(bf[u][0][t], af[u][0][t >> 2][t & 3], acc[0][0], 0, 0, 0);
      } else {
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bf[u][j][t], af[u][i][t >> 2][t & 3], acc[i][j], 0, 0, 0);
      }
    };
    constexpr int MFMAS = 8 * TM * TN * KSUB;   // of a K tile
    constexpr int FIRST = FIRST_T * TM * TN;    // in front of the barrier: they cover the gathering of the workgroup
    constexpr int LAND = ONE ? 1 : 2;           // the last ones, with nothing behind them
    constexpr int READ_SLOTS = MFMAS - FIRST - REQS - LAND;
    constexpr int PER_MFMA = (READS + READ_SLOTS - 1) / READ_SLOTS;
    static_assert(READ_SLOTS > 0, "every request and read has its place");
#pragma unroll
    for (int q = 0; q < FIRST; ++q) mfma_nth(q);
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(WAIT_NEXT);  // tile kt+1 has landed (this wave's share)
    // ... everyone's, and everyone holds its operands of tile kt.  The barrier alone: with the fences of
    // __syncthreads() the compiler waits for every request in flight, those of the later tiles included.
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    const unsigned next = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)(smem + ((kt + 1) % STAGES) * STAGE);
    unsigned char *freed = smem + (kt % STAGES) * STAGE;
#pragma unroll
    for (int q = FIRST; q < MFMAS; ++q) {
      mfma_nth(q);
      const int slot = q - FIRST;
      if (slot < REQS) {
        dma_nth(freed, (kt + STAGES) * BK, slot);
      } else {
#pragma unroll
        for (int x = 0; x < PER_MFMA; ++x) {
          const int r = (slot - REQS) * PER_MFMA + x;
          if (r < READS) read_nth(next, af_next, bf_next, r);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  const int nk = (K - kb + BK - 1) / BK;
#pragma unroll
  for (int s = 0; s < STAGES; ++s) dma(smem + s * STAGE, s * BK);
  __builtin_amdgcn_s_waitcnt(WAIT_FIRST);
  __syncthreads();
  f32x4 af0[KSUB][TM][2], af1[KSUB][TM][2];
  float bf0[KSUB][TN][8], bf1[KSUB][TN][8];
  read_operands(smem, af0, bf0);
  for (int kt = 0; kt < nk; kt += 2) {
    step(kt, af0, bf0, af1, bf1);
    if (kt + 1 < nk) step(kt + 1, af1, bf1, af0, bf0);
  }
  // requests past the end of K may still be writing zeros where the epilogue stages, and the last operand reads
  // (of a tile nobody multiplies) may still be writing their registers
  __builtin_amdgcn_s_waitcnt(0x0070);
  operands_landed(af0, bf0);
  operands_landed(af1, bf1);
  __syncthreads();
  if constexpr (ONE) {
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[0][0][e] += acc_odd[e];
  }

  // One-launch split along K, as in the half-precision kernels: every workgroup leaves its partial product in
  // block (tile, K range) of a workspace, in accumulator order, with device-scope stores (the K ranges of a
  // tile may run on XCDs whose L2s do not see each other's lines), and takes a ticket; the workgroup that draws
  // the tile's last ticket sums the blocks in K order, its own included, and runs the epilogue.  Nobody waits.
  if (fused) {
    __shared__ unsigned s_ticket;
    constexpr int DEVICE_SCOPE = 16;  // the sc1 bit of a buffer instruction
    const unsigned splits = gridDim.y;
    constexpr unsigned TILE_BYTES = BM * BN * 4, WAVE_BYTES = TILE_BYTES / 4;
    __amdgpu_buffer_rsrc_t rsrc_ws = __builtin_amdgcn_make_buffer_rsrc((void *)args.fuse_ws, 0, 0x7fffffff, 0x00020000);
    const unsigned first = blockIdx.x * splits * TILE_BYTES + wave_u * WAVE_BYTES + lane * 16;
    const unsigned mine = first + blockIdx.y * TILE_BYTES;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const f32x4 v = {acc[i][j][g * 4 + 0], acc[i][j][g * 4 + 1], acc[i][j][g * 4 + 2], acc[i][j][g * 4 + 3]};
          __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), rsrc_ws, (int)(mine + ((i * TN + j) * 4 + g) * 1024), 0,
                                                 DEVICE_SCOPE);
        }
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): the stores are acknowledged
    __syncthreads();
    if (tid == 0) s_ticket = __hip_atomic_fetch_add(args.fuse_count + blockIdx.x, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (s_ticket != splits - 1) return;
    if (tid == 0) __hip_atomic_store(args.fuse_count + blockIdx.x, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;
#pragma unroll 1
    for (unsigned z = 0; z < splits; ++z) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const f32x4 v = __builtin_bit_cast(
                f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_ws, (int)(first + z * TILE_BYTES + ((i * TN + j) * 4 + g) * 1024), 0,
                                                           DEVICE_SCOPE));
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[i][j][g * 4 + e] += v[e];
          }
    }
  }
  f32_tile_epilogue<32, TM, TN>(acc, (float *)smem + wave_u * (32 * 32 * TN), args, m0 + wm * (32 * TM), n0 + wn * (32 * TN),
                              zrow, lane);
}

int launch_gemm_f32(const ContractionArgs &a, int tile, hipStream_t stream) {
  ContractionArgs args = a;
  // the 64x64 tiles exist in the direct-to-LDS form only (operands below 2 GiB, a_bytes / b_bytes set by the dispatcher)
  const bool dma = a.a_bytes != 0 && a.b_bytes != 0;
  if ((tile != 64 && tile != 6432) || !dma) tile = 128;
  const int edge = tile == 128 ? 128 : 64;
  args.grid_m = (a.M + edge - 1) / edge;
  args.grid_n = (a.N + edge - 1) / edge;
  args.group_m = 4;
  const unsigned splits = a.k_split > 0 ? (unsigned)((a.K + a.k_split - 1) / a.k_split) : 1u;
  const dim3 grid((unsigned)(args.grid_m * args.grid_n), splits);
  if (!dma) hipLaunchKernelGGL(gemm_f32_kernel, grid, dim3(256), 0, stream, args);
  else if (tile == 64) hipLaunchKernelGGL((gemm_f32_dma_kernel<1, 1, 4, 1>), grid, dim3(256), 0, stream, args);
  else if (tile == 6432) hipLaunchKernelGGL((gemm_f32_dma_kernel<1, 1, 4, 2>), grid, dim3(256), 0, stream, args);
  else hipLaunchKernelGGL((gemm_f32_dma_kernel<2, 2, 2, 1>), grid, dim3(256), 0, stream, args);
  return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------
// Fallback GEMM: any element strides, any of f32/f16/bf16 per operand, no
// alignment requirement.  One output element per thread, fp32 FMA on the
// vector ALU.  Correct everywhere, fast nowhere; the dispatcher only uses it
// when no matrix-core kernel applies.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float load_scalar(const void *p, int dtype, long long idx) {
  if (dtype == DT_F32) return ((const float *)p)[idx];
  if (dtype == DT_F16) return (float)((const _Float16 *)p)[idx];
  return (float)((const __bf16 *)p)[idx];
}

__global__ void __launch_bounds__(256) gemm_generic_kernel(const GenericGemmArgs a) {
  const int n = blockIdx.x * 16 + (threadIdx.x & 15);
  const int m = blockIdx.y * 16 + (threadIdx.x >> 4);
  if (m >= a.M || n >= a.N) return;
  float acc = 0.0f;
  for (int k = 0; k < a.K; ++k)
    acc = fmaf(load_scalar(a.A, a.a_dtype, (long long)m * a.sam + (long long)k * a.sak),
               load_scalar(a.B, a.b_dtype, (long long)k * a.sbk + (long long)n * a.sbn), acc);
  float v[1] = {acc};
  apply_epilogue<1>(v, m, n, 1, a.epi);
  store_from_float<1>(a.C, a.c_dtype, (long long)m * a.scm + (long long)n * a.scn, 1, v);
}

// (row r of the padded side = ((r0 * n1) + r1) * n2 + r2; its first element on the strided side lies at
// r0 * rs + r1 * s1 + r2 * s2.  TO_PADDED: strided -> padded rows, zeros behind the data; else the way back,
// data only.)
template <typename T, bool TO_PADDED>
__global__ void __launch_bounds__(256) pad_copy_kernel(const T *src, T *dst, long long rows, long long cols, long long rs, long long cs,
                                                       long long n1, long long s1, long long n2, long long s2, long long pitch,
                                                       long long total) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const long long width = TO_PADDED ? pitch : cols;
  const long long r = idx / width, c = idx - r * width;
  const long long r01 = r / n2, r2 = r - r01 * n2;
  const long long r0 = r01 / n1, r1 = r01 - r0 * n1;
  const long long strided = r0 * rs + r1 * s1 + r2 * s2 + c * cs;
  if constexpr (TO_PADDED) dst[idx] = (r < rows && c < cols) ? src[strided] : T(0);
  else dst[strided] = src[r * pitch + c];
}

int launch_pad_copy(const void *src, void *dst, int elt_bytes, long long rows_src, long long cols_src, long long rs,
                    long long cs, long long rows_dst, long long pitch, hipStream_t stream, long long n1, long long s1,
                    long long n2, long long s2) {
  const long long total = rows_dst * pitch;
  if (total <= 0) return 0;
  const long long blocks = (total + 255) / 256;
  if (blocks >= (1ll << 31) || (elt_bytes != 2 && elt_bytes != 4) || n1 < 1 || n2 < 1) return (int)hipErrorInvalidValue;
  if (elt_bytes == 2)
    hipLaunchKernelGGL((pad_copy_kernel<unsigned short, true>), dim3((unsigned)blocks), dim3(256), 0, stream,
                       (const unsigned short *)src, (unsigned short *)dst, rows_src, cols_src, rs, cs, n1, s1, n2, s2, pitch, total);
  else
    hipLaunchKernelGGL((pad_copy_kernel<unsigned, true>), dim3((unsigned)blocks), dim3(256), 0, stream, (const unsigned *)src,
                       (unsigned *)dst, rows_src, cols_src, rs, cs, n1, s1, n2, s2, pitch, total);
  return (int)hipGetLastError();
}

int launch_unpad_copy(const void *src, void *dst, int elt_bytes, long long rows, long long cols, long long rs, long long cs,
                      long long pitch, hipStream_t stream, long long n1, long long s1, long long n2, long long s2) {
  const long long total = rows * cols;
  if (total <= 0) return 0;
  const long long blocks = (total + 255) / 256;
  if (blocks >= (1ll << 31) || (elt_bytes != 2 && elt_bytes != 4) || n1 < 1 || n2 < 1) return (int)hipErrorInvalidValue;
  if (elt_bytes == 2)
    hipLaunchKernelGGL((pad_copy_kernel<unsigned short, false>), dim3((unsigned)blocks), dim3(256), 0, stream,
                       (const unsigned short *)src, (unsigned short *)dst, rows, cols, rs, cs, n1, s1, n2, s2, pitch, total);
  else
    hipLaunchKernelGGL((pad_copy_kernel<unsigned, false>), dim3((unsigned)blocks), dim3(256), 0, stream, (const unsigned *)src,
                       (unsigned *)dst, rows, cols, rs, cs, n1, s1, n2, s2, pitch, total);
  return (int)hipGetLastError();
}

int launch_gemm_generic(const GenericGemmArgs &a, hipStream_t stream) {
  const dim3 grid((unsigned)((a.N + 15) / 16), (unsigned)((a.M + 15) / 16));
  hipLaunchKernelGGL(gemm_generic_kernel, grid, dim3(256), 0, stream, a);
  return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------
// Split-K reduction: sums the fp32 partial products of the K ranges, applies the
// operator chain and stores.  One thread per row and 4 channels (1 when N % 4).
// ---------------------------------------------------------------------------
template <int V>
__global__ void __launch_bounds__(256) splitk_reduce_kernel(const SplitKReduceArgs a) {
  // (every argument of the prologue in one batch of scalar loads instead of one round trip per field)
  asm volatile("" ::"s"(a.partial), "s"(a.out), "s"(a.out_dtype), "s"(a.splits), "s"(a.M), "s"(a.N), "s"(a.ldc),
               "s"(a.tile_counts), "s"(a.epi.n_ops));
  const int groups = (a.N + V - 1) / V;
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long long)a.M * groups) return;
  const long long m = idx / groups;
  const int n = (int)(idx % groups) * V;
  const int nvalid = a.N - n;
  float v[V];
#pragma unroll
  for (int e = 0; e < V; ++e) v[e] = 0.0f;
  const float *p = a.partial + m * a.N + n;
  const long long plane = (long long)a.M * a.N;
  int splits = a.splits;
  if (a.tile_counts != nullptr) {
    splits = (int)a.tile_counts[(m / a.mt) * a.grid_n + n / a.nt];
    if (splits == 0) return;  // no record names this tile: its elements are not written
  }
  // eight planes at a time, loads first: with a few thousand threads and a serial chain of
  // loads per thread the kernel would be bound by memory latency times the split count
  int z = 0;
  for (; z + 8 <= splits; z += 8) {
    if constexpr (V == 4) {
      f32x4 t[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) t[u] = *(const f32x4 *)(p + (z + u) * plane);
#pragma unroll
      for (int u = 0; u < 8; ++u)
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] += t[u][e];
    } else {
      float t[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) t[u] = p[(z + u) * plane];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[0] += t[u];
    }
  }
  for (; z < splits; ++z) {
    if constexpr (V == 4) {
      const f32x4 t = *(const f32x4 *)(p + z * plane);
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] += t[e];
    } else {
      v[0] += p[z * plane];
    }
  }
  apply_epilogue<V>(v, m, n, nvalid, a.epi);
  store_from_float<V>(a.out, a.out_dtype, m * a.ldc + n, nvalid, v);
}

int launch_splitk_reduce(const SplitKReduceArgs &a, hipStream_t stream) {
  const bool vec = a.N % 4 == 0 && (((uintptr_t)a.partial) & 15) == 0;
  const long long groups = vec ? a.N / 4 : a.N;
  const long long blocks = ((long long)a.M * groups + 255) / 256;
  if (blocks <= 0) return 0;
  if (blocks >= (1ll << 31)) return (int)hipErrorInvalidValue;
  if (vec) hipLaunchKernelGGL(splitk_reduce_kernel<4>, dim3((unsigned)blocks), dim3(256), 0, stream, a);
  else hipLaunchKernelGGL(splitk_reduce_kernel<1>, dim3((unsigned)blocks), dim3(256), 0, stream, a);
  return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------
// Split-K workspace for callers that cannot allocate device memory (code under HIP
// graph capture, serving loops, harnesses that forbid hipMalloc): a file-scope device
// array instead of the per-stream buffer the other entry points grow on demand.  Every
// GPU the library runs on holds its own copy of the array, at its own address, until the
// process ends.  In host code the array's name is only a stand-in for the symbol: the
// address kernels may use comes from hipGetSymbolAddress, asked once per device with that
// device current, and is what every launch and copy is given.
// ---------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[TRACEA_STATIC_SCRATCH_BYTES];

int static_scratch_address(int device, void **ptr) {
  constexpr int kMaxDevices = 64;
  static std::mutex mu;
  static void *address[kMaxDevices] = {};
  if (device < 0 || device >= kMaxDevices) return (int)hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(mu);
  if (address[device] == nullptr) {
    int current = -1;
    hipError_t e = hipGetDevice(&current);
    if (e != hipSuccess) return (int)e;
    if (current != device && (e = hipSetDevice(device)) != hipSuccess) return (int)e;
    void *p = nullptr;
    e = hipGetSymbolAddress((void **)&p, HIP_SYMBOL(scratch));
    if (current != device) (void)hipSetDevice(current);
    if (e != hipSuccess) return (int)e;
    if (p == nullptr) return (int)hipErrorInvalidSymbol;
    address[device] = p;
  }
  *ptr = address[device];
  return 0;
}

// ---------------------------------------------------------------------------
// Coordinate tables of the convolution, computed on the device with the same
// fast_divmod the contraction kernel uses, for bit-exact comparison with the
// CPU statement of src/emitter/cuda/conv.rs:176-191, 208-210.
// ---------------------------------------------------------------------------
__global__ void conv_coords_kernel(TraceaConvParamsBlock p, int32_t *rows, int64_t *base_off,
                                   int32_t *cols) {
  const int m_gemm = p.batch * p.h_out * p.w_out;
  const int k_gemm = p.r_sz * p.s_sz * p.c_in;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < m_gemm) {
    int bn, rem, ho, wo;
    fast_divmod(i, p.hw_m, p.hw_s, p.h_out * p.w_out, bn, rem);
    fast_divmod(rem, p.w_m, p.w_s, p.w_out, ho, wo);
    rows[3 * i] = bn;
    rows[3 * i + 1] = ho;
    rows[3 * i + 2] = wo;
    base_off[i] = (int64_t)bn * p.h_in * p.w_in * p.c_in;
  }
  if (i < k_gemm) {
    int rf, rem, sf, ci;
    fast_divmod(i, p.sic_m, p.sic_s, p.s_sz * p.c_in, rf, rem);
    fast_divmod(rem, p.c_m, p.c_s, p.c_in, sf, ci);
    cols[3 * i] = rf;
    cols[3 * i + 1] = sf;
    cols[3 * i + 2] = ci;
  }
}

int launch_conv_coords(const TraceaConvParamsBlock &p, int32_t *rows, int64_t *base_off,
                       int32_t *cols, hipStream_t stream) {
  const int m_gemm = p.batch * p.h_out * p.w_out;
  const int k_gemm = p.r_sz * p.s_sz * p.c_in;
  const int n = m_gemm > k_gemm ? m_gemm : k_gemm;
  hipLaunchKernelGGL(conv_coords_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, p,
                     rows, base_off, cols);
  return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------
// Synthetic operand fill for the tuner: splitmix-style hash of the element
// index, uniform in [-amplitude, amplitude].
// ---------------------------------------------------------------------------
__global__ void fill_uniform_kernel(void *ptr, size_t n, int dtype, unsigned seed, float amplitude) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    unsigned long long z = (i + 1) * 0x9E3779B97F4A7C15ull + ((unsigned long long)seed << 32);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    const float u = (float)(z >> 40) * (1.0f / 16777216.0f);  // [0,1)
    const float v = (2.0f * u - 1.0f) * amplitude;
    if (dtype == DT_F32) ((float *)ptr)[i] = v;
    else if (dtype == DT_F16) ((_Float16 *)ptr)[i] = (_Float16)v;
    else ((__bf16 *)ptr)[i] = (__bf16)v;
  }
}

int launch_fill_uniform(void *ptr, size_t n, int dtype, unsigned seed, float amplitude,
                        hipStream_t stream) {
  if (n == 0) return 0;
  size_t blocks = (n + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(fill_uniform_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, ptr, n,
                     dtype, seed, amplitude);
  return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------
// Shader-clock probe: one wave that, `samples` times, writes the pair (s_memtime = shader clock ticks,
// s_memrealtime = the constant 100 MHz counter) and sleeps for about `gap` times 64 clocks.  Launched on
// a stream of its own beside the kernels under measurement it shares their clock domain and costs them a
// wave slot on one CU; the slope of ticks over real time between two samples is the clock the device ran
// at in between.  The loop is bounded by its arguments and waits for nothing.
// ---------------------------------------------------------------------------
__global__ void clock_probe_kernel(unsigned long long *out, int samples, int gap) {
  if (threadIdx.x != 0) return;
  for (int i = 0; i < samples; ++i) {
    const unsigned long long ticks = __builtin_amdgcn_s_memtime();
    const unsigned long long real = __builtin_amdgcn_s_memrealtime();
    out[2 * i] = ticks;
    out[2 * i + 1] = real;
    for (int g = 0; g < gap; ++g) __builtin_amdgcn_s_sleep(64);
  }
}

int launch_clock_probe(unsigned long long *out, int samples, int gap, hipStream_t stream) {
  if (out == nullptr || samples <= 0 || samples > (1 << 20) || gap < 0 || gap > 4096) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(clock_probe_kernel, dim3(1), dim3(64), 0, stream, out, samples, gap);
  return (int)hipGetLastError();
}

}  // namespace tracea_amd
