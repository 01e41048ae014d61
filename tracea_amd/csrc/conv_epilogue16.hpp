// Register epilogue of the convolution kernels on 16x16x32 MFMAs (gfx950).
//
// The filter fragment is the first MFMA operand, so a lane ends with 4 consecutive output channels
// (4q .. 4q+3 of a 16-filter block, q = lane >> 4) of pixel lane & 15 of a 16-pixel block.  For the chains
// of the form [affine] [ReLU] [residual] [ReLU] (affine: v*a + b per channel -- a bias, a scale-shift or a
// folded BatchNorm; same functors as the reference's epilogue, src/kernels/gpu/epilogue.cuh:12-63, in the
// order of its emitter, src/emitter/cuda/conv.rs:91-116) everything happens in registers: per pair of
// filter blocks one v_permlane16_swap per packed register gives every lane 8 consecutive channels of its
// pixel, one 16-byte store; a residual is fetched in that layout, 16 bytes per lane, and taken back to the
// accumulators' layout by the same swap.  F: bit 0 affine, 1 first ReLU, 2 residual, 3 second ReLU.
#pragma once
#include "contraction_kernel.hpp"

namespace tracea_amd {

template <int DT, int F>
struct Epilogue16 {
  static constexpr bool AFF = (F & 1) != 0, RELU1 = (F & 2) != 0, RES = (F & 4) != 0, RELU2 = (F & 8) != 0;
  // the chain's last ReLU on the packed halves (one v_pk_max_f16 per two values; rounding is monotonic and
  // keeps zero, so max before or after it is the same value)
  static constexpr bool PK = DT == DT_F16 && (RELU2 || (RELU1 && !RES));
  static constexpr bool RELU1_F32 = RELU1 && !(PK && !RES), RELU2_F32 = RELU2 && !PK;
  static constexpr unsigned OOB = 0x80000000u;  // beyond every buffer: a load returns zeros, a store is dropped

  static __device__ __forceinline__ unsigned pack2(float x, float y) {
    unsigned u;
    if constexpr (DT == DT_F16) {
      const f16x2 h = {(_Float16)x, (_Float16)y};
      u = __builtin_bit_cast(unsigned, h);
    } else {
      const bf16x2 h = {(__bf16)x, (__bf16)y};
      u = __builtin_bit_cast(unsigned, h);
    }
    if constexpr (PK) {
      const f16x2 z = {(_Float16)0.0f, (_Float16)0.0f};
      u = __builtin_bit_cast(unsigned, __builtin_elementwise_max(__builtin_bit_cast(f16x2, u), z));
    }
    return u;
  }
  static __device__ __forceinline__ void unpack2(unsigned u, float &x, float &y) {
    if constexpr (DT == DT_F16) {
      x = (float)__builtin_bit_cast(_Float16, (unsigned short)(u & 0xffffu));
      y = (float)__builtin_bit_cast(_Float16, (unsigned short)(u >> 16));
    } else {
      x = __builtin_bit_cast(float, u << 16);
      y = __builtin_bit_cast(float, u & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ f32x4 finish(f32x4 v, f32x4 a, f32x4 b, const float (&r)[4]) {
    if constexpr (AFF) v = v * a + b;
    if constexpr (RELU1_F32) {
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = fmaxf(0.0f, v[e]);
    }
    if constexpr (RES) {
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] += r[e];
    }
    if constexpr (RELU2_F32) {
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = fmaxf(0.0f, v[e]);
    }
    return v;
  }
  // One pixel block x two filter blocks fa, fb (accumulators acc_a, acc_b): after the swap the lanes of
  // 16-lane group q hold channels (q>>1)*8 .. +7 of block (q&1 ? fb : fa), one 16-byte store per lane.
  // ta/tb: the affine operands of the lane's four channels per block; prow: the pixel's row in the tile's
  // output (and residual) window, < 0 for a pixel outside the tile; row_c/row_r: row pitches in bytes.
  // pair_offset: the lane's byte offset into that window (output or residual alike, by the pitch).
  static __device__ __forceinline__ int pair_offset(int fa, int fb, int prow, int q, int pitch) {
    const int ch = ((q & 1) ? fb : fa) * 16 + (q >> 1) * 8;
    return prow >= 0 ? prow * pitch + ch * 2 : (int)OOB;
  }
  // (the residual's 16 bytes of the lane, as pair_block's store would write them; zeros without a residual
  // buffer.  A kernel with registers to spare asks for them in front of its main loop and hands them to
  // pair_block_with: fetched in the epilogue they are a round trip to memory with nothing left to hide it.)
  static __device__ __forceinline__ u32x4 fetch_pair_residual(int fa, int fb, int prow, int q, __amdgpu_buffer_rsrc_t rsrc_r,
                                                              int row_r) {
    return __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_r, pair_offset(fa, fb, prow, q, row_r), 0, 0));
  }
  static __device__ __forceinline__ void pair_block_with(f32x4 acc_a, f32x4 acc_b, int fa, int fb, f32x4 ta_a, f32x4 tb_a,
                                                         f32x4 ta_b, f32x4 tb_b, int prow, int q, __amdgpu_buffer_rsrc_t rsrc_c,
                                                         int row_c, u32x4 r8) {
    float ra[4] = {0, 0, 0, 0}, rb[4] = {0, 0, 0, 0};
    if constexpr (RES) {
      unsigned r0 = r8[0], r1 = r8[1], r2 = r8[2], r3 = r8[3];
      asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %2\n\tv_permlane16_swap_b32 %1, %3"
                   : "+v"(r0), "+v"(r1), "+v"(r2), "+v"(r3));
      unpack2(r0, ra[0], ra[1]);
      unpack2(r1, ra[2], ra[3]);
      unpack2(r2, rb[0], rb[1]);
      unpack2(r3, rb[2], rb[3]);
    }
    const f32x4 va = finish(acc_a, ta_a, tb_a, ra);
    const f32x4 vb = finish(acc_b, ta_b, tb_b, rb);
    unsigned a_lo = pack2(va[0], va[1]), a_hi = pack2(va[2], va[3]);
    unsigned b_lo = pack2(vb[0], vb[1]), b_hi = pack2(vb[2], vb[3]);
    // (as instructions: the compiler's builtin for the swap returns its first result twice; the s_nop is the
    // wait the hardware asks for between a vector-ALU write of an operand and the swap)
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %2\n\tv_permlane16_swap_b32 %1, %3"
                 : "+v"(a_lo), "+v"(a_hi), "+v"(b_lo), "+v"(b_hi));
    const u32x4 row8 = {a_lo, a_hi, b_lo, b_hi};
    __builtin_amdgcn_raw_buffer_store_b128(row8, rsrc_c, pair_offset(fa, fb, prow, q, row_c), 0, 0);
  }
  static __device__ __forceinline__ void pair_block(f32x4 acc_a, f32x4 acc_b, int fa, int fb, f32x4 ta_a, f32x4 tb_a, f32x4 ta_b,
                                                    f32x4 tb_b, int prow, int q, __amdgpu_buffer_rsrc_t rsrc_c,
                                                    __amdgpu_buffer_rsrc_t rsrc_r, int row_c, int row_r) {
    u32x4 r8 = {0u, 0u, 0u, 0u};
    if constexpr (RES) r8 = fetch_pair_residual(fa, fb, prow, q, rsrc_r, row_r);
    pair_block_with(acc_a, acc_b, fa, fb, ta_a, tb_a, ta_b, tb_b, prow, q, rsrc_c, row_c, r8);
  }
  // One pixel block x 64 filters: acc[i] the accumulators of filter block fb[i]; fb[2j] and fb[2j+1] share a store.
  static __device__ __forceinline__ void pixel_block(const f32x4 (&acc)[4], const int (&fb)[4], const f32x4 (&ta)[4],
                                                     const f32x4 (&tb)[4], int prow, int q, __amdgpu_buffer_rsrc_t rsrc_c,
                                                     __amdgpu_buffer_rsrc_t rsrc_r, int row_c, int row_r) {
#pragma unroll
    for (int j = 0; j < 2; ++j)
      pair_block(acc[2 * j], acc[2 * j + 1], fb[2 * j], fb[2 * j + 1], ta[2 * j], tb[2 * j], ta[2 * j + 1], tb[2 * j + 1], prow, q, rsrc_c,
                 rsrc_r, row_c, row_r);
  }
  // (the same with the residual's two 16-byte pieces already in registers: res[j] = fetch_pair_residual of pair j)
  static __device__ __forceinline__ void pixel_block_with(const f32x4 (&acc)[4], const int (&fb)[4], const f32x4 (&ta)[4],
                                                          const f32x4 (&tb)[4], int prow, int q, __amdgpu_buffer_rsrc_t rsrc_c,
                                                          int row_c, const u32x4 (&res)[2]) {
#pragma unroll
    for (int j = 0; j < 2; ++j)
      pair_block_with(acc[2 * j], acc[2 * j + 1], fb[2 * j], fb[2 * j + 1], ta[2 * j], tb[2 * j], ta[2 * j + 1], tb[2 * j + 1], prow, q,
                      rsrc_c, row_c, res[j]);
  }
  // One pixel block x one filter block (channels ch .. ch+3 of the lane): 8 bytes per lane.
  static __device__ __forceinline__ u32x2 fetch_single_residual(int ch, int prow, __amdgpu_buffer_rsrc_t rsrc_r, int row_r) {
    return __builtin_bit_cast(u32x2,
                              __builtin_amdgcn_raw_buffer_load_b64(rsrc_r, prow >= 0 ? prow * row_r + ch * 2 : (int)OOB, 0, 0));
  }
  static __device__ __forceinline__ void single_block_with(f32x4 acc, f32x4 ta, f32x4 tb, int ch, int prow,
                                                           __amdgpu_buffer_rsrc_t rsrc_c, int row_c, u32x2 r4) {
    float rr[4] = {0, 0, 0, 0};
    if constexpr (RES) {
      unpack2(r4[0], rr[0], rr[1]);
      unpack2(r4[1], rr[2], rr[3]);
    }
    const f32x4 v = finish(acc, ta, tb, rr);
    const u32x2 o = {pack2(v[0], v[1]), pack2(v[2], v[3])};
    __builtin_amdgcn_raw_buffer_store_b64(o, rsrc_c, prow >= 0 ? prow * row_c + ch * 2 : (int)OOB, 0, 0);
  }
  static __device__ __forceinline__ void single_block(f32x4 acc, f32x4 ta, f32x4 tb, int ch, int prow,
                                                      __amdgpu_buffer_rsrc_t rsrc_c, __amdgpu_buffer_rsrc_t rsrc_r, int row_c,
                                                      int row_r) {
    u32x2 r4 = {0u, 0u};
    if constexpr (RES) r4 = fetch_single_residual(ch, prow, rsrc_r, row_r);
    single_block_with(acc, ta, tb, ch, prow, rsrc_c, row_c, r4);
  }
};

// switch (sig) over the 16 forms: BODY(F) with F a compile-time constant
#define TRACEA_EPILOGUE16_FORMS(sig, BODY)                                                                              \
  switch (sig) {                                                                                                        \
    case 0: BODY(0); break;  case 1: BODY(1); break;  case 2: BODY(2); break;  case 3: BODY(3); break;                  \
    case 4: BODY(4); break;  case 5: BODY(5); break;  case 6: BODY(6); break;  case 7: BODY(7); break;                  \
    case 8: BODY(8); break;  case 9: BODY(9); break;  case 10: BODY(10); break; case 11: BODY(11); break;               \
    case 12: BODY(12); break; case 13: BODY(13); break; case 14: BODY(14); break; case 15: BODY(15); break;             \
    default: break;                                                                                                     \
  }

}  // namespace tracea_amd
