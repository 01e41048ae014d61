// One member of the contraction kernel family per translation unit; the build
// compiles this file once per line of contraction_variants.def with
// -DV_NAME=... -DV_BM=... -DV_BN=... -DV_BK=... -DV_WM=... -DV_WN=... -DV_STAGES=... -DV_DIRECT=<pipeline mode>
#include "contraction_kernel.hpp"
#include "conv_patch_kernel.hpp"
#include "conv_resident_kernel.hpp"
#include "conv_wave16_kernel.hpp"
#include "conv_ksplit16_kernel.hpp"
#include "conv_thin8_kernel.hpp"

#define TRACEA_CAT2(a, b) a##b
#define TRACEA_CAT(a, b) TRACEA_CAT2(a, b)
#define TRACEA_STR2(a) #a
#define TRACEA_STR(a) TRACEA_STR2(a)

namespace tracea_amd {
// Host-side accessor (a function, so that nothing here is emitted for the device).
const ContractionVariant &TRACEA_CAT(contraction_variant_, V_NAME)() {
  static const ContractionVariant v = {
      TRACEA_STR(V_NAME), V_BM, V_BN, V_BK, V_WM, V_WN, V_STAGES, (V_DIRECT == 6 ? 2 : V_DIRECT),
#if V_DIRECT == 4
      (size_t)V_STAGES * V_BN * V_BK * 2,  // filter ring only; the patch size depends on the problem
      &launch_conv_patch<V_BM, V_BN, V_WM, V_WN, V_STAGES>, 32};
#elif V_DIRECT == 5
      (size_t)rs_filter_bytes(V_STAGES) + RS_TABLE_BYTES,  // the patch, sized by the problem, comes on top
      &launch_conv_resident<V_STAGES, 4>, 32};  // 64 input channels: 4 k-steps per tap
#elif V_DIRECT == 7
      (size_t)CW_TABLE_BYTES,  // patch and filter slab, sized by the problem, come on top
      &launch_conv_wave16<V_BK, (V_BM / 16 - 1) / V_WM, 0, V_WM>, 16};  // waves_m multiplying waves
#elif V_DIRECT == 8
      (size_t)V_STAGES * cw_ring_stage_bytes(V_BK) + CW_TABLE_BYTES,  // the patch comes on top
      &launch_conv_wave16<V_BK, (V_BM / 16 - 1) / 4, V_STAGES>, 16};
#elif V_DIRECT == 9
      (size_t)V_STAGES * CK_STAGE_BYTES + CK_TABLE_BYTES,  // the patch comes on top
      &launch_conv_ksplit16<V_BK, V_BM / 16, V_STAGES>, 16};
#elif V_DIRECT == 10
      (size_t)CT_TABLE_BYTES,  // the patch, sized by the problem, comes on top
      &launch_conv_thin8<V_STAGES>, 16};
#elif V_DIRECT == 6
      (size_t)V_STAGES * (V_BM + V_BN) * V_BK * 2,
      &launch_contraction<V_BM, V_BN, V_BK, V_WM, V_WN, V_STAGES, 2, 16>, 16};  // pipeline 2 on 16x16x32 MFMAs
#else
      (size_t)V_STAGES * (V_BM + V_BN) * V_BK * 2,
      &launch_contraction<V_BM, V_BN, V_BK, V_WM, V_WN, V_STAGES, V_DIRECT>, 32};
#endif
  return v;
}
}  // namespace tracea_amd
