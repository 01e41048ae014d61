// Compile-and-link check of include/tracea.hpp against libtracea.so (host only, no GPU needed):
// exercises the wrapper types exactly as a caller of the reference's header would.
#include <cstdio>
#include <cstring>

#include "tracea.hpp"
#include "tracea_plan.h"
#include "tracea_ttg.h"

int main() {
  if (tracea::version() != "0.1.0") return 1;
  float buf[16] = {0};
  tracea::TensorView a(buf, {4, 4}, tracea::DType::Float32, -1);
  if (a.stride[0] != 4 || a.stride[1] != 1) return 2;
  tracea::TensorView c(buf, {4, 4}, tracea::DType::Float32, -1);
  tracea::GemmParams gp;
  bool threw = false;
  try {
    tracea::gemm(a, a, nullptr, nullptr, c, gp);  // no tracea_init -> must throw with the prefix
  } catch (const std::runtime_error &e) {
    threw = std::strncmp(e.what(), "tracea::gemm failed: ", 21) == 0;
  }
  if (!threw) return 3;
  tracea::Conv2dParams cp;
  if (cp.to_c().groups != 1 || cp.to_c().dilation_h != 1) return 4;
  tracea::AttentionParams ap;
  if (ap.to_c().causal != 1 || ap.to_c().scale != 0.0f) return 5;
  // tile lists are host-side objects until they are launched: usable without a device
  TraceaTtgLayout *lay = tracea_ttg_from_diagonal(256, 256, 256, 64, 64, 32);
  if (lay == nullptr || tracea_ttg_num_active_tiles(lay) != 4) return 6;
  TraceaTileMetadata recs[4];
  if (tracea_ttg_l2_table(lay, recs, 4) != 4 || recs[3].region_m != 3 || recs[3].region_n != 3 || recs[3].k_end != 256)
    return 7;
  tracea_ttg_destroy(lay);
  if (tracea_ttg_from_dense(256, 256, 256, 0, 64, 32) != nullptr) return 8;
  std::puts("tracea.hpp ok");
  return 0;
}
