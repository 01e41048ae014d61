// Table of the precompiled contraction kernel variants (one accessor per line
// of contraction_variants.def, each defined in its own translation unit).
#include "common.hpp"

namespace tracea_amd {

#define TRACEA_VARIANT(name, bm, bn, bk, wm, wn, stages, direct) \
  const ContractionVariant &contraction_variant_##name();
#include "contraction_variants.def"
#undef TRACEA_VARIANT

namespace {
typedef const ContractionVariant &(*Accessor)();
const Accessor kAccessors[] = {
#define TRACEA_VARIANT(name, bm, bn, bk, wm, wn, stages, direct) &contraction_variant_##name,
#include "contraction_variants.def"
#undef TRACEA_VARIANT
};
}  // namespace

int contraction_variant_count() { return (int)(sizeof(kAccessors) / sizeof(kAccessors[0])); }
const ContractionVariant &contraction_variant(int i) { return kAccessors[i](); }

}  // namespace tracea_amd
