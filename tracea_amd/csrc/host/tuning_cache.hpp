// Persistent tuning cache: key -> {config, score, timestamp}, stored as pretty
// JSON in .tracea/tuning_cache_v2.json (same path, key strings and entry layout
// as the reference: src/core/tuning.rs:14-64, 66-78).
#pragma once
#include <string>

#include "pipeline_config.hpp"

namespace tracea_amd {

struct CacheEntry {
  PipelineConfig config;
  float score = 0.0f;  // TFLOP/s
  uint64_t timestamp = 0;
};

// Name of device 0 as the cache keys spell it ("" before tracea_init succeeds).
const char *tuning_device_name();

// Path of the cache file; TRACEA_TUNING_CACHE overrides the default.
std::string tuning_cache_path();

bool tuning_cache_get(const std::string &key, CacheEntry *out);
void tuning_cache_put(const std::string &key, const CacheEntry &e, bool persist);
// Drops the in-memory copy so that the next lookup re-reads the file.
void tuning_cache_reload();

// Index of the contraction variant a cached config names, or -1.
int tuning_cache_lookup_variant(const std::string &key);

// PipelineConfig <-> kernel variant
PipelineConfig config_for_contraction_variant(int index);
int contraction_variant_for_config(const PipelineConfig &c);
PipelineConfig config_for_attention_variant(int index);

}  // namespace tracea_amd
