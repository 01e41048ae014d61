// Persistent tuning cache: key -> {config, score, timestamp}, stored as pretty
// JSON in .tracea/tuning_cache_v2.json (same path, key strings and entry layout
// as the reference: src/core/tuning.rs:14-64, 66-78).
#pragma once
#include <string>

#include "../common.hpp"
#include "pipeline_config.hpp"

namespace tracea_amd {

struct CacheEntry {
  PipelineConfig config;
  float score = 0.0f;  // TFLOP/s
  uint64_t timestamp = 0;
  // What the record was measured on.  The reference's keys (gemm_{m}_{n}_{k}_{dev}, src/core/tuning.rs:14-34)
  // carry neither the element type nor the layout of B, so a record of one would steer calls with the other:
  // the two are kept inside the entry (additional fields, ignored by a reader that does not know them) and a
  // lookup for other operands skips the record.  Empty (a record written without them, e.g. by the reference):
  // f16 with a K-contiguous B, which is what every tuner of this path measures.
  std::string operand_dtype;  // "f16" | "bf16"
  std::string b_layout;       // "k_contiguous" | "n_contiguous"
  bool matches(int dtype, bool b_ncontig) const {
    const std::string d = operand_dtype.empty() ? "f16" : operand_dtype;
    const std::string l = b_layout.empty() ? "k_contiguous" : b_layout;
    return d == (dtype == DT_BF16 ? "bf16" : "f16") && l == (b_ncontig ? "n_contiguous" : "k_contiguous");
  }
};

// Name of device 0 as the cache keys spell it ("" before tracea_init succeeds).
const char *tuning_device_name();

// Path of the cache file; TRACEA_TUNING_CACHE overrides the default.
std::string tuning_cache_path();

bool tuning_cache_get(const std::string &key, CacheEntry *out);
void tuning_cache_put(const std::string &key, const CacheEntry &e, bool persist);
// Drops the in-memory copy so that the next lookup re-reads the file.
void tuning_cache_reload();

// Tuning history (src/optimizer/history.rs:7-51): key -> {backend, config, tflops, timestamp, explanation}
// in tuning_history.json (TRACEA_TUNING_HISTORY overrides the path).
struct HistoryEntry {
  std::string backend = "Rocm";
  PipelineConfig config;
  float tflops = 0.0f;
  uint64_t timestamp = 0;
  std::string explanation;
};
std::string tuning_history_path();
std::string tuning_history_explanation(const std::string &backend, float tflops, const std::string &reason);
bool tuning_history_query(const std::string &key, HistoryEntry *out);
void tuning_history_record(const std::string &key, const HistoryEntry &e);
void tuning_history_reload();

// Index of the contraction variant a cached config names, or -1; a record measured on other operands
// (element type, layout of B) than the caller's does not count.
int tuning_cache_lookup_variant(const std::string &key, int dtype = DT_F16, bool b_ncontig = false);

// PipelineConfig <-> kernel variant
PipelineConfig config_for_contraction_variant(int index);
int contraction_variant_for_config(const PipelineConfig &c);
PipelineConfig config_for_attention_variant(int index);
// First attention variant with the config's queries per workgroup, wave count, ring depth and MFMA shape that is
// feasible for `a`, or -1; and the variant a cached record of the problem names (key of the reference's attention
// adapter, src/kernels/attention/cuda_adapter.rs), or -1.
int attention_variant_for_config(const PipelineConfig &c, const AttentionArgs &a);
int tuning_cache_lookup_attention(const AttentionArgs &a);
std::string attention_cache_key(size_t b, size_t s, size_t h, size_t d, bool causal);

}  // namespace tracea_amd
