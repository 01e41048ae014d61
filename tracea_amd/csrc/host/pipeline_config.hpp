// PipelineConfig: the tuning record and its JSON wire format.
// C++ mirror of the reference's struct (src/core/config.rs:297-340): same field
// names, same order, enum fields serialised as the reference's variant names,
// so that a tuning cache written here parses there and vice versa.
// validate() reproduces src/core/config.rs:376-396.
#pragma once
#include <cstdint>
#include <map>
#include <string>
#include <vector>

namespace tracea_amd {

// Minimal JSON value (objects keep insertion order for stable output).
struct Json {
  enum Type { Null, Bool, Number, String, Array, Object } type = Null;
  bool b = false;
  double num = 0.0;
  std::string str;
  std::vector<Json> arr;
  std::vector<std::pair<std::string, Json>> obj;

  static Json make_null() { return Json(); }
  static Json make_bool(bool v) { Json j; j.type = Bool; j.b = v; return j; }
  static Json make_num(double v) { Json j; j.type = Number; j.num = v; return j; }
  static Json make_str(const std::string &v) { Json j; j.type = String; j.str = v; return j; }
  static Json make_arr() { Json j; j.type = Array; return j; }
  static Json make_obj() { Json j; j.type = Object; return j; }

  const Json *find(const std::string &key) const;
  void set(const std::string &key, const Json &v);
  std::string dump(int indent = -1, int depth = 0) const;  // indent < 0: compact
  // Parses text; on failure returns false and sets *err.
  static bool parse(const std::string &text, Json *out, std::string *err);
};

struct PipelineConfig {
  uint32_t num_stages = 2;
  uint32_t m_tile = 64, n_tile = 64, k_tile = 32;
  std::string instruction = "None";       // SpecializedInstruction
  std::string swizzle_mode = "None";      // SwizzleMode
  std::string quantization = "None";      // QuantizationMode
  bool has_layout_policy = true;
  std::string layout_policy = "RowMajor"; // Option<LayoutPolicy>
  Json epilogue = Json::make_arr();       // Vec<EpilogueOp>, kept verbatim
  bool has_force_num_warps = false;
  uint32_t force_num_warps = 0;           // Option<u32>
  uint32_t micro_m = 1, micro_n = 1, k_unroll = 1;
  uint32_t prefetch_distance = 0, cp_async_distance = 0;
  std::string barrier_mode = "None";
  std::string softmax_granularity = "PerTile";
  std::string intrinsic_shape = "None";
  bool vectorize_epilogue = true;
  bool ttg_enabled = false;
  std::string attention_variant = "Naive";
  std::string gemm_variant = "Naive";
  bool double_buffer = false;
  std::string register_strategy = "Array";
  uint32_t bank_conflict_padding = 8;
  uint32_t fusion_count = 1;

  PipelineConfig() = default;
  // PipelineConfig::new(num_stages, m_tile, n_tile, k_tile)
  PipelineConfig(uint32_t stages, uint32_t mt, uint32_t nt, uint32_t kt)
      : num_stages(stages), m_tile(mt), n_tile(nt), k_tile(kt) {}

  // Empty string when valid, else the reference's message.
  std::string validate() const;
  Json to_json_value() const;
  std::string to_json() const { return to_json_value().dump(); }
  // Fields absent from the text keep their defaults (older cache files lack
  // the newer fields).  Returns false and sets *err on malformed input.
  static bool from_json_value(const Json &j, PipelineConfig *out, std::string *err);
  static bool from_json(const std::string &text, PipelineConfig *out, std::string *err);
  // Numeric feature vector: every number / bool of the JSON form in key-sorted
  // order, strings and null contributing 0 (src/core/config.rs:399-433).
  std::vector<float> to_vector() const;
};

}  // namespace tracea_amd
