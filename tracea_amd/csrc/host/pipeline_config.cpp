#include "pipeline_config.hpp"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>

namespace tracea_amd {

// ---- Json ---------------------------------------------------------------------
const Json *Json::find(const std::string &key) const {
  if (type != Object) return nullptr;
  for (const auto &kv : obj)
    if (kv.first == key) return &kv.second;
  return nullptr;
}

void Json::set(const std::string &key, const Json &v) {
  type = Object;
  for (auto &kv : obj)
    if (kv.first == key) {
      kv.second = v;
      return;
    }
  obj.emplace_back(key, v);
}

static void dump_string(const std::string &s, std::string *out) {
  out->push_back('"');
  for (unsigned char c : s) {
    switch (c) {
      case '"': *out += "\\\""; break;
      case '\\': *out += "\\\\"; break;
      case '\n': *out += "\\n"; break;
      case '\r': *out += "\\r"; break;
      case '\t': *out += "\\t"; break;
      default:
        if (c < 0x20) {
          char buf[8];
          snprintf(buf, sizeof(buf), "\\u%04x", c);
          *out += buf;
        } else {
          out->push_back((char)c);
        }
    }
  }
  out->push_back('"');
}

std::string Json::dump(int indent, int depth) const {
  std::string out;
  const bool pretty = indent >= 0;
  auto newline = [&](int d) {
    if (!pretty) return;
    out.push_back('\n');
    out.append((size_t)(d * indent), ' ');
  };
  switch (type) {
    case Null: out = "null"; break;
    case Bool: out = b ? "true" : "false"; break;
    case Number: {
      char buf[40];
      if (std::isfinite(num) && num == std::floor(num) && std::fabs(num) < 9.0e15)
        snprintf(buf, sizeof(buf), "%lld", (long long)num);
      else if (std::isfinite(num))
        snprintf(buf, sizeof(buf), "%.9g", num);
      else
        snprintf(buf, sizeof(buf), "null");
      out = buf;
    } break;
    case String: dump_string(str, &out); break;
    case Array:
      out.push_back('[');
      for (size_t i = 0; i < arr.size(); ++i) {
        if (i) out.push_back(',');
        newline(depth + 1);
        out += arr[i].dump(indent, depth + 1);
      }
      if (!arr.empty()) newline(depth);
      out.push_back(']');
      break;
    case Object:
      out.push_back('{');
      for (size_t i = 0; i < obj.size(); ++i) {
        if (i) out.push_back(',');
        newline(depth + 1);
        dump_string(obj[i].first, &out);
        out += pretty ? ": " : ":";
        out += obj[i].second.dump(indent, depth + 1);
      }
      if (!obj.empty()) newline(depth);
      out.push_back('}');
      break;
  }
  return out;
}

namespace {
struct Parser {
  const std::string &s;
  size_t i = 0;
  std::string err;
  explicit Parser(const std::string &text) : s(text) {}
  void ws() {
    while (i < s.size() && (s[i] == ' ' || s[i] == '\n' || s[i] == '\t' || s[i] == '\r')) ++i;
  }
  bool fail(const char *m) {
    if (err.empty()) err = std::string(m) + " at offset " + std::to_string(i);
    return false;
  }
  bool parse_string(std::string *out) {
    if (i >= s.size() || s[i] != '"') return fail("expected string");
    ++i;
    out->clear();
    while (i < s.size() && s[i] != '"') {
      char c = s[i++];
      if (c == '\\') {
        if (i >= s.size()) return fail("bad escape");
        char e = s[i++];
        switch (e) {
          case 'n': out->push_back('\n'); break;
          case 't': out->push_back('\t'); break;
          case 'r': out->push_back('\r'); break;
          case 'b': out->push_back('\b'); break;
          case 'f': out->push_back('\f'); break;
          case 'u': {
            if (i + 4 > s.size()) return fail("bad \\u escape");
            unsigned cp = (unsigned)strtoul(s.substr(i, 4).c_str(), nullptr, 16);
            i += 4;
            if (cp < 0x80) out->push_back((char)cp);
            else if (cp < 0x800) {
              out->push_back((char)(0xC0 | (cp >> 6)));
              out->push_back((char)(0x80 | (cp & 0x3F)));
            } else {
              out->push_back((char)(0xE0 | (cp >> 12)));
              out->push_back((char)(0x80 | ((cp >> 6) & 0x3F)));
              out->push_back((char)(0x80 | (cp & 0x3F)));
            }
          } break;
          default: out->push_back(e);
        }
      } else {
        out->push_back(c);
      }
    }
    if (i >= s.size()) return fail("unterminated string");
    ++i;
    return true;
  }
  bool parse_value(Json *out, int depth) {
    if (depth > 64) return fail("nesting too deep");
    ws();
    if (i >= s.size()) return fail("unexpected end");
    const char c = s[i];
    if (c == '{') {
      ++i;
      *out = Json::make_obj();
      ws();
      if (i < s.size() && s[i] == '}') { ++i; return true; }
      for (;;) {
        ws();
        std::string key;
        if (!parse_string(&key)) return false;
        ws();
        if (i >= s.size() || s[i] != ':') return fail("expected ':'");
        ++i;
        Json v;
        if (!parse_value(&v, depth + 1)) return false;
        out->obj.emplace_back(key, v);
        ws();
        if (i < s.size() && s[i] == ',') { ++i; continue; }
        if (i < s.size() && s[i] == '}') { ++i; return true; }
        return fail("expected ',' or '}'");
      }
    }
    if (c == '[') {
      ++i;
      *out = Json::make_arr();
      ws();
      if (i < s.size() && s[i] == ']') { ++i; return true; }
      for (;;) {
        Json v;
        if (!parse_value(&v, depth + 1)) return false;
        out->arr.push_back(v);
        ws();
        if (i < s.size() && s[i] == ',') { ++i; continue; }
        if (i < s.size() && s[i] == ']') { ++i; return true; }
        return fail("expected ',' or ']'");
      }
    }
    if (c == '"') {
      out->type = Json::String;
      return parse_string(&out->str);
    }
    if (s.compare(i, 4, "true") == 0) { i += 4; *out = Json::make_bool(true); return true; }
    if (s.compare(i, 5, "false") == 0) { i += 5; *out = Json::make_bool(false); return true; }
    if (s.compare(i, 4, "null") == 0) { i += 4; *out = Json::make_null(); return true; }
    char *end = nullptr;
    const double v = strtod(s.c_str() + i, &end);
    if (end == s.c_str() + i) return fail("unexpected character");
    i = (size_t)(end - s.c_str());
    *out = Json::make_num(v);
    return true;
  }
};
}  // namespace

bool Json::parse(const std::string &text, Json *out, std::string *err) {
  Parser p(text);
  if (!p.parse_value(out, 0)) {
    if (err) *err = p.err;
    return false;
  }
  p.ws();
  if (p.i != text.size()) {
    if (err) *err = "trailing characters at offset " + std::to_string(p.i);
    return false;
  }
  return true;
}

// ---- PipelineConfig -----------------------------------------------------------
std::string PipelineConfig::validate() const {
  char buf[160];
  if (m_tile % 16 != 0) {
    snprintf(buf, sizeof(buf), "m_tile (%u) must be a multiple of 16", m_tile);
    return buf;
  }
  if (n_tile % 16 != 0) {
    snprintf(buf, sizeof(buf), "n_tile (%u) must be a multiple of 16", n_tile);
    return buf;
  }
  if (num_stages < 2) {
    snprintf(buf, sizeof(buf), "num_stages (%u) must be at least 2 to prevent pipeline hazards",
             num_stages);
    return buf;
  }
  if (k_tile < 16) {
    snprintf(buf, sizeof(buf), "k_tile (%u) must be at least 16", k_tile);
    return buf;
  }
  if (has_force_num_warps && (force_num_warps == 0 || force_num_warps > 32)) {
    snprintf(buf, sizeof(buf), "force_num_warps (%u) must be between 1 and 32", force_num_warps);
    return buf;
  }
  return "";
}

Json PipelineConfig::to_json_value() const {
  Json j = Json::make_obj();
  j.set("num_stages", Json::make_num(num_stages));
  j.set("m_tile", Json::make_num(m_tile));
  j.set("n_tile", Json::make_num(n_tile));
  j.set("k_tile", Json::make_num(k_tile));
  j.set("instruction", Json::make_str(instruction));
  j.set("swizzle_mode", Json::make_str(swizzle_mode));
  j.set("quantization", Json::make_str(quantization));
  j.set("layout_policy", has_layout_policy ? Json::make_str(layout_policy) : Json::make_null());
  j.set("epilogue", epilogue);
  j.set("force_num_warps", has_force_num_warps ? Json::make_num(force_num_warps) : Json::make_null());
  j.set("micro_m", Json::make_num(micro_m));
  j.set("micro_n", Json::make_num(micro_n));
  j.set("k_unroll", Json::make_num(k_unroll));
  j.set("prefetch_distance", Json::make_num(prefetch_distance));
  j.set("cp_async_distance", Json::make_num(cp_async_distance));
  j.set("barrier_mode", Json::make_str(barrier_mode));
  j.set("softmax_granularity", Json::make_str(softmax_granularity));
  j.set("intrinsic_shape", Json::make_str(intrinsic_shape));
  j.set("vectorize_epilogue", Json::make_bool(vectorize_epilogue));
  j.set("ttg_enabled", Json::make_bool(ttg_enabled));
  j.set("attention_variant", Json::make_str(attention_variant));
  j.set("gemm_variant", Json::make_str(gemm_variant));
  j.set("double_buffer", Json::make_bool(double_buffer));
  j.set("register_strategy", Json::make_str(register_strategy));
  j.set("bank_conflict_padding", Json::make_num(bank_conflict_padding));
  j.set("fusion_count", Json::make_num(fusion_count));
  return j;
}

namespace {
bool get_u32(const Json &j, const char *key, uint32_t *out, std::string *err) {
  const Json *v = j.find(key);
  if (!v) return true;
  if (v->type != Json::Number || v->num < 0 || v->num > 4294967295.0 || v->num != std::floor(v->num)) {
    if (err) *err = std::string("field ") + key + " must be an unsigned integer";
    return false;
  }
  *out = (uint32_t)v->num;
  return true;
}
bool get_str(const Json &j, const char *key, std::string *out, std::string *err) {
  const Json *v = j.find(key);
  if (!v) return true;
  if (v->type != Json::String) {
    if (err) *err = std::string("field ") + key + " must be a string";
    return false;
  }
  *out = v->str;
  return true;
}
bool get_bool(const Json &j, const char *key, bool *out, std::string *err) {
  const Json *v = j.find(key);
  if (!v) return true;
  if (v->type != Json::Bool) {
    if (err) *err = std::string("field ") + key + " must be a boolean";
    return false;
  }
  *out = v->b;
  return true;
}
}  // namespace

bool PipelineConfig::from_json_value(const Json &j, PipelineConfig *out, std::string *err) {
  if (j.type != Json::Object) {
    if (err) *err = "PipelineConfig must be a JSON object";
    return false;
  }
  PipelineConfig c;
  bool ok = get_u32(j, "num_stages", &c.num_stages, err) && get_u32(j, "m_tile", &c.m_tile, err) &&
            get_u32(j, "n_tile", &c.n_tile, err) && get_u32(j, "k_tile", &c.k_tile, err) &&
            get_str(j, "instruction", &c.instruction, err) &&
            get_str(j, "swizzle_mode", &c.swizzle_mode, err) &&
            get_str(j, "quantization", &c.quantization, err) &&
            get_u32(j, "micro_m", &c.micro_m, err) && get_u32(j, "micro_n", &c.micro_n, err) &&
            get_u32(j, "k_unroll", &c.k_unroll, err) &&
            get_u32(j, "prefetch_distance", &c.prefetch_distance, err) &&
            get_u32(j, "cp_async_distance", &c.cp_async_distance, err) &&
            get_str(j, "barrier_mode", &c.barrier_mode, err) &&
            get_str(j, "softmax_granularity", &c.softmax_granularity, err) &&
            get_str(j, "intrinsic_shape", &c.intrinsic_shape, err) &&
            get_bool(j, "vectorize_epilogue", &c.vectorize_epilogue, err) &&
            get_bool(j, "ttg_enabled", &c.ttg_enabled, err) &&
            get_str(j, "attention_variant", &c.attention_variant, err) &&
            get_str(j, "gemm_variant", &c.gemm_variant, err) &&
            get_bool(j, "double_buffer", &c.double_buffer, err) &&
            get_str(j, "register_strategy", &c.register_strategy, err) &&
            get_u32(j, "bank_conflict_padding", &c.bank_conflict_padding, err) &&
            get_u32(j, "fusion_count", &c.fusion_count, err);
  if (!ok) return false;
  if (const Json *lp = j.find("layout_policy")) {
    if (lp->type == Json::Null) c.has_layout_policy = false;
    else if (lp->type == Json::String) { c.has_layout_policy = true; c.layout_policy = lp->str; }
    else { if (err) *err = "field layout_policy must be a string or null"; return false; }
  }
  if (const Json *fw = j.find("force_num_warps")) {
    if (fw->type == Json::Null) c.has_force_num_warps = false;
    else if (fw->type == Json::Number && fw->num >= 0) { c.has_force_num_warps = true; c.force_num_warps = (uint32_t)fw->num; }
    else { if (err) *err = "field force_num_warps must be an unsigned integer or null"; return false; }
  }
  if (const Json *ep = j.find("epilogue")) {
    if (ep->type != Json::Array) { if (err) *err = "field epilogue must be an array"; return false; }
    c.epilogue = *ep;
  }
  *out = c;
  return true;
}

bool PipelineConfig::from_json(const std::string &text, PipelineConfig *out, std::string *err) {
  Json j;
  if (!Json::parse(text, &j, err)) return false;
  return from_json_value(j, out, err);
}

static void flatten(const Json &v, std::vector<float> *out) {
  switch (v.type) {
    case Json::Number: out->push_back((float)v.num); break;
    case Json::Bool: out->push_back(v.b ? 1.0f : 0.0f); break;
    case Json::Array:
      for (const Json &e : v.arr) flatten(e, out);
      break;
    case Json::Object: {
      std::vector<const std::pair<std::string, Json> *> items;
      for (const auto &kv : v.obj) items.push_back(&kv);
      std::sort(items.begin(), items.end(),
                [](const std::pair<std::string, Json> *a, const std::pair<std::string, Json> *b) {
                  return a->first < b->first;
                });
      for (const auto *kv : items) flatten(kv->second, out);
    } break;
    default: out->push_back(0.0f);
  }
}

std::vector<float> PipelineConfig::to_vector() const {
  std::vector<float> v;
  flatten(to_json_value(), &v);
  return v;
}

}  // namespace tracea_amd
