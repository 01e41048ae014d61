// C++ convenience layer over the C ABI of include/tracea.h.
//
// Source-compatible with the wrapper half of the reference's include/tracea.hpp
// (namespace tracea: TensorView, Conv2dParams, ConvTranspose2dParams, GemmParams,
// AttentionParams, conv2d, conv_transpose2d, gemm, attention, get_last_error,
// version; reference lines 173-420): same type and member names, same default
// values, same exception type and message prefix.  Header-only; link against
// libtracea.so.
#pragma once

#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "tracea.h"

namespace tracea {

enum class DType : int {
  Float32 = TRACEA_DTYPE_FLOAT32,
  Float16 = TRACEA_DTYPE_FLOAT16,
  BFloat16 = TRACEA_DTYPE_BFLOAT16,
  Int32 = TRACEA_DTYPE_INT32,
  Int8 = TRACEA_DTYPE_INT8,
};

enum class EpilogueKind : int {
  Identity = TRACEA_EPILOGUE_IDENTITY,
  BiasAdd = TRACEA_EPILOGUE_BIAS_ADD,
  ReLU = TRACEA_EPILOGUE_RELU,
  Gelu = TRACEA_EPILOGUE_GELU,
  SiLU = TRACEA_EPILOGUE_SILU,
  BiasReLU = TRACEA_EPILOGUE_BIAS_RELU,
  BiasSiLU = TRACEA_EPILOGUE_BIAS_SILU,
  Residual = TRACEA_EPILOGUE_RESIDUAL,
  ResidualReLU = TRACEA_EPILOGUE_RESIDUAL_RELU,
};

enum class SoftmaxGranularity : int {
  Auto = TRACEA_SOFTMAX_AUTO,
  PerTile = TRACEA_SOFTMAX_PER_TILE,
  PerTwoTiles = TRACEA_SOFTMAX_PER_TWO_TILES,
};

// Borrowed view of a tensor.  Owns its shape/stride vectors, never the data.
// Strides are in elements; the two-argument-plus constructor fills in the
// contiguous row-major strides.  device_id -1 means host memory (which this
// library rejects), >= 0 a HIP device ordinal.
class TensorView {
 public:
  void *ptr = nullptr;
  std::vector<uint64_t> shape;
  std::vector<int64_t> stride;
  DType dtype = DType::Float32;
  int32_t device_id = -1;

  TensorView() = default;
  TensorView(void *data, std::vector<uint64_t> dims, DType type, int32_t device = -1)
      : ptr(data), shape(std::move(dims)), stride(shape.size(), 1), dtype(type), device_id(device) {
    int64_t run = 1;
    for (size_t i = shape.size(); i-- > 0;) {
      stride[i] = run;
      run *= static_cast<int64_t>(shape[i]);
    }
  }

  // The C struct borrows shape/stride from this object: keep it alive across the call.
  TraceaTensorView to_c() const {
    TraceaTensorView v;
    v.ptr = ptr;
    v.rank = static_cast<uint32_t>(shape.size());
    v.shape = shape.data();
    v.stride = stride.data();
    v.dtype = static_cast<TraceaDType>(dtype);
    v.device_id = device_id;
    return v;
  }
};

struct Conv2dParams {
  uint32_t stride_h = 1, stride_w = 1;
  uint32_t padding_h = 0, padding_w = 0;
  uint32_t dilation_h = 1, dilation_w = 1;
  uint32_t groups = 1;
  EpilogueKind epilogue = EpilogueKind::Identity;
  void *stream = nullptr;  // hipStream_t

  TraceaConv2dParams to_c() const {
    TraceaConv2dParams p;
    p.stride_h = stride_h; p.stride_w = stride_w;
    p.padding_h = padding_h; p.padding_w = padding_w;
    p.dilation_h = dilation_h; p.dilation_w = dilation_w;
    p.groups = groups;
    p.epilogue = static_cast<TraceaEpilogueKind>(epilogue);
    p.stream = stream;
    return p;
  }
};

struct ConvTranspose2dParams {
  uint32_t stride_h = 1, stride_w = 1;
  uint32_t padding_h = 0, padding_w = 0;
  uint32_t output_padding_h = 0, output_padding_w = 0;
  uint32_t dilation_h = 1, dilation_w = 1;
  uint32_t groups = 1;
  EpilogueKind epilogue = EpilogueKind::Identity;
  void *stream = nullptr;

  TraceaConvTranspose2dParams to_c() const {
    TraceaConvTranspose2dParams p;
    p.stride_h = stride_h; p.stride_w = stride_w;
    p.padding_h = padding_h; p.padding_w = padding_w;
    p.output_padding_h = output_padding_h; p.output_padding_w = output_padding_w;
    p.dilation_h = dilation_h; p.dilation_w = dilation_w;
    p.groups = groups;
    p.epilogue = static_cast<TraceaEpilogueKind>(epilogue);
    p.stream = stream;
    return p;
  }
};

struct GemmParams {
  EpilogueKind epilogue = EpilogueKind::Identity;
  void *stream = nullptr;
  TraceaGemmParams to_c() const {
    TraceaGemmParams p;
    p.epilogue = static_cast<TraceaEpilogueKind>(epilogue);
    p.stream = stream;
    return p;
  }
};

struct AttentionParams {
  bool causal = true;
  SoftmaxGranularity softmax_mode = SoftmaxGranularity::Auto;
  float scale = 0.0f;  // 0 selects 1/sqrt(head dim)
  void *stream = nullptr;
  TraceaAttentionParams to_c() const {
    TraceaAttentionParams p;
    p.causal = causal ? 1 : 0;
    p.softmax_mode = static_cast<TraceaSoftmaxGranularity>(softmax_mode);
    p.scale = scale;
    p.stream = stream;
    return p;
  }
};

inline std::string get_last_error() {
  uint8_t text[1024];
  const int32_t n = tracea_get_last_error(text, sizeof(text));
  return n > 0 ? std::string(reinterpret_cast<const char *>(text), static_cast<size_t>(n)) : std::string();
}

namespace detail {
// A nullable TraceaTensorView* built from a nullable TensorView*.
struct OptionalView {
  TraceaTensorView storage;
  const TraceaTensorView *ptr = nullptr;
  explicit OptionalView(const TensorView *v) {
    if (v != nullptr) {
      storage = v->to_c();
      ptr = &storage;
    }
  }
};
inline void require_success(TraceaStatus st, const char *what) {
  if (st != TRACEA_SUCCESS) throw std::runtime_error(std::string(what) + " failed: " + get_last_error());
}
}  // namespace detail

// x [N,H,W,C], w [K,R,S,C], out [N,Ho,Wo,K]; b / residual may be nullptr.
// Throws std::runtime_error("tracea::conv2d failed: <last error>") on failure.
inline void conv2d(const TensorView &x, const TensorView &w, const TensorView *b,
                   const TensorView *residual, TensorView &out, const Conv2dParams &params) {
  detail::OptionalView bias(b), res(residual);
  TraceaTensorView o = out.to_c();
  detail::require_success(tracea_conv2d(x.to_c(), w.to_c(), bias.ptr, res.ptr, &o, params.to_c()),
                          "tracea::conv2d");
}

inline void conv_transpose2d(const TensorView &x, const TensorView &w, const TensorView *b,
                             const TensorView *residual, TensorView &out,
                             const ConvTranspose2dParams &params) {
  detail::OptionalView bias(b), res(residual);
  TraceaTensorView o = out.to_c();
  detail::require_success(
      tracea_conv_transpose2d(x.to_c(), w.to_c(), bias.ptr, res.ptr, &o, params.to_c()),
      "tracea::conv_transpose2d");
}

// c [M,N] = epilogue(a [M,K] . b [K,N])
inline void gemm(const TensorView &a, const TensorView &b, const TensorView *bias,
                 const TensorView *residual, TensorView &c, const GemmParams &params) {
  detail::OptionalView bv(bias), res(residual);
  TraceaTensorView o = c.to_c();
  detail::require_success(tracea_gemm(a.to_c(), b.to_c(), bv.ptr, res.ptr, &o, params.to_c()),
                          "tracea::gemm");
}

// q, k, v, o [B,H,S,D]
inline void attention(const TensorView &q, const TensorView &k, const TensorView &v, TensorView &o,
                      const AttentionParams &params) {
  TraceaTensorView out = o.to_c();
  detail::require_success(tracea_attention(q.to_c(), k.to_c(), v.to_c(), &out, params.to_c()),
                          "tracea::attention");
}

inline std::string version() {
  return std::to_string(tracea_version_major()) + "." + std::to_string(tracea_version_minor()) + "." +
         std::to_string(tracea_version_patch());
}

}  // namespace tracea
