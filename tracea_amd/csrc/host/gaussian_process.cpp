// HardwareProfile and the Gaussian-process surrogate of the tuner.
//
// The model is the reference's (src/optimizer/mod.rs:297-576): an ARD squared-
// exponential kernel exp(-d^2/2) over [shape features ++ flattened config ++
// tile ratios], unit signal variance, noise sigma^2 on the diagonal, and the
// roofline estimate as the prior mean.  Linear algebra is a dense Cholesky in
// double precision (the reference factors in f32 through nalgebra).
#include <algorithm>
#include <cmath>
#include <cstdio>

#include "tuner.hpp"

namespace tracea_amd {

// ---- HardwareProfile ---------------------------------------------------------------
HardwareProfile HardwareProfile::mi355x() {
  HardwareProfile p;
  p.name = "AMD Instinct MI355X";
  p.backend = "Rocm";
  p.shared_memory_per_block = 160 * 1024;
  p.max_registers_per_thread = 512;
  p.registers_per_sm = 4 * 128 * 1024;  // four SIMDs x 512 KB of 32-bit registers
  p.max_registers_per_block = 4 * 128 * 1024;
  p.max_warps_per_sm = 32;
  p.wavefront_size = 64;
  p.max_blocks_per_sm = 16;
  p.shared_memory_per_sm = 160 * 1024;
  p.has_specialized_units = true;
  p.supported_intrinsic_shapes = {"M32N32K2", "M16N16K4"};
  p.max_threadgroup_memory = 160 * 1024;
  p.preferred_tile_shape[0] = 256;
  p.preferred_tile_shape[1] = 256;
  p.preferred_tile_shape[2] = 64;
  p.simd_width = 64;
  p.peak_tflops_standard = 157.3f;
  p.peak_tflops_tensor = 2500.0f;
  p.mem_bw_gbps = 8000.0f;
  return p;
}

HardwareProfile HardwareProfile::rtx3070() {
  HardwareProfile p;
  p.name = "NVIDIA GeForce RTX 3070";
  p.backend = "Cuda";
  p.shared_memory_per_block = 48 * 1024;
  p.max_registers_per_thread = 255;
  p.registers_per_sm = 65536;
  p.max_registers_per_block = 65536;
  p.max_warps_per_sm = 48;
  p.wavefront_size = 32;
  p.max_blocks_per_sm = 16;
  p.shared_memory_per_sm = 100 * 1024;
  p.has_specialized_units = true;
  p.supported_intrinsic_shapes = {"M16N8K16"};
  p.preferred_tile_shape[0] = 128;
  p.preferred_tile_shape[1] = 128;
  p.preferred_tile_shape[2] = 32;
  p.simd_width = 32;
  p.peak_tflops_standard = 20.3f;
  p.peak_tflops_tensor = 40.6f;
  p.mem_bw_gbps = 448.0f;
  return p;
}

HardwareProfile HardwareProfile::mi250() {
  HardwareProfile p;
  p.name = "AMD Instinct MI250X";
  p.backend = "Rocm";
  p.shared_memory_per_block = 64 * 1024;
  p.max_registers_per_thread = 256;
  p.registers_per_sm = 163840;
  p.max_registers_per_block = 65536;
  p.max_warps_per_sm = 32;
  p.wavefront_size = 64;
  p.max_blocks_per_sm = 16;
  p.shared_memory_per_sm = 64 * 1024;
  p.has_specialized_units = true;
  p.supported_intrinsic_shapes = {"M32N32K2", "M16N16K4"};
  p.max_threadgroup_memory = 64 * 1024;
  p.preferred_tile_shape[0] = 256;
  p.preferred_tile_shape[1] = 128;
  p.preferred_tile_shape[2] = 16;
  p.simd_width = 64;
  p.peak_tflops_standard = 47.9f;
  p.peak_tflops_tensor = 383.0f;
  p.mem_bw_gbps = 1600.0f;
  return p;
}

HardwareProfile HardwareProfile::a100() {
  HardwareProfile p;
  p.name = "NVIDIA A100-SXM4-40GB";
  p.backend = "Cuda";
  p.shared_memory_per_block = 164 * 1024;
  p.max_registers_per_thread = 255;
  p.registers_per_sm = 65536;
  p.max_registers_per_block = 65536;
  p.max_warps_per_sm = 64;
  p.wavefront_size = 32;
  p.max_blocks_per_sm = 32;
  p.shared_memory_per_sm = 164 * 1024;
  p.has_specialized_units = true;
  p.supported_intrinsic_shapes = {"M16N8K16"};
  p.preferred_tile_shape[0] = 128;
  p.preferred_tile_shape[1] = 256;
  p.preferred_tile_shape[2] = 32;
  p.simd_width = 32;
  p.peak_tflops_standard = 19.5f;
  p.peak_tflops_tensor = 312.0f;
  p.mem_bw_gbps = 1555.0f;
  return p;
}

bool HardwareProfile::by_name(const std::string &name, HardwareProfile *out) {
  if (name == "mi355x") *out = mi355x();
  else if (name == "rtx3070") *out = rtx3070();
  else if (name == "mi250") *out = mi250();
  else if (name == "a100") *out = a100();
  else return false;
  return true;
}

size_t estimate_smem_usage(const PipelineConfig &c) {
  const uint32_t tile_bytes = (c.m_tile * c.k_tile + c.k_tile * c.n_tile) * 2u;
  return (size_t)(tile_bytes * c.num_stages);
}

float HardwareProfile::estimate_occupancy(const PipelineConfig &c) const {
  const uint32_t warps_per_block = c.has_force_num_warps ? c.force_num_warps : 4u;
  if (warps_per_block == 0) return 0.0f;
  const uint32_t blocks_by_warps = max_warps_per_sm / warps_per_block;
  const float thread_count = (float)(warps_per_block * wavefront_size);
  const float tile_elements = (float)(c.m_tile * c.n_tile);
  uint32_t est_regs = 32;
  if (c.instruction == "CudaMMA" || c.instruction == "RocmMFMA") {
    const float load_regs = (tile_elements * (float)c.num_stages) / thread_count;
    est_regs = (uint32_t)(load_regs + 32.0f);
  }
  est_regs = std::min(est_regs, max_registers_per_thread);
  const uint32_t regs_per_block = warps_per_block * wavefront_size * est_regs;
  const uint32_t blocks_by_regs =
      (registers_per_sm > 0 && regs_per_block > 0) ? registers_per_sm / regs_per_block : max_blocks_per_sm;
  const uint32_t blocks = std::min(std::min(blocks_by_warps, blocks_by_regs), max_blocks_per_sm);
  return blocks == 0 ? 0.0f : (float)blocks / (float)max_blocks_per_sm;
}

std::string HardwareProfile::check_feasibility(const PipelineConfig &c, uint64_t m) const {
  if (estimate_smem_usage(c) > shared_memory_per_block) return "SharedMemoryOverflow";
  const float occ = estimate_occupancy(c);
  if (occ < 0.05f) {
    char buf[48];
    snprintf(buf, sizeof(buf), "LowOccupancy(%u)", (unsigned)(occ * 1000.0f));
    return buf;
  }
  if (m > 1024 && c.m_tile < 16) return "ForbiddenZone(\"Excessive tile-overhead for large M\")";
  if (c.num_stages > 8) return "ForbiddenZone(\"Unstable pipeline depth (>8 stages)\")";
  return std::string();
}

Json HardwareProfile::to_json_value() const {
  Json j = Json::make_obj();
  j.set("name", Json::make_str(name));
  j.set("backend", Json::make_str(backend));
  j.set("shared_memory_per_block", Json::make_num((double)shared_memory_per_block));
  j.set("max_registers_per_thread", Json::make_num(max_registers_per_thread));
  j.set("registers_per_sm", Json::make_num(registers_per_sm));
  j.set("max_registers_per_block", Json::make_num(max_registers_per_block));
  j.set("max_warps_per_sm", Json::make_num(max_warps_per_sm));
  j.set("wavefront_size", Json::make_num(wavefront_size));
  j.set("max_blocks_per_sm", Json::make_num(max_blocks_per_sm));
  j.set("shared_memory_per_sm", Json::make_num((double)shared_memory_per_sm));
  j.set("has_specialized_units", Json::make_bool(has_specialized_units));
  Json shapes = Json::make_arr();
  for (const auto &s : supported_intrinsic_shapes) shapes.arr.push_back(Json::make_str(s));
  j.set("supported_intrinsic_shapes", shapes);
  j.set("max_threadgroup_memory", Json::make_num((double)max_threadgroup_memory));
  Json tile = Json::make_arr();
  for (uint32_t t : preferred_tile_shape) tile.arr.push_back(Json::make_num(t));
  j.set("preferred_tile_shape", tile);
  j.set("simd_width", Json::make_num(simd_width));
  j.set("peak_tflops_standard", Json::make_num(peak_tflops_standard));
  j.set("peak_tflops_tensor", Json::make_num(peak_tflops_tensor));
  j.set("mem_bw_gbps", Json::make_num(mem_bw_gbps));
  return j;
}

void TuningStats::log_pruning(const std::string &reason) {
  pruned_count += 1;
  pruning_reasons[reason] += 1;
}

// ---- GaussianProcess ---------------------------------------------------------------
namespace {

// In-place lower Cholesky of the n x n row-major matrix; false when a pivot is
// not positive.
bool cholesky(std::vector<double> *a, size_t n) {
  std::vector<double> &m = *a;
  for (size_t j = 0; j < n; ++j) {
    double d = m[j * n + j];
    for (size_t p = 0; p < j; ++p) d -= m[j * n + p] * m[j * n + p];
    if (!(d > 0.0)) return false;
    const double l = std::sqrt(d);
    m[j * n + j] = l;
    for (size_t i = j + 1; i < n; ++i) {
      double s = m[i * n + j];
      for (size_t p = 0; p < j; ++p) s -= m[i * n + p] * m[j * n + p];
      m[i * n + j] = s / l;
    }
    for (size_t i = 0; i < j; ++i) m[i * n + j] = 0.0;
  }
  return true;
}

// L x = b
std::vector<double> solve_lower(const std::vector<double> &l, size_t n, const std::vector<double> &b) {
  std::vector<double> x(n);
  for (size_t i = 0; i < n; ++i) {
    double s = b[i];
    for (size_t p = 0; p < i; ++p) s -= l[i * n + p] * x[p];
    x[i] = s / l[i * n + i];
  }
  return x;
}

// L^T x = b
std::vector<double> solve_upper_t(const std::vector<double> &l, size_t n, const std::vector<double> &b) {
  std::vector<double> x(n);
  for (size_t ii = n; ii-- > 0;) {
    double s = b[ii];
    for (size_t p = ii + 1; p < n; ++p) s -= l[p * n + ii] * x[p];
    x[ii] = s / l[ii * n + ii];
  }
  return x;
}

std::vector<float> config_features(const PipelineConfig &c, uint32_t m, uint32_t n, uint32_t k) {
  std::vector<float> v = c.to_vector();
  v.push_back((float)c.m_tile / (float)m);
  v.push_back((float)c.n_tile / (float)n);
  v.push_back((float)c.k_tile / (float)k);
  return v;
}

uint64_t splitmix64(uint64_t *state) {
  uint64_t z = (*state += 0x9E3779B97F4A7C15ull);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

}  // namespace

GaussianProcess::GaussianProcess() : length_scales(15, 1.0f) {}

std::vector<float> GaussianProcess::full_features(uint32_t m, uint32_t n, uint32_t k, const PipelineConfig &c) {
  std::vector<float> f = {std::log2((float)m), std::log2((float)n), std::log2((float)k),
                          (float)m / std::max((float)n, 1.0f), (float)n / std::max((float)k, 1.0f)};
  const std::vector<float> cf = config_features(c, m, n, k);
  f.insert(f.end(), cf.begin(), cf.end());
  return f;
}

float GaussianProcess::roofline_prior(uint32_t m, uint32_t n, uint32_t k, const PipelineConfig &c,
                                      const HardwareProfile &gpu) {
  const float peak = c.instruction != "None" ? gpu.peak_tflops_tensor : gpu.peak_tflops_standard;
  const double ops = 2.0 * (double)m * (double)n * (double)k;
  const double bytes = ((double)m * k + (double)k * n + (double)m * n) * 2.0;
  const float intensity = (float)(ops / bytes);
  const float bw_limit = gpu.mem_bw_gbps * intensity / 1000.0f;
  return std::min(peak, bw_limit);
}

// The scale vector is sized to the config features but indexed by position in
// the full vector, whose first five entries are the shape features; positions
// past its end use scale 1 (mod.rs:466-473, 317-321).
float GaussianProcess::ard_distance_sq(const std::vector<float> &a, const std::vector<float> &b) const {
  float d = 0.0f;
  const size_t n = std::min(a.size(), b.size());
  for (size_t i = 0; i < n; ++i) {
    const float ls = i < length_scales.size() ? length_scales[i] : 1.0f;
    const float diff = a[i] - b[i];
    d += diff * diff / (ls * ls);
  }
  return d;
}

void GaussianProcess::observe(const Observation &obs, const HardwareProfile &gpu) {
  if (observations.empty()) {
    const size_t nf = config_features(obs.config, obs.m, obs.n, obs.k).size();
    length_scales.assign(nf, 1.0f);
  }
  observations.push_back(obs);
  if (observations.size() % 5 == 0 && observations.size() > 5) optimize_hyperparams(gpu);
}

bool GaussianProcess::factor(const HardwareProfile &gpu, std::vector<std::vector<float>> *feats,
                             std::vector<double> *chol, std::vector<double> *diff) const {
  const size_t n = observations.size();
  feats->resize(n);
  diff->resize(n);
  for (size_t i = 0; i < n; ++i) {
    const Observation &o = observations[i];
    (*feats)[i] = full_features(o.m, o.n, o.k, o.config);
    (*diff)[i] = (double)o.score - (double)roofline_prior(o.m, o.n, o.k, o.config, gpu);
  }
  chol->assign(n * n, 0.0);
  const double noise = (double)noise_sigma * (double)noise_sigma;
  for (size_t i = 0; i < n; ++i)
    for (size_t j = 0; j <= i; ++j) {
      double kv = std::exp(-(double)ard_distance_sq((*feats)[i], (*feats)[j]) / 2.0);
      if (i == j) kv += noise;
      (*chol)[i * n + j] = kv;
      (*chol)[j * n + i] = kv;
    }
  return cholesky(chol, n);
}

float GaussianProcess::marginal_log_likelihood(const HardwareProfile &gpu) const {
  if (observations.empty()) return 0.0f;
  const size_t n = observations.size();
  std::vector<std::vector<float>> feats;
  std::vector<double> l, diff;
  if (!factor(gpu, &feats, &l, &diff)) return -1e9f;
  const std::vector<double> beta = solve_lower(l, n, diff);
  double t1 = 0.0, t2 = 0.0;
  for (size_t i = 0; i < n; ++i) {
    t1 += beta[i] * beta[i];
    t2 += std::log(l[i * n + i]);
  }
  const double t3 = -0.5 * (double)n * std::log(2.0 * M_PI);
  return (float)(-0.5 * t1 - t2 + t3);
}

void GaussianProcess::optimize_hyperparams(const HardwareProfile &gpu) {
  if (observations.size() < 3) return;
  const float lr = 0.1f;
  for (int it = 0; it < 10; ++it) {
    const float current = marginal_log_likelihood(gpu);
    for (size_t d = 0; d < length_scales.size(); ++d) {
      const float orig = length_scales[d];
      length_scales[d] = orig * (1.0f + lr);
      const float up = marginal_log_likelihood(gpu);
      length_scales[d] = orig * (1.0f - lr);
      const float down = marginal_log_likelihood(gpu);
      if (up > current && up > down) length_scales[d] = orig * (1.0f + lr);
      else if (down > current) length_scales[d] = orig * (1.0f - lr);
      else length_scales[d] = orig;
      length_scales[d] = std::min(std::max(length_scales[d], 0.1f), 10.0f);
    }
  }
}

void GaussianProcess::predict(uint32_t m, uint32_t n, uint32_t k, const PipelineConfig &c,
                              const HardwareProfile &gpu, float *mean, float *stddev) const {
  const float prior = roofline_prior(m, n, k, c, gpu);
  *mean = prior;
  *stddev = 1.0f;
  if (observations.empty()) return;
  const size_t nobs = observations.size();
  std::vector<std::vector<float>> feats;
  std::vector<double> l, diff;
  if (!factor(gpu, &feats, &l, &diff)) return;
  const std::vector<double> alpha = solve_upper_t(l, nobs, solve_lower(l, nobs, diff));
  const std::vector<float> cur = full_features(m, n, k, c);
  std::vector<double> kstar(nobs);
  double mu = prior;
  for (size_t i = 0; i < nobs; ++i) {
    kstar[i] = std::exp(-(double)ard_distance_sq(cur, feats[i]) / 2.0);
    mu += kstar[i] * alpha[i];
  }
  const std::vector<double> v = solve_lower(l, nobs, kstar);
  double vv = 0.0;
  for (double x : v) vv += x * x;
  *mean = (float)mu;
  *stddev = (float)std::sqrt(std::max(1.0 - vv, 1e-6));
}

// EI with the exact normal density and the reference's tanh stand-in for the
// normal CDF: 0.5 (1 + tanh(z / sqrt 2))  (mod.rs:555-563).
float GaussianProcess::expected_improvement(uint32_t m, uint32_t n, uint32_t k, const PipelineConfig &c,
                                            float best_y, const HardwareProfile &gpu) const {
  float mu, sigma;
  predict(m, n, k, c, gpu, &mu, &sigma);
  if (sigma < 1e-6f) return 0.0f;
  const float z = (mu - best_y) / sigma;
  const float phi = std::exp(-0.5f * z * z) / std::sqrt(2.0f * (float)M_PI);
  const float cdf = 0.5f * (1.0f + std::tanh(z / std::sqrt(2.0f)));
  return (mu - best_y) * cdf + sigma * phi;
}

float GaussianProcess::ucb(uint32_t m, uint32_t n, uint32_t k, const PipelineConfig &c,
                           const HardwareProfile &gpu) const {
  float mu, sigma;
  predict(m, n, k, c, gpu, &mu, &sigma);
  return mu + exploration_beta * sigma;
}

float GaussianProcess::thompson_sample(uint32_t m, uint32_t n, uint32_t k, const PipelineConfig &c,
                                       const HardwareProfile &gpu, uint64_t *state) const {
  float mu, sigma;
  predict(m, n, k, c, gpu, &mu, &sigma);
  sigma = std::max(sigma, 1e-6f);
  // Box-Muller on two 53-bit uniforms
  const double u1 = ((double)(splitmix64(state) >> 11) + 1.0) * (1.0 / 9007199254740993.0);
  const double u2 = (double)(splitmix64(state) >> 11) * (1.0 / 9007199254740992.0);
  const double z = std::sqrt(-2.0 * std::log(u1)) * std::cos(2.0 * M_PI * u2);
  return mu + sigma * (float)z;
}

}  // namespace tracea_amd
