// tracea-tuner: command-line driver of the tuning entry points.
//
//   tracea-tuner gemm <m> <n> <k> [--out <file>]
//   tracea-tuner conv <n> <h> <w> <c_in> <c_out> <k_h> <k_w> [stride] [pad] [--out <file>]
//   tracea-tuner attention <b> <h> <s> <d> [--causal] [--out <file>]
//
// Same sub-commands, argument order, default output files and result record
// {timestamp, kernel, problem, best_config} as the reference's tuner binary
// (src/bin/tuner.rs:11-276); the record also carries the measured score.
// Uses nothing but the C ABI of libtracea.so.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <ctime>
#include <string>
#include <vector>

#include "tracea.h"
#include "tracea_tuner.h"

namespace {

std::string rfc3339_now() {
  const time_t t = time(nullptr);
  struct tm tmv;
  localtime_r(&t, &tmv);
  char buf[40], zone[8];
  strftime(buf, sizeof(buf), "%Y-%m-%dT%H:%M:%S", &tmv);
  strftime(zone, sizeof(zone), "%z", &tmv);  // +hhmm -> +hh:mm
  std::string z(zone);
  if (z.size() == 5) z.insert(3, ":");
  return std::string(buf) + z;
}

// Splits off "--out <file>" and "--causal"; the rest are positional.
struct Args {
  std::vector<std::string> pos;
  std::string out;
  bool causal = false;
};

Args split(int argc, char **argv, int from, const char *default_out) {
  Args a;
  a.out = default_out;
  for (int i = from; i < argc; ++i) {
    if (!strcmp(argv[i], "--out") && i + 1 < argc) a.out = argv[++i];
    else if (!strcmp(argv[i], "--causal")) a.causal = true;
    else a.pos.push_back(argv[i]);
  }
  return a;
}

bool parse_sizes(const std::vector<std::string> &pos, size_t need, std::vector<size_t> *out) {
  if (pos.size() < need) return false;
  for (const std::string &s : pos) {
    char *end = nullptr;
    const unsigned long long v = strtoull(s.c_str(), &end, 10);
    if (end == s.c_str() || *end != 0) {
      fprintf(stderr, "not a number: %s\n", s.c_str());
      return false;
    }
    out->push_back((size_t)v);
  }
  return true;
}

int finish(const TraceaResult &r, const char *kernel, const std::string &problem_json, const std::string &path) {
  if (!r.success) {
    fprintf(stderr, "tuning failed: %s\n", r.error_msg ? r.error_msg : "unknown error");
    tracea_free_string(r.error_msg);
    return 1;
  }
  const char *cfg = static_cast<const char *>(r.config_ptr);
  printf("Tuning Complete.\nBest Configuration: %s\nBest Score: %.2f TFLOPS\n", cfg, r.score);
  FILE *f = fopen(path.c_str(), "w");
  if (f == nullptr) {
    perror(path.c_str());
    tracea_free_string(static_cast<char *>(r.config_ptr));
    return 1;
  }
  fprintf(f, "{\n  \"timestamp\": \"%s\",\n  \"kernel\": \"%s\",\n  \"problem\": %s,\n  \"best_config\": %s,\n"
             "  \"score_tflops\": %.4f\n}\n",
          rfc3339_now().c_str(), kernel, problem_json.c_str(), cfg, r.score);
  fclose(f);
  printf("Results saved to %s\n", path.c_str());
  tracea_free_string(static_cast<char *>(r.config_ptr));
  return 0;
}

void usage() {
  fprintf(stderr,
          "Usage: tracea-tuner <subcommand> [args]\nSubcommands:\n"
          "  gemm <m> <n> <k> [--out <file>]\n"
          "  conv <n> <h> <w> <c_in> <c_out> <k_h> <k_w> [stride] [pad] [--out <file>]\n"
          "  attention <b> <h> <s> <d> [--causal] [--out <file>]\n");
}

}  // namespace

int main(int argc, char **argv) {
  if (argc < 2) {
    usage();
    return 0;
  }
  const std::string sub = argv[1];
  if (sub != "gemm" && sub != "conv" && sub != "attention") {
    fprintf(stderr, "Unknown subcommand: %s\n", sub.c_str());
    usage();
    return 2;
  }
  char problem[256];
  std::vector<size_t> v;
  if (sub == "gemm") {
    const Args a = split(argc, argv, 2, "bench_results.json");
    if (!parse_sizes(a.pos, 3, &v)) {
      fprintf(stderr, "Usage: tracea-tuner gemm <m> <n> <k> [--out <file>]\n");
      return 2;
    }
    printf("Starting Tuner for GEMM %zux%zux%zu\n", v[0], v[1], v[2]);
    if (tracea_init() != 0) {
      fprintf(stderr, "Runtime init failed\n");
      return 1;
    }
    snprintf(problem, sizeof(problem), "{ \"m\": %zu, \"n\": %zu, \"k\": %zu }", v[0], v[1], v[2]);
    return finish(tracea_autotune_gemm(v[0], v[1], v[2], 0), "gemm", problem, a.out);
  }
  if (sub == "conv") {
    const Args a = split(argc, argv, 2, "conv_bench_results.json");
    if (!parse_sizes(a.pos, 7, &v)) {
      fprintf(stderr, "Usage: tracea-tuner conv <n> <h> <w> <c_in> <c_out> <k_h> <k_w> [stride] [pad] [--out <file>]\n");
      return 2;
    }
    const size_t stride = v.size() > 7 ? v[7] : 1, pad = v.size() > 8 ? v[8] : 0;
    printf("Starting Tuner for Conv2d %zux%zux%zux%zu -> %zux%zux%zu\n", v[0], v[1], v[2], v[3], v[4], v[5], v[6]);
    if (tracea_init() != 0) {
      fprintf(stderr, "Runtime init failed\n");
      return 1;
    }
    snprintf(problem, sizeof(problem),
             "{ \"n\": %zu, \"h\": %zu, \"w\": %zu, \"c_in\": %zu, \"c_out\": %zu, \"r\": %zu, \"s\": %zu, "
             "\"stride\": %zu, \"pad\": %zu }",
             v[0], v[1], v[2], v[3], v[4], v[5], v[6], stride, pad);
    return finish(tracea_autotune_conv2d(v[0], v[3], v[1], v[2], v[4], v[5], v[6], stride, pad, 1, 0), "conv2d",
                  problem, a.out);
  }
  const Args a = split(argc, argv, 2, "attention_bench_results.json");
  if (!parse_sizes(a.pos, 4, &v)) {
    fprintf(stderr, "Usage: tracea-tuner attention <b> <h> <s> <d> [--causal] [--out <file>]\n");
    return 2;
  }
  printf("Starting Tuner for Attention B%zu H%zu S%zu D%zu%s\n", v[0], v[1], v[2], v[3], a.causal ? " causal" : "");
  if (tracea_init() != 0) {
    fprintf(stderr, "Runtime init failed\n");
    return 1;
  }
  snprintf(problem, sizeof(problem), "{ \"b\": %zu, \"h\": %zu, \"s\": %zu, \"d\": %zu, \"causal\": %s }", v[0], v[1],
           v[2], v[3], a.causal ? "true" : "false");
  return finish(tracea_tune_fa2(v[0], v[1], v[2], v[3], a.causal), "attention", problem, a.out);
}
