// Shared pieces of the GPU op-test command lines (the counterparts of the
// reference's tests/npu_op_test_util.{h,cpp}): flag parsing, a seeded input
// generator, and the C entry points of the CPU oracle (test infrastructure).
#pragma once
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "../../llm_simple_amd/csrc/device_hip.hpp"

extern "C" {
void orc_round_array(uint16_t *out, const float *in, int64_t count, int dt);
void orc_widen_array(float *out, const uint16_t *in, int64_t count, int dt);
void orc_init_freq_cis(float *freq_cis, int head_dim, int max_seq_len, float theta, int dt, int use_powf);
void orc_rope(uint16_t *out, const uint16_t *in, const float *freq_cis, int start_pos, int cur_size,
              int n_heads, int head_dim, int is_neox, int dt);
void orc_kv_append(uint16_t *cache, const uint16_t *src, int prev_pos, int cur_size, int row_elems);
void orc_attention_f32(float *out, const uint16_t *q, const uint16_t *k, const uint16_t *v, int batch,
                       int m, int n, int offset, int group_size, int kv_head_num, int head_dim,
                       int64_t kv_seq_stride, int dt, int n_threads);
void orc_matmul_bias(uint16_t *out, const uint16_t *lhs, const uint16_t *w, const float *bias, int m, int n,
                     int k, int dt, int n_threads);
void orc_add(uint16_t *out, const uint16_t *lhs, const uint16_t *rhs, int64_t count, int dt);
int64_t orc_all_close(const float *a, const float *b, int64_t count, float abs_err, float rel_err,
                      float *max_abs_out);
}

namespace optest {

// --name value / --name=value
inline std::string flag(int argc, char **argv, const char *name, const char *dflt) {
  const std::string key = std::string("--") + name;
  for (int i = 1; i < argc; ++i) {
    const std::string a = argv[i];
    if (a == key && i + 1 < argc) return argv[i + 1];
    if (a.rfind(key + "=", 0) == 0) return a.substr(key.size() + 1);
  }
  return dflt;
}
inline long flag_int(int argc, char **argv, const char *name, long dflt) {
  return std::atol(flag(argc, argv, name, std::to_string(dflt).c_str()).c_str());
}

// N(0,1) from a seed: splitmix64 -> Box-Muller, rounded to the storage type.
// The rounded bits go to the device and to the golden alike (the round-trip of
// tests/flash_attn_test.cpp:88-104).
struct Rng {
  uint64_t s;
  explicit Rng(uint64_t seed) : s(seed) {}
  uint64_t next() {
    uint64_t z = (s += 0x9E3779B97F4A7C15ULL);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    return z ^ (z >> 31);
  }
  double uniform() { return (static_cast<double>(next() >> 11) + 0.5) * (1.0 / 9007199254740992.0); }
  float normal() {
    const double u1 = uniform(), u2 = uniform();
    return static_cast<float>(std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586 * u2));
  }
};

inline std::vector<uint16_t> normal_bits(uint64_t seed, size_t count, int dt) {
  Rng r(seed);
  std::vector<float> f(count);
  for (auto &x : f) x = r.normal();
  std::vector<uint16_t> b(count);
  orc_round_array(b.data(), f.data(), static_cast<int64_t>(count), dt);
  return b;
}

// N(0, sigma) weights rounded to the storage type
inline std::vector<uint16_t> scaled_normal_bits(uint64_t seed, size_t count, float sigma, int dt) {
  Rng r(seed);
  std::vector<float> f(count);
  for (auto &x : f) x = sigma * r.normal();
  std::vector<uint16_t> b(count);
  orc_round_array(b.data(), f.data(), static_cast<int64_t>(count), dt);
  return b;
}
inline std::vector<float> normal_f32(uint64_t seed, size_t count, float sigma) {
  Rng r(seed);
  std::vector<float> f(count);
  for (auto &x : f) x = sigma * r.normal();
  return f;
}

inline std::shared_ptr<llm_simple_amd::Tensor> to_gpu(const void *host, size_t elems,
                                                      llm_simple_amd::DataType dt) {
  auto h = llm_simple_amd::Tensor::MakeCPUTensor(elems, dt);
  std::memcpy(h->data_ptr, host, llm_simple_amd::SizeOfTensor(elems, dt));
  return h->to(llm_simple_amd::DEV_GPU);
}

inline llm_simple_amd::DataType parse_dtype(const std::string &s) {
  return (s == "bf16" || s == "bfloat16") ? llm_simple_amd::DT_BFLOAT16 : llm_simple_amd::DT_FLOAT16;
}

}  // namespace optest
