// Device layer for the GPU backend: the DEV_GPU arm of the reference's
// Tensor / allocator pair (src/device.hpp:9-55; src/device_gpu.cpp is an empty
// file there).  Host-only C++: everything that touches the GPU goes through
// the C ABI of libllmhip.so.
#pragma once
#include <chrono>
#include <cstddef>
#include <cstdint>
#include <fstream>
#include <map>
#include <memory>
#include <string>
#include <unordered_map>

#include "../../include/hip_ops.hpp"

namespace llm_simple_amd {

// malloc / free (src/device_cpu.cpp:5-16).
class CPUAllocator {
 public:
  static CPUAllocator &GetInstance();
  static void *Allocate(size_t size);
  static void Deallocate(void *ptr);
};

// Pooling device allocator with the contract of the reference's NPUAllocator
// (src/device_npu.cpp:26-67): Allocate takes the smallest cached block that is
// large enough, else asks the device and then, while more than dev_mem_max
// bytes are owned, gives cached blocks back smallest first; Deallocate returns
// a block to the cache.  Not thread safe, and -- as in the reference -- a
// freed block can be handed out again at once, so the caller drains the stream
// before temporaries go out of scope (src/llama2_layer_npu.cpp:605-608).
class GPUAllocator {
 public:
  using RawAlloc = int (*)(void **, size_t);
  using RawFree = int (*)(void *);

  static GPUAllocator &GetInstance();
  static void *Allocate(size_t size);
  static void Deallocate(void *ptr);

  // Test hooks: replace the device calls (default llmhip_malloc / llmhip_free)
  // and the 8 GiB trim threshold; ReleaseAll frees every cached block.
  void SetBackend(RawAlloc a, RawFree f);
  void SetByteCap(size_t cap) { dev_mem_max_ = cap; }
  void ReleaseAll();
  size_t OwnedBytes() const { return owned_bytes_; }
  size_t CachedBlocks() const { return cache_.size(); }

 private:
  GPUAllocator();
  void *AllocateImpl(size_t size);
  void DeallocateImpl(void *ptr);

  std::multimap<size_t, void *> cache_;         // free blocks by size
  std::unordered_map<void *, size_t> ptr_size_;  // every block this allocator owns
  size_t dev_mem_max_{8ULL << 30};
  size_t owned_bytes_{0};
  RawAlloc raw_alloc_;
  RawFree raw_free_;
};

// src/device.hpp:41-55.  data_size counts elements, bytes = SizeOfTensor().
class Tensor : public std::enable_shared_from_this<Tensor> {
 public:
  Tensor() = default;
  ~Tensor();
  static std::shared_ptr<Tensor> MakeCPUTensor(size_t size, DataType dtype);
  static std::shared_ptr<Tensor> MakeGPUTensor(size_t size, DataType dtype);

  // Same device: this tensor; other device: a new tensor filled by a blocking
  // copy (src/device.cpp:22-52).
  std::shared_ptr<Tensor> to(DeviceType to_dev);
  void to_file(const char *path);

  void *data_ptr{nullptr};
  size_t data_size{0};
  DataType data_type{DT_FLOAT16};
  DeviceType dev_type{DEV_CPU};
};

// Chrome-trace ("chrome://tracing", Perfetto) writer of the reference's profiler
// (src/profiling.hpp, src/profiling.cpp:11-38): a JSON array of complete events
// {"name", "ph":"X", "pid":0, "ts" (us since StartLogging), "dur" (us, GPU time between two
// stream events), "args":{"file","lineno","info"}}.
class AppProfiler {
 public:
  bool StartLogging(const std::string &log_path);
  void RecordEvent(const std::string &name, const std::string &info, const char *file, int lineno,
                   uint64_t ts_us_steady, double dur_us);
  void Finish();
  size_t EventCount() const { return count_; }

 private:
  std::ofstream profile_file_;
  bool first_record_{true};
  uint64_t start_us_count_{0};
  size_t count_{0};
};

// Scope guard (src/profiling.cpp:40-94): records a stream event at construction; at
// destruction records a second one, drains the stream and writes one trace record whose
// duration is the GPU time between the two events.
class AppProfileGuard {
 public:
  AppProfileGuard(const char *name, const char *info, gpuStream_t stream, AppProfiler *profiler,
                  const char *fname, int lineno, bool is_profiling);
  ~AppProfileGuard();
  AppProfileGuard(const AppProfileGuard &) = delete;
  AppProfileGuard &operator=(const AppProfileGuard &) = delete;

 private:
  std::string record_name_, record_info_;
  const char *record_file_name_;
  int record_file_lineno_;
  gpuStream_t stream_;
  AppProfiler *profiler_;
  bool is_profiling_;
  void *event_{nullptr};
  uint64_t start_us_{0};
};

#define LLM_AMD_CONCAT2(x, y) x##y
#define LLM_AMD_CONCAT(x, y) LLM_AMD_CONCAT2(x, y)
// Same argument list as the reference's macro (src/profiling.hpp:47-48).
#define APP_PROFILE(name, info, stream, profiler, isprofiling)                                   \
  ::llm_simple_amd::AppProfileGuard LLM_AMD_CONCAT(temp_perf_obj_, __LINE__)(                    \
      name, info, stream, profiler, __FILE__, __LINE__, isprofiling)

// Positions of one step (src/model_base.hpp:40-48): cur_size = cur_pos - prev_pos
// query tokens, keys [0, cur_pos) valid after the append.
struct InferenceCtx {
  InferenceCtx(size_t cur_pos_, size_t prev_pos_, gpuStream_t stream = nullptr)
      : cur_pos(cur_pos_), prev_pos(prev_pos_), cur_size(cur_pos_ - prev_pos_), gpu_stream(stream) {}
  size_t cur_pos;
  size_t prev_pos;
  size_t cur_size;
  gpuStream_t gpu_stream;
  // the reference reaches these through ctx.model (src/llama2_layer_npu.cpp:1169-1171)
  AppProfiler *profiler{nullptr};
  bool is_profiling{false};
};

// Host rotary table [max_seq_len][head_dim/2][2] = (cos, sin), built the way
// ModelBase::InitFreqCIS does (src/model_base.cpp:27-83): inverse frequencies
// through a double pow, angles and cos/sin in fp32, every entry rounded to bf16
// and widened back for bf16 models.
std::shared_ptr<Tensor> MakeFreqCIS(int head_dim, int max_seq_len, float theta, DataType dt);

// The attention block of one transformer layer on the GPU: what
// Qwen2TransformerLayerNPUImpl::Forward does between the q/k/v projections
// and o_proj (src/llama2_layer_npu.cpp:780-869), and, with n_kv_heads ==
// n_heads and fp16, what the Llama-2 layer does (:206-208, :325-374).
// Owns the per-layer contiguous KV cache [max_seq_len][n_kv_heads][head_dim]
// (src/llama2_layer_npu.cpp:1148-1149).
class AttentionGPUImpl {
 public:
  bool Init(int n_heads, int n_kv_heads, int head_dim, int max_seq_len, DataType dtype,
            bool rope_is_neox_style, std::shared_ptr<Tensor> freq_cis_gpu);
  // q: [cur_size][n_heads*head_dim], k, v: [cur_size][n_kv_heads*head_dim], on the GPU.
  // Returns [cur_size][n_heads*head_dim].  Asynchronous on ctx.gpu_stream.
  std::shared_ptr<Tensor> Forward(std::shared_ptr<Tensor> q, std::shared_ptr<Tensor> k,
                                  std::shared_ptr<Tensor> v, InferenceCtx &ctx);
  std::shared_ptr<Tensor> k_cache, v_cache;

 private:
  int n_heads_{0}, n_kv_heads_{0}, head_dim_{0}, max_seq_len_{0};
  DataType dtype_{DT_FLOAT16};
  bool neox_{false};
  std::shared_ptr<Tensor> freq_cis_;
};

// Dense projection y = x W^T (+ bias) on the GPU: MatmulLayerNPUImpl without quantisation
// (src/llama2_layer_npu.cpp:1158-1181).  The weight is kept as W[n][k] row-major (checkpoint
// layout); the reference's nz repacking is an Ascend detail.  bias is fp32 [n] or null
// (src/llama2_layer_npu.cpp:1323-1338).
class MatmulLayerGPUImpl {
 public:
  // host_weight: n*k elements of dtype; host_bias: n floats or nullptr.  Blocking copies.
  bool Init(const void *host_weight, const float *host_bias, size_t n, size_t k, DataType dtype);
  // input [cur_size][k] on the GPU -> [cur_size][n].  Asynchronous on ctx.gpu_stream.
  std::shared_ptr<Tensor> Forward(std::shared_ptr<Tensor> input, InferenceCtx &ctx);
  size_t n{0}, k{0};

 private:
  DataType dtype_{DT_FLOAT16};
  std::shared_ptr<Tensor> weight_, bias_;
};

// The whole attention block of a Qwen2 / Llama-2 layer between input_norm and post_norm
// (src/llama2_layer_npu.cpp:760-901): q/k/v projections (bias for Qwen2), RoPE + cache
// append, attention, o_proj, residual add.
class AttentionBlockGPUImpl {
 public:
  struct Weights {  // host pointers; biases may be null (Llama-2)
    const void *wq, *wk, *wv, *wo;
    const float *bq, *bk, *bv;
  };
  bool Init(const Weights &w, int hidden_dim, int n_heads, int n_kv_heads, int max_seq_len,
            DataType dtype, bool rope_is_neox_style, std::shared_ptr<Tensor> freq_cis_gpu);
  // normed: output of input_norm [cur_size][hidden]; residual: the layer input.  Returns
  // residual + o_proj(attention(...)).
  std::shared_ptr<Tensor> Forward(std::shared_ptr<Tensor> normed, std::shared_ptr<Tensor> residual,
                                  InferenceCtx &ctx);
  AttentionGPUImpl attention;
  MatmulLayerGPUImpl q_proj, k_proj, v_proj, o_proj;

 private:
  int hidden_dim_{0};
  DataType dtype_{DT_FLOAT16};
};

}  // namespace llm_simple_amd
