// Device layer for the GPU backend: the DEV_GPU arm of the reference's
// Tensor / allocator pair (src/device.hpp:9-55; src/device_gpu.cpp is an empty
// file there).  Host-only C++: everything that touches the GPU goes through
// the C ABI of libllmhip.so.
#pragma once
#include <cstddef>
#include <map>
#include <memory>
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

// Positions of one step (src/model_base.hpp:40-48): cur_size = cur_pos - prev_pos
// query tokens, keys [0, cur_pos) valid after the append.
struct InferenceCtx {
  InferenceCtx(size_t cur_pos_, size_t prev_pos_, gpuStream_t stream = nullptr)
      : cur_pos(cur_pos_), prev_pos(prev_pos_), cur_size(cur_pos_ - prev_pos_), gpu_stream(stream) {}
  size_t cur_pos;
  size_t prev_pos;
  size_t cur_size;
  gpuStream_t gpu_stream;
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

}  // namespace llm_simple_amd
