// Device layer for the GPU backend: the DEV_GPU arm of the reference's
// Tensor / allocator pair (src/device.hpp:9-55; src/device_gpu.cpp is an empty
// file there).  Host-only C++: everything that touches the GPU goes through
// the C ABI of libllmhip.so.
#pragma once
#include <chrono>
#include <cstddef>
#include <cstdint>
#include <fstream>
#include <tuple>
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

// Pooling device allocator with the pooling contract of the reference's NPUAllocator
// (src/device_npu.cpp:26-67): Allocate takes the smallest cached block that is large enough, else
// asks the device and then, while more than dev_mem_max bytes are owned, gives cached blocks back
// smallest first; Deallocate returns a block to the cache.
//
// Unlike the reference's pool this one is stream-ordered.  In the reference a freed block can be
// handed out again at once, so every layer drains its stream before its temporaries go out of scope
// (src/llama2_layer_npu.cpp:605-608, :990-993): one host round trip per layer per token.  Here a
// block that is freed remembers the stream whose queued work may still touch it and a ticket of that
// stream.  A request that names the same stream may take the block at once (its new use is queued
// behind the old one); any other request -- another stream, or host code that names none -- gets it
// only once an event recorded on that stream after the free has completed.  Such an event is recorded
// when a request first needs it, not at every free, so a model that runs on one stream makes no event
// call at all.  A block freed without a stream (never handed to a launch, or whose user drained the
// stream itself) is free for everybody.  Not thread safe, like the reference's.
class GPUAllocator {
 public:
  using RawAlloc = int (*)(void **, size_t);
  using RawFree = int (*)(void *);
  // event backend: create / record on a stream / query (0 = complete, anything else = not yet) /
  // wait / destroy; by default the llmhip_event_* calls of the C ABI
  struct EventBackend {
    int (*create)(void **event);
    int (*record)(void *event, void *stream);
    int (*query)(void *event);
    int (*sync)(void *event);
    int (*destroy)(void *event);
    int (*device_sync)();
  };
  // Stream tags of a block: kNoStream = no queued work touches it; kAnyStream = some stream does but
  // the caller did not say which (only a drained device makes it reusable).
  static gpuStream_t NoStream() { return reinterpret_cast<gpuStream_t>(static_cast<uintptr_t>(1)); }
  static gpuStream_t AnyStream() { return reinterpret_cast<gpuStream_t>(static_cast<uintptr_t>(2)); }

  static GPUAllocator &GetInstance();
  // stream: the stream the block will be used on (nullptr is the default stream, a stream like any
  // other), or NoStream() for a request from host code that will touch the block with blocking calls.
  static void *Allocate(size_t size, gpuStream_t stream = NoStream());
  // stream: the stream whose queued work may still read or write the block, NoStream() if none can,
  // AnyStream() if unknown.
  static void Deallocate(void *ptr, gpuStream_t stream = NoStream());

  // Test hooks: replace the device calls (default llmhip_malloc / llmhip_free, llmhip_event_*)
  // and the 8 GiB trim threshold; ReleaseAll frees every cached block (after draining the device
  // when any is still pending).
  void SetBackend(RawAlloc a, RawFree f);
  void SetEventBackend(const EventBackend *b);
  void SetByteCap(size_t cap) { dev_mem_max_ = cap; }
  void ReleaseAll();
  // Before a stream is destroyed: drain it, then tell the pool, which frees its blocks for everybody
  // (a later stream may get the same handle).
  void ForgetStream(gpuStream_t stream);
  size_t OwnedBytes() const { return owned_bytes_; }
  size_t CachedBlocks() const { return cache_.size(); }
  size_t PendingBlocks() const;
  size_t FenceEvents() const { return fence_events_; }  // events recorded so far (a single-stream model: 0)

 private:
  struct Block {
    void *ptr;
    gpuStream_t stream;  // NoStream(): free for everybody
    uint64_t ticket;     // position in that stream's sequence of frees
  };
  struct StreamState {
    uint64_t next_ticket{1};   // ticket of the next free on this stream
    uint64_t fenced{0};        // frees up to this ticket are covered by `event`
    uint64_t completed{0};     // frees up to this ticket are known complete
    void *event{nullptr};
  };
  GPUAllocator();
  void *AllocateImpl(size_t size, gpuStream_t stream);
  void DeallocateImpl(void *ptr, gpuStream_t stream);
  bool Usable(const Block &b, gpuStream_t requester, bool may_wait);
  void DrainAll();

  std::multimap<size_t, Block> cache_;           // free and pending blocks by size
  std::unordered_map<void *, size_t> ptr_size_;  // every block this allocator owns
  std::unordered_map<gpuStream_t, StreamState> streams_;
  size_t dev_mem_max_{8ULL << 30};
  size_t owned_bytes_{0};
  size_t fence_events_{0};
  RawAlloc raw_alloc_;
  RawFree raw_free_;
  EventBackend ev_;
};

// src/device.hpp:41-55.  data_size counts elements, bytes = SizeOfTensor().
class Tensor : public std::enable_shared_from_this<Tensor> {
 public:
  Tensor() = default;
  ~Tensor();
  static std::shared_ptr<Tensor> MakeCPUTensor(size_t size, DataType dtype);
  // stream: the stream whose launches will use the tensor (the pool is stream-ordered, see
  // GPUAllocator); without one the block comes from what no queued work can touch.
  static std::shared_ptr<Tensor> MakeGPUTensor(size_t size, DataType dtype,
                                               gpuStream_t stream = GPUAllocator::NoStream());
  // Tells the tensor that work queued on `stream` reads or writes it, so that its block is not
  // handed to anybody else before that work is done.  Layers call it on every tensor they pass
  // to a launch; a tensor used on two different streams is kept until the device has drained.
  void RecordStream(gpuStream_t stream);

  // Same device: this tensor; other device: a new tensor filled by a blocking
  // copy (src/device.cpp:22-52).
  std::shared_ptr<Tensor> to(DeviceType to_dev);
  void to_file(const char *path);

  void *data_ptr{nullptr};
  size_t data_size{0};
  DataType data_type{DT_FLOAT16};
  DeviceType dev_type{DEV_CPU};
  gpuStream_t stream_tag{GPUAllocator::NoStream()};  // see RecordStream
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

class ModelBase;

// Positions of one step (src/model_base.hpp:40-48): cur_size = cur_pos - prev_pos
// query tokens, keys [0, cur_pos) valid after the append.
struct InferenceCtx {
  InferenceCtx(size_t cur_pos_, size_t prev_pos_, gpuStream_t stream = nullptr)
      : cur_pos(cur_pos_), prev_pos(prev_pos_), cur_size(cur_pos_ - prev_pos_), gpu_stream(stream) {}
  // the reference's constructor (src/model_base.hpp:42); stream, profiler and profiling flag come from the model
  InferenceCtx(ModelBase *model, size_t cur_pos_, size_t prev_pos_);
  ModelBase *model{nullptr};
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
  // the same with the rotary table as a bare device pointer that somebody else owns (ModelBase::freq_cis)
  bool Init(int n_heads, int n_kv_heads, int head_dim, int max_seq_len, DataType dtype,
            bool rope_is_neox_style, float *freq_cis_dev);
  // q: [cur_size][n_heads*head_dim], k, v: [cur_size][n_kv_heads*head_dim], on the GPU.
  // Returns [cur_size][n_heads*head_dim].  Asynchronous on ctx.gpu_stream.
  std::shared_ptr<Tensor> Forward(std::shared_ptr<Tensor> q, std::shared_ptr<Tensor> k,
                                  std::shared_ptr<Tensor> v, InferenceCtx &ctx);
  std::shared_ptr<Tensor> k_cache, v_cache;

 private:
  int n_heads_{0}, n_kv_heads_{0}, head_dim_{0}, max_seq_len_{0};
  DataType dtype_{DT_FLOAT16};
  bool neox_{false};
  float *freqs_cis_{nullptr};
  std::shared_ptr<Tensor> freq_cis_owner_;
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

// ---------------------------------------------------------------------------
// Device dispatch: the layer facades of the reference (src/model_base.hpp, src/model_base.cpp)
// for the layers on this path, with the DEV_GPU arm that the reference leaves out.
// ---------------------------------------------------------------------------

// What these layers read of the reference's ModelConfig (src/model_base.hpp:18-36) ...
class ModelConfig {
 public:
  DeviceType device_type{DEV_GPU};
  DataType data_type{DT_FLOAT16};
  int max_seq_len{2048};
  bool rope_is_neox_style{false};
  bool debug_print{false};
};

// ... and of ModelBase (src/model_base.hpp:324-354): dimensions, the model's one stream, the
// rotary table and the profiler.
class ModelBase {
 public:
  virtual ~ModelBase() = default;
  // src/model_base.cpp:27-83 with the device arm for DEV_GPU: the table is built on the host and,
  // for DEV_GPU, copied to the device once; freq_cis then is a device pointer.
  bool InitFreqCIS(const float theta = 10000.0f, const DataType dt = DT_FLOAT32);

  ModelConfig config;
  int hidden_dim{0};
  int head_dim{0};
  int n_heads{0};
  int n_kv_heads{0};
  gpuStream_t model_stream{nullptr};
  float *freq_cis{nullptr};
  bool is_profiling{false};
  AppProfiler profiler;

 private:
  std::shared_ptr<Tensor> freq_cis_holder_;
};

// src/model_base.hpp:106-133.
class RoPELayerImpl {
 public:
  virtual ~RoPELayerImpl();
  virtual std::tuple<std::shared_ptr<Tensor>, std::shared_ptr<Tensor>> Forward(std::shared_ptr<Tensor> input_q,
                                                                              std::shared_ptr<Tensor> input_k,
                                                                              InferenceCtx &ctx) = 0;
  virtual bool Init(ModelBase *model, const std::string &weight_path);
  virtual void UnInit();

  size_t hidden_dim{0};
  size_t n_heads{0};
  size_t head_dim{0};
  size_t rope_dim{0};
  size_t weight_size{0};
  bool rope_is_neox_style{false};
  DataType dtype{DT_FLOAT16};
  float *freqs_cis{nullptr};
};

// The GPU sibling of RoPELayerNPUImpl (src/llama2_layer_npu.cpp:183-222): q and k of the same head
// count rotated by one hip_rope_layer call, outputs from the pool.
class RoPELayerGPUImpl : public RoPELayerImpl {
 public:
  ~RoPELayerGPUImpl() override;
  std::tuple<std::shared_ptr<Tensor>, std::shared_ptr<Tensor>> Forward(std::shared_ptr<Tensor> input_q,
                                                                      std::shared_ptr<Tensor> input_k,
                                                                      InferenceCtx &ctx) override;
  bool Init(ModelBase *model, const std::string &weight_path) override;
};

class RoPELayer {
 public:
  ~RoPELayer();
  std::tuple<std::shared_ptr<Tensor>, std::shared_ptr<Tensor>> Forward(std::shared_ptr<Tensor> input_q,
                                                                      std::shared_ptr<Tensor> input_k,
                                                                      InferenceCtx &ctx);
  // src/model_base.cpp:620-635: picks the implementation by model->config.device_type.
  bool Init(ModelBase *model, const std::string &weight_path);
  void UnInit();
  RoPELayerImpl *impl{nullptr};
};

// The attention part of a transformer layer -- between the q/k/v projections and o_proj -- behind
// the same kind of facade as the reference's Llamma2TransformerLayer / Qwen2TransformerLayer
// (src/model_base.hpp; the rest of those layers, norms and FFN, is outside this path).
class AttentionLayerImpl {
 public:
  virtual ~AttentionLayerImpl();
  // q [cur_size][n_heads*head_dim], k, v [cur_size][n_kv_heads*head_dim] on the device, unrotated;
  // returns [cur_size][n_heads*head_dim].
  virtual std::shared_ptr<Tensor> Forward(std::shared_ptr<Tensor> q, std::shared_ptr<Tensor> k,
                                          std::shared_ptr<Tensor> v, InferenceCtx &ctx) = 0;
  virtual bool Init(ModelBase *model, int layer_no);
  virtual void UnInit();

  size_t hidden_dim{0};
  size_t head_dim{0};
  size_t n_heads{0};
  size_t n_kv_heads{0};
  size_t max_seq_len{0};
  DataType dtype{DT_FLOAT16};
  std::shared_ptr<Tensor> k_cache, v_cache;
};

// Llama-2 on the GPU, call for call what Llamma2TransformerLayerNPUImpl::Forward does
// (src/llama2_layer_npu.cpp:284, :325-339, :370-374): rope_emb.Forward, two device-to-device copies
// into the caches, hip_flash_attn_opt_prefill_layer.  n_kv_heads == n_heads.
class Llama2AttentionGPUImpl : public AttentionLayerImpl {
 public:
  std::shared_ptr<Tensor> Forward(std::shared_ptr<Tensor> q, std::shared_ptr<Tensor> k, std::shared_ptr<Tensor> v,
                                  InferenceCtx &ctx) override;
  bool Init(ModelBase *model, int layer_no) override;
  RoPELayer rope_emb;
};

// Qwen2 on the GPU (src/llama2_layer_npu.cpp:790-869): the fused operators of AttentionGPUImpl.
class Qwen2AttentionGPUImpl : public AttentionLayerImpl {
 public:
  std::shared_ptr<Tensor> Forward(std::shared_ptr<Tensor> q, std::shared_ptr<Tensor> k, std::shared_ptr<Tensor> v,
                                  InferenceCtx &ctx) override;
  bool Init(ModelBase *model, int layer_no) override;

 private:
  AttentionGPUImpl impl_;
};

// src/model_base.cpp:248-264.
class Llama2AttentionLayer {
 public:
  ~Llama2AttentionLayer();
  std::shared_ptr<Tensor> Forward(std::shared_ptr<Tensor> q, std::shared_ptr<Tensor> k, std::shared_ptr<Tensor> v,
                                  InferenceCtx &ctx);
  bool Init(ModelBase *model, int layer_no);
  void UnInit();
  AttentionLayerImpl *impl{nullptr};
};

// src/model_base.cpp:294-306.
class Qwen2AttentionLayer {
 public:
  ~Qwen2AttentionLayer();
  std::shared_ptr<Tensor> Forward(std::shared_ptr<Tensor> q, std::shared_ptr<Tensor> k, std::shared_ptr<Tensor> v,
                                  InferenceCtx &ctx);
  bool Init(ModelBase *model, int layer_no);
  void UnInit();
  AttentionLayerImpl *impl{nullptr};
};

}  // namespace llm_simple_amd
