#include "device_hip.hpp"

#include <cstdio>

#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <fstream>

namespace llm_simple_amd {

CPUAllocator &CPUAllocator::GetInstance() {
  static CPUAllocator instance;
  return instance;
}
void *CPUAllocator::Allocate(size_t size) { return std::malloc(size); }
void CPUAllocator::Deallocate(void *ptr) { std::free(ptr); }

GPUAllocator::GPUAllocator() : raw_alloc_(&llmhip_malloc), raw_free_(&llmhip_free) {}

GPUAllocator &GPUAllocator::GetInstance() {
  static GPUAllocator instance;
  return instance;
}
void *GPUAllocator::Allocate(size_t size) { return GetInstance().AllocateImpl(size); }
void GPUAllocator::Deallocate(void *ptr) { GetInstance().DeallocateImpl(ptr); }

void GPUAllocator::SetBackend(RawAlloc a, RawFree f) {
  ReleaseAll();
  raw_alloc_ = a ? a : &llmhip_malloc;
  raw_free_ = f ? f : &llmhip_free;
}

void GPUAllocator::ReleaseAll() {
  for (auto &kv : cache_) {
    raw_free_(kv.second);
    owned_bytes_ -= kv.first;
    ptr_size_.erase(kv.second);
  }
  cache_.clear();
}

void *GPUAllocator::AllocateImpl(size_t size) {
  auto hit = cache_.lower_bound(size);  // smallest cached block that fits
  if (hit != cache_.end()) {
    void *p = hit->second;
    cache_.erase(hit);
    return p;
  }
  void *p = nullptr;
  int rc = raw_alloc_(&p, size);
  if (rc != LLMHIP_OK || p == nullptr) {
    hip_last_status() = rc ? rc : LLMHIP_ERR_INVALID_ARG;
    std::fprintf(stderr, "GPUAllocator: device allocation of %zu bytes failed: %s\n", size,
                 llmhip_error_string(rc));
    return nullptr;
  }
  owned_bytes_ += size;
  ptr_size_[p] = size;
  // after a miss, trim the cache while the pool owns more than the threshold
  while (owned_bytes_ > dev_mem_max_ && !cache_.empty()) {
    auto small = cache_.begin();
    raw_free_(small->second);
    owned_bytes_ -= small->first;
    ptr_size_.erase(small->second);
    cache_.erase(small);
  }
  return p;
}

void GPUAllocator::DeallocateImpl(void *ptr) {
  if (ptr == nullptr) return;
  auto it = ptr_size_.find(ptr);
  if (it == ptr_size_.end()) {
    std::fprintf(stderr, "GPUAllocator: %p was not allocated here\n", ptr);
    return;
  }
  cache_.emplace(it->second, ptr);
}

Tensor::~Tensor() {
  if (dev_type == DEV_GPU)
    GPUAllocator::Deallocate(data_ptr);
  else if (dev_type == DEV_CPU)
    CPUAllocator::Deallocate(data_ptr);
}

std::shared_ptr<Tensor> Tensor::MakeCPUTensor(size_t size, DataType dtype) {
  auto t = std::make_shared<Tensor>();
  t->data_size = size;
  t->data_type = dtype;
  t->dev_type = DEV_CPU;
  t->data_ptr = CPUAllocator::Allocate(SizeOfTensor(size, dtype));
  return t;
}

std::shared_ptr<Tensor> Tensor::MakeGPUTensor(size_t size, DataType dtype) {
  auto t = std::make_shared<Tensor>();
  t->data_size = size;
  t->data_type = dtype;
  t->dev_type = DEV_GPU;
  t->data_ptr = GPUAllocator::Allocate(SizeOfTensor(size, dtype));
  return t;
}

std::shared_ptr<Tensor> Tensor::to(DeviceType to_dev) {
  if (to_dev == dev_type) return shared_from_this();
  const size_t bytes = SizeOfTensor(data_size, data_type);
  if (dev_type == DEV_GPU && to_dev == DEV_CPU) {
    auto r = MakeCPUTensor(data_size, data_type);
    CHECK_LLMHIP(llmhip_memcpy_d2h(r->data_ptr, data_ptr, bytes));
    return r;
  }
  if (dev_type == DEV_CPU && to_dev == DEV_GPU) {
    auto r = MakeGPUTensor(data_size, data_type);
    if (r->data_ptr) CHECK_LLMHIP(llmhip_memcpy_h2d(r->data_ptr, data_ptr, bytes));
    return r;
  }
  return std::shared_ptr<Tensor>();
}

void Tensor::to_file(const char *path) {
  std::shared_ptr<Tensor> host = (dev_type == DEV_CPU) ? shared_from_this() : to(DEV_CPU);
  std::ofstream ofs(path, std::ios::binary);
  ofs.write(static_cast<const char *>(host->data_ptr),
            static_cast<std::streamsize>(SizeOfTensor(data_size, data_type)));
}

static inline float bf16_round_trip(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  u = (u + 0x7FFFu + ((u >> 16) & 1u)) & 0xFFFF0000u;  // nearest even, as src/util.cpp:33-72
  std::memcpy(&f, &u, 4);
  return f;
}

std::shared_ptr<Tensor> MakeFreqCIS(int head_dim, int max_seq_len, float theta, DataType dt) {
  const int freq_len = head_dim / 2;
  auto t = Tensor::MakeCPUTensor(static_cast<size_t>(max_seq_len) * freq_len * 2, DT_FLOAT32);
  float *tab = static_cast<float *>(t->data_ptr);
  for (int j = 0; j < freq_len; ++j) {
    const float inv = static_cast<float>(
        1.0f / std::pow(static_cast<double>(theta), static_cast<double>(2 * j) / head_dim));
    for (int pos = 0; pos < max_seq_len; ++pos) {
      const float angle = static_cast<float>(pos) * inv;
      float c = std::cos(angle), s = std::sin(angle);
      if (dt == DT_BFLOAT16) {
        c = bf16_round_trip(c);
        s = bf16_round_trip(s);
      }
      tab[(static_cast<size_t>(pos) * freq_len + j) * 2] = c;
      tab[(static_cast<size_t>(pos) * freq_len + j) * 2 + 1] = s;
    }
  }
  return t;
}

bool AttentionGPUImpl::Init(int n_heads, int n_kv_heads, int head_dim, int max_seq_len,
                            DataType dtype, bool rope_is_neox_style,
                            std::shared_ptr<Tensor> freq_cis_gpu) {
  if (n_heads < 1 || n_kv_heads < 1 || n_heads % n_kv_heads != 0 || head_dim != 128 ||
      max_seq_len < 1 || (dtype != DT_FLOAT16 && dtype != DT_BFLOAT16) || !freq_cis_gpu)
    return false;
  n_heads_ = n_heads;
  n_kv_heads_ = n_kv_heads;
  head_dim_ = head_dim;
  max_seq_len_ = max_seq_len;
  dtype_ = dtype;
  neox_ = rope_is_neox_style;
  freq_cis_ = freq_cis_gpu;
  const size_t cache_elems = static_cast<size_t>(max_seq_len) * n_kv_heads * head_dim;
  k_cache = Tensor::MakeGPUTensor(cache_elems, dtype);
  v_cache = Tensor::MakeGPUTensor(cache_elems, dtype);
  return k_cache->data_ptr != nullptr && v_cache->data_ptr != nullptr;
}

std::shared_ptr<Tensor> AttentionGPUImpl::Forward(std::shared_ptr<Tensor> q,
                                                  std::shared_ptr<Tensor> k,
                                                  std::shared_ptr<Tensor> v, InferenceCtx &ctx) {
  const int cur_size = static_cast<int>(ctx.cur_size);
  const int hidden = n_heads_ * head_dim_;
  if (ctx.cur_pos > static_cast<size_t>(max_seq_len_)) return nullptr;
  if (!q || !k || !v || !q->data_ptr || !k->data_ptr || !v->data_ptr) return nullptr;
  auto q_emb = Tensor::MakeGPUTensor(static_cast<size_t>(hidden) * cur_size, dtype_);
  auto out = Tensor::MakeGPUTensor(static_cast<size_t>(hidden) * cur_size, dtype_);
  if (!q_emb || !out || !q_emb->data_ptr || !out->data_ptr) return nullptr;  // nothing launched yet
  hip_last_status() = 0;
  if (cur_size == 1 && n_heads_ / n_kv_heads_ <= 16) {
    // a decode step: rotary embedding, append and attention in one pass over the cache
    hip_decode_step_gqa_layer(out->data_ptr, k_cache->data_ptr, v_cache->data_ptr, freq_cis_->data_ptr,
                              q->data_ptr, k->data_ptr, v->data_ptr, static_cast<int>(ctx.prev_pos),
                              n_heads_ / n_kv_heads_, n_kv_heads_, head_dim_, neox_, dtype_, ctx.gpu_stream);
  } else {
    hip_rope_kv_append_layer(q_emb->data_ptr, k_cache->data_ptr, v_cache->data_ptr,
                             freq_cis_->data_ptr, q->data_ptr, k->data_ptr, v->data_ptr,
                             static_cast<int>(ctx.prev_pos), cur_size, n_heads_, n_kv_heads_,
                             head_dim_, neox_, dtype_, ctx.gpu_stream);
    hip_flash_attn_gqa_layer(out->data_ptr, q_emb->data_ptr, k_cache->data_ptr, v_cache->data_ptr,
                             cur_size, static_cast<int>(ctx.cur_pos), static_cast<int>(ctx.prev_pos),
                             n_heads_ / n_kv_heads_, n_kv_heads_, head_dim_, dtype_, ctx.gpu_stream);
  }
  // q_emb goes back to the pool when this scope ends while the attention launch may
  // still read it: drain the stream first, the rule the reference states at
  // src/llama2_layer_npu.cpp:605-608.
  CHECK_LLMHIP(llmhip_stream_sync(ctx.gpu_stream));
  // a rejected or failed launch leaves `out` unwritten: report it instead of returning garbage
  if (hip_last_status() != 0) return nullptr;
  return out;
}

// ---------------------------------------------------------------------------
// profiler
// ---------------------------------------------------------------------------
static uint64_t steady_us() {
  return static_cast<uint64_t>(std::chrono::duration_cast<std::chrono::microseconds>(
                                   std::chrono::steady_clock::now().time_since_epoch())
                                   .count());
}

static std::string json_escape(const std::string &in) {
  std::string out;
  out.reserve(in.size() + 2);
  for (char ch : in) {
    switch (ch) {
      case '"': out += "\\\""; break;
      case '\\': out += "\\\\"; break;
      case '\n': out += "\\n"; break;
      case '\t': out += "\\t"; break;
      default:
        if (static_cast<unsigned char>(ch) < 0x20) {
          char buf[8];
          snprintf(buf, sizeof(buf), "\\u%04x", ch);
          out += buf;
        } else {
          out += ch;
        }
    }
  }
  return out;
}

bool AppProfiler::StartLogging(const std::string &log_path) {
  profile_file_.open(log_path.c_str());
  if (!profile_file_) return false;
  profile_file_ << "[\n";
  first_record_ = true;
  count_ = 0;
  start_us_count_ = steady_us();
  return true;
}

void AppProfiler::RecordEvent(const std::string &name, const std::string &info, const char *file,
                              int lineno, uint64_t ts_us_steady, double dur_us) {
  if (!profile_file_.is_open()) return;
  if (first_record_)
    first_record_ = false;
  else
    profile_file_ << ",\n";
  profile_file_ << "{\"name\":\"" << json_escape(name) << "\",\"ph\":\"X\",\"pid\":0,\"ts\":"
                << (ts_us_steady - start_us_count_) << ",\"dur\":" << dur_us
                << ",\"args\":{\"file\":\"" << json_escape(file ? file : "") << "\",\"lineno\":" << lineno
                << ",\"info\":\"" << json_escape(info) << "\"}}";
  ++count_;
}

void AppProfiler::Finish() {
  if (!profile_file_.is_open()) return;
  profile_file_ << "\n]\n";
  profile_file_.close();
}

AppProfileGuard::AppProfileGuard(const char *name, const char *info, gpuStream_t stream,
                                 AppProfiler *profiler, const char *fname, int lineno,
                                 bool is_profiling)
    : record_name_(name), record_info_(info), record_file_name_(fname), record_file_lineno_(lineno),
      stream_(stream), profiler_(profiler), is_profiling_(is_profiling && profiler != nullptr) {
  if (is_profiling_) {
    CHECK_LLMHIP(llmhip_event_create(&event_));
    CHECK_LLMHIP(llmhip_event_record(event_, stream_));
    start_us_ = steady_us();
  }
}

AppProfileGuard::~AppProfileGuard() {
  if (!is_profiling_) return;
  void *end_event = nullptr;
  CHECK_LLMHIP(llmhip_event_create(&end_event));
  CHECK_LLMHIP(llmhip_event_record(end_event, stream_));
  CHECK_LLMHIP(llmhip_stream_sync(stream_));
  float duration_ms = 0.0f;
  CHECK_LLMHIP(llmhip_event_elapsed_ms(&duration_ms, event_, end_event));
  CHECK_LLMHIP(llmhip_event_destroy(event_));
  CHECK_LLMHIP(llmhip_event_destroy(end_event));
  profiler_->RecordEvent(record_name_, record_info_, record_file_name_, record_file_lineno_,
                         start_us_, static_cast<double>(duration_ms) * 1000.0);
}

// ---------------------------------------------------------------------------
// projections and the whole attention block
// ---------------------------------------------------------------------------
bool MatmulLayerGPUImpl::Init(const void *host_weight, const float *host_bias, size_t n_, size_t k_,
                              DataType dtype) {
  if (!host_weight || n_ == 0 || k_ == 0 || n_ % 16 != 0 || k_ % 16 != 0 ||
      (dtype != DT_FLOAT16 && dtype != DT_BFLOAT16))
    return false;
  n = n_;
  k = k_;
  dtype_ = dtype;
  weight_ = Tensor::MakeGPUTensor(n * k, dtype);
  if (!weight_ || !weight_->data_ptr) return false;
  if (llmhip_memcpy_h2d(weight_->data_ptr, host_weight, n * k * SizeOfTensor(1, dtype)) != 0) return false;
  bias_.reset();
  if (host_bias) {
    bias_ = Tensor::MakeGPUTensor(n, DT_FLOAT32);
    if (!bias_ || !bias_->data_ptr) return false;
    if (llmhip_memcpy_h2d(bias_->data_ptr, host_bias, n * sizeof(float)) != 0) return false;
  }
  return true;
}

std::shared_ptr<Tensor> MatmulLayerGPUImpl::Forward(std::shared_ptr<Tensor> input, InferenceCtx &ctx) {
  const int m = static_cast<int>(ctx.cur_size);
  if (!input || !input->data_ptr) return nullptr;
  auto output = Tensor::MakeGPUTensor(n * ctx.cur_size, dtype_);
  if (!output || !output->data_ptr) return nullptr;
  char info[96];
  snprintf(info, sizeof(info), "m %d n %zu k %zu", m, n, k);
  APP_PROFILE("MatmulLayer", info, ctx.gpu_stream, ctx.profiler, ctx.is_profiling);
  if (bias_)
    hip_matmul_bias_layer(output->data_ptr, input->data_ptr, weight_->data_ptr, bias_->data_ptr, m,
                          static_cast<int>(n), static_cast<int>(k), dtype_, ctx.gpu_stream);
  else
    hip_matmul_layer(output->data_ptr, input->data_ptr, weight_->data_ptr, m, static_cast<int>(n),
                     static_cast<int>(k), dtype_, ctx.gpu_stream);
  return output;
}

bool AttentionBlockGPUImpl::Init(const Weights &w, int hidden_dim, int n_heads, int n_kv_heads,
                                 int max_seq_len, DataType dtype, bool rope_is_neox_style,
                                 std::shared_ptr<Tensor> freq_cis_gpu) {
  if (hidden_dim < 1 || n_heads < 1 || hidden_dim % n_heads != 0) return false;
  const int head_dim = hidden_dim / n_heads;
  hidden_dim_ = hidden_dim;
  dtype_ = dtype;
  const size_t kv_dim = static_cast<size_t>(n_kv_heads) * head_dim;
  return attention.Init(n_heads, n_kv_heads, head_dim, max_seq_len, dtype, rope_is_neox_style,
                        freq_cis_gpu) &&
         q_proj.Init(w.wq, w.bq, hidden_dim, hidden_dim, dtype) &&
         k_proj.Init(w.wk, w.bk, kv_dim, hidden_dim, dtype) &&
         v_proj.Init(w.wv, w.bv, kv_dim, hidden_dim, dtype) &&
         o_proj.Init(w.wo, nullptr, hidden_dim, hidden_dim, dtype);
}

std::shared_ptr<Tensor> AttentionBlockGPUImpl::Forward(std::shared_ptr<Tensor> normed,
                                                       std::shared_ptr<Tensor> residual,
                                                       InferenceCtx &ctx) {
  if (!residual || !residual->data_ptr) return nullptr;
  hip_last_status() = 0;
  auto q = q_proj.Forward(normed, ctx);
  auto k = k_proj.Forward(normed, ctx);
  auto v = v_proj.Forward(normed, ctx);
  // Every early return below drains the stream first: the temporaries go back to the pool at scope
  // exit while launches that read or write them may still be queued.
  auto bail = [&]() -> std::shared_ptr<Tensor> {
    CHECK_LLMHIP(llmhip_stream_sync(ctx.gpu_stream));
    return nullptr;
  };
  if (!q || !k || !v || hip_last_status() != 0) return bail();
  std::shared_ptr<Tensor> attn;
  {
    char info[96];
    snprintf(info, sizeof(info), "cur_size %zu cur_pos %zu", ctx.cur_size, ctx.cur_pos);
    APP_PROFILE("RoPE+KVAppend+FlashAttnGQA", info, ctx.gpu_stream, ctx.profiler, ctx.is_profiling);
    attn = attention.Forward(q, k, v, ctx);
  }
  if (!attn) return bail();
  auto proj = o_proj.Forward(attn, ctx);
  auto out = Tensor::MakeGPUTensor(static_cast<size_t>(hidden_dim_) * ctx.cur_size, dtype_);
  if (!proj || !out || !out->data_ptr) return bail();
  {
    APP_PROFILE("Add", "attn output + input", ctx.gpu_stream, ctx.profiler, ctx.is_profiling);
    hip_add_layer(out->data_ptr, residual->data_ptr, proj->data_ptr,
                  static_cast<int>(ctx.cur_size) * hidden_dim_, dtype_, ctx.gpu_stream);
  }
  // temporaries return to the pool at scope exit: drain first (src/llama2_layer_npu.cpp:605-608)
  CHECK_LLMHIP(llmhip_stream_sync(ctx.gpu_stream));
  if (hip_last_status() != 0) return nullptr;
  return out;
}

}  // namespace llm_simple_amd
