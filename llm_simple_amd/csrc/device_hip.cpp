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

static const GPUAllocator::EventBackend kHipEvents = {&llmhip_event_create, &llmhip_event_record, &llmhip_event_query,
                                                      &llmhip_event_sync,   &llmhip_event_destroy, &llmhip_device_sync};

GPUAllocator::GPUAllocator() : raw_alloc_(&llmhip_malloc), raw_free_(&llmhip_free), ev_(kHipEvents) {}

GPUAllocator &GPUAllocator::GetInstance() {
  static GPUAllocator instance;
  return instance;
}
void *GPUAllocator::Allocate(size_t size, gpuStream_t stream) { return GetInstance().AllocateImpl(size, stream); }
void GPUAllocator::Deallocate(void *ptr, gpuStream_t stream) { GetInstance().DeallocateImpl(ptr, stream); }

void GPUAllocator::SetBackend(RawAlloc a, RawFree f) {
  ReleaseAll();
  raw_alloc_ = a ? a : &llmhip_malloc;
  raw_free_ = f ? f : &llmhip_free;
}

void GPUAllocator::SetEventBackend(const EventBackend *b) {
  ReleaseAll();
  ev_ = b ? *b : kHipEvents;
}

size_t GPUAllocator::PendingBlocks() const {
  size_t n = 0;
  for (const auto &kv : cache_)
    if (kv.second.stream != NoStream()) ++n;
  return n;
}

// Waits until nothing queued on the device can touch a cached block; every block is then free for
// everybody.
void GPUAllocator::DrainAll() {
  if (PendingBlocks() == 0) return;
  int rc = ev_.device_sync();
  if (rc != LLMHIP_OK) hip_last_status() = rc;
  for (auto &kv : cache_) kv.second.stream = NoStream();
  for (auto &st : streams_) st.second.completed = st.second.fenced = st.second.next_ticket - 1;
}

void GPUAllocator::ForgetStream(gpuStream_t stream) {
  for (auto &kv : cache_)
    if (kv.second.stream == stream) kv.second.stream = NoStream();
  auto it = streams_.find(stream);
  if (it != streams_.end()) {
    if (it->second.event) ev_.destroy(it->second.event);
    streams_.erase(it);
  }
}

void GPUAllocator::ReleaseAll() {
  DrainAll();
  for (auto &kv : cache_) {
    raw_free_(kv.second.ptr);
    owned_bytes_ -= kv.first;
    ptr_size_.erase(kv.second.ptr);
  }
  cache_.clear();
  for (auto &st : streams_)
    if (st.second.event) ev_.destroy(st.second.event);
  streams_.clear();
}

// May `requester` take block b now?  A block pending on another stream needs an event of that
// stream, recorded after the block was freed, to have completed.  The event is recorded here, when
// somebody first asks (it then covers every block the stream has freed so far); with may_wait the
// call blocks until it has completed.
bool GPUAllocator::Usable(const Block &b, gpuStream_t requester, bool may_wait) {
  if (b.stream == NoStream()) return true;
  if (b.stream == AnyStream()) {
    if (!may_wait) return false;
    DrainAll();
    return true;
  }
  if (b.stream == requester) return true;  // queued behind its last use
  StreamState &st = streams_[b.stream];
  if (b.ticket <= st.completed) return true;
  const bool fence_in_flight = st.fenced > st.completed;
  if (fence_in_flight && ev_.query(st.event) == LLMHIP_OK) {
    st.completed = st.fenced;
    if (b.ticket <= st.completed) return true;
  }
  if (st.fenced < b.ticket && (may_wait || st.fenced == st.completed)) {
    // no event in flight covers this block (re-recording one that is in flight would only move it
    // later, so that is left to a caller that waits anyway)
    if (!st.event && ev_.create(&st.event) != LLMHIP_OK) return false;
    if (ev_.record(st.event, b.stream) != LLMHIP_OK) return false;
    st.fenced = st.next_ticket - 1;
    ++fence_events_;
  }
  if (!may_wait) return false;
  int rc = ev_.sync(st.event);
  if (rc != LLMHIP_OK) {
    hip_last_status() = rc;
    return false;
  }
  st.completed = st.fenced;
  return b.ticket <= st.completed;
}

void *GPUAllocator::AllocateImpl(size_t size, gpuStream_t stream) {
  // smallest cached block that fits and that this requester may take now
  auto first_fit = cache_.lower_bound(size);
  for (auto it = first_fit; it != cache_.end(); ++it) {
    if (Usable(it->second, stream, false)) {
      void *p = it->second.ptr;
      cache_.erase(it);
      return p;
    }
  }
  // Everything that fits is pending on other streams.  Below the byte cap a fresh block is cheaper
  // than a wait; at the cap, wait for the smallest one.
  if (first_fit != cache_.end() && owned_bytes_ + size > dev_mem_max_ && Usable(first_fit->second, stream, true)) {
    first_fit = cache_.lower_bound(size);  // (a drain may have rewritten tags, not positions)
    void *p = first_fit->second.ptr;
    cache_.erase(first_fit);
    return p;
  }
  void *p = nullptr;
  int rc = raw_alloc_(&p, size);
  if ((rc != LLMHIP_OK || p == nullptr) && first_fit != cache_.end() && Usable(first_fit->second, stream, true)) {
    // the device is out of memory but a pending block fits: wait for it
    first_fit = cache_.lower_bound(size);
    p = first_fit->second.ptr;
    cache_.erase(first_fit);
    return p;
  }
  if (rc != LLMHIP_OK || p == nullptr) {
    hip_last_status() = rc ? rc : LLMHIP_ERR_INVALID_ARG;
    std::fprintf(stderr, "GPUAllocator: device allocation of %zu bytes failed: %s\n", size,
                 llmhip_error_string(rc));
    return nullptr;
  }
  owned_bytes_ += size;
  ptr_size_[p] = size;
  // after a miss, trim the cache while the pool owns more than the threshold (blocks that queued
  // work may still touch are given back only after a drain)
  if (owned_bytes_ > dev_mem_max_ && !cache_.empty()) {
    DrainAll();
    while (owned_bytes_ > dev_mem_max_ && !cache_.empty()) {
      auto small = cache_.begin();
      raw_free_(small->second.ptr);
      owned_bytes_ -= small->first;
      ptr_size_.erase(small->second.ptr);
      cache_.erase(small);
    }
  }
  return p;
}

void GPUAllocator::DeallocateImpl(void *ptr, gpuStream_t stream) {
  if (ptr == nullptr) return;
  auto it = ptr_size_.find(ptr);
  if (it == ptr_size_.end()) {
    std::fprintf(stderr, "GPUAllocator: %p was not allocated here\n", ptr);
    return;
  }
  Block b{ptr, stream, 0};
  if (stream != NoStream() && stream != AnyStream()) b.ticket = streams_[stream].next_ticket++;
  cache_.emplace(it->second, b);
}

Tensor::~Tensor() {
  if (dev_type == DEV_GPU)
    GPUAllocator::Deallocate(data_ptr, stream_tag);
  else if (dev_type == DEV_CPU)
    CPUAllocator::Deallocate(data_ptr);
}

void Tensor::RecordStream(gpuStream_t stream) {
  if (stream_tag == GPUAllocator::NoStream())
    stream_tag = stream;
  else if (stream_tag != stream)
    stream_tag = GPUAllocator::AnyStream();
}

std::shared_ptr<Tensor> Tensor::MakeCPUTensor(size_t size, DataType dtype) {
  auto t = std::make_shared<Tensor>();
  t->data_size = size;
  t->data_type = dtype;
  t->dev_type = DEV_CPU;
  t->data_ptr = CPUAllocator::Allocate(SizeOfTensor(size, dtype));
  return t;
}

std::shared_ptr<Tensor> Tensor::MakeGPUTensor(size_t size, DataType dtype, gpuStream_t stream) {
  auto t = std::make_shared<Tensor>();
  t->data_size = size;
  t->data_type = dtype;
  t->dev_type = DEV_GPU;
  t->data_ptr = GPUAllocator::Allocate(SizeOfTensor(size, dtype), stream);
  // a block obtained for a stream may still be in use by work queued on it: the tag stays with
  // the tensor from birth, so that freeing it unused does not release the block to everybody
  t->stream_tag = stream;
  return t;
}

std::shared_ptr<Tensor> Tensor::to(DeviceType to_dev) {
  if (to_dev == dev_type) return shared_from_this();
  const size_t bytes = SizeOfTensor(data_size, data_type);
  if (dev_type == DEV_GPU && to_dev == DEV_CPU) {
    auto r = MakeCPUTensor(data_size, data_type);
    // the copy must see what work queued on the tensor's stream produces
    if (stream_tag == GPUAllocator::AnyStream())
      CHECK_LLMHIP(llmhip_device_sync());
    else if (stream_tag != GPUAllocator::NoStream())
      CHECK_LLMHIP(llmhip_stream_sync(stream_tag));
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
  if (!freq_cis_gpu || !freq_cis_gpu->data_ptr) return false;
  freq_cis_owner_ = freq_cis_gpu;
  return Init(n_heads, n_kv_heads, head_dim, max_seq_len, dtype, rope_is_neox_style,
              static_cast<float *>(freq_cis_gpu->data_ptr));
}

bool AttentionGPUImpl::Init(int n_heads, int n_kv_heads, int head_dim, int max_seq_len,
                            DataType dtype, bool rope_is_neox_style, float *freq_cis_dev) {
  if (n_heads < 1 || n_kv_heads < 1 || n_heads % n_kv_heads != 0 || head_dim != 128 ||
      max_seq_len < 1 || (dtype != DT_FLOAT16 && dtype != DT_BFLOAT16) || !freq_cis_dev)
    return false;
  n_heads_ = n_heads;
  n_kv_heads_ = n_kv_heads;
  head_dim_ = head_dim;
  max_seq_len_ = max_seq_len;
  dtype_ = dtype;
  neox_ = rope_is_neox_style;
  freqs_cis_ = freq_cis_dev;
  const size_t cache_elems = static_cast<size_t>(max_seq_len) * n_kv_heads * head_dim;
  k_cache = Tensor::MakeGPUTensor(cache_elems, dtype);
  v_cache = Tensor::MakeGPUTensor(cache_elems, dtype);
  return k_cache->data_ptr != nullptr && v_cache->data_ptr != nullptr;
}

// True when the positions of a step are consistent with a cache of max_seq_len rows: the step appends
// rows [prev_pos, cur_pos) and reads rows [0, cur_pos).  Anything else would write past the cache.
static bool ctx_fits_cache(const InferenceCtx &ctx, size_t max_seq_len) {
  return ctx.cur_size >= 1 && ctx.prev_pos + ctx.cur_size == ctx.cur_pos && ctx.cur_pos <= max_seq_len &&
         ctx.cur_pos <= static_cast<size_t>(INT32_MAX);
}

std::shared_ptr<Tensor> AttentionGPUImpl::Forward(std::shared_ptr<Tensor> q,
                                                  std::shared_ptr<Tensor> k,
                                                  std::shared_ptr<Tensor> v, InferenceCtx &ctx) {
  const int cur_size = static_cast<int>(ctx.cur_size);
  const int hidden = n_heads_ * head_dim_;
  if (!ctx_fits_cache(ctx, static_cast<size_t>(max_seq_len_))) return nullptr;
  if (!q || !k || !v || !q->data_ptr || !k->data_ptr || !v->data_ptr) return nullptr;
  // Every tensor of this step is tied to the stream: the pool hands a freed block to another stream,
  // or to host code, only after the work queued here is done, so nothing below waits for the GPU
  // (the reference drains the stream once per layer instead, src/llama2_layer_npu.cpp:990-993).
  gpuStream_t stream = ctx.gpu_stream;
  auto out = Tensor::MakeGPUTensor(static_cast<size_t>(hidden) * cur_size, dtype_, stream);
  if (!out || !out->data_ptr) return nullptr;  // nothing launched yet
  for (Tensor *t : {q.get(), k.get(), v.get(), k_cache.get(), v_cache.get()}) t->RecordStream(stream);
  if (freq_cis_owner_) freq_cis_owner_->RecordStream(stream);
  hip_last_status() = 0;
  if (cur_size == 1 && n_heads_ / n_kv_heads_ <= 16) {
    // a decode step: rotary embedding, append and attention in one pass over the cache
    hip_decode_step_gqa_layer(out->data_ptr, k_cache->data_ptr, v_cache->data_ptr, freqs_cis_,
                              q->data_ptr, k->data_ptr, v->data_ptr, static_cast<int>(ctx.prev_pos),
                              n_heads_ / n_kv_heads_, n_kv_heads_, head_dim_, neox_, dtype_, ctx.gpu_stream);
  } else {
    auto q_emb = Tensor::MakeGPUTensor(static_cast<size_t>(hidden) * cur_size, dtype_, stream);
    if (!q_emb || !q_emb->data_ptr) return nullptr;
    hip_rope_kv_append_layer(q_emb->data_ptr, k_cache->data_ptr, v_cache->data_ptr,
                             freqs_cis_, q->data_ptr, k->data_ptr, v->data_ptr,
                             static_cast<int>(ctx.prev_pos), cur_size, n_heads_, n_kv_heads_,
                             head_dim_, neox_, dtype_, ctx.gpu_stream);
    hip_flash_attn_gqa_layer(out->data_ptr, q_emb->data_ptr, k_cache->data_ptr, v_cache->data_ptr,
                             cur_size, static_cast<int>(ctx.cur_pos), static_cast<int>(ctx.prev_pos),
                             n_heads_ / n_kv_heads_, n_kv_heads_, head_dim_, dtype_, ctx.gpu_stream);
    // q_emb returns to the pool here, tagged with the stream: the attention launch that still reads it
    // is queued ahead of whatever gets the block next
  }
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
  auto output = Tensor::MakeGPUTensor(n * ctx.cur_size, dtype_, ctx.gpu_stream);
  if (!output || !output->data_ptr) return nullptr;
  input->RecordStream(ctx.gpu_stream);
  weight_->RecordStream(ctx.gpu_stream);
  if (bias_) bias_->RecordStream(ctx.gpu_stream);
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
  // No return below waits for the GPU: every temporary carries the stream's tag, and the pool keeps
  // its block away from other streams and from host code until the work queued here is done.
  if (!q || !k || !v || hip_last_status() != 0) return nullptr;
  std::shared_ptr<Tensor> attn;
  {
    char info[96];
    snprintf(info, sizeof(info), "cur_size %zu cur_pos %zu", ctx.cur_size, ctx.cur_pos);
    APP_PROFILE("RoPE+KVAppend+FlashAttnGQA", info, ctx.gpu_stream, ctx.profiler, ctx.is_profiling);
    attn = attention.Forward(q, k, v, ctx);
  }
  if (!attn) return nullptr;
  auto proj = o_proj.Forward(attn, ctx);
  auto out = Tensor::MakeGPUTensor(static_cast<size_t>(hidden_dim_) * ctx.cur_size, dtype_, ctx.gpu_stream);
  if (!proj || !out || !out->data_ptr) return nullptr;
  residual->RecordStream(ctx.gpu_stream);
  {
    APP_PROFILE("Add", "attn output + input", ctx.gpu_stream, ctx.profiler, ctx.is_profiling);
    hip_add_layer(out->data_ptr, residual->data_ptr, proj->data_ptr,
                  static_cast<int>(ctx.cur_size) * hidden_dim_, dtype_, ctx.gpu_stream);
  }
  if (hip_last_status() != 0) return nullptr;
  return out;
}

// ---------------------------------------------------------------------------
// device dispatch
// ---------------------------------------------------------------------------
InferenceCtx::InferenceCtx(ModelBase *model_, size_t cur_pos_, size_t prev_pos_)
    : model(model_), cur_pos(cur_pos_), prev_pos(prev_pos_), cur_size(cur_pos_ - prev_pos_),
      gpu_stream(model_ ? model_->model_stream : nullptr), profiler(model_ ? &model_->profiler : nullptr),
      is_profiling(model_ ? model_->is_profiling : false) {}

bool ModelBase::InitFreqCIS(const float theta, const DataType dt) {
  if (n_heads < 1 || hidden_dim < 1 || config.max_seq_len < 1) return false;
  const int hd = hidden_dim / n_heads;
  auto host = MakeFreqCIS(hd, config.max_seq_len, theta, dt);
  if (config.device_type == DEV_GPU) {
    freq_cis_holder_ = host->to(DEV_GPU);
    if (!freq_cis_holder_ || !freq_cis_holder_->data_ptr) return false;
  } else {
    freq_cis_holder_ = host;
  }
  freq_cis = static_cast<float *>(freq_cis_holder_->data_ptr);
  return true;
}

RoPELayerImpl::~RoPELayerImpl() {}

bool RoPELayerImpl::Init(ModelBase *model, const std::string & /*weight_path*/) {
  if (!model || model->n_heads < 1 || model->hidden_dim % model->n_heads != 0) return false;
  hidden_dim = model->hidden_dim;
  head_dim = model->hidden_dim / model->n_heads;
  n_heads = model->n_heads;
  rope_dim = static_cast<size_t>(model->config.max_seq_len) * model->hidden_dim;
  weight_size = sizeof(float) * rope_dim;
  freqs_cis = model->freq_cis;
  rope_is_neox_style = model->config.rope_is_neox_style;
  dtype = model->config.data_type;
  return true;
}

void RoPELayerImpl::UnInit() {}

RoPELayerGPUImpl::~RoPELayerGPUImpl() {}

bool RoPELayerGPUImpl::Init(ModelBase *model, const std::string &weight_path) {
  if (!RoPELayerImpl::Init(model, weight_path)) return false;
  return freqs_cis != nullptr && head_dim == 128 && (dtype == DT_FLOAT16 || dtype == DT_BFLOAT16);
}

std::tuple<std::shared_ptr<Tensor>, std::shared_ptr<Tensor>> RoPELayerGPUImpl::Forward(
    std::shared_ptr<Tensor> input_q, std::shared_ptr<Tensor> input_k, InferenceCtx &ctx) {
  std::shared_ptr<Tensor> none;
  if (!input_q || !input_k || !input_q->data_ptr || !input_k->data_ptr || ctx.cur_size < 1)
    return std::make_tuple(none, none);
  auto output_q = Tensor::MakeGPUTensor(hidden_dim * ctx.cur_size, dtype, ctx.gpu_stream);
  auto output_k = Tensor::MakeGPUTensor(hidden_dim * ctx.cur_size, dtype, ctx.gpu_stream);
  if (!output_q->data_ptr || !output_k->data_ptr) return std::make_tuple(none, none);
  input_q->RecordStream(ctx.gpu_stream);
  input_k->RecordStream(ctx.gpu_stream);
  char info[128];
  snprintf(info, sizeof(info), "pos: %zu seq len: %zu n_head %zu head_dim %zu hidden_dim %zu", ctx.prev_pos,
           ctx.cur_size, n_heads, head_dim, hidden_dim);
  APP_PROFILE("RoPELayer", info, ctx.gpu_stream, ctx.profiler, ctx.is_profiling);
  hip_rope_layer(output_q->data_ptr, output_k->data_ptr, freqs_cis, input_q->data_ptr, input_k->data_ptr,
                 static_cast<int>(ctx.prev_pos), static_cast<int>(ctx.cur_size), static_cast<int>(n_heads),
                 static_cast<int>(hidden_dim), rope_is_neox_style, dtype, ctx.gpu_stream);
  return std::make_tuple(output_q, output_k);
}

RoPELayer::~RoPELayer() { delete impl; }

std::tuple<std::shared_ptr<Tensor>, std::shared_ptr<Tensor>> RoPELayer::Forward(std::shared_ptr<Tensor> input_q,
                                                                              std::shared_ptr<Tensor> input_k,
                                                                              InferenceCtx &ctx) {
  return impl->Forward(input_q, input_k, ctx);
}

bool RoPELayer::Init(ModelBase *model, const std::string &weight_path) {
  delete impl;
  impl = nullptr;
  if (!model) return false;
  switch (model->config.device_type) {
    case DEV_GPU:
      impl = new RoPELayerGPUImpl();
      break;
    default:  // DEV_NPU and DEV_CPU implementations live in the reference, not here
      std::fprintf(stderr, "invalid device type\n");
      return false;
  }
  return impl->Init(model, weight_path);
}

void RoPELayer::UnInit() {}

AttentionLayerImpl::~AttentionLayerImpl() {}

bool AttentionLayerImpl::Init(ModelBase *model, int /*layer_no*/) {
  if (!model || model->n_heads < 1 || model->hidden_dim % model->n_heads != 0) return false;
  hidden_dim = model->hidden_dim;
  head_dim = model->hidden_dim / model->n_heads;
  n_heads = model->n_heads;
  n_kv_heads = model->n_kv_heads > 0 ? model->n_kv_heads : model->n_heads;
  max_seq_len = model->config.max_seq_len;
  dtype = model->config.data_type;
  return true;
}

void AttentionLayerImpl::UnInit() {}

bool Llama2AttentionGPUImpl::Init(ModelBase *model, int layer_no) {
  if (!AttentionLayerImpl::Init(model, layer_no)) return false;
  if (n_kv_heads != n_heads || head_dim != 128 || max_seq_len < 1 || (dtype != DT_FLOAT16 && dtype != DT_BFLOAT16))
    return false;
  if (!rope_emb.Init(model, "")) return false;
  // src/llama2_layer_npu.cpp:726-727
  k_cache = Tensor::MakeGPUTensor(n_heads * head_dim * max_seq_len, dtype);
  v_cache = Tensor::MakeGPUTensor(n_heads * head_dim * max_seq_len, dtype);
  return k_cache->data_ptr != nullptr && v_cache->data_ptr != nullptr;
}

std::shared_ptr<Tensor> Llama2AttentionGPUImpl::Forward(std::shared_ptr<Tensor> q, std::shared_ptr<Tensor> k,
                                                        std::shared_ptr<Tensor> v, InferenceCtx &ctx) {
  if (!ctx_fits_cache(ctx, max_seq_len) || !v || !v->data_ptr) return nullptr;
  hip_last_status() = 0;
  auto q_k_emb = rope_emb.Forward(q, k, ctx);
  auto q_emb = std::get<0>(q_k_emb);
  auto k_emb = std::get<1>(q_k_emb);
  if (!q_emb || !k_emb) return nullptr;
  // update kv cache
  const size_t copy_size = ctx.cur_size * n_heads * head_dim * sizeof(uint16_t);
  const size_t copy_offset = ctx.prev_pos * n_heads * head_dim * sizeof(uint16_t);
  for (Tensor *t : {v.get(), k_cache.get(), v_cache.get()}) t->RecordStream(ctx.gpu_stream);
  {
    char info[64];
    snprintf(info, sizeof(info), "copy_size %zu byte", copy_size);
    APP_PROFILE("UpdateKVCache", info, ctx.gpu_stream, ctx.profiler, ctx.is_profiling);
    CHECK_LLMHIP(llmhip_memcpy_d2d_async(static_cast<uint8_t *>(k_cache->data_ptr) + copy_offset, k_emb->data_ptr,
                                         copy_size, ctx.gpu_stream));
    CHECK_LLMHIP(llmhip_memcpy_d2d_async(static_cast<uint8_t *>(v_cache->data_ptr) + copy_offset, v->data_ptr,
                                         copy_size, ctx.gpu_stream));
  }
  auto tmp_output_tensor = Tensor::MakeGPUTensor(hidden_dim * ctx.cur_size, dtype, ctx.gpu_stream);
  if (!tmp_output_tensor->data_ptr) return nullptr;
  hip_flash_attn_opt_prefill_layer(tmp_output_tensor->data_ptr, q_emb->data_ptr, k_cache->data_ptr,
                                   v_cache->data_ptr, static_cast<int>(ctx.cur_size), static_cast<int>(ctx.cur_pos),
                                   static_cast<int>(ctx.prev_pos), static_cast<int>(n_heads),
                                   static_cast<int>(head_dim), dtype, ctx.gpu_stream);
  if (hip_last_status() != 0) return nullptr;
  return tmp_output_tensor;
}

bool Qwen2AttentionGPUImpl::Init(ModelBase *model, int layer_no) {
  if (!AttentionLayerImpl::Init(model, layer_no)) return false;
  if (!impl_.Init(static_cast<int>(n_heads), static_cast<int>(n_kv_heads), static_cast<int>(head_dim),
                  static_cast<int>(max_seq_len), dtype, model->config.rope_is_neox_style, model->freq_cis))
    return false;
  k_cache = impl_.k_cache;
  v_cache = impl_.v_cache;
  return true;
}

std::shared_ptr<Tensor> Qwen2AttentionGPUImpl::Forward(std::shared_ptr<Tensor> q, std::shared_ptr<Tensor> k,
                                                       std::shared_ptr<Tensor> v, InferenceCtx &ctx) {
  return impl_.Forward(q, k, v, ctx);
}

Llama2AttentionLayer::~Llama2AttentionLayer() { delete impl; }

std::shared_ptr<Tensor> Llama2AttentionLayer::Forward(std::shared_ptr<Tensor> q, std::shared_ptr<Tensor> k,
                                                      std::shared_ptr<Tensor> v, InferenceCtx &ctx) {
  return impl->Forward(q, k, v, ctx);
}

bool Llama2AttentionLayer::Init(ModelBase *model, int layer_no) {
  delete impl;
  impl = nullptr;
  if (!model) return false;
  switch (model->config.device_type) {
    case DEV_GPU:
      impl = new Llama2AttentionGPUImpl();
      break;
    default:
      std::fprintf(stderr, "invalid device type\n");
      return false;
  }
  return impl->Init(model, layer_no);
}

void Llama2AttentionLayer::UnInit() {}

Qwen2AttentionLayer::~Qwen2AttentionLayer() { delete impl; }

std::shared_ptr<Tensor> Qwen2AttentionLayer::Forward(std::shared_ptr<Tensor> q, std::shared_ptr<Tensor> k,
                                                     std::shared_ptr<Tensor> v, InferenceCtx &ctx) {
  return impl->Forward(q, k, v, ctx);
}

bool Qwen2AttentionLayer::Init(ModelBase *model, int layer_no) {
  delete impl;
  impl = nullptr;
  if (!model) return false;
  switch (model->config.device_type) {
    case DEV_GPU:
      impl = new Qwen2AttentionGPUImpl();
      break;
    default:
      std::fprintf(stderr, "invalid device type\n");
      return false;
  }
  return impl->Init(model, layer_no);
}

void Qwen2AttentionLayer::UnInit() {}

}  // namespace llm_simple_amd
