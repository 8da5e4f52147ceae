// Host-only checks of the device layer and of the C ABI's argument validation.
// Needs no GPU: the allocator runs on an injected host backend and every ABI
// call below is rejected (or reports "no device") before anything is launched.
#include <cmath>
#include <chrono>
#include <cstdio>
#include <fstream>
#include <iterator>
#include <string>
#include <cstdlib>
#include <vector>

#include "../../llm_simple_amd/csrc/device_hip.hpp"

using namespace llm_simple_amd;

static int g_fail = 0, g_allocs = 0, g_frees = 0;
#define EXPECT(c)                                                       \
  do {                                                                  \
    if (!(c)) {                                                         \
      std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #c);          \
      ++g_fail;                                                         \
    }                                                                   \
  } while (0)

static int host_alloc(void **p, size_t n) {
  *p = std::malloc(n ? n : 1);
  ++g_allocs;
  return *p ? 0 : 2;
}
static int host_free(void *p) {
  std::free(p);
  ++g_frees;
  return 0;
}
static int failing_alloc(void **p, size_t) {
  *p = nullptr;
  return 2;  // hipErrorOutOfMemory
}

static void test_sizes() {
  EXPECT(SizeOfTensor(10, DT_FLOAT16) == 20);
  EXPECT(SizeOfTensor(10, DT_BFLOAT16) == 20);
  EXPECT(SizeOfTensor(10, DT_FLOAT32) == 40);
  EXPECT(SizeOfTensor(3, DT_INT64) == 24);
  EXPECT(SizeOfTensor(3, DT_UINT8) == 3);
  EXPECT(SizeOfTensor(1, static_cast<DataType>(99)) == static_cast<size_t>(-1));
  EXPECT(DEV_GPU == 1 && DT_FLOAT16 == 4 && DT_BFLOAT16 == 5);
}

static void test_allocator_pool() {
  GPUAllocator &a = GPUAllocator::GetInstance();
  a.SetBackend(host_alloc, host_free);
  a.SetByteCap(1 << 20);
  g_allocs = g_frees = 0;
  void *p1 = GPUAllocator::Allocate(1000);
  void *p2 = GPUAllocator::Allocate(4000);
  void *p3 = GPUAllocator::Allocate(2000);
  EXPECT(g_allocs == 3 && a.OwnedBytes() == 7000);
  GPUAllocator::Deallocate(p2);
  GPUAllocator::Deallocate(p1);
  GPUAllocator::Deallocate(p3);
  EXPECT(a.CachedBlocks() == 3 && g_frees == 0);
  // smallest cached block that fits: 1500 -> the 2000-byte block, not the 4000-byte one
  void *q = GPUAllocator::Allocate(1500);
  EXPECT(q == p3 && g_allocs == 3);
  void *q2 = GPUAllocator::Allocate(1000);
  EXPECT(q2 == p1);
  void *q3 = GPUAllocator::Allocate(5000);  // nothing fits: a fresh block
  EXPECT(g_allocs == 4 && q3 != p2);
  GPUAllocator::Deallocate(q);
  GPUAllocator::Deallocate(q2);
  GPUAllocator::Deallocate(q3);
  // trim: with a 6000-byte threshold a miss frees cached blocks, smallest first,
  // until the pool owns no more than the threshold (or the cache is empty)
  a.SetByteCap(6000);
  void *big = GPUAllocator::Allocate(9000);
  EXPECT(big != nullptr && g_frees == 4 && a.CachedBlocks() == 0 && a.OwnedBytes() == 9000);
  GPUAllocator::Deallocate(big);
  a.ReleaseAll();
  EXPECT(a.OwnedBytes() == 0 && g_frees == 5);
  // exhaustion is reported, not fatal
  a.SetBackend(failing_alloc, host_free);
  hip_last_status() = 0;
  EXPECT(GPUAllocator::Allocate(64) == nullptr && hip_last_status() != 0);
  a.SetBackend(nullptr, nullptr);
  a.SetByteCap(8ULL << 30);
}

// A fake event backend: an event completes when the test says so.  Records what the pool asked for.
struct FakeEvent {
  void *stream = nullptr;
  bool recorded = false, complete = false;
};
static int g_ev_created = 0, g_ev_destroyed = 0, g_ev_records = 0, g_ev_syncs = 0, g_dev_syncs = 0;
static std::vector<FakeEvent *> g_events;
static int fake_create(void **e) {
  auto *ev = new FakeEvent();
  g_events.push_back(ev);
  *e = ev;
  ++g_ev_created;
  return 0;
}
static int fake_record(void *e, void *stream) {
  auto *ev = static_cast<FakeEvent *>(e);
  ev->stream = stream;
  ev->recorded = true;
  ev->complete = false;
  ++g_ev_records;
  return 0;
}
static int fake_query(void *e) { return static_cast<FakeEvent *>(e)->complete ? 0 : LLMHIP_NOT_READY; }
static int fake_sync(void *e) {
  static_cast<FakeEvent *>(e)->complete = true;  // waiting makes it complete
  ++g_ev_syncs;
  return 0;
}
static int fake_destroy(void *e) {
  delete static_cast<FakeEvent *>(e);
  ++g_ev_destroyed;
  return 0;
}
static int fake_device_sync() {
  ++g_dev_syncs;
  return 0;
}

// The pool is stream-ordered: a block freed under work queued on one stream goes back to that
// stream at once, and to anybody else only after an event of that stream has completed.
static void test_allocator_stream_order() {
  GPUAllocator &a = GPUAllocator::GetInstance();
  const GPUAllocator::EventBackend fake = {fake_create, fake_record, fake_query, fake_sync, fake_destroy,
                                           fake_device_sync};
  a.SetBackend(host_alloc, host_free);
  a.SetEventBackend(&fake);
  a.SetByteCap(1 << 20);
  g_allocs = g_frees = 0;
  int sa = 0, sb = 0;  // two stream handles
  gpuStream_t A = &sa, B = &sb;

  // same stream: immediate reuse, no event at all
  void *p = GPUAllocator::Allocate(4096, A);
  GPUAllocator::Deallocate(p, A);
  EXPECT(a.PendingBlocks() == 1);
  void *p_again = GPUAllocator::Allocate(4096, A);
  EXPECT(p_again == p && g_allocs == 1 && a.FenceEvents() == 0 && g_ev_records == 0);

  // another stream while the first one's work is pending: the block is NOT reused, a fresh one is
  // allocated, and an event now guards the pending block
  GPUAllocator::Deallocate(p, A);
  void *q = GPUAllocator::Allocate(4096, B);
  EXPECT(q != p && g_allocs == 2 && a.FenceEvents() == 1 && g_ev_records == 1 && g_ev_syncs == 0);
  EXPECT(!g_events.empty() && g_events.back()->stream == A);
  // host code (no stream) is treated like another stream
  void *h = GPUAllocator::Allocate(4096);
  EXPECT(h != p && h != q && g_allocs == 3 && g_ev_records == 1);  // the event in flight already covers p
  // once the event has completed the block is anybody's
  g_events.back()->complete = true;
  void *r = GPUAllocator::Allocate(4096, B);
  EXPECT(r == p && g_allocs == 3);

  // a block freed after the event was recorded is not covered by it
  GPUAllocator::Deallocate(r, B);   // pending on B, ticket 1
  GPUAllocator::Deallocate(q, B);   // pending on B, ticket 2
  void *x = GPUAllocator::Allocate(4096, A);  // asks for B's blocks: records a fence on B (covers both)
  EXPECT(x != r && x != q && g_allocs == 4 && g_ev_records == 2);
  FakeEvent *fence_b = g_events.back();
  EXPECT(fence_b->stream == B);
  GPUAllocator::Deallocate(h, B);   // ticket 3: freed after the fence
  fence_b->complete = true;
  void *y1 = GPUAllocator::Allocate(4096, A), *y2 = GPUAllocator::Allocate(4096, A);
  EXPECT((y1 == r || y1 == q) && (y2 == r || y2 == q) && y1 != y2 && g_allocs == 4);
  void *y3 = GPUAllocator::Allocate(4096, A);  // only h is cached, and the completed fence does not cover it
  EXPECT(y3 != h && g_allocs == 5 && g_ev_records == 3);

  // at the byte cap the pool waits for a pending block instead of allocating
  a.SetByteCap(a.OwnedBytes());
  const int syncs_before = g_ev_syncs;
  void *w = GPUAllocator::Allocate(4096);
  EXPECT(w == h && g_allocs == 5 && g_ev_syncs == syncs_before + 1);
  a.SetByteCap(1 << 20);

  // a block whose user did not name its stream comes back only after the device has drained
  GPUAllocator::Deallocate(w, GPUAllocator::AnyStream());
  void *z = GPUAllocator::Allocate(4096, A);
  EXPECT(z != w && g_dev_syncs == 0);
  a.SetByteCap(a.OwnedBytes());
  void *z2 = GPUAllocator::Allocate(4096, A);
  EXPECT(z2 == w && g_dev_syncs == 1);
  a.SetByteCap(1 << 20);

  // ForgetStream: a drained stream's blocks are free for everybody
  GPUAllocator::Deallocate(z2, A);
  a.ForgetStream(A);
  EXPECT(a.PendingBlocks() == 0);
  EXPECT(GPUAllocator::Allocate(4096, B) == z2);

  // Tensor tags: born with the stream it was allocated for, one stream stays, two become "any"
  {
    auto t = Tensor::MakeGPUTensor(16, DT_FLOAT16);
    EXPECT(t->stream_tag == GPUAllocator::NoStream());
    t->RecordStream(A);
    EXPECT(t->stream_tag == A);
    t->RecordStream(A);
    EXPECT(t->stream_tag == A);
    t->RecordStream(B);
    EXPECT(t->stream_tag == GPUAllocator::AnyStream());
    auto u = Tensor::MakeGPUTensor(16, DT_FLOAT16, B);
    EXPECT(u->stream_tag == B);
  }
  EXPECT(a.PendingBlocks() == 2);
  for (void *blk : {z2, z, y1, y2, y3, x}) GPUAllocator::Deallocate(blk);
  a.ReleaseAll();
  EXPECT(a.OwnedBytes() == 0 && g_ev_created == g_ev_destroyed);
  a.SetEventBackend(nullptr);
  a.SetBackend(nullptr, nullptr);
  a.SetByteCap(8ULL << 30);
}

// The layer facades pick their implementation by model->config.device_type
// (src/model_base.cpp:248-264, :294-306, :620-635): the GPU arm exists, everything else is refused.
namespace {
struct TestModel : ModelBase {};
}  // namespace
static void test_device_dispatch() {
  GPUAllocator &a = GPUAllocator::GetInstance();
  a.SetBackend(host_alloc, host_free);  // cache tensors come from the host in this test
  TestModel model;
  model.hidden_dim = 4 * 128;
  model.n_heads = 4;
  model.n_kv_heads = 4;
  model.head_dim = 128;
  model.config.max_seq_len = 32;
  model.config.data_type = DT_FLOAT16;
  model.config.rope_is_neox_style = false;
  float dummy_table[4] = {1, 0, 1, 0};
  model.freq_cis = dummy_table;  // never dereferenced on the host
  for (DeviceType dev : {DEV_CPU, DEV_NPU}) {
    model.config.device_type = dev;
    RoPELayer rope;
    Llama2AttentionLayer llama;
    Qwen2AttentionLayer qwen;
    EXPECT(!rope.Init(&model, "") && rope.impl == nullptr);
    EXPECT(!llama.Init(&model, 0) && llama.impl == nullptr);
    EXPECT(!qwen.Init(&model, 0) && qwen.impl == nullptr);
  }
  model.config.device_type = DEV_GPU;
  {
    RoPELayer rope;
    EXPECT(rope.Init(&model, "") && dynamic_cast<RoPELayerGPUImpl *>(rope.impl) != nullptr);
    EXPECT(rope.impl->hidden_dim == 512 && rope.impl->n_heads == 4 && rope.impl->head_dim == 128 &&
           rope.impl->freqs_cis == dummy_table && !rope.impl->rope_is_neox_style);
    Llama2AttentionLayer llama;
    EXPECT(llama.Init(&model, 0) && dynamic_cast<Llama2AttentionGPUImpl *>(llama.impl) != nullptr);
    EXPECT(llama.impl->k_cache && llama.impl->k_cache->data_size == (size_t)32 * 512);
    model.n_kv_heads = 2;
    model.config.data_type = DT_BFLOAT16;
    model.config.rope_is_neox_style = true;
    Qwen2AttentionLayer qwen;
    EXPECT(qwen.Init(&model, 0) && dynamic_cast<Qwen2AttentionGPUImpl *>(qwen.impl) != nullptr);
    EXPECT(qwen.impl->n_kv_heads == 2 && qwen.impl->k_cache->data_size == (size_t)32 * 256);
    // Llama-2 has as many kv heads as heads: the Llama sequence refuses a GQA model
    Llama2AttentionLayer bad;
    EXPECT(!bad.Init(&model, 0));
    // positions that do not fit the cache are refused before anything is queued
    auto t = Tensor::MakeGPUTensor(512, DT_BFLOAT16);
    InferenceCtx past_end(33, 32, nullptr), inconsistent(8, 2, nullptr);
    inconsistent.cur_size = 3;
    EXPECT(qwen.Forward(t, t, t, past_end) == nullptr);
    EXPECT(qwen.Forward(t, t, t, inconsistent) == nullptr);
    // a head size the kernels do not take
    model.hidden_dim = 4 * 64;
    RoPELayer small;
    EXPECT(!small.Init(&model, ""));
  }
  // the reference's context constructor takes stream and profiler from the model
  int s = 0;
  model.model_stream = &s;
  model.is_profiling = true;
  InferenceCtx ctx(&model, 10, 7);
  EXPECT(ctx.model == &model && ctx.gpu_stream == &s && ctx.cur_size == 3 && ctx.profiler == &model.profiler &&
         ctx.is_profiling);
  a.ReleaseAll();
  a.SetBackend(nullptr, nullptr);
}

static void test_tensor_cpu() {
  auto t = Tensor::MakeCPUTensor(16, DT_FLOAT32);
  EXPECT(t->dev_type == DEV_CPU && t->data_size == 16 && t->data_ptr != nullptr);
  EXPECT(t->to(DEV_CPU).get() == t.get());
  float *f = static_cast<float *>(t->data_ptr);
  for (int i = 0; i < 16; ++i) f[i] = static_cast<float>(i);
  t->to_file("/tmp/llm_simple_amd_tensor_test.bin");
  std::vector<float> back(16);
  FILE *fp = std::fopen("/tmp/llm_simple_amd_tensor_test.bin", "rb");
  EXPECT(fp != nullptr);
  if (fp) {
    EXPECT(std::fread(back.data(), 4, 16, fp) == 16);
    std::fclose(fp);
    EXPECT(back[7] == 7.0f);
  }
}

static void test_freq_cis() {
  auto t = MakeFreqCIS(128, 64, 10000.0f, DT_FLOAT16);
  const float *tab = static_cast<const float *>(t->data_ptr);
  for (int j = 0; j < 64; ++j) EXPECT(tab[2 * j] == 1.0f && tab[2 * j + 1] == 0.0f);
  double worst = 0;
  for (int pos = 0; pos < 64; ++pos)
    for (int j = 0; j < 64; ++j) {
      const double ang = pos * std::pow(10000.0, -2.0 * j / 128.0);
      worst = std::fmax(worst, std::fabs(tab[(pos * 64 + j) * 2] - std::cos(ang)));
      worst = std::fmax(worst, std::fabs(tab[(pos * 64 + j) * 2 + 1] - std::sin(ang)));
    }
  EXPECT(worst < 2e-5);
  auto b = MakeFreqCIS(128, 64, 1e6f, DT_BFLOAT16);
  const uint32_t *bits = static_cast<const uint32_t *>(b->data_ptr);
  for (int i = 0; i < 64 * 64 * 2; ++i) EXPECT((bits[i] & 0xFFFFu) == 0);  // bf16 values
}

static void test_abi_validation() {
  alignas(16) char x[32];
  void *p = x;  // 16-byte aligned: misaligned pointers are refused as invalid arguments
  // rejected before any launch, with or without a device
  EXPECT(llmhip_flash_attn(nullptr, p, p, p, 1, 1, 0, 1, 128, 4, nullptr) == LLMHIP_ERR_INVALID_ARG);
  EXPECT(llmhip_flash_attn(p, x + 2, p, p, 1, 1, 0, 1, 128, 4, nullptr) == LLMHIP_ERR_INVALID_ARG);  // misaligned q
  EXPECT(llmhip_flash_attn(p, p, p, p, 0, 1, 0, 1, 128, 4, nullptr) == LLMHIP_ERR_INVALID_ARG);
  EXPECT(llmhip_flash_attn(p, p, p, p, 1, 0, 0, 1, 128, 4, nullptr) == LLMHIP_ERR_INVALID_ARG);
  EXPECT(llmhip_flash_attn(p, p, p, p, 1, 1, -1, 1, 128, 4, nullptr) == LLMHIP_ERR_INVALID_ARG);
  EXPECT(llmhip_flash_attn(p, p, p, p, 1, 1, 0, 1, 128, 6, nullptr) == LLMHIP_ERR_INVALID_ARG);
  EXPECT(llmhip_flash_attn(p, p, p, p, 1, 1, 0, 1, 64, 4, nullptr) == LLMHIP_ERR_UNSUPPORTED);
  EXPECT(llmhip_flash_attn_gqa(p, p, p, p, 1, 1, 0, 0, 1, 128, 5, nullptr) == LLMHIP_ERR_INVALID_ARG);
  EXPECT(llmhip_flash_attn_gqa(p, p, p, p, 1, 1, 0, 2, 0, 128, 5, nullptr) == LLMHIP_ERR_INVALID_ARG);
  EXPECT(llmhip_flash_attn_opt_prefill(p, nullptr, p, p, 1, 1, 0, 1, 128, 4, nullptr) == LLMHIP_ERR_INVALID_ARG);
  EXPECT(llmhip_flash_decode_gqa(p, p, p, p, nullptr, 0, 1, 8, 4, 1, 1, 128, 1, 5, nullptr) == LLMHIP_ERR_INVALID_ARG);  // stride < n
  EXPECT(llmhip_flash_decode_gqa(p, p, p, p, nullptr, 0, 1, 8, 8, 17, 1, 128, 1, 5, nullptr) == LLMHIP_ERR_UNSUPPORTED);  // group > 16
  EXPECT(llmhip_flash_decode_gqa(p, p, p, p, nullptr, 0, 1, 4096, 4096, 5, 8, 128, 4, 5, nullptr) == LLMHIP_ERR_WORKSPACE);
  EXPECT(llmhip_flash_decode_workspace_bytes(1, 5, 8, 128, 1) == 0);
  EXPECT(llmhip_flash_decode_workspace_bytes(2, 5, 8, 128, 4) == (size_t)2 * 8 * 4 * 16 * 130 * 4);
  EXPECT(llmhip_flash_decode_default_splits(16, 32768, 8) == 2);
  EXPECT(llmhip_flash_decode_default_splits(1, 100, 8) == 1);
  EXPECT(llmhip_flash_decode_default_splits(0, 100, 8) == LLMHIP_ERR_INVALID_ARG);
  EXPECT(llmhip_rope(p, p, p, p, p, 0, 1, 2, 200, 0, 4, nullptr) == LLMHIP_ERR_UNSUPPORTED);  // hidden != heads*128
  EXPECT(llmhip_rope(p, p, p, p, p, -1, 1, 2, 256, 0, 4, nullptr) == LLMHIP_ERR_INVALID_ARG);
  EXPECT(llmhip_rope_single(p, p, nullptr, 0, 1, 2, 256, 0, 4, nullptr) == LLMHIP_ERR_INVALID_ARG);
  EXPECT(llmhip_rope_kv_append(p, p, p, p, p, p, p, 0, 0, 2, 2, 128, 0, 4, nullptr) == LLMHIP_ERR_INVALID_ARG);
  EXPECT(llmhip_rope_kv_append(p, p, p, p, p, p, p, 0, 1, 2, 2, 96, 0, 4, nullptr) == LLMHIP_ERR_UNSUPPORTED);
  EXPECT(llmhip_error_string(LLMHIP_ERR_WORKSPACE) != nullptr);
  if (llmhip_device_count() == 0) {
    void *d = nullptr, *s = nullptr;
    EXPECT(llmhip_malloc(&d, 16) == LLMHIP_ERR_NO_DEVICE);
    EXPECT(llmhip_stream_create(&s) == LLMHIP_ERR_NO_DEVICE);
    EXPECT(llmhip_set_device(0) == LLMHIP_ERR_NO_DEVICE);
    hip_last_status() = 0;
    auto t = Tensor::MakeGPUTensor(8, DT_FLOAT16);
    EXPECT(t->data_ptr == nullptr && hip_last_status() == LLMHIP_ERR_NO_DEVICE);
    std::printf("no device visible: GPU paths report LLMHIP_ERR_NO_DEVICE\n");
  }
}

// The profiler's file is a JSON array of Chrome-trace complete events
// (src/profiling.cpp:11-38, :80-93); RecordEvent is exercised directly, the GPU-timed guard
// belongs to the GPU tests.
static void test_profiler_file() {
  const char *path = "/tmp/llm_simple_amd_profiler_test.json";
  AppProfiler prof;
  EXPECT(prof.StartLogging(path));
  const uint64_t now = static_cast<uint64_t>(std::chrono::duration_cast<std::chrono::microseconds>(
                                                 std::chrono::steady_clock::now().time_since_epoch())
                                                 .count());
  prof.RecordEvent("MatmulLayer", "m 1 n 16 k \"16\"", "a\\b.cpp", 42, now + 5, 12.5);
  prof.RecordEvent("Add", "attn output + input", "x.cpp", 7, now + 30, 1.0);
  EXPECT(prof.EventCount() == 2);
  prof.Finish();
  std::ifstream in(path);
  std::string text((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
  EXPECT(text.rfind("[\n", 0) == 0);
  EXPECT(text.find("{\"name\":\"MatmulLayer\",\"ph\":\"X\",\"pid\":0,\"ts\":") != std::string::npos);
  EXPECT(text.find("\"dur\":12.5,\"args\":{\"file\":\"a\\\\b.cpp\",\"lineno\":42,\"info\":\"m 1 n 16 k \\\"16\\\"\"}}") !=
        std::string::npos);
  EXPECT(text.find("},\n{\"name\":\"Add\"") != std::string::npos);
  EXPECT(text.size() > 3 && text.substr(text.size() - 3) == "\n]\n");
  AppProfiler closed;
  closed.RecordEvent("x", "y", "z", 1, now, 1.0);  // not started: ignored
  EXPECT(closed.EventCount() == 0);
  EXPECT(!closed.StartLogging("/nonexistent-dir/trace.json"));
  // a projection layer refuses what the kernels cannot take, before touching the device
  MatmulLayerGPUImpl mm;
  uint16_t dummy = 0;
  EXPECT(!mm.Init(&dummy, nullptr, 15, 16, DT_FLOAT16));
  EXPECT(!mm.Init(&dummy, nullptr, 16, 16, DT_FLOAT32));
  EXPECT(!mm.Init(nullptr, nullptr, 16, 16, DT_FLOAT16));
}

int main() {
  test_profiler_file();
  test_sizes();
  test_allocator_pool();
  test_allocator_stream_order();
  test_device_dispatch();
  test_tensor_cpu();
  test_freq_cis();
  test_abi_validation();
  if (g_fail) {
    std::printf("%d check(s) failed\n", g_fail);
    return 1;
  }
  std::printf("device layer host checks: all passed\n");
  return 0;
}
