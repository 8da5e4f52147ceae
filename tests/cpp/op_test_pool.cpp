// The stream-ordered pool on a real device: a block freed while work queued on one stream still uses it must not
// reach another stream or host code before that work is done, and must go back to its own stream at once.
// A long attention launch reads a pooled q tensor on stream A; the tensor is freed right after the launch; requests
// from stream B and from the host then get other blocks (or the same one only once an event of A has completed),
// a request from stream A gets the very block; the attention output is checked against the oracle to show that
// nobody scribbled over q while the kernel was reading it.
#include "op_test_common.hpp"

using namespace llm_simple_amd;

int main() {
  std::printf("pool test (stream-ordered GPUAllocator on the device)\n");
  if (llmhip_device_count() < 1) {
    std::printf("no GPU\n");
    return 3;
  }
  const int H = 8, hd = 128, S = 2048;
  const DataType dt = DT_BFLOAT16;
  gpuStream_t A = nullptr, B = nullptr;
  CHECK_LLMHIP(llmhip_stream_create(&A));
  CHECK_LLMHIP(llmhip_stream_create(&B));
  auto q = optest::normal_bits(1, (size_t)S * H * hd, dt), k = optest::normal_bits(2, (size_t)S * H * hd, dt),
       v = optest::normal_bits(3, (size_t)S * H * hd, dt);
  auto d_k = optest::to_gpu(k.data(), k.size(), dt), d_v = optest::to_gpu(v.data(), v.size(), dt);
  auto d_out = Tensor::MakeGPUTensor(q.size(), dt, A);
  GPUAllocator &pool = GPUAllocator::GetInstance();
  bool ok = true;
  void *q_block = nullptr;
  const size_t q_bytes = SizeOfTensor(q.size(), dt);
  {
    auto d_q = optest::to_gpu(q.data(), q.size(), dt);
    q_block = d_q->data_ptr;
    d_q->RecordStream(A);
    d_k->RecordStream(A);
    d_v->RecordStream(A);
    for (int rep = 0; rep < 300; ++rep)  // several milliseconds of queued work that reads q
      hip_flash_attn_layer(d_out->data_ptr, d_q->data_ptr, d_k->data_ptr, d_v->data_ptr, S, S, 0, H, hd, dt, A);
  }  // d_q freed here, its launches still queued
  const size_t fences0 = pool.FenceEvents();
  // another stream and the host: not the pending block (scribble over what they get)
  auto other = Tensor::MakeGPUTensor(q.size(), dt, B);
  auto host_side = Tensor::MakeGPUTensor(q.size(), dt);
  ok = ok && other->data_ptr != q_block && host_side->data_ptr != q_block;
  CHECK_LLMHIP(llmhip_memset_async(other->data_ptr, 0xFF, q_bytes, B));
  std::vector<uint16_t> junk(q.size(), 0x7FC0);
  CHECK_LLMHIP(llmhip_memcpy_h2d(host_side->data_ptr, junk.data(), q_bytes));
  ok = ok && pool.FenceEvents() == fences0 + 1;  // one event on A guards the block now
  // its own stream gets it back at once
  auto same = Tensor::MakeGPUTensor(q.size(), dt, A);
  ok = ok && same->data_ptr == q_block;
  // A reads through `same` after the attention launches in stream order: harmless; give it back
  same.reset();
  auto hout = d_out->to(DEV_CPU);  // waits for stream A
  // Once A has drained, the block is anybody's -- after an event says so: `same` was freed after the first
  // event was recorded, so the first request from B records a second one (and takes a fresh block), the next
  // request finds that event complete.
  auto asks = Tensor::MakeGPUTensor(q.size(), dt, B);
  CHECK_LLMHIP(llmhip_stream_sync(A));
  auto later = Tensor::MakeGPUTensor(q.size(), dt, B);
  ok = ok && asks->data_ptr != q_block && later->data_ptr == q_block && pool.FenceEvents() == fences0 + 2;
  std::vector<float> golden(q.size()), got(q.size());
  orc_attention_f32(golden.data(), q.data(), k.data(), v.data(), 1, S, S, 0, 1, H, hd, S, dt, 0);
  orc_widen_array(got.data(), static_cast<const uint16_t *>(hout->data_ptr), (int64_t)got.size(), dt);
  float mx = 0;
  orc_all_close(got.data(), golden.data(), (int64_t)got.size(), 1e-3f, 1e-3f, &mx);
  std::printf("max-abs %.3e, fence events %zu, pointers %s\n", mx, pool.FenceEvents() - fences0, ok ? "as expected" : "WRONG");
  ok = ok && mx <= 1e-2f && hip_last_status() == 0;
  CHECK_LLMHIP(llmhip_stream_sync(A));
  CHECK_LLMHIP(llmhip_stream_sync(B));
  std::printf(ok ? "PASS\n" : "FAIL\n");
  return ok ? 0 : 1;
}
