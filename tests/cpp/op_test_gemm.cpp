// Counterpart of the reference's op_test_gemm (tests/gemm_main.cpp:34-45 flags --m --n --k
// --bias --dtype; tests/gemm_test.cpp:60-163): out = lhs . W^T (+ fp32 bias) on the GPU against
// the fp32 golden rounded to the storage type, judged by all_close(0.01, 0.01).  The weight is
// handed over as W[n][k] row-major instead of the Ascend nz repacking.
#include "op_test_common.hpp"

using namespace llm_simple_amd;

int main(int argc, char **argv) {
  const int m = optest::flag_int(argc, argv, "m", 2048), n = optest::flag_int(argc, argv, "n", 2048),
            k = optest::flag_int(argc, argv, "k", 2048);
  const std::string bias_s = optest::flag(argc, argv, "bias", "0");
  const bool bias = bias_s == "1" || bias_s == "true";
  const DataType dt = optest::parse_dtype(optest::flag(argc, argv, "dtype", "fp16"));
  const uint64_t seed = optest::flag_int(argc, argv, "seed", 1);
  std::printf("gemm test {m=%d,n=%d,k=%d,bias=%d} dtype %s\n", m, n, k, (int)bias, dt == DT_BFLOAT16 ? "bf16" : "fp16");
  if (llmhip_device_count() < 1) {
    std::printf("no GPU\n");
    return 3;
  }
  auto lhs = optest::normal_bits(seed, (size_t)m * k, dt);
  auto w = optest::scaled_normal_bits(seed + 1, (size_t)n * k, 1.0f / std::sqrt((float)k), dt);
  auto b = optest::normal_f32(seed + 2, n, 1.0f);
  gpuStream_t stream = nullptr;
  CHECK_LLMHIP(llmhip_stream_create(&stream));
  auto d_lhs = optest::to_gpu(lhs.data(), lhs.size(), dt), d_w = optest::to_gpu(w.data(), w.size(), dt);
  auto d_b = optest::to_gpu(b.data(), b.size(), DT_FLOAT32);
  auto d_out = Tensor::MakeGPUTensor((size_t)m * n, dt);
  void *e0 = nullptr, *e1 = nullptr;
  CHECK_LLMHIP(llmhip_event_create(&e0));
  CHECK_LLMHIP(llmhip_event_create(&e1));
  auto run = [&]() {
    if (bias)
      hip_matmul_bias_layer(d_out->data_ptr, d_lhs->data_ptr, d_w->data_ptr, d_b->data_ptr, m, n, k, dt, stream);
    else
      hip_matmul_layer(d_out->data_ptr, d_lhs->data_ptr, d_w->data_ptr, m, n, k, dt, stream);
  };
  run();  // plan creation
  CHECK_LLMHIP(llmhip_event_record(e0, stream));
  run();
  CHECK_LLMHIP(llmhip_event_record(e1, stream));
  CHECK_LLMHIP(llmhip_stream_sync(stream));
  float ms = 0;
  CHECK_LLMHIP(llmhip_event_elapsed_ms(&ms, e0, e1));
  std::printf("kernel duration %.4fms (%.1f TFLOP/s)\n", ms, 2.0 * m * n * k / (ms * 1e-3) / 1e12);
  auto h_out = d_out->to(DEV_CPU);
  std::vector<uint16_t> golden((size_t)m * n);
  orc_matmul_bias(golden.data(), lhs.data(), w.data(), bias ? b.data() : nullptr, m, n, k, dt, 0);
  std::vector<float> got_f(golden.size()), gold_f(golden.size());
  orc_widen_array(got_f.data(), static_cast<const uint16_t *>(h_out->data_ptr), (int64_t)got_f.size(), dt);
  orc_widen_array(gold_f.data(), golden.data(), (int64_t)gold_f.size(), dt);
  float mx = 0;
  const int64_t bad = orc_all_close(got_f.data(), gold_f.data(), (int64_t)got_f.size(), 0.01f, 0.01f, &mx);
  std::printf("max abs err %.3e, %lld elements outside all_close(0.01, 0.01)\n", mx, (long long)bad);
  CHECK_LLMHIP(llmhip_event_destroy(e0));
  CHECK_LLMHIP(llmhip_event_destroy(e1));
  CHECK_LLMHIP(llmhip_stream_destroy(stream));
  const bool ok = bad == 0 && hip_last_status() == 0;
  std::printf(ok ? "test success\n" : "test failed\n");
  return ok ? 0 : 1;
}
