// GPU counterpart of the reference's op_test_flash_attn (tests/flash_attn_main.cpp:5-52,
// tests/flash_attn_test.cpp:67-236): same flags (--m --n --offset --head_num --head_dim),
// extended with --kv_head_num, --dtype {fp16,bf16} and --seed.  Inputs are generated on
// the host, rounded to the storage type, sent through Tensor::to(DEV_GPU); the operator
// is called through hip_ops.hpp; the result is compared with the fp32 golden under the
// reference's all_close rule (tests/npu_op_test_util.cpp:33-48) and the max-abs bound.
#include "op_test_common.hpp"

using namespace llm_simple_amd;

int main(int argc, char **argv) {
  const int m = optest::flag_int(argc, argv, "m", 2048), n = optest::flag_int(argc, argv, "n", 2048);
  const int offset = optest::flag_int(argc, argv, "offset", 0);
  const int head_num = optest::flag_int(argc, argv, "head_num", 32);
  const int head_dim = optest::flag_int(argc, argv, "head_dim", 128);
  const int kv_head_num = optest::flag_int(argc, argv, "kv_head_num", head_num);
  const uint64_t seed = optest::flag_int(argc, argv, "seed", 1);
  const DataType dt = optest::parse_dtype(optest::flag(argc, argv, "dtype", "fp16"));
  if (head_num % kv_head_num != 0) {
    std::printf("head_num must be a multiple of kv_head_num\n");
    return 2;
  }
  std::printf("flash_attn op test {m=%d,n=%d,offset=%d,head_num=%d,kv_head_num=%d,head_dim=%d,%s}\n", m,
              n, offset, head_num, kv_head_num, head_dim, dt == DT_BFLOAT16 ? "bf16" : "fp16");
  if (llmhip_device_count() < 1) {
    std::printf("no GPU\n");
    return 3;
  }
  const size_t qn = (size_t)m * head_num * head_dim, kn = (size_t)n * kv_head_num * head_dim;
  auto q = optest::normal_bits(seed, qn, dt), k = optest::normal_bits(seed + 1, kn, dt),
       v = optest::normal_bits(seed + 2, kn, dt);
  auto dq = optest::to_gpu(q.data(), qn, dt), dk = optest::to_gpu(k.data(), kn, dt),
       dv = optest::to_gpu(v.data(), kn, dt);
  auto dout = Tensor::MakeGPUTensor(qn, dt);
  gpuStream_t stream = nullptr;
  CHECK_LLMHIP(llmhip_stream_create(&stream));
  CHECK_LLMHIP(llmhip_memset_async(dout->data_ptr, 0, SizeOfTensor(qn, dt), stream));
  if (kv_head_num == head_num)
    hip_flash_attn_layer(dout->data_ptr, dq->data_ptr, dk->data_ptr, dv->data_ptr, m, n, offset, head_num,
                         head_dim, dt, stream);
  else
    hip_flash_attn_gqa_layer(dout->data_ptr, dq->data_ptr, dk->data_ptr, dv->data_ptr, m, n, offset,
                             head_num / kv_head_num, kv_head_num, head_dim, dt, stream);
  CHECK_LLMHIP(llmhip_stream_sync(stream));
  auto hout = dout->to(DEV_CPU);
  std::vector<float> got(qn), golden(qn);
  orc_widen_array(got.data(), static_cast<const uint16_t *>(hout->data_ptr), (int64_t)qn, dt);
  orc_attention_f32(golden.data(), q.data(), k.data(), v.data(), 1, m, n, offset, head_num / kv_head_num,
                    kv_head_num, head_dim, n, dt, 0);
  float max_abs = 0;
  const int64_t bad = orc_all_close(got.data(), golden.data(), (int64_t)qn, 1e-3f, 1e-3f, &max_abs);
  const float tol = dt == DT_BFLOAT16 ? 1e-2f : 2e-3f;
  std::printf("max abs error %.3e (bound %.0e); all_close(1e-3,1e-3) failing elements: %lld of %zu\n", max_abs,
              tol, (long long)bad, qn);
  CHECK_LLMHIP(llmhip_stream_destroy(stream));
  const bool ok = hip_last_status() == 0 && max_abs <= tol && (dt == DT_BFLOAT16 || bad == 0);
  std::printf(ok ? "PASS\n" : "FAIL\n");
  return ok ? 0 : 1;
}
