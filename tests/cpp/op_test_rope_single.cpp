// GPU counterpart of the reference's op_test_rope_single (tests/rope_single_layer_main.cpp,
// tests/rope_single_layer_test.cpp:52-122): flags --max_seq_len --head_num --head_dim
// --offset --seq_len --dtype --is_neox --theta.  The golden is the oracle's RoPE, which
// rounds once to the storage type like the reference's golden (:97); the check is bit
// exactness, stricter than the reference's all_close.
#include "op_test_common.hpp"

using namespace llm_simple_amd;

int main(int argc, char **argv) {
  const int max_seq_len = optest::flag_int(argc, argv, "max_seq_len", 2048);
  const int head_num = optest::flag_int(argc, argv, "head_num", 40);
  const int head_dim = optest::flag_int(argc, argv, "head_dim", 128);
  const int offset = optest::flag_int(argc, argv, "offset", 0);
  const int seq_len = optest::flag_int(argc, argv, "seq_len", 128);
  const bool is_neox = optest::flag_int(argc, argv, "is_neox", 1) != 0;
  const float theta = std::atof(optest::flag(argc, argv, "theta", "10000").c_str());
  const DataType dt = optest::parse_dtype(optest::flag(argc, argv, "dtype", "fp16"));
  std::printf("rope_single op test {max_seq_len=%d,head_num=%d,head_dim=%d,offset=%d,seq_len=%d,is_neox=%d,%s}\n",
              max_seq_len, head_num, head_dim, offset, seq_len, (int)is_neox, dt == DT_BFLOAT16 ? "bf16" : "fp16");
  if (offset + seq_len > max_seq_len) {
    std::printf("offset + seq_len exceeds max_seq_len\n");
    return 2;
  }
  if (llmhip_device_count() < 1) {
    std::printf("no GPU\n");
    return 3;
  }
  auto table = MakeFreqCIS(head_dim, max_seq_len, theta, dt);
  auto dtable = table->to(DEV_GPU);
  const size_t cnt = (size_t)seq_len * head_num * head_dim;
  auto x = optest::normal_bits(11, cnt, dt);
  std::vector<uint16_t> golden(cnt);
  orc_rope(golden.data(), x.data(), static_cast<const float *>(table->data_ptr), offset, seq_len, head_num,
           head_dim, is_neox, dt);
  auto dx = optest::to_gpu(x.data(), cnt, dt);
  auto dout = Tensor::MakeGPUTensor(cnt, dt);
  gpuStream_t stream = nullptr;
  CHECK_LLMHIP(llmhip_stream_create(&stream));
  hip_rope_single_layer(dout->data_ptr, dtable->data_ptr, dx->data_ptr, offset, seq_len, head_num,
                        head_num * head_dim, is_neox, dt, stream);
  CHECK_LLMHIP(llmhip_stream_sync(stream));
  auto hout = dout->to(DEV_CPU);
  const uint16_t *got = static_cast<const uint16_t *>(hout->data_ptr);
  size_t diff = 0;
  for (size_t i = 0; i < cnt; ++i) diff += got[i] != golden[i];
  std::printf("%zu of %zu elements differ from the golden\n", diff, cnt);
  CHECK_LLMHIP(llmhip_stream_destroy(stream));
  const bool ok = diff == 0 && hip_last_status() == 0;
  std::printf(ok ? "PASS\n" : "FAIL\n");
  return ok ? 0 : 1;
}
