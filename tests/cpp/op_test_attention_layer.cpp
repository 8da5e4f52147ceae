// Drives AttentionGPUImpl the way a model step drives a transformer layer's attention
// block (src/llama2_layer_npu.cpp:780-869): one prefill of --prompt tokens, then
// --steps decode steps with the KV cache growing in place, then (--chunk N) one more chunk of N
// tokens over the whole cache (chunked prefill), checked after every step against the oracle's
// unfused rope -> append -> attention sequence.
#include "op_test_common.hpp"

using namespace llm_simple_amd;

int main(int argc, char **argv) {
  const int H = optest::flag_int(argc, argv, "head_num", 12), Hkv = optest::flag_int(argc, argv, "kv_head_num", 2);
  const int prompt = optest::flag_int(argc, argv, "prompt", 64), steps = optest::flag_int(argc, argv, "steps", 8);
  const int max_seq_len = optest::flag_int(argc, argv, "max_seq_len", 512);
  const int chunk = optest::flag_int(argc, argv, "chunk", 0);
  const bool is_neox = optest::flag_int(argc, argv, "is_neox", 1) != 0;
  const float theta = std::atof(optest::flag(argc, argv, "theta", "1000000").c_str());
  const DataType dt = optest::parse_dtype(optest::flag(argc, argv, "dtype", "bf16"));
  const int hd = 128;
  std::printf("attention layer test {head_num=%d,kv_head_num=%d,prompt=%d,steps=%d,%s,neox=%d}\n", H, Hkv, prompt,
              steps, dt == DT_BFLOAT16 ? "bf16" : "fp16", (int)is_neox);
  if (llmhip_device_count() < 1) {
    std::printf("no GPU\n");
    return 3;
  }
  auto table = MakeFreqCIS(hd, max_seq_len, theta, dt);
  const float *tab = static_cast<const float *>(table->data_ptr);
  AttentionGPUImpl layer;
  if (!layer.Init(H, Hkv, hd, max_seq_len, dt, is_neox, table->to(DEV_GPU))) {
    std::printf("Init failed\n");
    return 1;
  }
  gpuStream_t stream = nullptr;
  CHECK_LLMHIP(llmhip_stream_create(&stream));
  std::vector<uint16_t> kc((size_t)max_seq_len * Hkv * hd, 0), vc(kc.size(), 0);
  const float tol = dt == DT_BFLOAT16 ? 1e-2f : 2e-3f;
  float worst = 0;
  size_t prev = 0;
  const int total_steps = steps + (chunk > 0 ? 1 : 0);
  for (int step = 0; step <= total_steps; ++step) {
    const size_t cur = step == 0 ? prompt : (step > steps ? prev + chunk : prev + 1);
    InferenceCtx ctx(cur, prev, stream);
    const size_t m = ctx.cur_size;
    auto q = optest::normal_bits(100 + step, m * H * hd, dt), k = optest::normal_bits(200 + step, m * Hkv * hd, dt),
         v = optest::normal_bits(300 + step, m * Hkv * hd, dt);
    auto out = layer.Forward(optest::to_gpu(q.data(), q.size(), dt), optest::to_gpu(k.data(), k.size(), dt),
                             optest::to_gpu(v.data(), v.size(), dt), ctx);
    if (!out) {
      std::printf("Forward failed at step %d\n", step);
      return 1;
    }
    auto hout = out->to(DEV_CPU);
    // oracle: rope(q), rope(k) -> cache, v -> cache, attention over [0, cur)
    std::vector<uint16_t> qr(q.size()), kr(k.size());
    orc_rope(qr.data(), q.data(), tab, (int)prev, (int)m, H, hd, is_neox, dt);
    orc_rope(kr.data(), k.data(), tab, (int)prev, (int)m, Hkv, hd, is_neox, dt);
    orc_kv_append(kc.data(), kr.data(), (int)prev, (int)m, Hkv * hd);
    orc_kv_append(vc.data(), v.data(), (int)prev, (int)m, Hkv * hd);
    std::vector<float> golden(q.size()), got(q.size());
    orc_attention_f32(golden.data(), qr.data(), kc.data(), vc.data(), 1, (int)m, (int)cur, (int)prev, H / Hkv, Hkv,
                      hd, max_seq_len, dt, 0);
    orc_widen_array(got.data(), static_cast<const uint16_t *>(hout->data_ptr), (int64_t)got.size(), dt);
    float mx = 0;
    orc_all_close(got.data(), golden.data(), (int64_t)got.size(), 1e-3f, 1e-3f, &mx);
    worst = std::fmax(worst, mx);
    prev = cur;
  }
  // the device caches must hold exactly what the oracle's caches hold
  auto hk = layer.k_cache->to(DEV_CPU), hv = layer.v_cache->to(DEV_CPU);
  const size_t valid = prev * Hkv * hd;
  const bool caches_equal = std::memcmp(hk->data_ptr, kc.data(), valid * 2) == 0 &&
                            std::memcmp(hv->data_ptr, vc.data(), valid * 2) == 0;
  std::printf("worst max-abs over %d steps: %.3e (bound %.0e); caches %s\n", total_steps + 1, worst, tol,
              caches_equal ? "bit-identical" : "DIFFER");
  CHECK_LLMHIP(llmhip_stream_destroy(stream));
  const bool ok = worst <= tol && caches_equal && hip_last_status() == 0;
  std::printf(ok ? "PASS\n" : "FAIL\n");
  return ok ? 0 : 1;
}
