// Drives the attention part of a transformer layer the way a model step drives it
// (src/llama2_layer_npu.cpp:780-869 for Qwen2, :284-374 for Llama-2): one prefill of --prompt
// tokens, then --steps decode steps with the KV cache growing in place, then (--chunk N) one more
// chunk of N tokens over the whole cache (chunked prefill), checked after every step against the
// oracle's unfused rope -> append -> attention sequence.
//
//   --model direct   AttentionGPUImpl itself (default)
//   --model qwen2    Qwen2AttentionLayer, the facade with the device switch (DEV_GPU arm)
//   --model llama2   Llama2AttentionLayer: RoPELayer::Forward, two device-to-device copies,
//                    hip_flash_attn_opt_prefill_layer, as the reference's Llama layer issues them; its
//                    outputs and caches must equal, bit for bit, those of the fused path run beside it
//   --time R         no checks: R rounds of (prefill, --steps decode steps), prints the median time per
//                    decode step through the layer and through bare llmhip_decode_step_gqa calls
#include <algorithm>
#include <chrono>

#include "op_test_common.hpp"

using namespace llm_simple_amd;

namespace {

struct Model : ModelBase {};

struct Args {
  int H, Hkv, prompt, steps, max_seq_len, chunk, rounds;
  bool is_neox;
  float theta;
  DataType dt;
  std::string model;
};

double now_us() {
  return std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

// One generated token per call with nothing between the calls but the layer's own host code: what
// a model's decode loop costs per layer.  Returns the median over rounds of the GPU time (stream
// events) and of the host time per step.
int time_mode(const Args &a, Model &model) {
  const int hd = 128;
  Qwen2AttentionLayer layer;
  if (!layer.Init(&model, 0)) {
    std::printf("Init failed\n");
    return 1;
  }
  gpuStream_t stream = model.model_stream;
  auto qp = optest::normal_bits(1, (size_t)a.prompt * a.H * hd, a.dt), kp = optest::normal_bits(2, (size_t)a.prompt * a.Hkv * hd, a.dt),
       vp = optest::normal_bits(3, (size_t)a.prompt * a.Hkv * hd, a.dt);
  auto q1 = optest::normal_bits(4, (size_t)a.H * hd, a.dt), k1 = optest::normal_bits(5, (size_t)a.Hkv * hd, a.dt),
       v1 = optest::normal_bits(6, (size_t)a.Hkv * hd, a.dt);
  auto d_qp = optest::to_gpu(qp.data(), qp.size(), a.dt), d_kp = optest::to_gpu(kp.data(), kp.size(), a.dt),
       d_vp = optest::to_gpu(vp.data(), vp.size(), a.dt);
  auto d_q1 = optest::to_gpu(q1.data(), q1.size(), a.dt), d_k1 = optest::to_gpu(k1.data(), k1.size(), a.dt),
       d_v1 = optest::to_gpu(v1.data(), v1.size(), a.dt);
  auto d_out = Tensor::MakeGPUTensor((size_t)a.H * hd, a.dt);
  void *ev0 = nullptr, *ev1 = nullptr;
  CHECK_LLMHIP(llmhip_event_create(&ev0));
  CHECK_LLMHIP(llmhip_event_create(&ev1));
  std::vector<double> layer_gpu, layer_host, abi_gpu, abi_host;
  const size_t fences_before = GPUAllocator::GetInstance().FenceEvents();
  for (int round = 0; round < a.rounds + 2; ++round) {  // two warm-up rounds
    for (int which = 0; which < 2; ++which) {
      InferenceCtx pre(&model, a.prompt, 0);
      if (!layer.Forward(d_qp, d_kp, d_vp, pre)) return 1;
      CHECK_LLMHIP(llmhip_event_record(ev0, stream));
      const double t0 = now_us();
      for (int s = 0; s < a.steps; ++s) {
        const size_t prev = a.prompt + s;
        if (which == 0) {
          InferenceCtx ctx(&model, prev + 1, prev);
          auto out = layer.Forward(d_q1, d_k1, d_v1, ctx);
          if (!out) return 1;
        } else {
          CHECK_LLMHIP(llmhip_decode_step_gqa(d_out->data_ptr, layer.impl->k_cache->data_ptr,
                                              layer.impl->v_cache->data_ptr, model.freq_cis, d_q1->data_ptr,
                                              d_k1->data_ptr, d_v1->data_ptr, (int)prev, a.H / a.Hkv, a.Hkv, hd,
                                              a.is_neox ? 1 : 0, a.dt, stream));
        }
      }
      const double t1 = now_us();
      CHECK_LLMHIP(llmhip_event_record(ev1, stream));
      CHECK_LLMHIP(llmhip_event_sync(ev1));
      float ms = 0;
      CHECK_LLMHIP(llmhip_event_elapsed_ms(&ms, ev0, ev1));
      if (round >= 2) {
        (which == 0 ? layer_gpu : abi_gpu).push_back(ms * 1e3 / a.steps);
        (which == 0 ? layer_host : abi_host).push_back((t1 - t0) / a.steps);
      }
    }
  }
  auto med = [](std::vector<double> v) {
    std::sort(v.begin(), v.end());
    return v[v.size() / 2];
  };
  std::printf("{\"layer_decode_us_per_step\": %.3f, \"layer_host_us_per_step\": %.3f, \"abi_decode_us_per_step\": %.3f, "
              "\"abi_host_us_per_step\": %.3f, \"steps\": %d, \"rounds\": %d, \"prompt\": %d, \"head_num\": %d, "
              "\"kv_head_num\": %d, \"pool_fence_events\": %zu, \"status\": %d}\n",
              med(layer_gpu), med(layer_host), med(abi_gpu), med(abi_host), a.steps, a.rounds, a.prompt, a.H, a.Hkv,
              GPUAllocator::GetInstance().FenceEvents() - fences_before, hip_last_status());
  CHECK_LLMHIP(llmhip_event_destroy(ev0));
  CHECK_LLMHIP(llmhip_event_destroy(ev1));
  return hip_last_status() == 0 ? 0 : 1;
}

}  // namespace

int main(int argc, char **argv) {
  Args a;
  a.H = optest::flag_int(argc, argv, "head_num", 12);
  a.Hkv = optest::flag_int(argc, argv, "kv_head_num", 2);
  a.prompt = optest::flag_int(argc, argv, "prompt", 64);
  a.steps = optest::flag_int(argc, argv, "steps", 8);
  a.max_seq_len = optest::flag_int(argc, argv, "max_seq_len", 512);
  a.chunk = optest::flag_int(argc, argv, "chunk", 0);
  a.rounds = optest::flag_int(argc, argv, "time", 0);
  a.is_neox = optest::flag_int(argc, argv, "is_neox", 1) != 0;
  a.theta = std::atof(optest::flag(argc, argv, "theta", "1000000").c_str());
  a.dt = optest::parse_dtype(optest::flag(argc, argv, "dtype", "bf16"));
  a.model = optest::flag(argc, argv, "model", "direct");
  const int H = a.H, Hkv = a.Hkv, hd = 128, max_seq_len = a.max_seq_len;
  const DataType dt = a.dt;
  std::printf("attention layer test {model=%s,head_num=%d,kv_head_num=%d,prompt=%d,steps=%d,%s,neox=%d}\n",
              a.model.c_str(), H, Hkv, a.prompt, a.steps, dt == DT_BFLOAT16 ? "bf16" : "fp16", (int)a.is_neox);
  if (llmhip_device_count() < 1) {
    std::printf("no GPU\n");
    return 3;
  }
  if (a.prompt + a.steps + a.chunk > max_seq_len) {
    std::printf("prompt + steps + chunk exceed max_seq_len\n");
    return 2;
  }
  // the model-level state the layers read (src/model_base.hpp:324-354)
  Model model;
  model.config.device_type = DEV_GPU;
  model.config.data_type = dt;
  model.config.max_seq_len = max_seq_len;
  model.config.rope_is_neox_style = a.is_neox;
  model.hidden_dim = H * hd;
  model.head_dim = hd;
  model.n_heads = H;
  model.n_kv_heads = Hkv;
  CHECK_LLMHIP(llmhip_stream_create(&model.model_stream));
  if (!model.InitFreqCIS(a.theta, dt)) {
    std::printf("InitFreqCIS failed\n");
    return 1;
  }
  if (a.rounds > 0) {
    const int rc = time_mode(a, model);
    CHECK_LLMHIP(llmhip_stream_sync(model.model_stream));
    return rc;
  }
  auto table = MakeFreqCIS(hd, max_seq_len, a.theta, dt);  // host copy for the oracle
  const float *tab = static_cast<const float *>(table->data_ptr);

  AttentionGPUImpl direct;
  Qwen2AttentionLayer qwen;   // the fused path behind the facade
  Llama2AttentionLayer llama;
  const bool use_llama = a.model == "llama2", use_qwen = a.model == "qwen2" || use_llama;
  if (use_llama && Hkv != H) {
    std::printf("--model llama2 needs kv_head_num == head_num\n");
    return 2;
  }
  bool init_ok = true;
  if (!use_qwen) init_ok = direct.Init(H, Hkv, hd, max_seq_len, dt, a.is_neox, model.freq_cis);
  if (use_qwen) init_ok = qwen.Init(&model, 0);
  if (use_llama) init_ok = init_ok && llama.Init(&model, 0);
  if (!init_ok) {
    std::printf("Init failed\n");
    return 1;
  }
  gpuStream_t stream = model.model_stream;
  std::vector<uint16_t> kc((size_t)max_seq_len * Hkv * hd, 0), vc(kc.size(), 0);
  const float tol = dt == DT_BFLOAT16 ? 1e-2f : 2e-3f;
  float worst = 0;
  size_t prev = 0;
  bool llama_equal = true;
  const int total_steps = a.steps + (a.chunk > 0 ? 1 : 0);
  for (int step = 0; step <= total_steps; ++step) {
    const size_t cur = step == 0 ? a.prompt : (step > a.steps ? prev + a.chunk : prev + 1);
    InferenceCtx ctx(&model, cur, prev);
    const size_t m = ctx.cur_size;
    auto q = optest::normal_bits(100 + step, m * H * hd, dt), k = optest::normal_bits(200 + step, m * Hkv * hd, dt),
         v = optest::normal_bits(300 + step, m * Hkv * hd, dt);
    auto d_q = optest::to_gpu(q.data(), q.size(), dt), d_k = optest::to_gpu(k.data(), k.size(), dt),
         d_v = optest::to_gpu(v.data(), v.size(), dt);
    auto out = use_qwen ? qwen.Forward(d_q, d_k, d_v, ctx) : direct.Forward(d_q, d_k, d_v, ctx);
    if (!out) {
      std::printf("Forward failed at step %d\n", step);
      return 1;
    }
    auto hout = out->to(DEV_CPU);
    if (use_llama) {
      auto out_l = llama.Forward(d_q, d_k, d_v, ctx);
      if (!out_l) {
        std::printf("Llama Forward failed at step %d\n", step);
        return 1;
      }
      auto hl = out_l->to(DEV_CPU);
      llama_equal = llama_equal && std::memcmp(hl->data_ptr, hout->data_ptr, q.size() * 2) == 0;
    }
    // oracle: rope(q), rope(k) -> cache, v -> cache, attention over [0, cur)
    std::vector<uint16_t> qr(q.size()), kr(k.size());
    orc_rope(qr.data(), q.data(), tab, (int)prev, (int)m, H, hd, a.is_neox, dt);
    orc_rope(kr.data(), k.data(), tab, (int)prev, (int)m, Hkv, hd, a.is_neox, dt);
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
  const size_t valid = prev * Hkv * hd;
  auto same_as_oracle = [&](std::shared_ptr<Tensor> dk, std::shared_ptr<Tensor> dv) {
    auto hk = dk->to(DEV_CPU), hv = dv->to(DEV_CPU);
    return std::memcmp(hk->data_ptr, kc.data(), valid * 2) == 0 && std::memcmp(hv->data_ptr, vc.data(), valid * 2) == 0;
  };
  bool caches_equal = use_qwen ? same_as_oracle(qwen.impl->k_cache, qwen.impl->v_cache)
                               : same_as_oracle(direct.k_cache, direct.v_cache);
  if (use_llama) caches_equal = caches_equal && same_as_oracle(llama.impl->k_cache, llama.impl->v_cache);
  std::printf("worst max-abs over %d steps: %.3e (bound %.0e); caches %s\n", total_steps + 1, worst, tol,
              caches_equal ? "bit-identical" : "DIFFER");
  if (use_llama)
    std::printf("Llama sequence (rope layer, two copies, opt_prefill attention) vs fused path: outputs %s\n",
                llama_equal ? "bit-identical" : "DIFFER");
  std::printf("pool: %zu fence events, %zu cached blocks\n", GPUAllocator::GetInstance().FenceEvents(),
              GPUAllocator::GetInstance().CachedBlocks());
  CHECK_LLMHIP(llmhip_stream_sync(stream));
  const bool ok = worst <= tol && caches_equal && llama_equal && hip_last_status() == 0;
  std::printf(ok ? "PASS\n" : "FAIL\n");
  return ok ? 0 : 1;
}
