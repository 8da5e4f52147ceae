// Drives AttentionBlockGPUImpl -- q/k/v projections (fp32 bias), RoPE + cache append,
// attention, o_proj, residual add: src/llama2_layer_npu.cpp:760-901 -- through one prefill and
// --steps decode steps with the profiler on, and checks every step against the oracle's chain
// of the same operators.  --trace PATH receives the Chrome-trace file (src/profiling.cpp).
#include "op_test_common.hpp"

using namespace llm_simple_amd;

int main(int argc, char **argv) {
  const int H = optest::flag_int(argc, argv, "head_num", 12), Hkv = optest::flag_int(argc, argv, "kv_head_num", 2);
  const int prompt = optest::flag_int(argc, argv, "prompt", 64), steps = optest::flag_int(argc, argv, "steps", 4);
  const int max_seq_len = optest::flag_int(argc, argv, "max_seq_len", 512);
  const bool is_neox = optest::flag_int(argc, argv, "is_neox", 1) != 0;
  const bool use_bias = optest::flag_int(argc, argv, "bias", 1) != 0;
  const float theta = std::atof(optest::flag(argc, argv, "theta", "1000000").c_str());
  const DataType dt = optest::parse_dtype(optest::flag(argc, argv, "dtype", "bf16"));
  const std::string trace = optest::flag(argc, argv, "trace", "");
  const int hd = 128, hidden = H * hd, kvd = Hkv * hd;
  std::printf("attention block test {hidden=%d,head_num=%d,kv_head_num=%d,prompt=%d,steps=%d,%s,bias=%d}\n", hidden, H,
              Hkv, prompt, steps, dt == DT_BFLOAT16 ? "bf16" : "fp16", (int)use_bias);
  if (llmhip_device_count() < 1) {
    std::printf("no GPU\n");
    return 3;
  }
  const float ws = 1.0f / std::sqrt((float)hidden);
  auto wq = optest::scaled_normal_bits(11, (size_t)hidden * hidden, ws, dt);
  auto wk = optest::scaled_normal_bits(12, (size_t)kvd * hidden, ws, dt);
  auto wv = optest::scaled_normal_bits(13, (size_t)kvd * hidden, ws, dt);
  auto wo = optest::scaled_normal_bits(14, (size_t)hidden * hidden, ws, dt);
  auto bq = optest::normal_f32(15, hidden, 0.02f), bk = optest::normal_f32(16, kvd, 0.02f),
       bv = optest::normal_f32(17, kvd, 0.02f);
  auto table = MakeFreqCIS(hd, max_seq_len, theta, dt);
  const float *tab = static_cast<const float *>(table->data_ptr);
  AttentionBlockGPUImpl block;
  AttentionBlockGPUImpl::Weights w{wq.data(), wk.data(), wv.data(), wo.data(),
                                   use_bias ? bq.data() : nullptr, use_bias ? bk.data() : nullptr,
                                   use_bias ? bv.data() : nullptr};
  if (!block.Init(w, hidden, H, Hkv, max_seq_len, dt, is_neox, table->to(DEV_GPU))) {
    std::printf("Init failed\n");
    return 1;
  }
  gpuStream_t stream = nullptr;
  CHECK_LLMHIP(llmhip_stream_create(&stream));
  AppProfiler profiler;
  const bool profiling = !trace.empty() && profiler.StartLogging(trace);
  std::vector<uint16_t> kc((size_t)max_seq_len * kvd, 0), vc(kc.size(), 0);
  int64_t bad_total = 0;
  float worst = 0;
  size_t prev = 0;
  for (int step = 0; step <= steps; ++step) {
    const size_t cur = step == 0 ? prompt : prev + 1;
    InferenceCtx ctx(cur, prev, stream);
    ctx.profiler = &profiler;
    ctx.is_profiling = profiling;
    const int m = (int)ctx.cur_size;
    auto x = optest::normal_bits(500 + step, (size_t)m * hidden, dt);      // input_norm output
    auto res = optest::normal_bits(600 + step, (size_t)m * hidden, dt);    // layer input
    auto out = block.Forward(optest::to_gpu(x.data(), x.size(), dt), optest::to_gpu(res.data(), res.size(), dt), ctx);
    if (!out) {
      std::printf("Forward failed at step %d\n", step);
      return 1;
    }
    auto hout = out->to(DEV_CPU);
    // the oracle's chain, every operator rounding to the storage type as the device ones do
    std::vector<uint16_t> q((size_t)m * hidden), k((size_t)m * kvd), v((size_t)m * kvd);
    orc_matmul_bias(q.data(), x.data(), wq.data(), use_bias ? bq.data() : nullptr, m, hidden, hidden, dt, 0);
    orc_matmul_bias(k.data(), x.data(), wk.data(), use_bias ? bk.data() : nullptr, m, kvd, hidden, dt, 0);
    orc_matmul_bias(v.data(), x.data(), wv.data(), use_bias ? bv.data() : nullptr, m, kvd, hidden, dt, 0);
    std::vector<uint16_t> qr(q.size()), kr(k.size());
    orc_rope(qr.data(), q.data(), tab, (int)prev, m, H, hd, is_neox, dt);
    orc_rope(kr.data(), k.data(), tab, (int)prev, m, Hkv, hd, is_neox, dt);
    orc_kv_append(kc.data(), kr.data(), (int)prev, m, kvd);
    orc_kv_append(vc.data(), v.data(), (int)prev, m, kvd);
    std::vector<float> attn_f((size_t)m * hidden);
    orc_attention_f32(attn_f.data(), qr.data(), kc.data(), vc.data(), 1, m, (int)cur, (int)prev, H / Hkv, Hkv, hd,
                      max_seq_len, dt, 0);
    std::vector<uint16_t> attn(attn_f.size()), proj(attn_f.size()), gold(attn_f.size());
    orc_round_array(attn.data(), attn_f.data(), (int64_t)attn.size(), dt);
    orc_matmul_bias(proj.data(), attn.data(), wo.data(), nullptr, m, hidden, hidden, dt, 0);
    orc_add(gold.data(), res.data(), proj.data(), (int64_t)gold.size(), dt);
    std::vector<float> got_f(gold.size()), gold_f(gold.size());
    orc_widen_array(got_f.data(), static_cast<const uint16_t *>(hout->data_ptr), (int64_t)got_f.size(), dt);
    orc_widen_array(gold_f.data(), gold.data(), (int64_t)gold_f.size(), dt);
    // The rule of the reference's projection test (tests/gemm_test.cpp:163), all_close(0.01, 0.01),
    // or two steps of the storage type: four rounded operators in a row (projection, attention,
    // projection, add) can each land one step apart when their fp32 sums are ordered differently,
    // and two steps at magnitude 2..4 in bf16 is 0.031.
    // (taken at the magnitude of the add's operands: where residual and projection cancel, a
    // one-step difference of the projection is many steps of the small sum).
    const int mant = dt == DT_BFLOAT16 ? 7 : 10;
    std::vector<float> res_f(res.size());
    orc_widen_array(res_f.data(), res.data(), (int64_t)res_f.size(), dt);
    for (size_t i = 0; i < got_f.size(); ++i) {
      const float d = std::fabs(got_f[i] - gold_f[i]);
      const float big = std::fmax(std::fabs(got_f[i]), std::fabs(gold_f[i]));
      const float ustep = std::ldexp(1.0f, std::ilogb(std::fmax(std::fmax(big, std::fabs(res_f[i])), 1e-30f)) - mant);
      worst = std::fmax(worst, d);
      if (d > 0.01f && d / big > 0.01f && d > 2.0f * ustep) {
        if (++bad_total <= 5) std::printf("  step %d elem %zu: got %.6f gold %.6f\n", step, i, got_f[i], gold_f[i]);
      }
    }
    prev = cur;
  }
  if (profiling) profiler.Finish();
  std::printf("worst max-abs over %d steps: %.3e; %lld elements outside all_close(0.01, 0.01) and two steps; %zu trace records\n",
              steps + 1, worst, (long long)bad_total, profiler.EventCount());
  CHECK_LLMHIP(llmhip_stream_destroy(stream));
  // 6 records per step: 4 projections, the attention sub-block, the add
  const bool trace_ok = !profiling || profiler.EventCount() == (size_t)6 * (steps + 1);
  const bool ok = bad_total == 0 && trace_ok && hip_last_status() == 0;
  std::printf(ok ? "PASS\n" : "FAIL\n");
  return ok ? 0 : 1;
}
