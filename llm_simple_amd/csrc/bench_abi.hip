// C ABI of libllmhip_bench.so (declared in include/llmhip_bench.h): the measurement aids of the
// benchmark.  Built with LLMHIP_BENCH defined, so the prefill kernel linked here is the library's own
// copy with the clock stamp; the product library libllmhip.so holds none of this.
#include "../../include/llmhip_bench.h"

#include <hip/hip_runtime.h>

#include "bench_kernels.hpp"
#include "kernels.hpp"

using namespace LLMHIP_NS;

namespace {
inline int from_hip(hipError_t e) { return e == hipSuccess ? LLMHIP_OK : (int)e; }
inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline int device_count() {
  int n = 0;
  return hipGetDeviceCount(&n) == hipSuccess ? n : 0;
}
}  // namespace

extern "C" {

int llmhip_bench_flash_attn_gqa_clocked(void *out, const void *q, const void *k, const void *v, int m, int n,
                                        int offset, int group_size, int kv_head_num, int head_dim, int dt,
                                        void *clock_probe, void *stream) {
  if (!out || !q || !k || !v || !clock_probe || !aligned16(out) || !aligned16(q) || !aligned16(k) ||
      !aligned16(v) || (reinterpret_cast<uintptr_t>(clock_probe) & 7u))
    return LLMHIP_ERR_INVALID_ARG;
  if (m < 1 || n < 1 || offset < 0 || group_size < 1 || kv_head_num < 1 ||
      (dt != LLMHIP_DT_FLOAT16 && dt != LLMHIP_DT_BFLOAT16))
    return LLMHIP_ERR_INVALID_ARG;
  if (head_dim != 128) return LLMHIP_ERR_UNSUPPORTED;
  if (kv_head_num > 65535 || (long long)group_size * kv_head_num > 65535) return LLMHIP_ERR_UNSUPPORTED;
  if ((long long)m * group_size <= 16) return LLMHIP_ERR_UNSUPPORTED;  // prefill kernel only
  if (device_count() < 1) return LLMHIP_ERR_NO_DEVICE;
  return from_hip(launch_flash_prefill(out, q, k, v, m, n, offset, group_size, kv_head_num, dt,
                                       static_cast<hipStream_t>(stream), nullptr, clock_probe));
}

int llmhip_bench_mfma_ceiling(int mix, double target_ms, double *tflops) {
  if (!tflops || (mix != 0 && mix != 1) || target_ms < 0.0 || target_ms > 2000.0) return LLMHIP_ERR_INVALID_ARG;
  if (device_count() < 1) return LLMHIP_ERR_NO_DEVICE;
  return from_hip(run_mfma_ceiling(mix, target_ms, tflops));
}

int llmhip_bench_stream_read(const void *src_a, const void *src_b, size_t bytes_each, void *sink, size_t sink_bytes,
                             int variant, void *stream) {
  if (!src_a || !src_b || !sink || bytes_each == 0 || bytes_each % 16 != 0 || (variant != 0 && variant != 1))
    return LLMHIP_ERR_INVALID_ARG;
  if (sink_bytes < kStreamReadSinkBytes) return LLMHIP_ERR_WORKSPACE;
  if (!aligned16(src_a) || !aligned16(src_b) || !aligned16(sink)) return LLMHIP_ERR_INVALID_ARG;
  if (device_count() < 1) return LLMHIP_ERR_NO_DEVICE;
  return from_hip(launch_stream_read(src_a, src_b, bytes_each, sink, variant, static_cast<hipStream_t>(stream)));
}

}  // extern "C"
