// C ABI of libllmhip.so (declared in include/llmhip.h): argument validation,
// dispatch to the gfx950 kernels, and thin wrappers over the HIP runtime so
// that the C++ device layer above needs no HIP header.
#include "../../include/llmhip.h"

#include <hip/hip_runtime.h>

#include <map>
#include <mutex>
#include <vector>

#include "kernels.hpp"

using namespace llmhip;

namespace {

constexpr int kMaxDecodeCols = 16;
constexpr int kMaxDecodeSplits = 256;

inline hipStream_t as_stream(void *s) { return static_cast<hipStream_t>(s); }
inline int from_hip(hipError_t e) { return e == hipSuccess ? LLMHIP_OK : (int)e; }
inline bool dtype_ok(int dt) { return dt == LLMHIP_DT_FLOAT16 || dt == LLMHIP_DT_BFLOAT16; }
// every kernel moves 16-byte pieces: a misaligned base pointer would fault on the device
inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
template <typename... P> inline bool all_aligned16(P... ptrs) { return (aligned16(ptrs) && ...); }

// Split-KV scratch for the entry points that mirror the reference signatures
// and therefore have no workspace argument: one buffer per stream that only grows.
// A buffer that has become too small is not freed when a larger one replaces it: launches already
// queued, and HIP graphs captured earlier, keep their pointer valid.  Retired buffers go with
// llmhip_stream_destroy / llmhip_release_internal_workspace.
struct StreamScratch {
  void *ptr = nullptr;
  size_t bytes = 0;
  std::vector<void *> retired;
};
std::mutex g_scratch_mu;
std::map<void *, StreamScratch> g_scratch;

// Caller holds g_scratch_mu.  Growing allocates, which a stream under capture must not do: such a
// call is refused with LLMHIP_ERR_WORKSPACE (warm the stream up with its largest shape first).
int scratch_for_locked(void *stream, size_t need, void **out) {
  StreamScratch &s = g_scratch[stream];
  if (s.bytes < need) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(as_stream(stream), &cap) != hipSuccess) (void)hipGetLastError();
    if (cap != hipStreamCaptureStatusNone) return LLMHIP_ERR_WORKSPACE;
    size_t want = need < (size_t)(4u << 20) ? (size_t)(4u << 20) : need;
    void *fresh = nullptr;
    hipError_t e = hipMalloc(&fresh, want);
    if (e != hipSuccess) return (int)e;
    if (s.ptr) s.retired.push_back(s.ptr);
    s.ptr = fresh;
    s.bytes = want;
  }
  *out = s.ptr;
  return LLMHIP_OK;
}

int attn_common(void *out, const void *q, const void *k, const void *v, int m, int n,
                int offset, int group_size, int kv_head_num, int head_dim, int dt,
                void *stream) {
  if (!out || !q || !k || !v || !all_aligned16(out, q, k, v)) return LLMHIP_ERR_INVALID_ARG;
  if (m < 1 || n < 1 || offset < 0 || group_size < 1 || kv_head_num < 1)
    return LLMHIP_ERR_INVALID_ARG;
  if (!dtype_ok(dt)) return LLMHIP_ERR_INVALID_ARG;
  if (head_dim != 128) return LLMHIP_ERR_UNSUPPORTED;
  // grid dimensions and the 32-bit row offsets of the tile loader
  if (kv_head_num > 65535 || (long long)group_size * kv_head_num > 65535) return LLMHIP_ERR_UNSUPPORTED;
  if ((long long)m * group_size <= kMaxDecodeCols) {
    // few query rows: stream the cache once with the split-KV kernel
    const int n_vis = (n < m + offset) ? n : m + offset;  // keys any row can see
    int splits = flash_decode_default_splits(1, n_vis, kv_head_num);
    void *ws = nullptr;
    const size_t need = flash_decode_workspace_bytes(1, m, group_size, kv_head_num, splits);
    if (!need)
      return from_hip(launch_flash_decode(out, q, k, v, nullptr, 1, m, n_vis, offset, n_vis, group_size,
                                          kv_head_num, splits, dt, as_stream(stream)));
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    int rc = scratch_for_locked(stream, need, &ws);
    if (rc != LLMHIP_OK) return rc;
    return from_hip(launch_flash_decode(out, q, k, v, ws, 1, m, n_vis, offset, n_vis,
                                        group_size, kv_head_num, splits, dt,
                                        as_stream(stream)));
  }
  // a chunk of few rows over a long cache is split over the key range: fp32 partials in the
  // per-stream scratch
  const size_t need = flash_prefill_workspace_bytes(m, n, offset, group_size, kv_head_num);
  if (!need)
    return from_hip(launch_flash_prefill(out, q, k, v, m, n, offset, group_size, kv_head_num, dt,
                                         as_stream(stream)));
  std::lock_guard<std::mutex> lk(g_scratch_mu);
  void *ws = nullptr;
  int rc = scratch_for_locked(stream, need, &ws);
  if (rc != LLMHIP_OK) return rc;
  return from_hip(launch_flash_prefill(out, q, k, v, m, n, offset, group_size, kv_head_num, dt,
                                       as_stream(stream), ws));
}

}  // namespace

extern "C" {

int llmhip_flash_attn(void *out, const void *q, const void *k, const void *v, int m, int n,
                      int offset, int head_num, int head_dim, int dt, void *stream) {
  return attn_common(out, q, k, v, m, n, offset, 1, head_num, head_dim, dt, stream);
}

int llmhip_flash_attn_gqa(void *out, const void *q, const void *k, const void *v, int m,
                          int n, int offset, int group_size, int kv_head_num, int head_dim,
                          int dt, void *stream) {
  return attn_common(out, q, k, v, m, n, offset, group_size, kv_head_num, head_dim, dt, stream);
}

int llmhip_flash_attn_opt_prefill(void *out, const void *q, const void *k, const void *v,
                                  int m, int n, int offset, int head_num, int head_dim,
                                  int dt, void *stream) {
  return attn_common(out, q, k, v, m, n, offset, 1, head_num, head_dim, dt, stream);
}

size_t llmhip_flash_attn_scratch_bytes(int m, int n, int offset, int group_size, int kv_head_num) {
  if (m < 1 || n < 1 || offset < 0 || group_size < 1 || kv_head_num < 1) return 0;
  if ((long long)m * group_size <= kMaxDecodeCols) {
    const int n_vis = (n < m + offset) ? n : m + offset;
    return flash_decode_workspace_bytes(1, m, group_size, kv_head_num,
                                        flash_decode_default_splits(1, n_vis, kv_head_num));
  }
  return flash_prefill_workspace_bytes(m, n, offset, group_size, kv_head_num);
}

int llmhip_flash_decode_default_splits(int batch, int n, int kv_head_num) {
  if (batch < 1 || n < 1 || kv_head_num < 1) return LLMHIP_ERR_INVALID_ARG;
  return flash_decode_default_splits(batch, n, kv_head_num);
}

size_t llmhip_flash_decode_workspace_bytes(int batch, int group_size, int kv_head_num,
                                           int head_dim, int num_splits) {
  if (batch < 1 || group_size < 1 || kv_head_num < 1 || head_dim != 128) return 0;
  if (num_splits <= 0) {
    // the largest count the default rule picks for any KV length
    num_splits = flash_decode_max_default_splits((long long)batch * kv_head_num);
  }
  if (num_splits > kMaxDecodeSplits) num_splits = kMaxDecodeSplits;
  return flash_decode_workspace_bytes(batch, 1, group_size, kv_head_num, num_splits);
}

int llmhip_flash_decode_gqa(void *out, const void *q, const void *k_cache,
                            const void *v_cache, void *workspace, size_t workspace_bytes,
                            int batch, int n, int64_t kv_seq_stride, int group_size,
                            int kv_head_num, int head_dim, int num_splits, int dt,
                            void *stream) {
  if (!out || !q || !k_cache || !v_cache || !all_aligned16(out, q, k_cache, v_cache, workspace))
    return LLMHIP_ERR_INVALID_ARG;
  if (batch < 1 || n < 1 || group_size < 1 || kv_head_num < 1 || kv_seq_stride < n)
    return LLMHIP_ERR_INVALID_ARG;
  if (!dtype_ok(dt)) return LLMHIP_ERR_INVALID_ARG;
  if (head_dim != 128 || group_size > kMaxDecodeCols) return LLMHIP_ERR_UNSUPPORTED;
  if (batch > 65535 || kv_head_num > 65535) return LLMHIP_ERR_UNSUPPORTED;
  if (num_splits <= 0) num_splits = flash_decode_default_splits(batch, n, kv_head_num);
  if (num_splits > kMaxDecodeSplits) num_splits = kMaxDecodeSplits;  // the combine kernel's limit
  const size_t need = flash_decode_workspace_bytes(batch, 1, group_size, kv_head_num, num_splits);
  if (need && (!workspace || workspace_bytes < need)) return LLMHIP_ERR_WORKSPACE;
  return from_hip(launch_flash_decode(out, q, k_cache, v_cache, workspace, batch, 1, n, n - 1,
                                      kv_seq_stride, group_size, kv_head_num, num_splits, dt,
                                      as_stream(stream)));
}

int llmhip_flash_decode_gqa_static(void *out, const void *q, const void *k_cache, const void *v_cache,
                                   int batch, int n, int64_t kv_seq_stride, int group_size,
                                   int kv_head_num, int head_dim, int num_splits, int dt, void *stream) {
  if (!out || !q || !k_cache || !v_cache || !all_aligned16(out, q, k_cache, v_cache))
    return LLMHIP_ERR_INVALID_ARG;
  if (batch < 1 || n < 1 || group_size < 1 || kv_head_num < 1 || kv_seq_stride < n)
    return LLMHIP_ERR_INVALID_ARG;
  if (!dtype_ok(dt)) return LLMHIP_ERR_INVALID_ARG;
  if (head_dim != 128 || group_size > kMaxDecodeCols) return LLMHIP_ERR_UNSUPPORTED;
  if (batch > 65535 || kv_head_num > 65535) return LLMHIP_ERR_UNSUPPORTED;
  if (num_splits <= 0) {
    // the default count, lowered until its partials fit the fixed array (one split needs none)
    num_splits = flash_decode_default_splits(batch, n, kv_head_num);
    while (num_splits > 1 &&
           flash_decode_workspace_bytes(batch, 1, group_size, kv_head_num, num_splits) > kStaticDecodeScratchBytes)
      --num_splits;
  }
  if (num_splits > kMaxDecodeSplits) num_splits = kMaxDecodeSplits;
  // the launch uses at most one split per 128 keys: a larger count is judged by what it becomes
  num_splits = flash_decode_effective_splits(num_splits, n);
  // the fixed array must hold the partials of every (sequence, kv head, split)
  if (flash_decode_workspace_bytes(batch, 1, group_size, kv_head_num, num_splits) > kStaticDecodeScratchBytes)
    return LLMHIP_ERR_WORKSPACE;
  return from_hip(launch_flash_decode_static(out, q, k_cache, v_cache, batch, n, kv_seq_stride, group_size,
                                             kv_head_num, num_splits, dt, as_stream(stream)));
}

size_t llmhip_flash_decode_static_scratch_bytes(void) { return kStaticDecodeScratchBytes; }

int llmhip_decode_step_gqa(void *out, void *k_cache, void *v_cache, const void *freq_cis, const void *in_q,
                           const void *in_k, const void *in_v, int pos, int group_size, int kv_head_num,
                           int head_dim, int is_neox_style, int dt, void *stream) {
  if (!out || !k_cache || !v_cache || !freq_cis || !in_q || !in_k || !in_v ||
      !all_aligned16(out, k_cache, v_cache, freq_cis, in_q, in_k, in_v))
    return LLMHIP_ERR_INVALID_ARG;
  if (pos < 0 || pos == INT32_MAX || group_size < 1 || kv_head_num < 1 || !dtype_ok(dt)) return LLMHIP_ERR_INVALID_ARG;
  if (head_dim != 128 || group_size > kMaxDecodeCols) return LLMHIP_ERR_UNSUPPORTED;
  if (kv_head_num > 65535) return LLMHIP_ERR_UNSUPPORTED;
  const int n = pos + 1;
  const int splits = flash_decode_default_splits(1, n, kv_head_num);
  const size_t need = flash_decode_workspace_bytes(1, 1, group_size, kv_head_num, splits);
  if (!need)
    return from_hip(launch_flash_decode_step(out, k_cache, v_cache, freq_cis, in_q, in_k, in_v, nullptr, pos,
                                             group_size, kv_head_num, is_neox_style, splits, dt,
                                             as_stream(stream)));
  std::lock_guard<std::mutex> lk(g_scratch_mu);
  void *ws = nullptr;
  int rc = scratch_for_locked(stream, need, &ws);
  if (rc != LLMHIP_OK) return rc;
  return from_hip(launch_flash_decode_step(out, k_cache, v_cache, freq_cis, in_q, in_k, in_v, ws, pos, group_size,
                                           kv_head_num, is_neox_style, splits, dt, as_stream(stream)));
}

int llmhip_rope(void *out_q, void *out_k, const void *freq_cis, const void *in_q,
                const void *in_k, int start_pos, int cur_size, int n_heads, int hidden_dim,
                int is_neox_style, int dt, void *stream) {
  if (!out_q || !out_k || !freq_cis || !in_q || !in_k || !all_aligned16(out_q, out_k, freq_cis, in_q, in_k))
    return LLMHIP_ERR_INVALID_ARG;
  if (start_pos < 0 || cur_size < 1 || n_heads < 1 || !dtype_ok(dt))
    return LLMHIP_ERR_INVALID_ARG;
  if (hidden_dim != n_heads * 128) return LLMHIP_ERR_UNSUPPORTED;
  return from_hip(launch_rope_kv_append(out_q, out_k, nullptr, freq_cis, in_q, in_k, nullptr,
                                        start_pos, cur_size, n_heads, n_heads, 0,
                                        is_neox_style, dt, as_stream(stream)));
}

int llmhip_rope_single(void *out, const void *freq_cis, const void *in, int start_pos,
                       int cur_size, int n_heads, int hidden_dim, int is_neox_style, int dt,
                       void *stream) {
  if (!out || !freq_cis || !in || !all_aligned16(out, freq_cis, in)) return LLMHIP_ERR_INVALID_ARG;
  if (start_pos < 0 || cur_size < 1 || n_heads < 1 || !dtype_ok(dt))
    return LLMHIP_ERR_INVALID_ARG;
  if (hidden_dim != n_heads * 128) return LLMHIP_ERR_UNSUPPORTED;
  return from_hip(launch_rope_kv_append(out, nullptr, nullptr, freq_cis, in, nullptr, nullptr,
                                        start_pos, cur_size, n_heads, 0, 0, is_neox_style, dt,
                                        as_stream(stream)));
}

int llmhip_rope_kv_append(void *out_q, void *k_cache, void *v_cache, const void *freq_cis,
                          const void *in_q, const void *in_k, const void *in_v,
                          int start_pos, int cur_size, int n_heads, int n_kv_heads,
                          int head_dim, int is_neox_style, int dt, void *stream) {
  if (!out_q || !k_cache || !v_cache || !freq_cis || !in_q || !in_k || !in_v ||
      !all_aligned16(out_q, k_cache, v_cache, freq_cis, in_q, in_k, in_v))
    return LLMHIP_ERR_INVALID_ARG;
  if (start_pos < 0 || cur_size < 1 || n_heads < 1 || n_kv_heads < 1 || !dtype_ok(dt))
    return LLMHIP_ERR_INVALID_ARG;
  if (head_dim != 128) return LLMHIP_ERR_UNSUPPORTED;
  return from_hip(launch_rope_kv_append(out_q, k_cache, v_cache, freq_cis, in_q, in_k, in_v,
                                        start_pos, cur_size, n_heads, n_kv_heads, start_pos,
                                        is_neox_style, dt, as_stream(stream)));
}

/* ---------------- runtime surface ---------------- */

int llmhip_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) return 0;
  return n;
}
int llmhip_device_props(int device, int *compute_units, int *max_clock_khz, size_t *total_mem_bytes) {
  if (llmhip_device_count() < 1) return LLMHIP_ERR_NO_DEVICE;
  hipDeviceProp_t prop;
  hipError_t e = hipGetDeviceProperties(&prop, device);
  if (e != hipSuccess) return (int)e;
  if (compute_units) *compute_units = prop.multiProcessorCount;
  if (max_clock_khz) *max_clock_khz = prop.clockRate;
  if (total_mem_bytes) *total_mem_bytes = prop.totalGlobalMem;
  return LLMHIP_OK;
}
int llmhip_set_device(int device) {
  if (llmhip_device_count() < 1) return LLMHIP_ERR_NO_DEVICE;
  return from_hip(hipSetDevice(device));
}
int llmhip_malloc(void **ptr, size_t bytes) {
  if (!ptr) return LLMHIP_ERR_INVALID_ARG;
  if (llmhip_device_count() < 1) return LLMHIP_ERR_NO_DEVICE;
  return from_hip(hipMalloc(ptr, bytes));
}
int llmhip_free(void *ptr) { return from_hip(hipFree(ptr)); }
int llmhip_memcpy_h2d(void *dst, const void *src, size_t bytes) {
  if (!dst || !src) return LLMHIP_ERR_INVALID_ARG;
  return from_hip(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
}
int llmhip_memcpy_d2h(void *dst, const void *src, size_t bytes) {
  if (!dst || !src) return LLMHIP_ERR_INVALID_ARG;
  return from_hip(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
}
int llmhip_memcpy_d2d_async(void *dst, const void *src, size_t bytes, void *stream) {
  if (!dst || !src) return LLMHIP_ERR_INVALID_ARG;
  return from_hip(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, as_stream(stream)));
}
int llmhip_memset_async(void *dst, int value, size_t bytes, void *stream) {
  if (!dst) return LLMHIP_ERR_INVALID_ARG;
  // a fill kernel, not hipMemsetAsync: the call may be captured into a HIP graph
  return from_hip(launch_fill(dst, value, bytes, as_stream(stream)));
}
int llmhip_stream_create(void **stream) {
  if (!stream) return LLMHIP_ERR_INVALID_ARG;
  if (llmhip_device_count() < 1) return LLMHIP_ERR_NO_DEVICE;
  hipStream_t s;
  hipError_t e = hipStreamCreate(&s);  // default priority
  if (e != hipSuccess) return (int)e;
  *stream = s;
  return LLMHIP_OK;
}
int llmhip_stream_destroy(void *stream) {
  {
    // the split-KV scratch kept for this stream goes with it
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    auto it = g_scratch.find(stream);
    if (it != g_scratch.end()) {
      if (it->second.ptr) {
        (void)hipStreamSynchronize(as_stream(stream));
        (void)hipFree(it->second.ptr);
      }
      for (void *old : it->second.retired) (void)hipFree(old);
      g_scratch.erase(it);
    }
  }
  return from_hip(hipStreamDestroy(as_stream(stream)));
}
int llmhip_stream_sync(void *stream) { return from_hip(hipStreamSynchronize(as_stream(stream))); }
int llmhip_device_sync(void) { return from_hip(hipDeviceSynchronize()); }
int llmhip_event_create(void **event) {
  if (!event) return LLMHIP_ERR_INVALID_ARG;
  if (llmhip_device_count() < 1) return LLMHIP_ERR_NO_DEVICE;
  hipEvent_t ev;
  hipError_t e = hipEventCreate(&ev);
  if (e != hipSuccess) return (int)e;
  *event = ev;
  return LLMHIP_OK;
}
int llmhip_event_destroy(void *event) {
  return from_hip(hipEventDestroy(static_cast<hipEvent_t>(event)));
}
int llmhip_event_record(void *event, void *stream) {
  return from_hip(hipEventRecord(static_cast<hipEvent_t>(event), as_stream(stream)));
}
int llmhip_event_sync(void *event) {
  return from_hip(hipEventSynchronize(static_cast<hipEvent_t>(event)));
}
int llmhip_event_query(void *event) {
  const hipError_t e = hipEventQuery(static_cast<hipEvent_t>(event));
  if (e == hipErrorNotReady) {
    (void)hipGetLastError();  // not an error: leave nothing behind for the next call to report
    return LLMHIP_NOT_READY;
  }
  return from_hip(e);
}
int llmhip_event_elapsed_ms(float *ms, void *start, void *stop) {
  if (!ms) return LLMHIP_ERR_INVALID_ARG;
  return from_hip(
      hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
}
const char *llmhip_error_string(int status) {
  switch (status) {
    case LLMHIP_OK: return "ok";
    case LLMHIP_ERR_INVALID_ARG: return "invalid argument";
    case LLMHIP_ERR_UNSUPPORTED: return "unsupported shape (head_dim must be 128)";
    case LLMHIP_ERR_WORKSPACE:
      return "workspace missing or too small (or batch * kv heads * splits beyond the fixed scratch of the "
             "allocation-free decode)";
    case LLMHIP_ERR_NO_DEVICE: return "no HIP device";
    case LLMHIP_NOT_READY: return "event not complete yet";
    default: break;
  }
  if (status > 0) return hipGetErrorString(static_cast<hipError_t>(status));
  return "unknown status";
}
int llmhip_release_internal_workspace(void) {
  std::lock_guard<std::mutex> lk(g_scratch_mu);
  int rc = LLMHIP_OK;
  if (!g_scratch.empty()) {
    // queued launches may still use the buffers
    hipError_t e = hipDeviceSynchronize();
    if (e != hipSuccess) rc = (int)e;
  }
  for (auto &kv : g_scratch) {
    if (kv.second.ptr) {
      hipError_t e = hipFree(kv.second.ptr);
      if (e != hipSuccess) rc = (int)e;
    }
    for (void *old : kv.second.retired) (void)hipFree(old);
  }
  g_scratch.clear();
  release_matmul_resources();
  return rc;
}

static int matmul_common(void *out, const void *lhs, const void *weight, const void *bias, int m,
                         int n, int k, int dt, void *stream) {
  if (!out || !lhs || !weight) return LLMHIP_ERR_INVALID_ARG;
  if (m < 1 || n < 1 || k < 1 || !dtype_ok(dt)) return LLMHIP_ERR_INVALID_ARG;
  if (n % 16 != 0 || k % 16 != 0) return LLMHIP_ERR_UNSUPPORTED;
  return from_hip(launch_matmul_bias(out, lhs, weight, static_cast<const float *>(bias), m, n, k, dt,
                                     as_stream(stream)));
}
int llmhip_matmul(void *out, const void *lhs, const void *weight, int m, int n, int k, int dt,
                  void *stream) {
  return matmul_common(out, lhs, weight, nullptr, m, n, k, dt, stream);
}
int llmhip_matmul_bias(void *out, const void *lhs, const void *weight, const void *bias_f32, int m,
                       int n, int k, int dt, void *stream) {
  if (!bias_f32) return LLMHIP_ERR_INVALID_ARG;
  return matmul_common(out, lhs, weight, bias_f32, m, n, k, dt, stream);
}
int llmhip_add(void *out, const void *lhs, const void *rhs, long long total_size, int dt,
               void *stream) {
  if (!out || !lhs || !rhs || total_size < 0 || !dtype_ok(dt) || !all_aligned16(out, lhs, rhs))
    return LLMHIP_ERR_INVALID_ARG;
  return from_hip(launch_add(out, lhs, rhs, (size_t)total_size, dt, as_stream(stream)));
}

}  // extern "C"
