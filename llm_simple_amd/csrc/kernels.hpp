// Launchers of the gfx950 kernels; called only by the C ABI in llmhip.hip after
// it has validated every argument.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "common.hpp"

namespace LLMHIP_NS {

// workspace: device memory of flash_prefill_workspace_bytes() bytes (0 = none needed) for the fp32
// partials of a key-range split; with a null workspace the call runs unsplit.
size_t flash_prefill_workspace_bytes(int m, int n, int offset, int group_size, int kv_head_num);
#ifdef LLMHIP_BENCH
// The measurement library's copy: clock_probe is a device pointer to two 64-bit counters that
// workgroup 0 fills with the shader-clock ticks and the reference-clock ticks of its lifetime.
hipError_t launch_flash_prefill(void *out, const void *q, const void *k, const void *v, int m,
                                int n, int offset, int group_size, int kv_head_num, int dt,
                                hipStream_t stream, void *workspace, void *clock_probe);
#else
hipError_t launch_flash_prefill(void *out, const void *q, const void *k, const void *v, int m,
                                int n, int offset, int group_size, int kv_head_num, int dt,
                                hipStream_t stream, void *workspace = nullptr);
#endif

// Compute units of the current device, cached per device; 256 when no device can be asked.
int device_compute_units();

// Split-KV decode.  rows = m * group_size <= 16 query rows per kv head.
size_t flash_decode_workspace_bytes(int batch, int m, int group_size, int kv_head_num,
                                    int num_splits);
int flash_decode_default_splits(int batch, int n, int kv_head_num);
int flash_decode_max_default_splits(long long pairs);
// The split count a launch really uses for n keys: at most one split per block of 128 keys.
int flash_decode_effective_splits(int num_splits, int n);
hipError_t launch_flash_decode(void *out, const void *q, const void *k, const void *v,
                               void *workspace, int batch, int m, int n, int offset,
                               int64_t kv_seq_stride, int group_size, int kv_head_num,
                               int num_splits, int dt, hipStream_t stream);

// One decode step of one sequence, rotary embedding and cache append fused into the decode kernel:
// q and the new K row are rotated with row `pos` of the table as they are loaded, the workgroups that own
// the last key range write row pos of both caches, attention runs over rows [0, pos].
hipError_t launch_flash_decode_step(void *out, void *k_cache, void *v_cache, const void *freq_cis,
                                    const void *in_q, const void *in_k, const void *in_v, void *workspace,
                                    int pos, int group_size, int kv_head_num, int is_neox, int num_splits,
                                    int dt, hipStream_t stream);

// Same decode with the split-KV partials in a fixed device array of kStaticDecodeScratchBytes inside
// the library: no allocation, no workspace argument.  The caller checks the size beforehand.
constexpr size_t kStaticDecodeScratchBytes = 4u << 20;
hipError_t launch_flash_decode_static(void *out, const void *q, const void *k, const void *v,
                                      int batch, int n, int64_t kv_seq_stride, int group_size,
                                      int kv_head_num, int num_splits, int dt, hipStream_t stream);

// q_heads may be 0 (rotate K only) and cache pointers may be null (no append):
// covers rope, rope_single and the fused rope + KV append.
hipError_t launch_rope_kv_append(void *out_q, void *out_k, void *out_v, const void *freq_cis,
                                 const void *in_q, const void *in_k, const void *in_v,
                                 int start_pos, int cur_size, int q_heads, int k_heads,
                                 int k_out_row_offset, int is_neox, int dt, hipStream_t stream);

// Projection GEMM through hipBLASLt: out[m][n] = round(lhs[m][k] . weight[n][k]^T + bias), bias
// fp32 [n] or null.  The first call creates the library handle and a 64 MiB workspace.
hipError_t launch_matmul_bias(void *out, const void *lhs, const void *weight, const float *bias,
                              int m, int n, int k, int dt, hipStream_t stream);
void release_matmul_resources();
hipError_t launch_add(void *out, const void *lhs, const void *rhs, size_t total, int dt,
                      hipStream_t stream);
// dst[0 .. bytes) = (unsigned char)value with a kernel (safe to capture into a HIP graph).
hipError_t launch_fill(void *dst, int value, size_t bytes, hipStream_t stream);

}  // namespace LLMHIP_NS
