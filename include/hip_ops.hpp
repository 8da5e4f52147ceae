// C++ face of the C ABI: the reference's operator names with the npu_ prefix
// replaced by hip_, same argument order and meaning (prebuild/npu_ops.h:6-18,
// :39-47), so that a *GPUImpl layer reads like its *NPUImpl sibling
// (src/llama2_layer_npu.cpp:790-869).  The stream is a hipStream_t carried as
// void* (the reference passes aclrtStream&).  Like the reference's void
// operators these return nothing; a failing status is logged to stderr and
// execution continues, the behaviour of CHECK_ACL (src/acl_util.hpp:6-12).
// hip_last_status() returns the most recent non-zero status for callers that
// want to check.
#pragma once
#include <cstdio>

#include "llmhip.h"

namespace llm_simple_amd {

enum DeviceType { DEV_CPU = 0, DEV_GPU, DEV_NPU };  // prebuild/defs.hpp:6

enum DataType : int32_t {  // prebuild/defs.hpp:8-18
  DT_UINT8 = 0,
  DT_INT8,
  DT_UINT32,
  DT_INT32,
  DT_FLOAT16,
  DT_BFLOAT16,
  DT_FLOAT32,
  DT_UINT64,
  DT_INT64,
};

// Bytes of `size` elements (prebuild/defs.hpp:20-41); (size_t)-1 for an unknown type.
inline size_t SizeOfTensor(size_t size, DataType dt) {
  static const int width[] = {1, 1, 4, 4, 2, 2, 4, 8, 8};
  if (dt < DT_UINT8 || dt > DT_INT64) return static_cast<size_t>(-1);
  return size * static_cast<size_t>(width[dt]);
}

using gpuStream_t = void *;

inline int &hip_last_status() {
  static thread_local int status = 0;
  return status;
}

#define CHECK_LLMHIP(x)                                                                  \
  do {                                                                                   \
    int ret__ = (x);                                                                     \
    if (ret__ != LLMHIP_OK) {                                                            \
      ::llm_simple_amd::hip_last_status() = ret__;                                       \
      std::fprintf(stderr, "%s:%d llmhip error %d: %s\n", __FILE__, __LINE__, ret__,     \
                   llmhip_error_string(ret__));                                          \
    }                                                                                    \
  } while (0)

inline void hip_flash_attn_layer(void *output_dev, void *q_dev, void *k_dev, void *v_dev, int m,
                                 int n, int offset, int head_num, int head_dim, DataType dt,
                                 gpuStream_t &stream) {
  CHECK_LLMHIP(llmhip_flash_attn(output_dev, q_dev, k_dev, v_dev, m, n, offset, head_num,
                                 head_dim, dt, stream));
}

inline void hip_flash_attn_gqa_layer(void *output_dev, void *q_dev, void *k_dev, void *v_dev,
                                     int m, int n, int offset, int group_size, int kv_head_num,
                                     int head_dim, DataType dt, gpuStream_t &stream) {
  CHECK_LLMHIP(llmhip_flash_attn_gqa(output_dev, q_dev, k_dev, v_dev, m, n, offset, group_size,
                                     kv_head_num, head_dim, dt, stream));
}

inline void hip_flash_attn_opt_prefill_layer(void *output_dev, void *q_dev, void *k_dev,
                                             void *v_dev, int m, int n, int offset, int head_num,
                                             int head_dim, DataType dt, gpuStream_t &stream) {
  CHECK_LLMHIP(llmhip_flash_attn_opt_prefill(output_dev, q_dev, k_dev, v_dev, m, n, offset,
                                             head_num, head_dim, dt, stream));
}

inline void hip_rope_layer(void *output_q_dev, void *output_k_dev, void *freqs_cis_dev,
                           void *input_q_dev, void *input_k_dev, int start_pos, int cur_size,
                           int n_heads, int hidden_dim, bool is_neox_style, DataType dt,
                           gpuStream_t &stream) {
  CHECK_LLMHIP(llmhip_rope(output_q_dev, output_k_dev, freqs_cis_dev, input_q_dev, input_k_dev,
                           start_pos, cur_size, n_heads, hidden_dim, is_neox_style ? 1 : 0, dt,
                           stream));
}

inline void hip_rope_single_layer(void *output_x_dev, void *freqs_cis_dev, void *input_x_dev,
                                  int start_pos, int cur_size, int n_heads, int hidden_dim,
                                  bool is_neox_style, DataType dt, gpuStream_t &stream) {
  CHECK_LLMHIP(llmhip_rope_single(output_x_dev, freqs_cis_dev, input_x_dev, start_pos, cur_size,
                                  n_heads, hidden_dim, is_neox_style ? 1 : 0, dt, stream));
}

// npu_matmul_nz_layer / npu_matmul_bias_nz_layer (prebuild/npu_ops.h:87-92) with the weight
// as W[n][k] row-major, and npu_add_layer (prebuild/npu_ops.h:81-82).
inline void hip_matmul_layer(void *output_dev, void *lhs_dev, void *rhs_dev, int m, int n, int k,
                             DataType dt, gpuStream_t &stream) {
  CHECK_LLMHIP(llmhip_matmul(output_dev, lhs_dev, rhs_dev, m, n, k, dt, stream));
}
inline void hip_matmul_bias_layer(void *output_dev, void *lhs_dev, void *rhs_dev, void *bias_dev,
                                  int m, int n, int k, DataType dt, gpuStream_t &stream) {
  CHECK_LLMHIP(llmhip_matmul_bias(output_dev, lhs_dev, rhs_dev, bias_dev, m, n, k, dt, stream));
}
inline void hip_add_layer(void *output_dev, void *lhs, void *rhs, int total_size, DataType dt,
                          gpuStream_t &stream) {
  CHECK_LLMHIP(llmhip_add(output_dev, lhs, rhs, total_size, dt, stream));
}

// rope(Q), rope(K) -> k_cache[start_pos:], V -> v_cache[start_pos:] in one launch: the
// sequence src/llama2_layer_npu.cpp:790-798 + :830-844 performs with four calls.
inline void hip_rope_kv_append_layer(void *output_q_dev, void *k_cache_dev, void *v_cache_dev,
                                     void *freqs_cis_dev, void *input_q_dev, void *input_k_dev,
                                     void *input_v_dev, int start_pos, int cur_size, int n_heads,
                                     int n_kv_heads, int head_dim, bool is_neox_style,
                                     DataType dt, gpuStream_t &stream) {
  CHECK_LLMHIP(llmhip_rope_kv_append(output_q_dev, k_cache_dev, v_cache_dev, freqs_cis_dev,
                                     input_q_dev, input_k_dev, input_v_dev, start_pos, cur_size,
                                     n_heads, n_kv_heads, head_dim, is_neox_style ? 1 : 0, dt,
                                     stream));
}

// Batched decode: one query token for each of `batch` sequences that each own a cache of
// kv_seq_stride rows (n valid).  No counterpart in the reference header, where decode is
// npu_flash_attn_gqa_layer with m = 1 (src/llama2_layer_npu.cpp:866-869) and batch is always 1.
// workspace_dev: llmhip_flash_decode_workspace_bytes(...) bytes of device memory owned by the caller.
inline void hip_flash_decode_gqa_layer(void *output_dev, void *q_dev, void *k_cache_dev, void *v_cache_dev,
                                       void *workspace_dev, size_t workspace_bytes, int batch, int n,
                                       int64_t kv_seq_stride, int group_size, int kv_head_num, int head_dim,
                                       int num_splits, DataType dt, gpuStream_t &stream) {
  CHECK_LLMHIP(llmhip_flash_decode_gqa(output_dev, q_dev, k_cache_dev, v_cache_dev, workspace_dev,
                                       workspace_bytes, batch, n, kv_seq_stride, group_size, kv_head_num,
                                       head_dim, num_splits, dt, stream));
}

// The same decode for callers that cannot allocate or carry a workspace (HIP graph capture, serving
// loops): the partials live in a fixed 4 MiB device array inside the library.
inline void hip_flash_decode_gqa_static_layer(void *output_dev, void *q_dev, void *k_cache_dev,
                                              void *v_cache_dev, int batch, int n, int64_t kv_seq_stride,
                                              int group_size, int kv_head_num, int head_dim, int num_splits,
                                              DataType dt, gpuStream_t &stream) {
  CHECK_LLMHIP(llmhip_flash_decode_gqa_static(output_dev, q_dev, k_cache_dev, v_cache_dev, batch, n,
                                              kv_seq_stride, group_size, kv_head_num, head_dim, num_splits,
                                              dt, stream));
}

// One decode step in one pass over the cache: the two npu_rope_single_layer calls, the two cache
// copies and npu_flash_attn_gqa_layer(m = 1) of src/llama2_layer_npu.cpp:790-869 in one operator.
inline void hip_decode_step_gqa_layer(void *output_dev, void *k_cache_dev, void *v_cache_dev,
                                      void *freqs_cis_dev, void *input_q_dev, void *input_k_dev,
                                      void *input_v_dev, int pos, int group_size, int kv_head_num, int head_dim,
                                      bool is_neox_style, DataType dt, gpuStream_t &stream) {
  CHECK_LLMHIP(llmhip_decode_step_gqa(output_dev, k_cache_dev, v_cache_dev, freqs_cis_dev, input_q_dev,
                                      input_k_dev, input_v_dev, pos, group_size, kv_head_num, head_dim,
                                      is_neox_style ? 1 : 0, dt, stream));
}

}  // namespace llm_simple_amd
