/*
 * llmhip.h -- C ABI of the MI355X (gfx950) attention path for llm_simple.
 *
 * One shared library, libllmhip.so, exports everything declared here.  Every
 * entry point is extern "C", takes plain pointers and integers, enqueues its
 * work on the HIP stream it is given (a hipStream_t passed as void*, NULL =
 * the default stream) and returns without waiting, exactly like the
 * reference's operator functions, which are asynchronous on their aclrtStream
 * (prebuild/npu_ops.h).  Unlike the reference's void functions every call
 * returns a status: 0 on success, a negative LLMHIP_ERR_* for arguments
 * rejected before anything is launched, or a positive hipError_t value.
 *
 * Element type T is selected by `dt`, numbered as the reference's DataType
 * (prebuild/defs.hpp:8-18): 4 = fp16, 5 = bf16.  All tensors are dense,
 * row-major and token-major.  head_dim must be 128 (every model the reference
 * supports has hidden/n_heads == 128).
 */
#ifndef LLMHIP_H_
#define LLMHIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LLMHIP_DT_FLOAT16 4  /* prebuild/defs.hpp:13 */
#define LLMHIP_DT_BFLOAT16 5 /* prebuild/defs.hpp:14 */

#define LLMHIP_OK 0
#define LLMHIP_ERR_INVALID_ARG (-1)   /* null or misaligned pointer, non-positive size, bad dtype */
#define LLMHIP_ERR_UNSUPPORTED (-2)   /* head_dim != 128, group too large for the kernel */
#define LLMHIP_ERR_WORKSPACE (-3)     /* workspace missing or too small */
#define LLMHIP_ERR_NO_DEVICE (-4)     /* no HIP device visible */
#define LLMHIP_NOT_READY (-5)         /* llmhip_event_query: the event has not completed yet (no error) */

/* Every device pointer handed to the operators below must be 16-byte aligned (anything the
 * runtime's allocator returns is; so is any row of a cache whose base is): the kernels move
 * 16-byte pieces, and a misaligned pointer is rejected with LLMHIP_ERR_INVALID_ARG before any
 * launch rather than left to fault on the device. */

/* ------------------------------------------------------------------ */
/* attention                                                           */
/* ------------------------------------------------------------------ */

/* Replaces npu_flash_attn_layer (prebuild/npu_ops.h:6-8; exercised by
 * tests/flash_attn_test.cpp:206-207).
 * out[m][head_num*head_dim] = softmax(scale * q k^T + causal(offset)) v with
 * q[m][head_num][head_dim], k and v = cache base pointers of which rows
 * [0, n) are read, key c masked for query r iff c > r + offset, scale =
 * 1/sqrt(head_dim) computed inside. */
int llmhip_flash_attn(void *out, const void *q, const void *k, const void *v, int m, int n,
                      int offset, int head_num, int head_dim, int dt, void *stream);

/* Replaces npu_flash_attn_gqa_layer (prebuild/npu_ops.h:10-13; call site
 * src/llama2_layer_npu.cpp:866-869).  k, v are [n][kv_head_num][head_dim];
 * query head h reads kv head h / group_size. */
int llmhip_flash_attn_gqa(void *out, const void *q, const void *k, const void *v, int m,
                          int n, int offset, int group_size, int kv_head_num, int head_dim,
                          int dt, void *stream);

/* Replaces npu_flash_attn_opt_prefill_layer (prebuild/npu_ops.h:15-18; call
 * site src/llama2_layer_npu.cpp:370-374).  Same contract as llmhip_flash_attn. */
int llmhip_flash_attn_opt_prefill(void *out, const void *q, const void *k, const void *v,
                                  int m, int n, int offset, int head_num, int head_dim,
                                  int dt, void *stream);

/* How many bytes of the library's per-stream scratch buffer a llmhip_flash_attn* call with these
 * arguments uses (head_num of the MHA entry points = kv_head_num with group_size 1): the fp32
 * partials of the split-KV decode kernel (m * group_size <= 16) or of a key-range split of the
 * prefill kernel (a chunk of few rows over a cache at least 8 times longer); 0 for ordinary
 * prefill shapes.  The buffer is allocated on the first call that needs it on a stream (at least
 * 4 MiB) and replaced by a larger one when a later call needs more; a replaced buffer is kept, not
 * freed, so launches already queued and HIP graphs captured earlier keep a valid pointer.  All of
 * them go with llmhip_stream_destroy or llmhip_release_internal_workspace.  HIP graphs: a call made
 * while its stream is capturing cannot allocate and is refused with LLMHIP_ERR_WORKSPACE when the
 * buffer would have to grow -- warm the stream up with its largest shape before capturing. */
size_t llmhip_flash_attn_scratch_bytes(int m, int n, int offset, int group_size, int kv_head_num);

/* Batched split-KV decode over a contiguous per-sequence KV cache: one query
 * token per sequence, `batch` independent sequences of the same valid length n.
 * q, out: [batch][group_size*kv_head_num][head_dim];
 * k_cache, v_cache: [batch][kv_seq_stride][kv_head_num][head_dim] (rows [0,n)
 * of each sequence are read; kv_seq_stride >= n is the allocated row count,
 * the reference's max_seq_len, src/llama2_layer_npu.cpp:1148-1149).
 * The reference has no batch dimension and no split-KV (decode there is
 * npu_flash_attn_gqa_layer with m = 1, src/llama2_layer_npu.cpp:866-869);
 * for batch == 1 this call returns what llmhip_flash_attn_gqa(m=1,
 * offset=n-1) returns.  num_splits <= 0 picks llmhip_flash_decode_default_splits;
 * values above 256 are treated as 256.
 * workspace: device memory of at least llmhip_flash_decode_workspace_bytes()
 * bytes, owned by the caller, so that the call allocates nothing. */
int llmhip_flash_decode_gqa(void *out, const void *q, const void *k_cache,
                            const void *v_cache, void *workspace, size_t workspace_bytes,
                            int batch, int n, int64_t kv_seq_stride, int group_size,
                            int kv_head_num, int head_dim, int num_splits, int dt,
                            void *stream);

/* Workspace size of llmhip_flash_decode_gqa for the same (batch, group_size, kv_head_num, num_splits);
 * 0 for one split.  num_splits <= 0 gives the size that covers the default split count at any KV
 * length (at most about one workgroup per compute unit of the device), so a caller that passes num_splits <= 0
 * to the decode call can size its workspace once. */
size_t llmhip_flash_decode_workspace_bytes(int batch, int group_size, int kv_head_num,
                                           int head_dim, int num_splits);

/* The split count the decode call uses for num_splits <= 0: about one workgroup per compute unit of the
 * current device, from a small model of the launch (whole rounds of workgroups preferred). */
int llmhip_flash_decode_default_splits(int batch, int n, int kv_head_num);

/* llmhip_flash_decode_gqa for callers that cannot allocate device memory or carry a workspace
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  Same arguments and results as llmhip_flash_decode_gqa without
 * `workspace`: the split-KV partials go to a fixed array of
 * llmhip_flash_decode_static_scratch_bytes() (4 MiB) of device memory inside the library, which
 * every GPU the library runs on holds until the process ends.  The call allocates and frees
 * nothing.  Limit: batch * kv_head_num * num_splits * 8320 bytes must fit the array (504 slots);
 * an explicit num_splits beyond that is rejected with LLMHIP_ERR_WORKSPACE before anything is
 * launched, the default count (num_splits <= 0) is lowered until it fits (one split needs no
 * scratch and always fits).  All calls on a GPU share the array: calls that overlap on one GPU (different streams,
 * different threads) race; calls on one stream are ordered and safe. */
int llmhip_flash_decode_gqa_static(void *out, const void *q, const void *k_cache,
                                   const void *v_cache, int batch, int n, int64_t kv_seq_stride,
                                   int group_size, int kv_head_num, int head_dim, int num_splits,
                                   int dt, void *stream);
size_t llmhip_flash_decode_static_scratch_bytes(void);

/* One decode step of one sequence in a single pass over the cache: what the reference does per
 * generated token with four calls -- npu_rope_single_layer on q and on k, two cache copies and
 * npu_flash_attn_gqa_layer with m = 1 (src/llama2_layer_npu.cpp:790-798, :830-844, :866-869) --
 * with the rotary embedding and the append inside the decode kernel.  in_q [group_size*kv_head_num]
 * [head_dim], in_k, in_v [kv_head_num][head_dim]: the projections of the token at position pos,
 * unrotated.  Rows [0, pos) of the caches are read; row pos of k_cache receives rope(in_k), row pos
 * of v_cache receives in_v; out = attention of rope(in_q) over rows [0, pos].  The results (output
 * and both cache rows) are bit-identical to llmhip_rope_kv_append(start_pos = pos, cur_size = 1)
 * followed by llmhip_flash_attn_gqa(m = 1, n = pos + 1, offset = pos).  Split-KV partials come from
 * the same per-stream scratch as llmhip_flash_attn_gqa. */
int llmhip_decode_step_gqa(void *out, void *k_cache, void *v_cache, const void *freq_cis,
                           const void *in_q, const void *in_k, const void *in_v, int pos,
                           int group_size, int kv_head_num, int head_dim, int is_neox_style, int dt,
                           void *stream);

/* ------------------------------------------------------------------ */
/* rotary embedding and KV-cache append                                */
/* ------------------------------------------------------------------ */

/* Replaces npu_rope_layer (prebuild/npu_ops.h:39-42; call site
 * src/llama2_layer_npu.cpp:206-208): rotates q and k, both
 * [cur_size][n_heads][hidden_dim/n_heads], by rows start_pos.. of
 * freq_cis[max_seq_len][head_dim/2][2] fp32 (cos, sin). */
int llmhip_rope(void *out_q, void *out_k, const void *freq_cis, const void *in_q,
                const void *in_k, int start_pos, int cur_size, int n_heads, int hidden_dim,
                int is_neox_style, int dt, void *stream);

/* Replaces npu_rope_single_layer (prebuild/npu_ops.h:44-47; call sites
 * src/llama2_layer_npu.cpp:790-798).  hidden_dim = n_heads*head_dim of the
 * tensor being rotated. */
int llmhip_rope_single(void *out, const void *freq_cis, const void *in, int start_pos,
                       int cur_size, int n_heads, int hidden_dim, int is_neox_style, int dt,
                       void *stream);

/* One launch for the reference's rope -> cache-append sequence
 * (npu_rope_single_layer x2, src/llama2_layer_npu.cpp:790-798, then two
 * aclrtMemcpyAsync device-to-device copies, :830-844; Llama: :206-208 and
 * :325-339): out_q = rope(in_q); k_cache[start_pos:start_pos+cur_size] =
 * rope(in_k); v_cache[start_pos:start_pos+cur_size] = in_v (bytes).
 * k_cache, v_cache: [max_seq_len][n_kv_heads][head_dim] base pointers. */
int llmhip_rope_kv_append(void *out_q, void *k_cache, void *v_cache, const void *freq_cis,
                          const void *in_q, const void *in_k, const void *in_v,
                          int start_pos, int cur_size, int n_heads, int n_kv_heads,
                          int head_dim, int is_neox_style, int dt, void *stream);

/* ------------------------------------------------------------------ */
/* runtime surface used by the device layer                            */
/* ------------------------------------------------------------------ */
/* Thin wrappers so that C++ host code needs no HIP header.  They stand where
 * the reference calls aclInit / aclrtSetDevice (src/qwen2_model.cpp:111-117),
 * aclrtMalloc / aclrtFree (src/device_npu.cpp:42,49), aclrtMemcpy
 * (src/device.cpp:31,42), aclrtMemcpyAsync (src/llama2_layer_npu.cpp:333-338),
 * aclrtSynchronizeStream (src/llama2_layer_npu.cpp:605-608) and the event
 * calls of src/profiling.cpp:48-78. */
int llmhip_device_count(void);
/* Compute units, maximum shader clock (kHz) and memory size of a device (any pointer may be null):
 * hipGetDeviceProperties for host code that includes no HIP header. */
int llmhip_device_props(int device, int *compute_units, int *max_clock_khz, size_t *total_mem_bytes);
int llmhip_set_device(int device);
int llmhip_malloc(void **ptr, size_t bytes);
int llmhip_free(void *ptr);
int llmhip_memcpy_h2d(void *dst, const void *src, size_t bytes);
int llmhip_memcpy_d2h(void *dst, const void *src, size_t bytes);
int llmhip_memcpy_d2d_async(void *dst, const void *src, size_t bytes, void *stream);
/* Fills with a kernel (any alignment, any size), so the call may be captured into a HIP graph. */
int llmhip_memset_async(void *dst, int value, size_t bytes, void *stream);
int llmhip_stream_create(void **stream);
int llmhip_stream_destroy(void *stream);
int llmhip_stream_sync(void *stream);
int llmhip_device_sync(void);
int llmhip_event_create(void **event);
int llmhip_event_destroy(void *event);
int llmhip_event_record(void *event, void *stream);
int llmhip_event_sync(void *event);
/* LLMHIP_OK once everything queued before the event's record has completed, LLMHIP_NOT_READY
 * before that; never blocks (hipEventQuery).  The device layer's stream-ordered pool asks this
 * before it hands a block freed on one stream to another. */
int llmhip_event_query(void *event);
int llmhip_event_elapsed_ms(float *ms, void *start, void *stop);
const char *llmhip_error_string(int status);
/* Frees the split-KV scratch the reference-signature attention entry points
 * keep per stream (they take no workspace argument, npu_ops.h:10-13), and the
 * hipBLASLt handle, plans and workspace of llmhip_matmul*. */
int llmhip_release_internal_workspace(void);

/* ---- projections around the attention block (the callers either side of the path) ---- */

/* Replaces npu_matmul_nz_layer (prebuild/npu_ops.h:87-88; call site
 * src/llama2_layer_npu.cpp:1178-1180): out[m][n] = lhs[m][k] . W^T, fp32 accumulation, one
 * rounding to dt.  `weight` is W[n][k] row-major -- the checkpoint layout -- not the
 * reference's Ascend "nz" repacking [n/16][k][16] (tests/gemm_test.cpp:95-101).  n and k
 * must be multiples of 16 (src/llama2_layer_npu.cpp:1211-1218).  Runs on hipBLASLt; the first
 * call allocates the library's handle and a 64 MiB workspace. */
int llmhip_matmul(void *out, const void *lhs, const void *weight, int m, int n, int k, int dt,
                  void *stream);

/* Replaces npu_matmul_bias_nz_layer (prebuild/npu_ops.h:90-92; call site
 * src/llama2_layer_npu.cpp:1174-1177): as llmhip_matmul with bias[n] in fp32 added to the
 * fp32 accumulator before the single rounding (golden tests/gemm_test.cpp:138-149). */
int llmhip_matmul_bias(void *out, const void *lhs, const void *weight, const void *bias_f32,
                       int m, int n, int k, int dt, void *stream);

/* Replaces npu_add_layer (prebuild/npu_ops.h:81-82; call site
 * src/llama2_layer_npu.cpp:900-901, the residual add after o_proj):
 * out[i] = round_dt(float(lhs[i]) + float(rhs[i])). */
int llmhip_add(void *out, const void *lhs, const void *rhs, long long total_size, int dt,
               void *stream);

#ifdef __cplusplus
}
#endif
#endif /* LLMHIP_H_ */
