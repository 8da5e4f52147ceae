/*
 * llmhip_bench.h -- C ABI of libllmhip_bench.so: measurement aids of the benchmark.
 *
 * None of these has a counterpart in the reference and none is part of the product library
 * (libllmhip.so, include/llmhip.h): they exist so that the benchmark can print, next to each
 * kernel's figure, what the machine it ran on delivers -- the shader clock under the prefill
 * kernel's load, the rate the matrix pipe sustains, the rate of a kernel that only reads.  Status
 * codes and the dtype numbering are those of llmhip.h.
 */
#ifndef LLMHIP_BENCH_H_
#define LLMHIP_BENCH_H_

#include "llmhip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* llmhip_flash_attn_gqa (llmhip.h) on this library's own copy of the prefill kernel
 * (m * group_size > 16, LLMHIP_ERR_UNSUPPORTED otherwise; square and ragged prefill shapes, no
 * key-range split), which also makes the first scheduled workgroup store two 64-bit counters at
 * clock_probe (device memory, 16 bytes): the shader-clock ticks and the ticks of the constant
 * 100 MHz reference clock between its start and its end.  Their ratio x 100 MHz is the shader
 * clock under this kernel's load. */
int llmhip_bench_flash_attn_gqa_clocked(void *out, const void *q, const void *k, const void *v, int m,
                                        int n, int offset, int group_size, int kv_head_num, int head_dim,
                                        int dt, void *clock_probe, void *stream);

/* Runs, for about target_ms (<= 2000), a loop of back-to-back bf16 32x32x16 MFMAs on N(0,1)
 * operands on every CU and returns the sustained TFLOP/s.  mix 0: the MFMAs alone (what the matrix
 * pipe sustains at the clock its own power draw allows); mix 1: the same MFMAs with the LDS
 * fragment reads and vector instructions of a flash-attention inner loop beside them, no memory
 * traffic, no barriers, no dependences.  Allocates and frees two small device buffers; runs on the
 * default stream. */
int llmhip_bench_mfma_ceiling(int mix, double target_ms, double *tflops);

/* A plain streaming read of two device arrays of bytes_each bytes (a multiple of 16), every byte
 * read once and nothing else done -- what the memory system delivers to a kernel that only reads,
 * to set beside the decode kernel's rate on the same byte count.  variant 0: one workgroup per CU
 * with 8 loads in flight per thread; variant 1: two per CU with 4 (the better one below about
 * 256 MiB).  sink: LLMHIP_BENCH_STREAM_READ_SINK_BYTES bytes of device memory that receive a
 * checksum per wave.  Asynchronous on `stream`; allocates nothing. */
#define LLMHIP_BENCH_STREAM_READ_SINK_BYTES 65536
int llmhip_bench_stream_read(const void *src_a, const void *src_b, size_t bytes_each, void *sink,
                             size_t sink_bytes, int variant, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* LLMHIP_BENCH_H_ */
