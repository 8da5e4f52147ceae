// Launchers of the measurement library (libllmhip_bench.so): probes that the benchmark sets beside
// the kernels' figures.  Nothing here is part of the product library.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

#include "common.hpp"

namespace LLMHIP_NS {

// Sustained MFMA TFLOP/s of this GPU on N(0,1) bf16 operands, mix 0 = MFMAs alone, mix 1 = MFMAs
// with the LDS reads and vector instructions of an attention loop (ceiling_probe.hip).
hipError_t run_mfma_ceiling(int mix, double target_ms, double *tflops_out);
// A kernel that only reads two arrays once (ceiling_probe.hip).
hipError_t launch_stream_read(const void *a, const void *b, size_t bytes_each, void *sink, int variant,
                              hipStream_t stream);
constexpr size_t kStreamReadSinkBytes = 65536;  // 4 bytes per wave of the largest grid (2 workgroups per CU)

}  // namespace LLMHIP_NS
