// Measurement aid: what the matrix pipe of this GPU sustains on bf16 operands drawn from N(0,1).
//
// The published dense bf16 peak assumes the maximum shader clock.  On normally distributed operands
// the MFMA pipe alone already draws enough power for the clock to drop well below it, and every LDS
// read and vector instruction issued beside the MFMAs takes issue slots and register-file
// bandwidth from them.  Two loops with no memory traffic, no barriers and no data dependences
// between iterations bracket what an attention kernel can reach on this machine:
//   mix 0: back-to-back v_mfma_f32_32x32x16_bf16 on register operands;
//   mix 1: the same MFMAs with the other instructions of a flash-attention inner loop beside
//          them in the measured proportion of the prefill kernel: per 4 MFMAs, 6 LDS fragment
//          reads of 1 KiB (ds_read_b128), 13 fp32 vector instructions and 4 v_exp_f32.
// 8 waves per CU (2 per SIMD), one workgroup per CU, like the prefill kernel.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include <vector>

#include "bench_kernels.hpp"
#include "common.hpp"

namespace LLMHIP_NS {

namespace {

template <int MIX>
__global__ __launch_bounds__(512, 1) void mfma_ceiling_kernel(const u32x4_t *ops, float *out, int iters) {
  __shared__ __attribute__((aligned(16))) char lds[65536];
  const int tid = threadIdx.x, lane = tid & 63;
  for (int i = tid; i < 4096; i += 512) *reinterpret_cast<u32x4_t *>(lds + i * 16) = ops[i];
  __syncthreads();
  u32x4_t a[4], b[8];
  for (int i = 0; i < 4; ++i) a[i] = ops[i * 512 + tid];
  for (int i = 0; i < 8; ++i) b[i] = ops[(8 + i) * 512 + tid];
  f32x16_t c[4];
  for (int j = 0; j < 4; ++j)
    for (int i = 0; i < 16; ++i) c[j][i] = 0.f;
  float x[16];
  for (int i = 0; i < 16; ++i) x[i] = 0.001f * (tid + i);
  int laddr = lane * 16;
  asm volatile("" : "+v"(laddr));
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      u32x4_t av[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) av[j] = a[j];
      if (MIX == 1) {
        // 6 LDS reads per 4 MFMAs: 4 feed the MFMAs, 2 more are folded into the vector work.  Vector
        // instructions per 4 MFMAs: 4 (below) + 5 + 4 (the arguments of the exponentials) = 13, plus 4 v_exp_f32
#pragma unroll
        for (int j = 0; j < 4; ++j)
          av[j] = lds_read_b128(lds, laddr + ((i * 4 + j) & 31) * 1024 + (it & 1) * 32768);
        const u32x4_t e0 = lds_read_b128(lds, laddr + ((i * 4 + 5) & 31) * 1024);
        const u32x4_t e1 = lds_read_b128(lds, laddr + ((i * 4 + 9) & 31) * 1024);
        x[0] += __builtin_bit_cast(float, e0[0] & 0x3f800000u) + __builtin_bit_cast(float, e1[1] & 0x3f800000u);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        c[j] = Elem<__bf16>::mfma32(av[j], b[i], c[j]);
        if (MIX == 1) {
#pragma unroll
          for (int q = 0; q < (5 + 3 - j) / 4; ++q)
            x[(j * 4 + q) & 15] = __builtin_fmaf(x[(j * 4 + q) & 15], 0.9999f, 0.37f);
          x[12 + j] = fast_exp2(x[12 + j] * 0.5f - 1.0f);
        }
      }
    }
    if ((it & 63) == 63)  // keep the accumulators bounded
      for (int j = 0; j < 4; ++j)
        for (int i = 0; i < 16; ++i) c[j][i] *= 1e-3f;
  }
  float r = 0.f;
  for (int j = 0; j < 4; ++j)
    for (int i = 0; i < 16; ++i) r += c[j][i];
  for (int i = 0; i < 16; ++i) r += x[i];
  out[(size_t)blockIdx.x * 512 + tid] = r;
}

// Plain streaming read of two arrays of n16 16-byte pieces each, every piece read once with non-temporal
// loads (ordinary loads stream about 11 % slower at 2 GiB), U loads in flight per thread, consecutive threads of the whole grid on consecutive pieces (all CUs walk through memory
// together, which the DRAM channels serve best).  The XOR of everything read goes to sink[wave], so that
// no load can be dropped.
template <int U>
__global__ __launch_bounds__(256) void stream_read_kernel(const u32x4_t *__restrict__ a, const u32x4_t *__restrict__ b,
                                                          size_t n16, unsigned *sink) {
  const size_t total = (size_t)gridDim.x * 256;
  u32x4_t acc = {0u, 0u, 0u, 0u};
#pragma unroll 1
  for (int half = 0; half < 2; ++half) {
    const u32x4_t *src = half ? b : a;
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    for (; i + (U - 1) * total < n16; i += U * total) {
      u32x4_t v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) v[u] = global_load_b128_nt(&src[i + u * total]);
#pragma unroll
      for (int u = 0; u < U; ++u) acc ^= v[u];
    }
    for (; i < n16; i += total) acc ^= global_load_b128_nt(&src[i]);
  }
  unsigned r = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
#pragma unroll
  for (int o = 32; o; o >>= 1) r ^= (unsigned)__shfl_xor((int)r, o, 64);
  if ((threadIdx.x & 63) == 0) sink[blockIdx.x * 4 + (threadIdx.x >> 6)] = r;
}

// N(0,1) rounded to bf16 from a fixed counter-based generator (splitmix64 + Box-Muller).
uint16_t normal_bf16(uint64_t i) {
  auto mix = [](uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
  };
  const double u1 = ((mix(2 * i) >> 11) + 1.0) / 9007199254740993.0, u2 = (mix(2 * i + 1) >> 11) / 9007199254740992.0;
  const float g = (float)(sqrt(-2.0 * log(u1)) * cos(6.283185307179586 * u2));
  uint32_t u = __builtin_bit_cast(uint32_t, g);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

}  // namespace

// variant 0: one workgroup per CU, 8 loads in flight per thread (best from 256 MiB up); variant 1: two
// per CU, 4 in flight (best below).  sink: 4 bytes per wave of the grid.
hipError_t launch_stream_read(const void *a, const void *b, size_t bytes_each, void *sink, int variant,
                              hipStream_t stream) {
  static std::atomic<int> cus_of[64];  // per device; every writer stores the same value
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= 64) return hipErrorInvalidDevice;
  int cus = cus_of[dev].load(std::memory_order_relaxed);
  if (cus <= 0) {
    e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess || cus <= 0) return e != hipSuccess ? e : hipErrorInvalidDevice;
    cus_of[dev].store(cus, std::memory_order_relaxed);
  }
  const u32x4_t *pa = static_cast<const u32x4_t *>(a), *pb = static_cast<const u32x4_t *>(b);
  unsigned *ps = static_cast<unsigned *>(sink);
  if (variant == 0)
    hipLaunchKernelGGL(stream_read_kernel<8>, dim3(cus), dim3(256), 0, stream, pa, pb, bytes_each / 16, ps);
  else
    hipLaunchKernelGGL(stream_read_kernel<4>, dim3(2 * cus), dim3(256), 0, stream, pa, pb, bytes_each / 16, ps);
  return hipGetLastError();
}

// Runs one of the two loops on every CU for about `target_ms` and returns the sustained TFLOP/s of
// its MFMAs (0 on error).  Allocates and frees its own small buffers.
hipError_t run_mfma_ceiling(int mix, double target_ms, double *tflops_out) {
  *tflops_out = 0.0;
  int dev = 0, cus = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (e != hipSuccess) return e;
  const size_t n_ops = 16 * 512 * 8;  // 16-bit elements
  std::vector<uint16_t> host(n_ops);
  for (size_t i = 0; i < n_ops; ++i) host[i] = normal_bf16(i);
  u32x4_t *d_ops = nullptr;
  float *d_out = nullptr;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  auto cleanup = [&]() {
    if (d_ops) (void)hipFree(d_ops);
    if (d_out) (void)hipFree(d_out);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
  };
  if ((e = hipMalloc(&d_ops, n_ops * 2)) != hipSuccess || (e = hipMalloc(&d_out, (size_t)cus * 512 * 4)) != hipSuccess ||
      (e = hipMemcpy(d_ops, host.data(), n_ops * 2, hipMemcpyHostToDevice)) != hipSuccess ||
      (e = hipEventCreate(&e0)) != hipSuccess || (e = hipEventCreate(&e1)) != hipSuccess) {
    cleanup();
    return e;
  }
  const int iters = 400;  // 12800 MFMAs per wave per launch, ~0.25-0.4 ms
  auto launch = [&]() {
    if (mix == 1)
      hipLaunchKernelGGL(mfma_ceiling_kernel<1>, dim3(cus), dim3(512), 0, nullptr, d_ops, d_out, iters);
    else
      hipLaunchKernelGGL(mfma_ceiling_kernel<0>, dim3(cus), dim3(512), 0, nullptr, d_ops, d_out, iters);
  };
  const int reps = target_ms > 1.0 ? (int)(target_ms / 0.3) + 1 : 4;
  for (int i = 0; i < reps; ++i) launch();  // settle the clocks
  (void)hipEventRecord(e0, nullptr);
  for (int i = 0; i < reps; ++i) launch();
  (void)hipEventRecord(e1, nullptr);
  e = hipEventSynchronize(e1);
  float ms = 0.f;
  if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
  if (e == hipSuccess && ms > 0.f) {
    const double flops = (double)cus * 8 * iters * 32 * 32768.0 * reps;
    *tflops_out = flops / (ms * 1e-3) / 1e12;
  }
  cleanup();
  return e == hipSuccess ? hipGetLastError() : e;
}

}  // namespace LLMHIP_NS
