// Projection GEMMs around the attention path, through hipBLASLt.
//
// out[m][n] = round_T( lhs[m][k] . W^T + bias ) with fp32 accumulation and an fp32 bias
// added before the single rounding: the arithmetic of the reference's npu_matmul_nz_layer /
// npu_matmul_bias_nz_layer (prebuild/npu_ops.h:87-92; golden tests/gemm_test.cpp:138-149:
// fp32 contraction + fp32 bias, then one cast to the storage type).  The reference stores
// the weight in Ascend's fractal "nz" layout [n/16][k][16]; here the weight is the plain
// checkpoint layout W[n][k] (row-major, k contiguous), which is what hipBLASLt reads as a
// transposed column-major operand -- no repacking on this device.
//
// Row-major out[m][n] is the column-major n x m matrix D = W(n x k) * X(k x m): A = W
// (stored k x n column-major, op T), B = X (k x m column-major, op N), bias along the rows
// of D (one value per output feature) in the epilogue.
//
// Also here: the elementwise residual add (npu_add_layer, prebuild/npu_ops.h:81-82).
#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>

#include <map>
#include <mutex>
#include <tuple>

#include "common.hpp"
#include "kernels.hpp"

namespace llmhip {

namespace {

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t la = nullptr, lb = nullptr, lc = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
  bool ok = false;
  uint64_t last_use = 0;
};

// One handle, workspace and plan cache per device.
struct DeviceBlas {
  hipblasLtHandle_t handle = nullptr;
  void *workspace = nullptr;
  std::map<std::tuple<int, int, int, int, int>, Plan> plans;  // m, n, k, dt, bias
  uint64_t tick = 0;
};
constexpr size_t kMaxPlans = 64;  // per device; the least recently used plan is dropped beyond this

void destroy_plan(Plan &pl) {
  if (pl.la) hipblasLtMatrixLayoutDestroy(pl.la);
  if (pl.lb) hipblasLtMatrixLayoutDestroy(pl.lb);
  if (pl.lc) hipblasLtMatrixLayoutDestroy(pl.lc);
  if (pl.desc) hipblasLtMatmulDescDestroy(pl.desc);
  pl = Plan();
}
struct Blas {
  std::mutex mu;
  static constexpr size_t kWorkspaceBytes = 64u << 20;
  std::map<int, DeviceBlas> dev;
};

Blas &blas() {
  static Blas b;
  return b;
}

hipError_t to_hip(hipblasStatus_t s) { return s == HIPBLAS_STATUS_SUCCESS ? hipSuccess : hipErrorUnknown; }

hipError_t make_plan(DeviceBlas &b, Plan &pl, int m, int n, int k, int dt, bool has_bias) {
  const hipDataType t = dt == kDtFloat16 ? HIP_R_16F : HIP_R_16BF;
  hipblasStatus_t s = hipblasLtMatmulDescCreate(&pl.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F);
  if (s != HIPBLAS_STATUS_SUCCESS) return to_hip(s);
  const hipblasOperation_t op_t = HIPBLAS_OP_T, op_n = HIPBLAS_OP_N;
  hipblasLtMatmulDescSetAttribute(pl.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &op_t, sizeof(op_t));
  hipblasLtMatmulDescSetAttribute(pl.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &op_n, sizeof(op_n));
  if (has_bias) {
    const hipblasLtEpilogue_t epi = HIPBLASLT_EPILOGUE_BIAS;
    const hipDataType bias_t = HIP_R_32F;
    hipblasLtMatmulDescSetAttribute(pl.desc, HIPBLASLT_MATMUL_DESC_EPILOGUE, &epi, sizeof(epi));
    hipblasLtMatmulDescSetAttribute(pl.desc, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &bias_t,
                                    sizeof(bias_t));
  }
  if ((s = hipblasLtMatrixLayoutCreate(&pl.la, t, k, n, k)) != HIPBLAS_STATUS_SUCCESS) return to_hip(s);
  if ((s = hipblasLtMatrixLayoutCreate(&pl.lb, t, k, m, k)) != HIPBLAS_STATUS_SUCCESS) return to_hip(s);
  if ((s = hipblasLtMatrixLayoutCreate(&pl.lc, t, n, m, n)) != HIPBLAS_STATUS_SUCCESS) return to_hip(s);
  hipblasLtMatmulPreference_t pref;
  if ((s = hipblasLtMatmulPreferenceCreate(&pref)) != HIPBLAS_STATUS_SUCCESS) return to_hip(s);
  const size_t ws = Blas::kWorkspaceBytes;
  hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws, sizeof(ws));
  hipblasLtMatmulHeuristicResult_t res[1];
  int found = 0;
  s = hipblasLtMatmulAlgoGetHeuristic(b.handle, pl.desc, pl.la, pl.lb, pl.lc, pl.lc, pref, 1, res, &found);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (s != HIPBLAS_STATUS_SUCCESS || found == 0) return hipErrorNotSupported;
  pl.algo = res[0].algo;
  pl.workspace = res[0].workspaceSize;
  pl.ok = true;
  return hipSuccess;
}

}  // namespace

hipError_t launch_matmul_bias(void *out, const void *lhs, const void *weight, const float *bias,
                              int m, int n, int k, int dt, hipStream_t stream) {
  Blas &all = blas();
  std::lock_guard<std::mutex> lock(all.mu);
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  DeviceBlas &b = all.dev[dev];
  if (!b.handle) {
    if (hipblasLtCreate(&b.handle) != HIPBLAS_STATUS_SUCCESS) return hipErrorUnknown;
    e = hipMalloc(&b.workspace, Blas::kWorkspaceBytes);
    if (e != hipSuccess) {
      hipblasLtDestroy(b.handle);
      b.handle = nullptr;
      return e;
    }
  }
  const auto key = std::make_tuple(m, n, k, dt, bias ? 1 : 0);
  if (b.plans.find(key) == b.plans.end() && b.plans.size() >= kMaxPlans) {
    // every distinct prompt length m makes a plan: keep the cache bounded
    auto victim = b.plans.begin();
    for (auto it = b.plans.begin(); it != b.plans.end(); ++it)
      if (it->second.last_use < victim->second.last_use) victim = it;
    destroy_plan(victim->second);
    b.plans.erase(victim);
  }
  Plan &pl = b.plans[key];
  if (!pl.ok) {
    e = make_plan(b, pl, m, n, k, dt, bias != nullptr);
    if (e != hipSuccess) {  // nothing half-built stays behind
      destroy_plan(pl);
      b.plans.erase(key);
      return e;
    }
  }
  pl.last_use = ++b.tick;
  if (bias) {
    // the bias pointer is a per-call attribute of the (cached) descriptor; calls are
    // serialised by the mutex above
    hipblasLtMatmulDescSetAttribute(pl.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof(bias));
  }
  const float alpha = 1.0f, beta = 0.0f;
  const hipblasStatus_t s =
      hipblasLtMatmul(b.handle, pl.desc, &alpha, weight, pl.la, lhs, pl.lb, &beta, out, pl.lc, out,
                      pl.lc, &pl.algo, b.workspace, Blas::kWorkspaceBytes, stream);
  return to_hip(s);
}

void release_matmul_resources() {
  Blas &all = blas();
  std::lock_guard<std::mutex> lock(all.mu);
  int cur = 0;
  const bool have_cur = hipGetDevice(&cur) == hipSuccess;
  for (auto &dv : all.dev) {
    DeviceBlas &b = dv.second;
    (void)hipSetDevice(dv.first);
    for (auto &kv : b.plans) destroy_plan(kv.second);
    if (b.workspace) (void)hipFree(b.workspace);
    if (b.handle) hipblasLtDestroy(b.handle);
  }
  all.dev.clear();
  if (have_cur) (void)hipSetDevice(cur);
}

// out = round_T(float(lhs) + float(rhs)), 8 elements per thread (HBM-bound: 6 bytes per element).
template <typename T>
__global__ __launch_bounds__(256) void add_kernel(uint16_t *out, const uint16_t *lhs, const uint16_t *rhs,
                                                  size_t total) {
  using E = Elem<T>;
  const size_t i = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (i + 8 <= total) {
    const u32x4_t a = *reinterpret_cast<const u32x4_t *>(lhs + i);
    const u32x4_t b = *reinterpret_cast<const u32x4_t *>(rhs + i);
    u32x4_t r;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float lo = E::widen((uint16_t)(a[j] & 0xffffu)) + E::widen((uint16_t)(b[j] & 0xffffu));
      const float hi = E::widen((uint16_t)(a[j] >> 16)) + E::widen((uint16_t)(b[j] >> 16));
      r[j] = E::pack2(lo, hi);
    }
    *reinterpret_cast<u32x4_t *>(out + i) = r;
  } else {
    for (size_t j = i; j < total; ++j) out[j] = E::round(E::widen(lhs[j]) + E::widen(rhs[j]));
  }
}

hipError_t launch_add(void *out, const void *lhs, const void *rhs, size_t total, int dt, hipStream_t stream) {
  if (total == 0) return hipSuccess;
  const size_t threads = (total + 7) / 8;
  const dim3 grid((unsigned)((threads + 255) / 256));
  if (dt == kDtFloat16)
    hipLaunchKernelGGL(add_kernel<_Float16>, grid, dim3(256), 0, stream, (uint16_t *)out,
                       (const uint16_t *)lhs, (const uint16_t *)rhs, total);
  else
    hipLaunchKernelGGL(add_kernel<__bf16>, grid, dim3(256), 0, stream, (uint16_t *)out,
                       (const uint16_t *)lhs, (const uint16_t *)rhs, total);
  return hipGetLastError();
}

// Byte fill, the kernel behind llmhip_memset_async: a memset node recorded into a HIP graph has given wrong
// results on replays, a kernel node does not.  The bulk goes out as 16-byte stores from the first 16-byte
// boundary on, the ragged head and tail as bytes.
__global__ __launch_bounds__(256) void fill_kernel(unsigned char *dst, unsigned char value, size_t bytes) {
  const size_t head = min(bytes, (size_t)((16 - (reinterpret_cast<uintptr_t>(dst) & 15)) & 15));
  const size_t vecs = (bytes - head) / 16, tail0 = head + vecs * 16;
  const uint32_t w = value * 0x01010101u;
  const u32x4_t v = {w, w, w, w};
  u32x4_t *mid = reinterpret_cast<u32x4_t *>(dst + head);
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < vecs; i += stride) mid[i] = v;
  if (blockIdx.x == 0) {
    for (size_t i = threadIdx.x; i < head; i += blockDim.x) dst[i] = value;
    for (size_t i = tail0 + threadIdx.x; i < bytes; i += blockDim.x) dst[i] = value;
  }
}

hipError_t launch_fill(void *dst, int value, size_t bytes, hipStream_t stream) {
  if (bytes == 0) return hipSuccess;
  size_t blocks = (bytes / 16 + 255) / 256;
  if (blocks < 1) blocks = 1;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(fill_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, static_cast<unsigned char *>(dst),
                     (unsigned char)value, bytes);
  return hipGetLastError();
}

}  // namespace llmhip
