// Rotary embedding on Q and K fused with the KV-cache append, gfx950.
//
// Replaces, in one launch, what the reference does with two (or one) rope
// launches plus two device-to-device copies per layer and step
// (src/llama2_layer_npu.cpp:790-798 + :830-844; Llama :206-208 + :325-339):
//   out_q[s][h][:]              = rope(in_q[s][h][:], freq_cis[start_pos+s])
//   out_k[row_off + s][h][:]    = rope(in_k[s][h][:], freq_cis[start_pos+s])
//   out_v[row_off + s][h][:]    = in_v[s][h][:]                    (bytes)
// with out_k / out_v the cache base pointers and row_off = start_pos for the
// append, or plain output tensors with row_off = 0 for the stand-alone rope
// entry points.
//
// Arithmetic follows src/llama2_layer_cpu.cpp:835-856 with the position
// offset of the device contract (tests/rope_single_layer_test.cpp:78-97):
// widen to fp32, (a*c - b*d, a*d + b*c) with every product and sum rounded
// separately (this file is compiled with -ffp-contract=off), one rounding to
// the storage type.  Pairing: interleaved (2f, 2f+1) or neox (f, f + 64).
//
// Pure streaming: one thread rotates 8 pairs (two 128-bit loads, two 128-bit
// stores, 64 bytes of the fp32 table), 8 threads cover a head row, V rows are
// copied 16 bytes per thread.
#include "common.hpp"
#include "kernels.hpp"

namespace llmhip {

struct RopeParams {
  const char *in_q, *in_k, *in_v;
  char *out_q, *out_k, *out_v;
  const float *freq_cis;
  int start_pos, cur_size;
  int q_heads, k_heads;
  int k_out_row_offset;
  int is_neox;
  int v_units;  // 16 lanes of 16 bytes per V head row, 0 if no V
};

template <typename T>
__device__ __forceinline__ void rotate8(const char *in_row, char *out_row, const float *tab,
                                        int f0, int is_neox) {
  using E = Elem<T>;
  // the 8 pairs f0..f0+7
  const int off_a = is_neox ? f0 * 2 : f0 * 4;               // bytes
  const int off_b = is_neox ? (f0 + 64) * 2 : f0 * 4 + 16;   // bytes
  const u32x4_t va = global_load_b128(in_row + off_a);
  const u32x4_t vb = global_load_b128(in_row + off_b);
  const f32x4_t t0 = *reinterpret_cast<const f32x4_t *>(tab + 2 * f0);
  const f32x4_t t1 = *reinterpret_cast<const f32x4_t *>(tab + 2 * f0 + 4);
  const f32x4_t t2 = *reinterpret_cast<const f32x4_t *>(tab + 2 * f0 + 8);
  const f32x4_t t3 = *reinterpret_cast<const f32x4_t *>(tab + 2 * f0 + 12);
  const float cs[16] = {t0[0], t0[1], t0[2], t0[3], t1[0], t1[1], t1[2], t1[3],
                        t2[0], t2[1], t2[2], t2[3], t3[0], t3[1], t3[2], t3[3]};
  uint16_t ea[8], eb[8];  // element j of chunk a / chunk b
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    ea[2 * j] = (uint16_t)(va[j] & 0xFFFFu);
    ea[2 * j + 1] = (uint16_t)(va[j] >> 16);
    eb[2 * j] = (uint16_t)(vb[j] & 0xFFFFu);
    eb[2 * j + 1] = (uint16_t)(vb[j] >> 16);
  }
  uint16_t ra[8], rb[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    // neox: pair i = (ea[i], eb[i]); interleaved: pair i = elements 2i, 2i+1 of
    // the 16 contiguous elements (ea then eb)
    uint16_t xa, xb;
    if (is_neox) {
      xa = ea[i];
      xb = eb[i];
    } else {
      xa = (i < 4) ? ea[2 * i] : eb[2 * i - 8];
      xb = (i < 4) ? ea[2 * i + 1] : eb[2 * i - 7];
    }
    const float a = E::widen(xa), b = E::widen(xb);
    const float c = cs[2 * i], d = cs[2 * i + 1];
    const float r0 = a * c - b * d;
    const float r1 = a * d + b * c;
    const uint16_t o0 = E::round(r0), o1 = E::round(r1);
    if (is_neox) {
      ra[i] = o0;
      rb[i] = o1;
    } else if (i < 4) {
      ra[2 * i] = o0;
      ra[2 * i + 1] = o1;
    } else {
      rb[2 * i - 8] = o0;
      rb[2 * i - 7] = o1;
    }
  }
  u32x4_t wa, wb;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    wa[j] = (uint32_t)ra[2 * j] | ((uint32_t)ra[2 * j + 1] << 16);
    wb[j] = (uint32_t)rb[2 * j] | ((uint32_t)rb[2 * j + 1] << 16);
  }
  *reinterpret_cast<u32x4_t *>(out_row + off_a) = wa;
  *reinterpret_cast<u32x4_t *>(out_row + off_b) = wb;
}

// One thread per unit; units of a token are laid out as
// [q_heads*8 rotate units | k_heads*8 rotate units | v_units copy units].
template <typename T>
__global__ __launch_bounds__(256) void rope_kv_append_kernel(RopeParams p) {
  const int units_q = p.q_heads * 8, units_k = p.k_heads * 8;
  const int per_token = units_q + units_k + p.v_units;
  const long long gid = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= (long long)per_token * p.cur_size) return;
  const int s = (int)(gid / per_token);
  int u = (int)(gid % per_token);
  const float *tab = p.freq_cis + (size_t)(p.start_pos + s) * kHeadDim;  // 64 (cos,sin) pairs
  if (u < units_q) {
    const int h = u >> 3, f0 = (u & 7) * 8;
    const size_t row = ((size_t)s * p.q_heads + h) * kRowBytes;
    rotate8<T>(p.in_q + row, p.out_q + row, tab, f0, p.is_neox);
    return;
  }
  u -= units_q;
  if (u < units_k) {
    const int h = u >> 3, f0 = (u & 7) * 8;
    const size_t irow = ((size_t)s * p.k_heads + h) * kRowBytes;
    const size_t orow = ((size_t)(s + p.k_out_row_offset) * p.k_heads + h) * kRowBytes;
    rotate8<T>(p.in_k + irow, p.out_k + orow, tab, f0, p.is_neox);
    return;
  }
  u -= units_k;
  const size_t ioff = (size_t)s * p.k_heads * kRowBytes + (size_t)u * 16;
  const size_t ooff = (size_t)(s + p.k_out_row_offset) * p.k_heads * kRowBytes + (size_t)u * 16;
  *reinterpret_cast<u32x4_t *>(p.out_v + ooff) = global_load_b128(p.in_v + ioff);
}

hipError_t launch_rope_kv_append(void *out_q, void *out_k, void *out_v, const void *freq_cis,
                                 const void *in_q, const void *in_k, const void *in_v,
                                 int start_pos, int cur_size, int q_heads, int k_heads,
                                 int k_out_row_offset, int is_neox, int dt, hipStream_t stream) {
  RopeParams p;
  p.in_q = static_cast<const char *>(in_q);
  p.in_k = static_cast<const char *>(in_k);
  p.in_v = static_cast<const char *>(in_v);
  p.out_q = static_cast<char *>(out_q);
  p.out_k = static_cast<char *>(out_k);
  p.out_v = static_cast<char *>(out_v);
  p.freq_cis = static_cast<const float *>(freq_cis);
  p.start_pos = start_pos;
  p.cur_size = cur_size;
  p.q_heads = q_heads;
  p.k_heads = k_heads;
  p.k_out_row_offset = k_out_row_offset;
  p.is_neox = is_neox ? 1 : 0;
  p.v_units = (in_v != nullptr) ? k_heads * 16 : 0;
  const long long total = (long long)cur_size * (q_heads * 8 + k_heads * 8 + p.v_units);
  if (total == 0) return hipSuccess;
  const int grid = (int)((total + 255) / 256);
  if (dt == kDtFloat16)
    hipLaunchKernelGGL(rope_kv_append_kernel<_Float16>, dim3(grid), dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL(rope_kv_append_kernel<__bf16>, dim3(grid), dim3(256), 0, stream, p);
  return hipGetLastError();
}

}  // namespace llmhip
