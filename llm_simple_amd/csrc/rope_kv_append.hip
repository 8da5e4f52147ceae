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
// Pure streaming: a unit is 32 bytes of a 256-byte head row (8 units per row; 8 pairs: two 128-bit
// loads, 64 bytes of the fp32 table, two 128-bit stores), Q, K and V rows alike -- a V row is copied
// by the same 8 lanes without the arithmetic.  A thread takes kRopeUnits units a whole grid apart and
// issues all their loads before it computes.  The pairing style is a template parameter, the storage
// type is rounded by the hardware conversion (equal to round-to-nearest-even on the bit pattern for
// every non-NaN fp32), the token of a unit comes from a multiply-shift division, the stores are
// non-temporal.  (Measured at 4096 tokens of Qwen2.5-7B: 12.7 us with the buffers in the last-level
// cache, 16.5 us from and to HBM; the same kernel without arithmetic and table 12.2 us with ordinary
// stores, so the rest is the memory path of three separate streams of 256-byte rows.)
#include "common.hpp"
#include "kernels.hpp"

namespace llmhip {

constexpr int kRopeUnits = 2;  // 32-byte units per thread, a grid apart: twice the loads in flight per wave

struct RopeParams {
  const char *in_q, *in_k, *in_v;
  char *out_q, *out_k, *out_v;
  const float *freq_cis;
  int start_pos, cur_size;
  int q_heads, k_heads, v_heads;  // head rows of a token: q, then k, then v (v_heads = 0 without V)
  int k_out_row_offset;
  FastDiv rows_per_token;
  uint32_t total;  // threads with work: cur_size * rows per token * 8
};

// The 8 pairs of one thread: a = elements of the first 16-byte chunk, b = of the second.  NEOX: pair i
// = (a[i], b[i]) (dims f, f + 64); interleaved: pair i = elements 2i, 2i+1 of the 16 contiguous ones.
// Arithmetic of src/llama2_layer_cpu.cpp:835-856: every product and sum rounded on its own.
template <typename T, bool NEOX>
__device__ __forceinline__ void rotate8(u32x4_t &va, u32x4_t &vb, const float *tab) {
  using E = Elem<T>;
  const f32x4_t t0 = *reinterpret_cast<const f32x4_t *>(tab);
  const f32x4_t t1 = *reinterpret_cast<const f32x4_t *>(tab + 4);
  const f32x4_t t2 = *reinterpret_cast<const f32x4_t *>(tab + 8);
  const f32x4_t t3 = *reinterpret_cast<const f32x4_t *>(tab + 12);
  const float cs[16] = {t0[0], t0[1], t0[2], t0[3], t1[0], t1[1], t1[2], t1[3],
                        t2[0], t2[1], t2[2], t2[3], t3[0], t3[1], t3[2], t3[3]};
  float r0[8], r1[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    uint16_t xa, xb;
    if (NEOX) {
      xa = (uint16_t)(va[i >> 1] >> ((i & 1) * 16));
      xb = (uint16_t)(vb[i >> 1] >> ((i & 1) * 16));
    } else {
      const uint32_t w = (i < 4) ? va[i] : vb[i - 4];
      xa = (uint16_t)w;
      xb = (uint16_t)(w >> 16);
    }
    const float a = E::widen(xa), b = E::widen(xb);
    const float c = cs[2 * i], d = cs[2 * i + 1];
    r0[i] = a * c - b * d;
    r1[i] = a * d + b * c;
  }
  if (NEOX) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      va[j] = E::pack2(r0[2 * j], r0[2 * j + 1]);
      vb[j] = E::pack2(r1[2 * j], r1[2 * j + 1]);
    }
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      va[j] = E::pack2(r0[j], r1[j]);
      vb[j] = E::pack2(r0[j + 4], r1[j + 4]);
    }
  }
}

template <typename T, bool NEOX>
__global__ __launch_bounds__(256) void rope_kv_append_kernel(RopeParams p) {
  constexpr int U = kRopeUnits;
  const uint32_t stride = gridDim.x * 256u;
  const uint32_t gid0 = blockIdx.x * 256u + threadIdx.x;
  u32x4_t va[U], vb[U];
  char *outp[U];
  const float *tabp[U];
  bool rot[U], live[U];
  const uint32_t j = gid0 & 7u;  // stride is a multiple of 8
  const int off_a = NEOX ? (int)j * 16 : (int)j * 32;
  const int off_b = NEOX ? off_a + 128 : off_a + 16;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const uint32_t gid = gid0 + u * stride;
    live[u] = gid < p.total;
    const uint32_t rowid = (live[u] ? gid : 0u) >> 3;
    const uint32_t s = fast_div(rowid, p.rows_per_token);
    const int r = (int)(rowid - s * p.rows_per_token.d);
    const char *in;
    rot[u] = true;
    if (r < p.q_heads) {
      const size_t row = ((size_t)s * p.q_heads + r) * kRowBytes;
      in = p.in_q + row;
      outp[u] = p.out_q + row;
    } else if (r < p.q_heads + p.k_heads) {
      const int h = r - p.q_heads;
      in = p.in_k + ((size_t)s * p.k_heads + h) * kRowBytes;
      outp[u] = p.out_k + ((size_t)(s + p.k_out_row_offset) * p.k_heads + h) * kRowBytes;
    } else {
      const int h = r - p.q_heads - p.k_heads;
      in = p.in_v + ((size_t)s * p.v_heads + h) * kRowBytes;
      outp[u] = p.out_v + ((size_t)(s + p.k_out_row_offset) * p.v_heads + h) * kRowBytes;
      rot[u] = false;
    }
    tabp[u] = p.freq_cis + (size_t)(p.start_pos + s) * kHeadDim + 16 * j;
    va[u] = global_load_b128(in + off_a);
    vb[u] = global_load_b128(in + off_b);
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    if (rot[u]) rotate8<T, NEOX>(va[u], vb[u], tabp[u]);
    if (live[u]) {
      // Non-temporal stores for every output row (measured at 4096 tokens, H=28, Hkv=4: from and to HBM
      // 18.2 -> 16.5 us, buffers resident in the last-level cache 13.15 -> 12.70 us; the attention launch
      // that reads the rows next takes the same time either way).  Marking only the cache rows changes
      // nothing: 7 of 9 written rows are rotated q.
      __builtin_nontemporal_store(va[u], reinterpret_cast<u32x4_t *>(outp[u] + off_a));
      __builtin_nontemporal_store(vb[u], reinterpret_cast<u32x4_t *>(outp[u] + off_b));
    }
  }
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
  p.v_heads = (in_v != nullptr) ? k_heads : 0;
  p.k_out_row_offset = k_out_row_offset;
  const long long rows = (long long)q_heads + k_heads + p.v_heads;
  const long long total = (long long)cur_size * rows * 8;
  if (total == 0) return hipSuccess;
  if (rows > 0x7FFFFFFFLL || total > 0x7FFFFFFFLL) return hipErrorInvalidValue;  // 32-bit thread index
  p.rows_per_token = make_fast_div((uint32_t)rows);
  p.total = (uint32_t)total;
  const int grid = (int)((total + 256 * kRopeUnits - 1) / (256 * kRopeUnits));
  void (*kern)(RopeParams) =
      (dt == kDtFloat16) ? (is_neox ? rope_kv_append_kernel<_Float16, true> : rope_kv_append_kernel<_Float16, false>)
                         : (is_neox ? rope_kv_append_kernel<__bf16, true> : rope_kv_append_kernel<__bf16, false>);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), 0, stream, p);
  return hipGetLastError();
}

}  // namespace llmhip
