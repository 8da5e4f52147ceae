// Shared device helpers for the gfx950 attention kernels: 16-bit storage type
// traits, MFMA wrappers, LDS swizzles and cross-lane exchanges.
//
// MFMA operand layouts used throughout (64-lane wavefront, lane l):
//   32x32x16:  A[row = l%32][k = 8*(l/32) + e],  B[k = 8*(l/32) + e][col = l%32],
//              C[row = 8*(i/4) + 4*(l/32) + i%4][col = l%32],  e = 0..7, i = 0..15
//   16x16x32:  A[row = l%16][k = 8*(l/16) + e],  B[k = 8*(l/16) + e][col = l%16],
//              C[row = 4*(l/16) + i][col = l%16],               e = 0..7, i = 0..3
// ds_read_b64_tr_b16 (per 16-lane group): lane j receives element (j%4) of the
// 8-byte chunks addressed by lanes 4e + j/4, e = 0..3; when lane i addresses
// row i/4, columns 4*(i%4)..+3 of a 4x16 block, lane j ends up with column j of
// rows 0..3.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

// The measurement library (libllmhip_bench.so) compiles the prefill kernel a second time with
// LLMHIP_BENCH defined (a clock stamp in the kernel); its copy lives in a namespace of its own so
// that the two libraries never share a symbol.
#ifdef LLMHIP_BENCH
#define LLMHIP_NS llmhip_bench
#else
#define LLMHIP_NS llmhip
#endif

namespace LLMHIP_NS {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;

constexpr int kHeadDim = 128;         // every supported model: hidden / n_heads == 128
constexpr int kRowBytes = kHeadDim * 2;  // one head row of 16-bit elements

// Data type numbering of the reference (prebuild/defs.hpp:8-18).
constexpr int kDtFloat16 = 4;
constexpr int kDtBFloat16 = 5;

template <typename T> struct Elem;

template <> struct Elem<_Float16> {
  static __device__ __forceinline__ f32x16_t mfma32(u32x4_t a, u32x4_t b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a),
                                                  __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4_t mfma16(u32x4_t a, u32x4_t b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a),
                                                  __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    typedef __attribute__((ext_vector_type(2))) _Float16 h2;
    h2 v = {(_Float16)lo, (_Float16)hi};  // v_cvt_f16_f32 rounds to nearest even
    return __builtin_bit_cast(uint32_t, v);
  }
  static __device__ __forceinline__ float widen(uint16_t bits) {
    return (float)__builtin_bit_cast(_Float16, bits);
  }
  static __device__ __forceinline__ uint16_t round(float f) {
    return __builtin_bit_cast(uint16_t, (_Float16)f);
  }
};

template <> struct Elem<__bf16> {
  static __device__ __forceinline__ f32x16_t mfma32(u32x4_t a, u32x4_t b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                   __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4_t mfma16(u32x4_t a, u32x4_t b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                   __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    typedef __attribute__((ext_vector_type(2))) __bf16 b2;
    b2 v = {(__bf16)lo, (__bf16)hi};  // round to nearest even
    return __builtin_bit_cast(uint32_t, v);
  }
  static __device__ __forceinline__ float widen(uint16_t bits) {
    return __builtin_bit_cast(float, ((uint32_t)bits) << 16);
  }
  // Round to nearest even on the bit pattern; agrees with the reference's
  // fp32_to_bfloat16 (src/util.cpp:33-72) on every finite input.
  static __device__ __forceinline__ uint16_t round(float f) {
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
  }
};

// n / d for 32-bit n by multiply and shift (Granlund-Montgomery, round-up variant): exact for every n.
// The host fills the struct, kernels divide with two multiplications' worth of work instead of the
// ~25 dependent instructions of a run-time integer division.
struct FastDiv {
  uint32_t d, m, l;  // l = ceil(log2 d); m = floor(2^32 (2^l - d) / d) + 1
};
inline FastDiv make_fast_div(uint32_t d) {
  FastDiv f;
  f.d = d;
  f.l = 0;
  while ((1ull << f.l) < d) ++f.l;
  f.m = (uint32_t)((((1ull << f.l) - d) << 32) / d + 1);
  return f;
}
__device__ __forceinline__ uint32_t fast_div(uint32_t n, const FastDiv &f) {
  if (f.l == 0) return n;  // d == 1
  const uint32_t t = (uint32_t)(((uint64_t)n * f.m) >> 32);
  return (t + ((n - t) >> 1)) >> (f.l - 1);
}

// Exchange with the lane whose index differs in bit 5 / bit 4.
__device__ __forceinline__ float xor_lane(float v, int mask) { return __shfl_xor(v, mask, 64); }

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// acc + lo + hi of a packed pair of storage-type values.
template <typename T> __device__ __forceinline__ float dot2_ones(uint32_t packed, float acc);
template <> __device__ __forceinline__ float dot2_ones<__bf16>(uint32_t packed, float acc) {
  typedef __attribute__((ext_vector_type(2))) __bf16 b2;
  const b2 one = {(__bf16)1.0f, (__bf16)1.0f};
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(b2, packed), one, acc, false);
}
template <> __device__ __forceinline__ float dot2_ones<_Float16>(uint32_t packed, float acc) {
  typedef __attribute__((ext_vector_type(2))) _Float16 h2;
  const h2 one = {(_Float16)1.0f, (_Float16)1.0f};
  return __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, packed), one, acc, false);
}

// LDS tile of 16-bit head rows, 256 bytes per row, 16 granules of 16 bytes.
// K tiles are read with ds_read_b128 by 16 consecutive rows at one logical
// granule: XOR with the row spreads them over all 16 bank groups.
__device__ __forceinline__ int k_swizzle_off(int row, int granule) {
  return row * kRowBytes + ((granule ^ (row & 15)) << 4);
}
// V tiles are read with ds_read_b64_tr_b16: one instruction touches 8 rows x
// one 64-byte chunk; XOR of the chunk index with row%4 places the four rows of
// each half-wave in distinct 64-byte bank groups.
__device__ __forceinline__ int v_swizzle_off(int row, int granule) {
  return row * kRowBytes + ((((granule >> 2) ^ (row & 3)) << 6) | ((granule & 3) << 4));
}

typedef __attribute__((__vector_size__(4 * sizeof(short)))) short lds_s16x4_t;

// Transposed 8-byte LDS read (see header comment); byte_off is a byte offset
// into the dynamic LDS segment.
__device__ __forceinline__ u32x2_t lds_read_tr16(const char *lds_base, int byte_off) {
  auto p = reinterpret_cast<__attribute__((address_space(3))) lds_s16x4_t *>(
      (__attribute__((address_space(3))) char *)(lds_base) + byte_off);
  lds_s16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(p);
  return __builtin_bit_cast(u32x2_t, v);
}

__device__ __forceinline__ u32x4_t lds_read_b128(const char *lds_base, int byte_off) {
  return *reinterpret_cast<const u32x4_t *>(lds_base + byte_off);
}
__device__ __forceinline__ void lds_write_b128(char *lds_base, int byte_off, u32x4_t v) {
  *reinterpret_cast<u32x4_t *>(lds_base + byte_off) = v;
}

__device__ __forceinline__ u32x4_t global_load_b128(const void *p) {
  return *reinterpret_cast<const u32x4_t *>(p);
}
// The same load marked non-temporal (read once, not worth keeping in the caches): on this part a kernel
// that streams from HBM with such loads reaches 7.2 TB/s where ordinary loads reach 6.4.
__device__ __forceinline__ u32x4_t global_load_b128_nt(const void *p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(p));
}

}  // namespace LLMHIP_NS
