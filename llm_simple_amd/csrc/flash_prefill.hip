// Causal flash-attention prefill for gfx950 (MI355X).
//
// Computes what the reference's npu_flash_attn_layer / npu_flash_attn_gqa_layer
// compute (prebuild/npu_ops.h:6-18): out[m][H*128] = softmax(scale q k^T +
// mask) v, key c masked for query r iff c > r + offset
// (src/llama2_layer_cpu.cpp:687-701), scale = 1/sqrt(128) inside
// (src/llama2_layer_cpu.cpp:177), query head h reading kv head h / group_size.
//
// Common to both kernels below.  A wave owns 32 query rows.  The scores are
// produced transposed, S^T = K Q^T, with mfma_f32_32x32x16: every lane then
// holds 16 keys of ONE query column per 32-key block, so the softmax row
// reductions are in-register plus one exchange with lane^32
// (v_permlane32_swap).  The probabilities, rounded to the storage type, are
// already laid out as the B operand of O^T += V^T P^T (the contraction index is
// permuted consistently on the V side), so P never touches LDS.  K and V tiles
// of 64 keys are staged in LDS, XOR-swizzled 256-byte rows; K fragments are
// read with ds_read_b128, V^T fragments with ds_read_b64_tr_b16.  exp2 with the
// scale folded into one FMA; the reference maximum is kept in raw score units and
// moves lazily, so O is rarely rescaled.  Accumulation is fp32; out =
// O / l rounded once; l sums the ROUNDED probabilities (what P.V used).
//
// flash_prefill_kernel<T, NW>: NW waves share the K/V tiles of 32*NW query rows.
// NW = 8 (one workgroup per CU) once 256-row workgroups alone fill the chip, NW = 4
// (two workgroups per CU) for smaller problems.  Tiles travel global -> LDS without
// VGPR staging (global_load_lds_dwordx4), spread over the MFMA stream.
#include "common.hpp"
#include "kernels.hpp"

namespace llmhip {

constexpr int kTileN = 64;                      // keys per LDS tile
constexpr int kTileBytes = kTileN * kRowBytes;  // 16 KiB
constexpr float kLazyLog2 = 8.0f;                // rescale threshold, log2 units

struct PrefillParams {
  const char *q;
  const char *k;
  const char *v;
  char *out;
  int m, n, offset;
  int H, Hkv, g;
  int num_q_tiles;
  int sched_mode;  // 0: plain, 1: several XCDs per kv head, 2: several kv heads per XCD
  int sched_a;     // mode 1: XCDs per kv head; mode 2: heads per XCD
  float scale_log2e;
};

// blockIdx -> (query tile, head).  Workgroup ids are dealt round-robin to the 8
// XCDs by the hardware; heads that share a kv head are kept on the same XCD(s)
// so that its K/V stay in that XCD's L2, and within an XCD the heaviest (last)
// query tiles are issued first.
__device__ __forceinline__ bool prefill_schedule(const PrefillParams &p, int bid, int &tile,
                                                 int &head) {
  const int T = p.num_q_tiles;
  if (p.sched_mode == 1) {
    const int X = p.sched_a;
    const int xcd = bid & 7, slot = bid >> 3;
    const int kvh = xcd / X, sub = xcd % X;
    const int idx = slot * X + sub;
    if (idx >= p.g * T) return false;
    tile = T - 1 - idx / p.g;
    head = kvh * p.g + idx % p.g;
    return true;
  }
  if (p.sched_mode == 2) {
    const int hp = p.sched_a;
    const int xcd = bid & 7, slot = bid >> 3;
    if (slot >= hp * T) return false;
    tile = T - 1 - slot / hp;
    head = xcd * hp + slot % hp;
    return true;
  }
  if (bid >= T * p.H) return false;
  tile = T - 1 - bid / p.H;
  head = bid % p.H;
  return true;
}

// max / sum over the lane pair (l, l^32) without going through the LDS
// crossbar.  v_permlane32_swap(a, b) exchanges a[32..63] with b[0..31]; with
// a == b == x the two results are (x_lo, x_lo) and (x_hi, x_hi).  The results
// are copied to scalars before the bit cast: a bit cast applied directly to a
// vector element reads element 0.
__device__ __forceinline__ void pair_swap(float x, float &lo, float &hi) {
  typedef __attribute__((ext_vector_type(2))) unsigned u2;
  const unsigned u = __builtin_bit_cast(unsigned, x);
  const u2 r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  const unsigned r0 = r[0], r1 = r[1];
  lo = __builtin_bit_cast(float, r0);
  hi = __builtin_bit_cast(float, r1);
}
__device__ __forceinline__ float pair_max(float x) {
  float lo, hi;
  pair_swap(x, lo, hi);
  return fmaxf(lo, hi);
}
__device__ __forceinline__ float pair_sum(float x) {
  float lo, hi;
  pair_swap(x, lo, hi);
  return lo + hi;
}

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

// LDS visibility + workgroup barrier that does not drain outstanding global loads.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// State of one wave: 32 query rows (one per lane pair), fp32 O^T accumulators.
template <typename T> struct WaveAttn {
  using E = Elem<T>;
  f32x16_t o[4];       // O^T: d block x (16 d rows of this lane)
  f32x16_t s[2];       // S^T / P^T of the current tile: key block x 16 keys
  u32x4_t pf[2][2];    // P^T packed as B operand: key block x k-step
  u32x4_t qf[8];       // Q^T fragments (B operand), loaded once
  float m_run, l_run;  // running max (raw score units) and sum of this lane's keys
  int lane, l32, hh, g16, li;

  __device__ __forceinline__ void init(int lane_) {
    lane = lane_;
    l32 = lane & 31;
    hh = lane >> 5;
    g16 = lane >> 4;
    li = lane & 15;
    m_run = -INFINITY;
    l_run = 0.0f;
#pragma unroll
    for (int d = 0; d < 4; ++d)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[d][i] = 0.0f;
  }

  __device__ __forceinline__ void load_q(const char *q_row_head) {
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) qf[kk] = global_load_b128(q_row_head + hh * 16 + kk * 32);
  }
  // The Q loads are complete after this: no wait inside the key loop is ever
  // attributed to them.
  __device__ __forceinline__ void pin_q() {
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) asm volatile("" : "+v"(qf[kk]));
  }

  struct NoHook {
    __device__ __forceinline__ void operator()(int) const {}
  };
  // S^T = K Q^T for the 64 keys of the tile at ks.  hook(i) runs after MFMA i
  // (0..15): the callers spread their global loads over the MFMA stream with it.
  template <typename Hook = NoHook>
  __device__ __forceinline__ void qk(const char *ks, Hook hook = Hook()) {
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        const u32x4_t kf = lds_read_b128(ks, k_swizzle_off(kb * 32 + l32, 2 * kk + hh));
        if (kk == 0) {
          f32x16_t z;
#pragma unroll
          for (int i = 0; i < 16; ++i) z[i] = 0.0f;
          s[kb] = E::mfma32(kf, qf[kk], z);
        } else {
          s[kb] = E::mfma32(kf, qf[kk], s[kb]);
        }
        hook(kk * 2 + kb);
      }
    }
  }

  // O^T += V^T P^T.  Lane (d = 32*dblk + l32, hh): element e of k-step (kb, ks2)
  // is the key 32*kb + 16*ks2 + 8*(e/4) + 4*hh + e%4 -- the key P's element e
  // carries.
  template <typename Hook = NoHook>
  __device__ __forceinline__ void pv(const char *vs, Hook hook = Hook()) {
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int ks2 = 0; ks2 < 2; ++ks2) {
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const int kr0 = kb * 32 + ks2 * 16 + 4 * hh + (li >> 2);
          const int gran = d * 4 + (g16 & 1) * 2 + ((li & 3) >> 1);
          const int sub = (li & 1) * 8;
          const u32x2_t lo = lds_read_tr16(vs, v_swizzle_off(kr0, gran) + sub);
          const u32x2_t hi = lds_read_tr16(vs, v_swizzle_off(kr0 + 8, gran) + sub);
          const u32x4_t vf = {lo[0], lo[1], hi[0], hi[1]};
          o[d] = E::mfma32(vf, pf[kb][ks2], o[d]);
          hook((kb * 2 + ks2) * 4 + d);
        }
      }
  }

  // Online softmax of s -> pf.  qrow: query row of this lane's column; rows see
  // keys <= qrow + offset; `partial` says whether any key of the tile can be
  // masked for any row of the wave.
  __device__ __forceinline__ void softmax(int key0, int qrow, int offset, int n, bool partial,
                                          float scale_log2e) {
    if (partial) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = key0 + kb * 32 + 8 * (i >> 2) + 4 * hh + (i & 3);
          if (key > qrow + offset || key >= n) s[kb][i] = -INFINITY;
        }
    }
    float mloc = -INFINITY;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int i = 0; i < 16; ++i) mloc = fmaxf(mloc, s[kb][i]);
    mloc = pair_max(mloc);
    // m_run is the reference maximum used in the exponent, in raw score units.  It
    // moves only when a row maximum exceeds it by more than kLazyLog2 in log2 units
    // (probabilities then stay below 2^kLazyLog2, harmless in fp32 sums and in the
    // 16-bit P operand); a -inf reference always moves.  O and l are rescaled only
    // then, which after the first tiles is rare.
    const bool move = mloc > m_run + kLazyLog2 / scale_log2e;
    const float m_new = move ? mloc : m_run;
    const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
    const float neg_ms = -m_use * scale_log2e;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int i = 0; i < 16; ++i)
        s[kb][i] = fast_exp2(__builtin_fmaf(s[kb][i], scale_log2e, neg_ms));
    if (__builtin_amdgcn_ballot_w64(move) != 0) {
      const float alpha = move ? fast_exp2((m_run - m_use) * scale_log2e) : 1.0f;
      l_run *= alpha;
#pragma unroll
      for (int d = 0; d < 4; ++d)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[d][i] *= alpha;
    }
    m_run = m_new;
    float ps0 = 0.0f, ps1 = 0.0f;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int ks2 = 0; ks2 < 2; ++ks2) {
        u32x4_t w;
#pragma unroll
        for (int e2 = 0; e2 < 4; ++e2) {
          w[e2] = E::pack2(s[kb][8 * ks2 + 2 * e2], s[kb][8 * ks2 + 2 * e2 + 1]);
          if (e2 & 1)
            ps1 = dot2_ones<T>(w[e2], ps1);
          else
            ps0 = dot2_ones<T>(w[e2], ps0);
        }
        pf[kb][ks2] = w;
      }
    l_run += ps0 + ps1;
  }

  // out[qrow][head][d] = O^T / l, rounded once.
  __device__ __forceinline__ void store(char *out_row_head, bool valid) {
    const float l_tot = pair_sum(l_run);
    const float inv = (l_tot > 0.0f) ? 1.0f / l_tot : 0.0f;
    if (!valid) return;
#pragma unroll
    for (int d = 0; d < 4; ++d)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        u32x2_t w;
        w[0] = E::pack2(o[d][4 * i4] * inv, o[d][4 * i4 + 1] * inv);
        w[1] = E::pack2(o[d][4 * i4 + 2] * inv, o[d][4 * i4 + 3] * inv);
        const int dd = 32 * d + 8 * i4 + 4 * hh;
        *reinterpret_cast<u32x2_t *>(out_row_head + dd * 2) = w;
      }
  }
};

// Global -> LDS tile loader without VGPR staging (global_load_lds_dwordx4: lane l's 16
// bytes land at the wave-uniform LDS address + 16*l).  One wave instruction fills four
// 256-byte rows; the XOR swizzles are realised on the global side: the lane that owns
// physical granule pg of row r fetches the logical granule that belongs there.  A tile
// is 16 instructions, dealt to the NW waves; `slot` s of wave w covers rows
// 4*(s*NW + w) .. +3.  Completion needs s_waitcnt vmcnt(0) before the publishing barrier.
template <int NW> struct DirectLoader {
  static constexpr int kSlots = 16 / NW;  // instructions per wave per tile
  int wave, lane, n;
  size_t kv_row_bytes;
  __device__ __forceinline__ void init(int wave_, int lane_, size_t kv_row_bytes_, int n_) {
    wave = wave_;
    lane = lane_;
    n = n_;
    kv_row_bytes = kv_row_bytes_;
  }
  template <bool IS_V>
  __device__ __forceinline__ void issue(const char *base, int t, char *stage, int slot) const {
    const int r0 = 4 * (slot * NW + wave);
    const int r = r0 + (lane >> 4), pg = lane & 15;
    const int lg = IS_V ? ((((pg >> 2) ^ (r & 3)) << 2) | (pg & 3)) : (pg ^ (r & 15));
    const int key = min(t * kTileN + r, n - 1);
    const char *g = base + (size_t)key * kv_row_bytes + lg * 16;
    __builtin_amdgcn_global_load_lds(
        (const __attribute__((address_space(1))) void *)(g),
        (__attribute__((address_space(3))) void *)(stage + r0 * kRowBytes), 16, 0, 0);
  }
  __device__ __forceinline__ void issue_k(const char *base, int t, char *stage, int slot) const {
    issue<false>(base, t, stage, slot);
  }
  __device__ __forceinline__ void issue_v(const char *base, int t, char *stage, int slot) const {
    issue<true>(base, t, stage, slot);
  }
  static __device__ __forceinline__ void wait_all() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
};

// ---------------------------------------------------------------------------
// NW waves, 32*NW query rows, double-buffered K/V tiles, one barrier per tile.
// Every wave runs S = K Q^T, softmax and P.V of a tile as one instruction stream
// (the compiler interleaves the softmax VALU work with the MFMAs); the loads of
// the next tile are spread over that stream.  NW = 4: two workgroups per CU
// (small problems); NW = 8: one workgroup per CU, K/V tiles shared by 256 rows.
// ---------------------------------------------------------------------------
template <typename T, int NW>
__global__ __launch_bounds__(64 * NW, NW == 4 ? 2 : 1) void flash_prefill_kernel(PrefillParams p) {
  // SUB tiles of 64 keys per LDS stage and per barrier: with one workgroup per CU (NW = 8)
  // a stage holds 128 keys, which halves the number of times the waves are forced in step.
  constexpr int BM = 32 * NW, PER = 16 / NW, SUB = NW == 8 ? 2 : 1;
  constexpr int kStage = SUB * 2 * kTileBytes;  // [SUB x K tile | SUB x V tile]
  extern __shared__ __attribute__((aligned(16))) char lds[];  // 2 stages
  int tile, head;
  if (!prefill_schedule(p, blockIdx.x, tile, head)) return;

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int kvh = head / p.g;
  const int row0 = tile * BM;
  const int rows_end = min(p.m, row0 + BM);
  const int n_vis = min(p.n, rows_end + p.offset);  // keys any row of this tile can see
  const int J = (n_vis + kTileN - 1) / kTileN;      // 64-key tiles of the workgroup
  const int JS = (J + SUB - 1) / SUB;               // stages
  const size_t q_row_bytes = (size_t)p.H * kRowBytes;
  const size_t kv_row_bytes = (size_t)p.Hkv * kRowBytes;
  const char *kbase = p.k + (size_t)kvh * kRowBytes;
  const char *vbase = p.v + (size_t)kvh * kRowBytes;

  WaveAttn<T> w;
  w.init(lane);
  const int qblk0 = row0 + wave * 32;
  const int qrow = qblk0 + w.l32;
  const int last_row = min(qblk0 + 31, p.m - 1);
  const int Jw = (qblk0 < p.m) ? min(J, (min(p.n, last_row + p.offset + 1) + kTileN - 1) / kTileN) : 0;
  w.load_q(p.q + (size_t)min(qrow, p.m - 1) * q_row_bytes + (size_t)head * kRowBytes);

  // tile t lives in stage (t / SUB) & 1 at sub-slot t % SUB
  auto k_tile = [&](int t) { return lds + ((t / SUB) & 1) * kStage + (t % SUB) * kTileBytes; };
  auto v_tile = [&](int t) { return lds + ((t / SUB) & 1) * kStage + (SUB + t % SUB) * kTileBytes; };

  DirectLoader<NW> ld;
  ld.init(wave, lane, kv_row_bytes, p.n);
#pragma unroll
  for (int u = 0; u < SUB; ++u)
#pragma unroll
    for (int sl = 0; sl < PER; ++sl) {
      ld.issue_k(kbase, min(u, J - 1), k_tile(u), sl);
      ld.issue_v(vbase, min(u, J - 1), v_tile(u), sl);
    }
  w.pin_q();  // waits for every load issued so far, the tile loads included
  ld.wait_all();
  lds_barrier();

  for (int js = 0; js < JS; ++js) {
#pragma unroll
    for (int u = 0; u < SUB; ++u) {
      const int j = js * SUB + u;             // tile computed now
      const int jn = min(j + SUB, J - 1);     // tile fetched now, into the other stage
      char *kn = k_tile(j + SUB), *vn = v_tile(j + SUB);
      if (j < Jw) {
        const int key0 = j * kTileN;
        const bool partial = (key0 + kTileN - 1 > qblk0 + p.offset) || (key0 + kTileN > p.n);
        // a burst of loads would stall every wave behind the texture addresser's queue:
        // one load every 16 / PER MFMAs instead
        w.qk(k_tile(j), [&](int i) {
#pragma unroll
          for (int r = 0; r < PER; ++r)
            if (i == (16 / PER) * r + 1) ld.issue_k(kbase, jn, kn, r);
        });
        w.softmax(key0, qrow, p.offset, p.n, partial, p.scale_log2e);
        w.pv(v_tile(j), [&](int i) {
#pragma unroll
          for (int r = 0; r < PER; ++r)
            if (i == (16 / PER) * r + 1) ld.issue_v(vbase, jn, vn, r);
        });
      } else {
#pragma unroll
        for (int sl = 0; sl < PER; ++sl) {
          ld.issue_k(kbase, jn, kn, sl);
          ld.issue_v(vbase, jn, vn, sl);
        }
      }
    }
    ld.wait_all();
    lds_barrier();
  }
  w.store(p.out + (size_t)qrow * q_row_bytes + (size_t)head * kRowBytes, qrow < p.m);
}

template <typename T, int NW>
static hipError_t launch_prefill_t(const PrefillParams &p0, hipStream_t stream) {
  PrefillParams p = p0;
  constexpr int BM = 32 * NW;
  constexpr int NT = 64 * NW;
  p.num_q_tiles = (p.m + BM - 1) / BM;
  const int T_ = p.num_q_tiles;
  int grid;
  if (p.Hkv <= 8 && 8 % p.Hkv == 0) {
    p.sched_mode = 1;
    p.sched_a = 8 / p.Hkv;
    const int per_kvh = p.g * T_;
    grid = 8 * ((per_kvh + p.sched_a - 1) / p.sched_a);
  } else if (p.Hkv % 8 == 0) {
    p.sched_mode = 2;
    p.sched_a = (p.Hkv / 8) * p.g;
    grid = 8 * p.sched_a * T_;
  } else {
    p.sched_mode = 0;
    p.sched_a = 0;
    grid = T_ * p.H;
  }
  const size_t lds_bytes = (NW == 8 ? 2 : 1) * 4 * kTileBytes;
  void (*kern)(PrefillParams) = flash_prefill_kernel<T, NW>;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)lds_bytes);
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  hipLaunchKernelGGL(kern, dim3(grid), dim3(NT), lds_bytes, stream, p);
  return hipGetLastError();
}

hipError_t launch_flash_prefill(void *out, const void *q, const void *k, const void *v, int m,
                                int n, int offset, int group_size, int kv_head_num, int dt,
                                hipStream_t stream) {
  PrefillParams p;
  p.q = static_cast<const char *>(q);
  p.k = static_cast<const char *>(k);
  p.v = static_cast<const char *>(v);
  p.out = static_cast<char *>(out);
  p.m = m;
  p.n = n;
  p.offset = offset;
  p.g = group_size;
  p.Hkv = kv_head_num;
  p.H = group_size * kv_head_num;
  p.scale_log2e = 1.4426950408889634f / sqrtf((float)kHeadDim);
  // 256-row workgroups once they alone fill the 256 CUs; 128-row ones (two per
  // CU) for smaller problems.
  const bool big = (long long)((m + 255) / 256) * p.H >= 256;
  if (dt == kDtFloat16)
    return big ? launch_prefill_t<_Float16, 8>(p, stream) : launch_prefill_t<_Float16, 4>(p, stream);
  return big ? launch_prefill_t<__bf16, 8>(p, stream) : launch_prefill_t<__bf16, 4>(p, stream);
}

}  // namespace llmhip
