// Causal flash-attention prefill for gfx950 (MI355X).
//
// Computes what the reference's npu_flash_attn_layer / npu_flash_attn_gqa_layer
// compute (prebuild/npu_ops.h:6-18): out[m][H*128] = softmax(scale q k^T +
// mask) v, key c masked for query r iff c > r + offset
// (src/llama2_layer_cpu.cpp:687-701), scale = 1/sqrt(128) inside
// (src/llama2_layer_cpu.cpp:177), query head h reading kv head h / group_size.
//
// Work decomposition.  One workgroup = 4 wavefronts = one (query tile, query
// head).  A query tile is 4*QB blocks of 32 rows; wave w owns blocks {w} (QB=1)
// or {w, 7-w} (QB=2) so that the causal diagonal costs every wave the same.
// The workgroup walks the visible keys in tiles of 64; K and V tiles are staged
// in LDS (double buffered, XOR-swizzled 256-byte rows) by all 256 threads with
// 128-bit loads and are shared by the four waves.
//
// Per wave and tile the scores are produced transposed, S^T = K Q^T, with
// mfma_f32_32x32x16: every lane then holds 16 keys of ONE query column, so the
// softmax row reductions are in-register plus one exchange with lane^32.  The
// probabilities, rounded to the storage type, are already laid out as the B
// operand of O^T += V^T P^T (the contraction index is permuted consistently on
// the V side), so P never touches LDS.  V^T fragments come from
// ds_read_b64_tr_b16.  Accumulation is fp32; out = O / l rounded once.
#include "common.hpp"
#include "kernels.hpp"

namespace llmhip {

constexpr int kTileN = 64;                        // keys per LDS tile
constexpr int kTileBytes = kTileN * kRowBytes;    // 16 KiB
constexpr int kPrefillThreads = 256;

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

template <typename T, int QB>
__global__ __launch_bounds__(kPrefillThreads) void flash_prefill_kernel(PrefillParams p) {
  using E = Elem<T>;
  constexpr int BM = 4 * QB * 32;
  extern __shared__ __attribute__((aligned(16))) char lds[];
  // lds: [2 stages][K tile | V tile]
  int tile, head;
  if (!prefill_schedule(p, blockIdx.x, tile, head)) return;

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int l32 = lane & 31;
  const int hh = lane >> 5;
  const int kvh = head / p.g;
  const int row0 = tile * BM;
  const int rows_end = min(p.m, row0 + BM);
  // keys any row of this tile can see
  const int n_vis = min(p.n, rows_end + p.offset);
  const int num_tiles = (n_vis + kTileN - 1) / kTileN;

  const size_t q_row_bytes = (size_t)p.H * kRowBytes;
  const size_t kv_row_bytes = (size_t)p.Hkv * kRowBytes;
  const char *kbase = p.k + (size_t)kvh * kRowBytes;
  const char *vbase = p.v + (size_t)kvh * kRowBytes;

  // ---- this wave's query blocks and Q^T fragments (B operand) ----
  int qrow[QB];     // query row of this lane's column
  int qblk0[QB];    // first row of the block
  u32x4_t qf[QB][8];
#pragma unroll
  for (int b = 0; b < QB; ++b) {
    const int blk = (b == 0) ? wave : (4 * QB - 1 - wave);
    qblk0[b] = row0 + blk * 32;
    qrow[b] = qblk0[b] + l32;
    const int rr = min(qrow[b], p.m - 1);
    const char *qp = p.q + (size_t)rr * q_row_bytes + (size_t)head * kRowBytes + hh * 16;
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) qf[b][kk] = global_load_b128(qp + kk * 32);
  }

  f32x16_t o[QB][4];
  float m_run[QB], l_run[QB];
#pragma unroll
  for (int b = 0; b < QB; ++b) {
    m_run[b] = -INFINITY;
    l_run[b] = 0.0f;
#pragma unroll
    for (int d = 0; d < 4; ++d)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[b][d][i] = 0.0f;
  }

  // ---- cooperative tile loader: thread -> 4 granules of K and 4 of V ----
  u32x4_t kreg[4], vreg[4];
  auto load_tile_regs = [&](int j) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = tid + i * kPrefillThreads;
      const int r = c >> 4, gi = c & 15;
      const int key = min(j * kTileN + r, p.n - 1);
      const size_t off = (size_t)key * kv_row_bytes + gi * 16;
      kreg[i] = global_load_b128(kbase + off);
      vreg[i] = global_load_b128(vbase + off);
    }
  };
  auto store_tile_lds = [&](int stage) {
    char *ks = lds + stage * 2 * kTileBytes;
    char *vs = ks + kTileBytes;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = tid + i * kPrefillThreads;
      const int r = c >> 4, gi = c & 15;
      lds_write_b128(ks, k_swizzle_off(r, gi), kreg[i]);
      lds_write_b128(vs, v_swizzle_off(r, gi), vreg[i]);
    }
  };

  if (num_tiles > 0) {
    load_tile_regs(0);
    store_tile_lds(0);
  }
  __syncthreads();

  for (int j = 0; j < num_tiles; ++j) {
    const int stage = j & 1;
    const bool has_next = (j + 1) < num_tiles;
    if (has_next) load_tile_regs(j + 1);

    const char *ks = lds + stage * 2 * kTileBytes;
    const char *vs = ks + kTileBytes;
    const int key0 = j * kTileN;

    // which of this wave's query blocks see any key of this tile
    bool active[QB], partial[QB];
    bool any_active = false;
#pragma unroll
    for (int b = 0; b < QB; ++b) {
      const int last_row = min(qblk0[b] + 31, p.m - 1);
      active[b] = (qblk0[b] < p.m) && (key0 <= last_row + p.offset);
      partial[b] = (key0 + kTileN - 1 > qblk0[b] + p.offset) || (key0 + kTileN > p.n);
      any_active |= active[b];
    }

    if (any_active) {
      // ---- S^T = K Q^T ----
      f32x16_t s[QB][2];
#pragma unroll
      for (int b = 0; b < QB; ++b)
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int i = 0; i < 16; ++i) s[b][kb][i] = 0.0f;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        const int r = kb * 32 + l32;
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) {
          const u32x4_t kf = lds_read_b128(ks, k_swizzle_off(r, 2 * kk + hh));
#pragma unroll
          for (int b = 0; b < QB; ++b)
            if (active[b]) s[b][kb] = E::mfma32(kf, qf[b][kk], s[b][kb]);
        }
      }

      // ---- online softmax per query column, P packed as B operand ----
      u32x4_t pf[QB][2][2];
#pragma unroll
      for (int b = 0; b < QB; ++b) {
        if (!active[b]) continue;
        float mloc = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            float t = s[b][kb][i] * p.scale_log2e;
            if (partial[b]) {
              const int key = key0 + kb * 32 + 8 * (i >> 2) + 4 * hh + (i & 3);
              if (key > qrow[b] + p.offset || key >= p.n) t = -INFINITY;
            }
            s[b][kb][i] = t;
            mloc = fmaxf(mloc, t);
          }
        mloc = fmaxf(mloc, xor_lane(mloc, 32));
        const float m_new = fmaxf(m_run[b], mloc);
        const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
        const float alpha = fast_exp2(m_run[b] - m_use);
        m_run[b] = m_new;
        float psum = 0.0f;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const float e = fast_exp2(s[b][kb][i] - m_use);
            s[b][kb][i] = e;
            psum += e;
          }
        l_run[b] = l_run[b] * alpha + psum;
#pragma unroll
        for (int d = 0; d < 4; ++d)
#pragma unroll
          for (int i = 0; i < 16; ++i) o[b][d][i] *= alpha;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int ks2 = 0; ks2 < 2; ++ks2) {
            u32x4_t w;
#pragma unroll
            for (int e2 = 0; e2 < 4; ++e2)
              w[e2] = E::pack2(s[b][kb][8 * ks2 + 2 * e2], s[b][kb][8 * ks2 + 2 * e2 + 1]);
            pf[b][kb][ks2] = w;
          }
      }

      // ---- O^T += V^T P^T ----
      // lane (d = 32*dblk + l32, hh): element e of k-step (kb, ks2) is the key
      // 32*kb + 16*ks2 + 8*(e/4) + 4*hh + e%4 -- the key P's element e carries.
      const int grp = lane >> 4;       // 16-lane group: d half = grp&1, hh = grp>>1
      const int li = lane & 15;
#pragma unroll
      for (int d = 0; d < 4; ++d) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int ks2 = 0; ks2 < 2; ++ks2) {
            const int kr0 = kb * 32 + ks2 * 16 + 4 * hh + (li >> 2);
            const int gran = d * 4 + (grp & 1) * 2 + ((li & 3) >> 1);
            const int sub = (li & 1) * 8;
            const u32x2_t lo = lds_read_tr16(vs, v_swizzle_off(kr0, gran) + sub);
            const u32x2_t hi = lds_read_tr16(vs, v_swizzle_off(kr0 + 8, gran) + sub);
            const u32x4_t vf = {lo[0], lo[1], hi[0], hi[1]};
#pragma unroll
            for (int b = 0; b < QB; ++b)
              if (active[b]) o[b][d] = E::mfma32(vf, pf[b][kb][ks2], o[b][d]);
          }
      }
    }

    if (has_next) store_tile_lds(stage ^ 1);
    __syncthreads();
  }

  // ---- epilogue: out[q][head][d] = O^T / l ----
#pragma unroll
  for (int b = 0; b < QB; ++b) {
    const float l_tot = l_run[b] + xor_lane(l_run[b], 32);
    const float inv = (l_tot > 0.0f) ? 1.0f / l_tot : 0.0f;
    if (qrow[b] < p.m) {
      char *op = p.out + (size_t)qrow[b] * q_row_bytes + (size_t)head * kRowBytes;
#pragma unroll
      for (int d = 0; d < 4; ++d)
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
          u32x2_t w;
          w[0] = E::pack2(o[b][d][4 * i4] * inv, o[b][d][4 * i4 + 1] * inv);
          w[1] = E::pack2(o[b][d][4 * i4 + 2] * inv, o[b][d][4 * i4 + 3] * inv);
          const int dd = 32 * d + 8 * i4 + 4 * hh;
          *reinterpret_cast<u32x2_t *>(op + dd * 2) = w;
        }
    }
  }
}

template <typename T, int QB>
static hipError_t launch_prefill_t(const PrefillParams &p0, hipStream_t stream) {
  PrefillParams p = p0;
  constexpr int BM = 4 * QB * 32;
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
  const size_t lds_bytes = 2 * 2 * kTileBytes;
  auto kern = flash_prefill_kernel<T, QB>;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)lds_bytes);
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  hipLaunchKernelGGL(kern, dim3(grid), dim3(kPrefillThreads), lds_bytes, stream, p);
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
  // Small problems: 128-row tiles give more workgroups; large ones: 256-row
  // tiles halve the LDS traffic per flop.
  const bool big = (long long)((m + 255) / 256) * p.H >= 256;
  if (dt == kDtFloat16)
    return big ? launch_prefill_t<_Float16, 2>(p, stream) : launch_prefill_t<_Float16, 1>(p, stream);
  return big ? launch_prefill_t<__bf16, 2>(p, stream) : launch_prefill_t<__bf16, 1>(p, stream);
}

}  // namespace llmhip
