// GQA-aware split-KV decode attention for gfx950 (MI355X).
//
// The reference decodes with the same operator as prefill, m = 1 and offset =
// n - 1 (npu_flash_attn_gqa_layer, src/llama2_layer_npu.cpp:866-869): one
// softmax row per head over the whole contiguous KV cache
// [max_seq_len][Hkv][128] (src/llama2_layer_npu.cpp:1148-1149).  That is a
// pure stream of K and V through the chip, so the kernel is organised around
// HBM: grid = (KV split, kv head, sequence); a workgroup takes every
// num_splits-th block of 128 keys of one kv head (the workgroups of a sequence
// walk through its cache side by side), each of its 4 waves 32 keys of a block,
// and K and V of every key are read from HBM exactly once for all group_size
// query heads (and all m <= 16/group_size query rows) that share the kv head.
//
// The m*group_size query rows are the 16 columns of mfma_f32_16x16x32
// (S^T = K Q^T, O^T += V^T P^T); unused columns are zero.  Every load
// instruction fetches whole 256-byte head rows (16 lanes per row); K and V are
// staged in wave-private LDS regions, K read back in the A-operand layout
// (loading K straight into that layout -- 16 rows x 16 bytes per quarter wave --
// costs the texture cache 16 tag look-ups where this costs 2, and measured 1-2 %
// slower), V read transposed with ds_read_b64_tr_b16.  K and V are read once, so
// their loads are non-temporal (7.1 TB/s at 2 GiB where ordinary loads give 6.2),
// and K and V of a step are fetched one after the other so that a CU has 32 KiB
// in flight, not 64 (see the loop).  Each wave keeps its own running (max, sum,
// O); the four
// waves are merged through LDS at the end and the workgroup writes either the
// final rows (one split) or an fp32 partial (max, sum, unnormalised O) that
// flash_decode_combine_kernel folds with the log-sum-exp rule.  (Folding inside
// the last-arriving workgroup instead was measured and rejected: the device-scope
// release/acquire fences it needs write back and invalidate the XCD's L2 and cost
// more than the second launch -- 91 us against 33 us at batch 1, 32768 keys.  Without
// fences, with the partials written through and read back at device scope (sc1 accesses)
// and one relaxed device-scope atomic, it is correct but still slower -- 35.9 us against
// 33.4 us, and 15.0 us against 10.6 us at 4096 keys: the chain store-acknowledge, atomic,
// two dependent rounds of memory-latency loads in ONE workgroup is longer than a launch.
// Eight-wave workgroups, half as many, merging pairs of splits through LDS: 4.5 TB/s
// against 6.0 at the time -- a CU draws about 31-35 GB/s however many waves ask, so all of
// them must stream.)
#include <atomic>

#include "common.hpp"
#include "kernels.hpp"

namespace llmhip {

constexpr int kDecThreads = 256;
constexpr int kDecWaveKeys = 32;                  // keys per wave per step
constexpr int kDecStepKeys = 4 * kDecWaveKeys;    // keys per workgroup per step
constexpr int kDecCols = 16;                      // query rows per kv head (MFMA N)
constexpr int kDecWaveLds = kDecWaveKeys * kRowBytes;  // 8 KiB of staging per wave, for K and for V
constexpr int kDecLdsPad = 24 * 1024;             // with the 64 KiB of staging: more than half a CU's LDS

struct DecodeParams {
  const char *q;
  const char *k;
  const char *v;
  char *out;
  float *ws_o;   // [batch][Hkv][splits][16][128]
  float *ws_ml;  // [batch][Hkv][splits][16][2]
  int batch, m, n, offset;
  int64_t kv_seq_stride;
  int g, Hkv, H;
  int rows;  // m * g
  int num_splits;
  float scale_log2e;
  // Fused decode step (FUSED kernels only): the token at row fused_pos = n - 1 is not in the cache yet.
  // q, new_k and new_v hold the unrotated projections of that token ([H][128], [Hkv][128] twice);
  // q and the new K row are rotated with table row freq_row (64 (cos, sin) pairs) as they are loaded,
  // and the workgroup that owns the last key range writes the rotated K row and the V row to the cache.
  const char *new_k;
  const char *new_v;
  const float *freq_row;
  int fused_pos, is_neox;
};

// RoPE of the four 16-byte fragments a lane holds of one head row: fragment kk = dims 8*cg + 32*kk .. +7.
// Arithmetic of the rotary kernel, unfused products and sums (src/llama2_layer_cpu.cpp:835-856):
// (a*c - b*s, a*s + b*c) rounded once; interleaved pairs (2f, 2f+1), neox pairs (f, f+64).
template <typename T>
__device__ __forceinline__ void rotate_frags(u32x4_t (&f)[4], const float *tab, int cg, int is_neox) {
#pragma clang fp contract(off)
  using E = Elem<T>;
  auto get = [](const u32x4_t &w, int e) { return (uint16_t)((w[e >> 1] >> ((e & 1) * 16)) & 0xFFFFu); };
  auto put = [](u32x4_t &w, int e, uint16_t v) {
    w[e >> 1] = (w[e >> 1] & ~(0xFFFFu << ((e & 1) * 16))) | ((uint32_t)v << ((e & 1) * 16));
  };
  if (is_neox) {
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      const int d0 = 8 * cg + 32 * kk;  // pair index of element 0: d0 < 64
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float a = E::widen(get(f[kk], e)), b = E::widen(get(f[kk + 2], e));
        const float c = tab[2 * (d0 + e)], sn = tab[2 * (d0 + e) + 1];
        const float ra = a * c - b * sn;
        const float rb = a * sn + b * c;
        put(f[kk], e, E::round(ra));
        put(f[kk + 2], e, E::round(rb));
      }
    }
  } else {
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      const int f0 = (8 * cg + 32 * kk) / 2;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float a = E::widen(get(f[kk], 2 * j)), b = E::widen(get(f[kk], 2 * j + 1));
        const float c = tab[2 * (f0 + j)], sn = tab[2 * (f0 + j) + 1];
        const float ra = a * c - b * sn;
        const float rb = a * sn + b * c;
        put(f[kk], 2 * j, E::round(ra));
        put(f[kk], 2 * j + 1, E::round(rb));
      }
    }
  }
}

// V staging swizzle for the 16x16x32 transposed reads: one instruction touches
// 8 rows x 32 bytes per half-wave, so the 32-byte slot index is XORed with
// row%8.
__device__ __forceinline__ int v_swizzle32_off(int row, int granule) {
  return row * kRowBytes + ((((granule >> 1) ^ (row & 7)) << 5) | ((granule & 1) << 4));
}

template <typename T, bool FUSED>
__global__ __launch_bounds__(kDecThreads) void flash_decode_kernel(DecodeParams p) {
  using E = Elem<T>;
  __shared__ __attribute__((aligned(16))) char lds[8 * kDecWaveLds];

  const int split = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int col = lane & 15, cg = lane >> 4;

  // A split is not a contiguous key range but every num_splits-th block of kDecStepKeys keys: the
  // workgroups of one sequence then walk through its cache side by side, which the DRAM channels
  // serve better than as many far-apart streams (the softmax merge does not care which keys a
  // partial covers).
  const int nblocks = (p.n + kDecStepKeys - 1) / kDecStepKeys;
  const int k_end = p.n;
  const int iters = (nblocks - split + p.num_splits - 1) / p.num_splits;  // blocks split, split + S, ...

  const size_t kv_row_bytes = (size_t)p.Hkv * kRowBytes;
  const size_t seq_off = (size_t)b * p.kv_seq_stride * kv_row_bytes + (size_t)kvh * kRowBytes;
  const char *kbase = p.k + seq_off;
  const char *vbase = p.v + seq_off;

  // query column of this lane
  const bool col_valid = col < p.rows;
  const int c_row = col_valid ? col / p.g : 0;
  const int c_head = kvh * p.g + (col_valid ? col % p.g : 0);
  const int c_limit = c_row + p.offset;  // last visible key of this column

  u32x4_t qf[4];
  {
    const char *qp = p.q + (((size_t)b * p.m + c_row) * p.H + c_head) * kRowBytes + cg * 16;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      u32x4_t z = {0u, 0u, 0u, 0u};
      qf[kk] = col_valid ? global_load_b128(qp + kk * 64) : z;
    }
    if (FUSED && col_valid) rotate_frags<T>(qf, p.freq_row, cg, p.is_neox);
  }

  f32x4_t o[8];
#pragma unroll
  for (int d = 0; d < 8; ++d) o[d] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.0f;

  char *vl = lds + wave * kDecWaveLds;
  char *kl = lds + (4 + wave) * kDecWaveLds;

  u32x4_t kn[8], vn[8];
  auto issue_k = [&](int it) {
    const int kb0 = (it * p.num_splits + split) * kDecStepKeys + wave * kDecWaveKeys;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int key = min(kb0 + 4 * i + cg, p.n - 1);
      const char *kp = kbase + (size_t)key * kv_row_bytes + col * 16;
      if (FUSED && key == p.fused_pos) kp = p.new_k + (size_t)kvh * kRowBytes + col * 16;
      kn[i] = global_load_b128_nt(kp);
    }
  };
  auto issue_v = [&](int it) {
    const int kb0 = (it * p.num_splits + split) * kDecStepKeys + wave * kDecWaveKeys;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int key = min(kb0 + 4 * i + cg, p.n - 1);
      const char *vp = vbase + (size_t)key * kv_row_bytes + col * 16;
      if (FUSED && key == p.fused_pos) vp = p.new_v + (size_t)kvh * kRowBytes + col * 16;
      vn[i] = global_load_b128_nt(vp);
    }
  };

  // K and V of a step are fetched one after the other, each while the other half of the step is
  // computed: a wave has 8 KiB of loads in flight at any time, the CU 32 KiB.  That is where this
  // memory system streams fastest -- with both in flight together (64 KiB per CU) every large shape
  // measured 2-3 % slower, and a plain read kernel shows the same optimum.
  // (The first step's K and V start together: one memory round trip less for a workgroup with one step.)
  if (iters > 0) {
    issue_k(0);
    issue_v(0);
  }

  for (int it = 0; it < iters; ++it) {
    const int kb0 = (it * p.num_splits + split) * kDecStepKeys + wave * kDecWaveKeys;
    u32x4_t kc[2][4];
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int i = 0; i < 8; ++i) lds_write_b128(kl, (4 * i + cg) * kRowBytes + ((col ^ ((4 * i + cg) & 15)) << 4), kn[i]);
    __builtin_amdgcn_wave_barrier();
    if (it > 0) issue_v(it);
    // K fragments (A operand): key blk*16+col, dims 32kk + 8cg .. +7
#pragma unroll
    for (int blk = 0; blk < 2; ++blk)
#pragma unroll
      for (int kk = 0; kk < 4; ++kk)
        kc[blk][kk] = lds_read_b128(kl, (blk * 16 + col) * kRowBytes + (((4 * kk + cg) ^ col) << 4));

    if (kb0 < k_end) {
      if (FUSED) {
        // the new token's row: rotate K in registers and append both rows to the cache (lanes whose
        // clamped key is the new row all hold and write the same bytes)
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
          const int key = min(kb0 + blk * 16 + col, p.n - 1);
          if (key == p.fused_pos) {
            rotate_frags<T>(kc[blk], p.freq_row, cg, p.is_neox);
            char *dst = const_cast<char *>(kbase) + (size_t)key * kv_row_bytes + cg * 16;
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) *reinterpret_cast<u32x4_t *>(dst + kk * 64) = kc[blk][kk];
          }
        }
      }
      // ---- S^T = K Q^T : 2 blocks of 16 keys ----
      f32x4_t s[2];
#pragma unroll
      for (int blk = 0; blk < 2; ++blk) {
        s[blk] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) s[blk] = E::mfma16(kc[blk][kk], qf[kk], s[blk]);
      }
      float mloc = -INFINITY;
#pragma unroll
      for (int blk = 0; blk < 2; ++blk)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = kb0 + blk * 16 + 4 * cg + i;
          float t = s[blk][i] * p.scale_log2e;
          if (key >= k_end || key > c_limit) t = -INFINITY;
          s[blk][i] = t;
          mloc = fmaxf(mloc, t);
        }
      mloc = fmaxf(mloc, xor_lane(mloc, 16));
      mloc = fmaxf(mloc, xor_lane(mloc, 32));
      const float m_new = fmaxf(m_run, mloc);
      const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
      const float alpha = fast_exp2(m_run - m_use);
      m_run = m_new;
#pragma unroll
      for (int blk = 0; blk < 2; ++blk)
#pragma unroll
        for (int i = 0; i < 4; ++i) s[blk][i] = fast_exp2(s[blk][i] - m_use);
      // P^T as B operand: slot e<4 -> block 0 key 4cg+e, e>=4 -> block 1 key 4cg+e-4
      u32x4_t pf;
      pf[0] = E::pack2(s[0][0], s[0][1]);
      pf[1] = E::pack2(s[0][2], s[0][3]);
      pf[2] = E::pack2(s[1][0], s[1][1]);
      pf[3] = E::pack2(s[1][2], s[1][3]);
      // the row sum takes the ROUNDED probabilities, the values P.V uses: numerator and
      // denominator then carry the same rounding (as in the prefill kernel)
      float psum = dot2_ones<T>(pf[0], 0.0f);
      psum = dot2_ones<T>(pf[1], psum);
      psum = dot2_ones<T>(pf[2], psum);
      psum = dot2_ones<T>(pf[3], psum);
      l_run = l_run * alpha + psum;
      // ---- O^T += V^T P^T ----
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int i = 0; i < 8; ++i) lds_write_b128(vl, v_swizzle32_off(4 * i + cg, col), vn[i]);
      if (FUSED) {  // the new token's V row goes to the cache
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int key = min(kb0 + 4 * i + cg, p.n - 1);
          if (key == p.fused_pos)
            *reinterpret_cast<u32x4_t *>(const_cast<char *>(vbase) + (size_t)key * kv_row_bytes + col * 16) = vn[i];
        }
      }
      __builtin_amdgcn_wave_barrier();
      if (it + 1 < iters) issue_k(it + 1);
      const int vr = 4 * cg + (col >> 2);
      const int sub = (col & 1) * 8;
#pragma unroll
      for (int d = 0; d < 8; ++d) {
        const int gran = 2 * d + ((col & 3) >> 1);
        const u32x2_t lo = lds_read_tr16(vl, v_swizzle32_off(vr, gran) + sub);
        const u32x2_t hi = lds_read_tr16(vl, v_swizzle32_off(vr + 16, gran) + sub);
        const u32x4_t vf = {lo[0], lo[1], hi[0], hi[1]};
        f32x4_t acc = o[d];
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] *= alpha;
        o[d] = E::mfma16(vf, pf, acc);
      }
    } else if (it + 1 < iters) {
      issue_k(it + 1);
    }
  }

  // ---- merge the four waves ----
  float l_tot = l_run + xor_lane(l_run, 16);
  l_tot += xor_lane(l_tot, 32);
  __syncthreads();
  float *lo_f = reinterpret_cast<float *>(lds);                      // [wave][col][128]
  float *lml = reinterpret_cast<float *>(lds + 4 * kDecWaveLds);     // [wave][col][2] (the K staging space)
#pragma unroll
  for (int d = 0; d < 8; ++d)
    *reinterpret_cast<f32x4_t *>(lo_f + ((wave * kDecCols + col) * kHeadDim + 16 * d + 4 * cg)) = o[d];
  if (cg == 0) {
    lml[(wave * kDecCols + col) * 2] = m_run;
    lml[(wave * kDecCols + col) * 2 + 1] = l_tot;
  }
  __syncthreads();

  {
    const int c = tid >> 4, dch = tid & 15;  // column, 8-wide d chunk
    float mw[4], M = -INFINITY;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      mw[w] = lml[(w * kDecCols + c) * 2];
      M = fmaxf(M, mw[w]);
    }
    const float M_use = (M == -INFINITY) ? 0.0f : M;
    float L = 0.0f, acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = 0.0f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float wt = fast_exp2(mw[w] - M_use);
      L += wt * lml[(w * kDecCols + c) * 2 + 1];
      const float *src = lo_f + ((w * kDecCols + c) * kHeadDim + 8 * dch);
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j] += wt * src[j];
    }
    if (c < p.rows) {
      if (p.num_splits == 1) {
        const float inv = (L > 0.0f) ? 1.0f / L : 0.0f;
        const int r = c / p.g, hq = c % p.g;
        char *op = p.out + (((size_t)b * p.m + r) * p.H + kvh * p.g + hq) * kRowBytes + dch * 16;
        u32x4_t w;
#pragma unroll
        for (int j = 0; j < 4; ++j) w[j] = E::pack2(acc[2 * j] * inv, acc[2 * j + 1] * inv);
        *reinterpret_cast<u32x4_t *>(op) = w;
      } else {
        const size_t slot = (((size_t)b * p.Hkv + kvh) * p.num_splits + split) * kDecCols + c;
        float *wo = p.ws_o + slot * kHeadDim + 8 * dch;
        *reinterpret_cast<f32x4_t *>(wo) = f32x4_t{acc[0], acc[1], acc[2], acc[3]};
        *reinterpret_cast<f32x4_t *>(wo + 4) = f32x4_t{acc[4], acc[5], acc[6], acc[7]};
        if (dch == 0) {
          p.ws_ml[slot * 2] = M;
          p.ws_ml[slot * 2 + 1] = L;
        }
      }
    }
  }
}

// Folds the splits of one output row (one query row of one head) with the log-sum-exp rule.
// grid (rows, Hkv, batch), 256 threads = 8 groups of 32: group sg takes splits sg, sg+8, ... (four
// dims per thread, all of a thread's loads issued before any is used), then the 8 groups are merged
// through LDS.  With few splits the surplus groups have nothing to load.
constexpr int kMaxSplits = 256;

template <typename T>
__global__ __launch_bounds__(256) void flash_decode_combine_kernel(DecodeParams p) {
  using E = Elem<T>;
  __shared__ float red_m[8], red_l[8];
  __shared__ f32x4_t red_o[8][32];
  const int c = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
  const int sg = threadIdx.x >> 5, d4 = threadIdx.x & 31;
  const int S = p.num_splits;
  const size_t base = ((size_t)b * p.Hkv + kvh) * S;
  const float *ml = p.ws_ml + (base * kDecCols + c) * 2;
  const float *src = p.ws_o + (base * kDecCols + c) * kHeadDim + 4 * d4;
  const size_t ml_stride = (size_t)kDecCols * 2, o_stride = (size_t)kDecCols * kHeadDim;
  float M = -INFINITY, L = 0.0f;
  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
  for (int s0 = sg; s0 < S; s0 += 32) {  // rounds of up to 4 splits per thread
    float mv[4], lv[4];
    f32x4_t ov[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int s = min(s0 + 8 * j, S - 1);
      mv[j] = ml[s * ml_stride];
      lv[j] = ml[s * ml_stride + 1];
      ov[j] = *reinterpret_cast<const f32x4_t *>(src + s * o_stride);
    }
    float Mn = M;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (s0 + 8 * j < S) Mn = fmaxf(Mn, mv[j]);
    const float M_use = (Mn == -INFINITY) ? 0.0f : Mn;
    const float resc = fast_exp2(M - M_use);  // 0 on the first round (M = -inf)
    L *= resc;
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] *= resc;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float wt = (s0 + 8 * j < S) ? fast_exp2(mv[j] - M_use) : 0.0f;
      L += wt * lv[j];
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] += wt * ov[j][i];
    }
    M = Mn;
  }
  if (d4 == 0) {
    red_m[sg] = M;
    red_l[sg] = L;
  }
  red_o[sg][d4] = acc;
  __syncthreads();
  if (sg != 0) return;
  float Mt = -INFINITY;
#pragma unroll
  for (int g8 = 0; g8 < 8; ++g8) Mt = fmaxf(Mt, red_m[g8]);
  const float Mt_use = (Mt == -INFINITY) ? 0.0f : Mt;
  float Lt = 0.0f;
  f32x4_t tot = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int g8 = 0; g8 < 8; ++g8) {
    const float wt = fast_exp2(red_m[g8] - Mt_use);  // 0 for a group without splits (-inf)
    Lt += wt * red_l[g8];
    const f32x4_t o = red_o[g8][d4];
#pragma unroll
    for (int i = 0; i < 4; ++i) tot[i] += wt * o[i];
  }
  const float inv = (Lt > 0.0f) ? 1.0f / Lt : 0.0f;
  const int r = c / p.g, hq = c % p.g;
  u32x2_t w;
  w[0] = E::pack2(tot[0] * inv, tot[1] * inv);
  w[1] = E::pack2(tot[2] * inv, tot[3] * inv);
  *reinterpret_cast<u32x2_t *>(p.out + (((size_t)b * p.m + r) * p.H + kvh * p.g + hq) * kRowBytes + d4 * 8) = w;
}

// Largest split count the default rule considers for batch * kv heads = pairs (any KV length): one
// round of workgroups, one workgroup per CU of the current device.
int flash_decode_max_default_splits(long long pairs) {
  const long long cus = device_compute_units();
  long long base = (cus + pairs - 1) / pairs;
  if (base < 8) base = 8;
  if (base > kMaxSplits) base = kMaxSplits;
  return (int)base;
}

// Split count that a simple model of the launch makes fastest.  Workgroups run one per CU in rounds
// of as many workgroups as the device has CUs; a CU of a full round streams 27.7 GB/s (all 256 of an
// MI355X together 7.1 TB/s, what its memory system gives a kernel that only reads), a CU of a thin
// round at most 32 GB/s (one workgroup keeps 32 KiB of loads in flight); a workgroup costs 3 us beyond
// its bytes, the combine launch 5 us.  Among the counts within 3 % of the best, one that fills its
// rounds exactly is preferred, else the smallest.  For the common shapes this is about one workgroup
// per CU (batch 16 x 8 kv heads -> 2 splits, batch 1 -> 32); for pair counts that do not divide a round
// it finds the count that fills the rounds.  Model / measured us on 256 CUs, bf16, cold: batch 1,
// n = 32768, 32 splits 26.9 / 26.2; batch 16, n = 4096, 2 splits 45.9 / 44.6; n = 8192: batch 12,
// 5 splits 68.6 / 68.6, batch 20, 3 splits 108.5 / 107.6, batch 40, 4 splits 209.3 / 206.8, batch 48,
// 2 splits 241.1 / 234.4 -- in a sweep of 38 shapes the count chosen is the fastest measured one or
// within 1.6 % of it.
static int default_splits_model(long long pairs, int nblocks, int cus) {
  int smax = flash_decode_max_default_splits(pairs);
  if (smax > nblocks) smax = nblocks;
  if (smax < 1) smax = 1;
  const double key_bytes = 2.0 * kRowBytes;  // K and V row of one kv head
  const double all_cus = 27.7e9 * cus;       // what the memory system gives all CUs together
  auto model = [&](int s) {
    const long long wgs = pairs * s;
    const long long full = wgs / cus, rest = wgs % cus;
    const double wg_bytes = key_bytes * kDecStepKeys * ((nblocks + s - 1) / s);
    double t = full * (wg_bytes / 27.7e9 + 3e-6);
    if (rest > 0) {
      double rate = all_cus / (double)rest;
      if (rate > 32e9) rate = 32e9;
      t += wg_bytes / rate + 3e-6;
    }
    return s > 1 ? t + 5e-6 : t;
  };
  double t_min = model(1);
  for (int s = 2; s <= smax; ++s) {
    const double t = model(s);
    if (t < t_min) t_min = t;
  }
  int first = 0;
  for (int s = 1; s <= smax; ++s) {
    if (model(s) > t_min * 1.03) continue;
    if (first == 0) first = s;
    if ((pairs * s) % cus == 0) return s;
  }
  return first;
}

// The model is evaluated a few hundred times per call; a decode loop asks for the same (pairs, key
// blocks) at every layer and for the next block count only every 128 tokens, so the last answers are
// kept per thread.
int flash_decode_default_splits(int batch, int n, int kv_head_num) {
  const long long pairs = (long long)batch * kv_head_num;
  const int nblocks = (n + kDecStepKeys - 1) / kDecStepKeys;
  const int cus = device_compute_units();
  struct Memo {
    long long pairs;
    int nblocks, cus, splits;
  };
  constexpr int kMemo = 8;
  static thread_local Memo memo[kMemo] = {};
  static thread_local unsigned next = 0;
  for (const Memo &e : memo)
    if (e.splits > 0 && e.pairs == pairs && e.nblocks == nblocks && e.cus == cus) return e.splits;
  const int s = default_splits_model(pairs, nblocks, cus);
  memo[next++ % kMemo] = Memo{pairs, nblocks, cus, s};
  return s;
}

int flash_decode_effective_splits(int num_splits, int n) {
  const int nblocks = (n + kDecStepKeys - 1) / kDecStepKeys;
  if (num_splits > nblocks) num_splits = nblocks;  // every split holds at least one block
  return num_splits < 1 ? 1 : num_splits;
}

size_t flash_decode_workspace_bytes(int batch, int m, int group_size, int kv_head_num,
                                    int num_splits) {
  (void)m;
  (void)group_size;
  if (num_splits <= 1) return 0;
  const size_t slots = (size_t)batch * kv_head_num * num_splits * kDecCols;
  return slots * (kHeadDim + 2) * sizeof(float);
}

static hipError_t launch_decode_impl(DecodeParams &p, void *workspace, int batch, int kv_head_num, int num_splits,
                                     int dt, bool fused, hipStream_t stream) {
  p.num_splits = flash_decode_effective_splits(num_splits, p.n);
  p.scale_log2e = 1.4426950408889634f / sqrtf((float)kHeadDim);
  const size_t slots = (size_t)batch * kv_head_num * p.num_splits * kDecCols;
  p.ws_o = static_cast<float *>(workspace);
  p.ws_ml = p.ws_o ? p.ws_o + slots * kHeadDim : nullptr;
  dim3 grid(p.num_splits, kv_head_num, batch);
  void (*kern)(DecodeParams) = (dt == kDtFloat16)
                                   ? (fused ? flash_decode_kernel<_Float16, true> : flash_decode_kernel<_Float16, false>)
                                   : (fused ? flash_decode_kernel<__bf16, true> : flash_decode_kernel<__bf16, false>);
  // kDecLdsPad bytes of dynamic LDS that nobody touches keep a second workgroup off the CU (two of
  // them would put 64 KiB of loads in flight again).  More than 64 KiB of LDS in total is an opt-in
  // per device and kernel.
  static std::atomic<uint64_t> attr_done[4] = {};
  const int which = (dt == kDtFloat16 ? 0 : 2) + (fused ? 1 : 0);
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const uint64_t bit = 1ull << (dev & 63);
  if (!(attr_done[which].load(std::memory_order_acquire) & bit)) {
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            kDecLdsPad);
    if (e != hipSuccess) return e;
    attr_done[which].fetch_or(bit, std::memory_order_release);
  }
  hipLaunchKernelGGL(kern, grid, dim3(kDecThreads), kDecLdsPad, stream, p);
  e = hipGetLastError();
  if (e != hipSuccess || p.num_splits == 1) return e;
  dim3 cgrid(p.rows, kv_head_num, batch);
  if (dt == kDtFloat16)
    hipLaunchKernelGGL(flash_decode_combine_kernel<_Float16>, cgrid, dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL(flash_decode_combine_kernel<__bf16>, cgrid, dim3(256), 0, stream, p);
  return hipGetLastError();
}

hipError_t launch_flash_decode(void *out, const void *q, const void *k, const void *v,
                               void *workspace, int batch, int m, int n, int offset,
                               int64_t kv_seq_stride, int group_size, int kv_head_num,
                               int num_splits, int dt, hipStream_t stream) {
  DecodeParams p = {};
  p.q = static_cast<const char *>(q);
  p.k = static_cast<const char *>(k);
  p.v = static_cast<const char *>(v);
  p.out = static_cast<char *>(out);
  p.batch = batch;
  p.m = m;
  p.n = n;
  p.offset = offset;
  p.kv_seq_stride = kv_seq_stride;
  p.g = group_size;
  p.Hkv = kv_head_num;
  p.H = group_size * kv_head_num;
  p.rows = m * group_size;
  return launch_decode_impl(p, workspace, batch, kv_head_num, num_splits, dt, false, stream);
}

// One decode step of one sequence with the rotary embedding and the cache append inside the decode
// kernel: rows [0, pos) of the caches are read, row pos is produced from in_k / in_v and written.
hipError_t launch_flash_decode_step(void *out, void *k_cache, void *v_cache, const void *freq_cis,
                                    const void *in_q, const void *in_k, const void *in_v, void *workspace,
                                    int pos, int group_size, int kv_head_num, int is_neox, int num_splits,
                                    int dt, hipStream_t stream) {
  DecodeParams p = {};
  p.q = static_cast<const char *>(in_q);
  p.k = static_cast<const char *>(k_cache);
  p.v = static_cast<const char *>(v_cache);
  p.out = static_cast<char *>(out);
  p.batch = 1;
  p.m = 1;
  p.n = pos + 1;
  p.offset = pos;
  p.kv_seq_stride = pos + 1;
  p.g = group_size;
  p.Hkv = kv_head_num;
  p.H = group_size * kv_head_num;
  p.rows = group_size;
  p.new_k = static_cast<const char *>(in_k);
  p.new_v = static_cast<const char *>(in_v);
  p.freq_row = static_cast<const float *>(freq_cis) + (size_t)pos * kHeadDim;
  p.fused_pos = pos;
  p.is_neox = is_neox ? 1 : 0;
  return launch_decode_impl(p, workspace, 1, kv_head_num, num_splits, dt, true, stream);
}

// ---------------------------------------------------------------------------
// Decode without any allocation: the split-KV partials live in a fixed array in device memory
// that is part of the library's code object (every GPU the library runs on holds its own copy
// until the process ends).  In host code the array's name is only a handle for
// hipGetSymbolAddress: the device address is looked up once per device and that pointer is what
// the kernels receive, exactly as they receive the caller's workspace in launch_flash_decode.
// Nothing in the buffer has to start at zero: every (sequence, kv head, split) slot that the
// combine kernel reads is written by the decode kernel of the same call.  All calls on one GPU
// share the array, so calls that overlap on one GPU (different streams) race.
// ---------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[kStaticDecodeScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
std::atomic<void *> g_scratch_ptr[kMaxDevices];
}  // namespace

hipError_t launch_flash_decode_static(void *out, const void *q, const void *k, const void *v,
                                      int batch, int n, int64_t kv_seq_stride, int group_size,
                                      int kv_head_num, int num_splits, int dt, hipStream_t stream) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  void *ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!ptr) {
    // first call on this device (which is current): each GPU has the array at its own address
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (!ptr) return hipErrorInvalidSymbol;
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);
  }
  return launch_flash_decode(out, q, k, v, ptr, batch, 1, n, n - 1, kv_seq_stride, group_size,
                             kv_head_num, num_splits, dt, stream);
}

}  // namespace llmhip
