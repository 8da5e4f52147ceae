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
// flash_prefill_kernel<T, NW, KB, NT>: NW waves share the K/V tiles of 16*NW*KB query rows.
// NW = 8, KB = 2 (256 rows, one workgroup per CU) once there are about 1.5 such workgroups per CU;
// NW = 4, KB = 2 (128 rows, two workgroups per CU) below that; NW = 8, KB = 1 (128 rows, two waves
// per row block, each taking one 32-key half of every tile) up to two 128-row workgroups per CU;
// NW = 4, KB = 1 (64 rows, paired waves, two workgroups per CU) up to about 1.2 per CU.  NT: the
// tile loads are non-temporal (chunks whose K/V tiles only one workgroup reads).
// Tiles travel global -> LDS without VGPR staging (global_load_lds_dwordx4), spread over the MFMA
// stream in the 8-wave kernels, issued beside the first MFMAs of a phase in the 4-wave ones.  The loop is software pipelined inside a wave: the MFMAs of S(j+1) are issued beside the
// softmax of tile j (the first ones beside the row-maximum chain, the rest, together with the
// MFMAs of P(j).V(j), beside the exponentials), so K is fetched one tile ahead of V.
// Every LDS fragment address is a loop-invariant register plus an immediate, and a
// tile load is a scalar base plus a loop-invariant lane offset: the loop spends its
// vector ALU instructions on the softmax only.
//
// A chunk of few query rows over a long cache (chunked prefill) has its key range split over
// workgroups: each leaves an fp32 partial (reference maximum, sum, unnormalised O) and
// prefill_combine_kernel (or, for few rows and many ranges, prefill_combine_wide_kernel) folds
// them; a chunk shorter than a tile packs the query heads of a kv head into the rows of one tile.  plan_prefill decides all of this from the shape and the
// device's CU count.
#include <atomic>

#include "common.hpp"
#include "kernels.hpp"

namespace LLMHIP_NS {

constexpr int kTileN = 64;                      // keys per LDS tile
constexpr int kTileBytes = kTileN * kRowBytes;  // 16 KiB
constexpr float kLazyLog2 = 8.0f;                // rescale threshold, log2 units
constexpr int kMaxPrefillSplits = 128;           // key ranges per call

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
  // Key-range split (chunked prefill: few query rows over a long cache).  Split s covers
  // keys [s*chunk, (s+1)*chunk); with more than one split every workgroup leaves an fp32 partial
  // (reference maximum, sum, unnormalised O) that prefill_combine_kernel folds.
  int num_splits, chunk;  // chunk: multiple of 64 keys
  // Split mode only: the rows of a tile are (token, head-in-group) pairs of ONE kv head, packed
  // token-major (row index = token * g + head % g), so a chunk shorter than a tile reads K and V of
  // its kv head once for all g query heads.
  int pack;
  float *ws_o;            // [split][m][H][128]
  float *ws_ml;           // [split][m][H][2]
#ifdef LLMHIP_BENCH
  // measurement library only: workgroup 0 stores {shader-clock ticks, 100 MHz ticks} of its lifetime
  unsigned long long *clock_probe;
#endif
};

// blockIdx -> (query tile, head, key range).  Workgroup ids are dealt round-robin to the 8
// XCDs by the hardware; heads that share a kv head are kept on the same XCD(s)
// so that its K/V stay in that XCD's L2, and within an XCD the heaviest (last)
// query tiles are issued first.  Key ranges (split mode) are the slowest index of an XCD's
// list, so that every XCD gets the same number of workgroups whatever the head count.
__device__ __forceinline__ bool prefill_schedule(const PrefillParams &p, int bid, int &tile,
                                                 int &head, int &split) {
  const int T = p.num_q_tiles;
  if (p.pack) {  // packed rows: items are (key range, tile, kv head)
    const int per = T * p.Hkv;
    if (bid >= per * p.num_splits) return false;
    split = bid / per;
    const int rem = bid % per;
    tile = T - 1 - rem / p.Hkv;
    head = (rem % p.Hkv) * p.g;  // first query head of the kv head
    return true;
  }
  if (p.sched_mode == 1) {
    const int X = p.sched_a;
    const int xcd = bid & 7, slot = bid >> 3;
    const int kvh = xcd / X, sub = xcd % X;
    const int idx = slot * X + sub, per = p.g * T;
    if (idx >= per * p.num_splits) return false;
    split = idx / per;
    const int rem = idx % per;
    tile = T - 1 - rem / p.g;
    head = kvh * p.g + rem % p.g;
    return true;
  }
  if (p.sched_mode == 2) {
    const int hp = p.sched_a;
    const int xcd = bid & 7, slot = bid >> 3, per = hp * T;
    if (slot >= per * p.num_splits) return false;
    split = slot / per;
    const int rem = slot % per;
    tile = T - 1 - rem / hp;
    head = xcd * hp + rem % hp;
    return true;
  }
  const int per = T * p.H;
  if (bid >= per * p.num_splits) return false;
  split = bid / per;
  const int rem = bid % per;
  tile = T - 1 - rem / p.H;
  head = rem % p.H;
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

// LDS visibility + workgroup barrier that does not drain outstanding global loads.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// State of one wave: 32 query rows (one per lane pair), fp32 O^T accumulators.  KB = 32-key blocks
// of every 64-key tile that the wave works on: 2 normally; 1 when two waves share the rows and
// each takes one half of every tile (short sequences: halves the serial MFMA chain of a wave).
template <typename T, int KB = 2> struct WaveAttn {
  using E = Elem<T>;
  f32x16_t o[4];       // O^T: d block x (16 d rows of this lane)
  u32x4_t pf[KB][2];   // P^T packed as B operand: key block x k-step
  u32x4_t qf[8];       // Q^T fragments (B operand), loaded once
  float m_run, l_run;  // running max (raw score units) and sum of this lane's keys
  int lane, l32, hh, g16, li;
  int k_addr[8];  // LDS byte offset of this lane's K fragment kk in tile slot 0, key block 0
  int v_addr[4];  // same for the V^T fragment of d block d (k-step 0, low half)

  // kb0: first 32-key block of a tile this wave works on (0, or 1 for the second wave of a pair)
  __device__ __forceinline__ void init(int lane_, int v_region, int kb0 = 0) {
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
    // Every other fragment address of the loop is one of these plus a compile-time constant
    // that fits the 16-bit offset field of the LDS instructions; the empty asm keeps the
    // compiler from recomputing them (it otherwise spends ~50 VALU instructions per tile).
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) {
      k_addr[kk] = k_swizzle_off(l32, 2 * kk + hh) + kb0 * 32 * kRowBytes;
      asm volatile("" : "+v"(k_addr[kk]));
    }
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const int gran = d * 4 + (g16 & 1) * 2 + ((li & 3) >> 1);
      v_addr[d] = v_region + v_swizzle_off(4 * hh + (li >> 2), gran) + (li & 1) * 8 + kb0 * 32 * kRowBytes;
      asm volatile("" : "+v"(v_addr[d]));
    }
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
  // S^T = K Q^T for the wave's keys of the K tile at byte offset `koff` of the LDS segment.
  // The fragments of step kk+1 are requested before the MFMAs of step kk.  hook(i) runs
  // after MFMA i (0..8*KB-1): the callers spread their global loads over the MFMA stream with it.
  template <int KK0 = 0, int KK1 = 8, typename Hook = NoHook>
  __device__ __forceinline__ void qk(const char *lds, int koff, f32x16_t (&s)[KB], Hook hook = Hook()) {
#pragma unroll
    for (int kk = KK0; kk < KK1; ++kk) {
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) {
        const u32x4_t kf = lds_read_b128(lds, k_addr[kk] + koff + kb * 32 * kRowBytes);
        if (kk == 0) {
          f32x16_t z;
#pragma unroll
          for (int i = 0; i < 16; ++i) z[i] = 0.0f;
          s[kb] = E::mfma32(kf, qf[kk], z);
        } else {
          s[kb] = E::mfma32(kf, qf[kk], s[kb]);
        }
        hook(kk * KB + kb);
      }
    }
  }

  // O^T += V^T P^T over the V tile at byte offset `voff` past the start of the V region.
  // Lane (d = 32*dblk + l32, hh): element e of k-step (kb, ks2) is the key
  // 32*kb + 16*ks2 + 8*(e/4) + 4*hh + e%4 -- the key P's element e carries.
  template <typename Hook = NoHook>
  __device__ __forceinline__ void pv(const char *lds, int voff, Hook hook = Hook()) {
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int ks2 = 0; ks2 < 2; ++ks2) {
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const int c = voff + (kb * 32 + ks2 * 16) * kRowBytes;
          const u32x2_t lo = lds_read_tr16(lds, v_addr[d] + c);
          const u32x2_t hi = lds_read_tr16(lds, v_addr[d] + c + 8 * kRowBytes);
          const u32x4_t vf = {lo[0], lo[1], hi[0], hi[1]};
          o[d] = E::mfma32(vf, pf[kb][ks2], o[d]);
          hook((kb * 2 + ks2) * 4 + d);
        }
      }
  }

  // Causal / length mask of one tile of scores (only called for tiles that can be cut); key0 =
  // first key of the wave's part of the tile.
  __device__ __forceinline__ void mask(f32x16_t (&s)[KB], int key0, int qrow, int offset, int n) {
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int key = key0 + kb * 32 + 8 * (i >> 2) + 4 * hh + (i & 3);
        if (key > qrow + offset || key >= n) s[kb][i] = -INFINITY;
      }
  }

  // P = exp2(s*c + neg_ms) rounded to T and packed as the B operand; returns this lane's sum
  // of the rounded values.
  __device__ __forceinline__ float probabilities(const f32x16_t (&s)[KB], float c, float neg_ms) {
    float ps0 = 0.0f, ps1 = 0.0f;
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int ks2 = 0; ks2 < 2; ++ks2) {
        u32x4_t w;
#pragma unroll
        for (int e2 = 0; e2 < 4; ++e2) {
          const float e0 = fast_exp2(__builtin_fmaf(s[kb][8 * ks2 + 2 * e2], c, neg_ms));
          const float e1 = fast_exp2(__builtin_fmaf(s[kb][8 * ks2 + 2 * e2 + 1], c, neg_ms));
          w[e2] = E::pack2(e0, e1);
          // l sums the ROUNDED probabilities, the values P.V really used: for rows that see few
          // keys the rounding errors of numerator and denominator then cancel.  (In a design that
          // separates MFMA and softmax phases these dot instructions are costly -- they queue
          // behind the MFMAs of every wave on the SIMD: a softmax pass beside an MFMA-issuing wave
          // takes 1690 cycles with them, 1070 with plain adds -- in this interleaved loop the
          // two versions time the same.)
          if (e2 & 1)
            ps1 = dot2_ones<T>(w[e2], ps1);
          else
            ps0 = dot2_ones<T>(w[e2], ps0);
        }
        pf[kb][ks2] = w;
      }
    return ps0 + ps1;
  }

  // First half of the online softmax of one tile of (already masked) scores: row maxima and,
  // rarely, the move of the reference.  m_run is the reference maximum used in the exponent,
  // in raw score units.  It moves only when a row maximum exceeds it by more than kLazyLog2
  // in log2 units (probabilities then stay below 2^kLazyLog2, harmless in fp32 sums and in
  // the 16-bit P operand); a -inf reference always moves.  O and l are rescaled only then,
  // which after the first tiles is rare.  Returns the additive term of the exponent.
  __device__ __forceinline__ float row_max(const f32x16_t (&s)[KB], float scale_log2e) {
    float m0 = -INFINITY, m1 = -INFINITY;  // two chains: half the dependent latency
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      if (KB == 2) {
        m0 = fmaxf(m0, s[0][i]);
        m1 = fmaxf(m1, s[KB - 1][i]);
      } else if (i & 1) {
        m1 = fmaxf(m1, s[0][i]);
      } else {
        m0 = fmaxf(m0, s[0][i]);
      }
    }
    const float mloc = pair_max(fmaxf(m0, m1));
    const bool move = mloc > m_run + kLazyLog2 / scale_log2e;
    if (__builtin_amdgcn_ballot_w64(move) != 0) {
      const float m_new = move ? mloc : m_run;
      const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
      const float alpha = move ? fast_exp2((m_run - m_use) * scale_log2e) : 1.0f;
      l_run *= alpha;
#pragma unroll
      for (int d = 0; d < 4; ++d)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[d][i] *= alpha;
      m_run = m_new;
    }
    return -((m_run == -INFINITY) ? 0.0f : m_run) * scale_log2e;
  }

  // Two waves that shared the rows (KB == 1): the second writes its state to LDS lane by lane
  // (66 floats per lane, stride 64 floats between a lane's values: conflict-free), the first folds
  // it into its own.  The reference maxima are uniform over a lane pair in both waves.
  __device__ __forceinline__ void export_state(float *lds_pair) const {
#pragma unroll
    for (int d = 0; d < 4; ++d)
#pragma unroll
      for (int i = 0; i < 16; ++i) lds_pair[(d * 16 + i) * 64 + lane] = o[d][i];
    lds_pair[64 * 64 + lane] = m_run;
    lds_pair[65 * 64 + lane] = l_run;
  }
  __device__ __forceinline__ void import_state(const float *lds_pair, float scale_log2e) {
    const float m_b = lds_pair[64 * 64 + lane], l_b = lds_pair[65 * 64 + lane];
    const float m_new = fmaxf(m_run, m_b);
    const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
    const float fa = fast_exp2((m_run - m_use) * scale_log2e), fb = fast_exp2((m_b - m_use) * scale_log2e);
    l_run = l_run * fa + l_b * fb;
#pragma unroll
    for (int d = 0; d < 4; ++d)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[d][i] = o[d][i] * fa + lds_pair[(d * 16 + i) * 64 + lane] * fb;
    m_run = m_new;
  }

  // out[row][head][0..127] = O^T / l, rounded once.  The lane layout of O^T (a lane holds 4
  // contiguous dims of one row at 16 places) would make every store instruction touch 32
  // rows with 16 bytes each; the tile goes through this wave's private 8 KiB of LDS instead
  // (16-byte granule XOR row%16: conflict-free both ways) and leaves as whole 256-byte rows,
  // 16 lanes per row.  lds_wave: this wave's region; out_blk: &out[first row of the wave][head];
  // rows_valid: how many of the wave's 32 rows exist.
  __device__ __forceinline__ void store(char *lds_wave, char *out_blk, size_t row_bytes, int rows_valid) {
    const float l_tot = pair_sum(l_run);
    const float inv = (l_tot > 0.0f) ? 1.0f / l_tot : 0.0f;
#pragma unroll
    for (int d = 0; d < 4; ++d)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        u32x2_t w;
        w[0] = E::pack2(o[d][4 * i4] * inv, o[d][4 * i4 + 1] * inv);
        w[1] = E::pack2(o[d][4 * i4 + 2] * inv, o[d][4 * i4 + 3] * inv);
        const int gran = 4 * d + i4;  // 16-byte granule of dims 32d + 8*i4 .. +7; hh picks its half
        *reinterpret_cast<u32x2_t *>(lds_wave + l32 * kRowBytes + ((gran ^ (l32 & 15)) << 4) + hh * 8) = w;
      }
    __builtin_amdgcn_wave_barrier();  // wave-private region: LDS ops of one wave complete in order
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      const int r = 4 * t + g16;
      const u32x4_t v = lds_read_b128(lds_wave, r * kRowBytes + ((li ^ (r & 15)) << 4));
      if (r < rows_valid) *reinterpret_cast<u32x4_t *>(out_blk + (size_t)r * row_bytes + li * 16) = v;
    }
  }
};

// Partial result of one key range (see PrefillParams::num_splits): this lane's row gets its
// unnormalised O^T as fp32, and (reference maximum in raw score units, sum) once per lane pair.
template <typename T, int KB>
__device__ __forceinline__ void store_partial(const WaveAttn<T, KB> &w, float *o_row, float *ml_row, bool row_valid) {
  const float l_tot = pair_sum(w.l_run);
  if (!row_valid) return;
#pragma unroll
  for (int d = 0; d < 4; ++d)
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      const f32x4_t v = {w.o[d][4 * i4], w.o[d][4 * i4 + 1], w.o[d][4 * i4 + 2], w.o[d][4 * i4 + 3]};
      *reinterpret_cast<f32x4_t *>(o_row + 32 * d + 8 * i4 + 4 * w.hh) = v;
    }
  if (w.hh == 0) {
    ml_row[0] = w.m_run;
    ml_row[1] = l_tot;
  }
}

// Global -> LDS tile loader without VGPR staging (global_load_lds_dwordx4: lane l's 16
// bytes land at the wave-uniform LDS address in M0 + 16*l).  One wave instruction fills four
// 256-byte rows; the XOR swizzles are realised on the global side: the lane that owns
// physical granule pg of row r fetches the logical granule that belongs there.  A tile
// is 16 instructions, dealt to the NW waves; `slot` s of wave w covers rows
// 4*(s*NW + w) .. +3.  The global address is a scalar tile base plus a per-lane 32-bit
// offset that never changes (except in a ragged last tile, whose rows are clamped to n-1),
// so a load costs no vector ALU work.  The loads are issued from inline asm: the compiler
// would order every later LDS read behind a transfer it knows about (s_waitcnt vmcnt(0)).
// Completion is waited for explicitly before the barrier that publishes a stage.
template <int NW, bool NT> struct DirectLoader {
  static constexpr int kSlots = 16 / NW;  // instructions per wave per tile
  int n, row_bytes;
  uint32_t lds_row0;          // LDS byte offset of row 4*wave (wave-uniform)
  int row[kSlots];            // tile row this lane fetches in slot s
  uint32_t lane_k[kSlots];    // logical granule byte offset within the row, K swizzle
  uint32_t lane_v[kSlots];    // same, V swizzle

  __device__ __forceinline__ void init(int wave, int lane, int row_bytes_, int n_) {
    n = n_;
    row_bytes = row_bytes_;
    lds_row0 = __builtin_amdgcn_readfirstlane(4 * wave * kRowBytes);
#pragma unroll
    for (int s = 0; s < kSlots; ++s) {
      const int r = 4 * (s * NW + wave) + (lane >> 4), pg = lane & 15;
      row[s] = r;
      lane_k[s] = (pg ^ (r & 15)) << 4;
      lane_v[s] = ((((pg >> 2) ^ (r & 3)) << 2) | (pg & 3)) << 4;
      asm volatile("" : "+v"(row[s]), "+v"(lane_k[s]), "+v"(lane_v[s]));
    }
  }
  // NT: the tile is read by this workgroup only (a packed chunk of one tile per kv head over a long
  // cache): non-temporal, like the decode kernel's loads (4 tokens over 131072 keys: 106 -> 93 us);
  // tiles that several workgroups read stay ordinary loads (non-temporal costs those 3-10 %).
  static __device__ __forceinline__ void dma(const char *tile_base, uint32_t lane_off, uint32_t lds_addr) {
    if (NT)
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt"
                   :
                   : "v"(lane_off), "s"(tile_base), "s"(lds_addr)
                   : "m0");
    else
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                   :
                   : "v"(lane_off), "s"(tile_base), "s"(lds_addr)
                   : "m0");
  }
  // t: key tile; lds_tile: LDS byte offset of the destination tile
  template <bool IS_V>
  __device__ __forceinline__ void issue(const char *base, int t, uint32_t lds_tile, int s) const {
    const char *tile_base = base + (size_t)t * kTileN * row_bytes;
    const uint32_t dst = lds_tile + lds_row0 + s * NW * 4 * kRowBytes;
    // rows past n-1 (ragged last tile) are clamped to row n-1: nothing beyond the caller's n
    // rows is read and the stale rows hold finite values; branch-free, two VALU instructions
    const int r = min(row[s], n - 1 - t * kTileN);
    dma(tile_base, r * row_bytes + (IS_V ? lane_v[s] : lane_k[s]), dst);
  }
  static __device__ __forceinline__ void wait_all() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
};

// ---------------------------------------------------------------------------
// NW waves, 32*NW query rows, two LDS stages of SUB 64-key tiles, one barrier per stage.
// Every wave runs S(j+1) = K Q^T, the softmax of tile j and P(j).V(j) as one instruction
// stream (the compiler interleaves the softmax VALU work with the MFMAs); the tile loads
// are spread over that stream.  NW = 4: two workgroups per CU (small problems); NW = 8:
// one workgroup per CU, K/V tiles shared by 256 rows.  KB = 1: every row block worked on by two
// waves that each take one 32-key half of every tile and are merged through LDS at the end (NW = 8:
// 128 rows; NW = 4: 64 rows, two workgroups per CU) -- for sequences so short that there is at most
// about one 128-row workgroup per CU, where the serial MFMA chain of a wave is what the launch
// waits for.
// ---------------------------------------------------------------------------
template <typename T, int NW, int KB, bool NT>
__global__ __launch_bounds__(64 * NW, NW == 4 ? 2 : 1) void flash_prefill_kernel(PrefillParams p) {
  // SUB tiles of 64 keys per stage and per barrier: with one workgroup per CU (NW = 8) a stage
  // holds 128 keys, which halves the number of times the waves are forced in step.
  // LDS: K tiles of both stages [2*SUB][16 KiB], then the V tiles likewise; tile t sits in
  // slot t % (2*SUB) of each region, so every fragment address is a per-lane register plus a
  // constant below 64 KiB.
  constexpr int BM = 16 * NW * KB, RB = BM / 32, PER = 16 / NW, SUB = NW == 8 ? 2 : 1, NSLOT = 2 * SUB;
  constexpr int kVRegion = NSLOT * kTileBytes;
  constexpr int kWaveKeys = 32 * KB;  // keys of a tile per wave
  constexpr int kSplitKK = 3;  // k-steps of S(j+1) issued beside the row-maximum chain
  extern __shared__ __attribute__((aligned(16))) char lds[];
  int tile, head, split;
  if (!prefill_schedule(p, blockIdx.x, tile, head, split)) return;
#ifdef LLMHIP_BENCH
  unsigned long long clk0 = 0, ref0 = 0;
  if (p.clock_probe) {
    clk0 = __builtin_amdgcn_s_memtime();
    ref0 = __builtin_amdgcn_s_memrealtime();
  }
#endif

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int kvh = head / p.g;
  // Rows of the tile.  Unpacked: rows are tokens of one head.  Packed: row index i stands for token
  // i / g of head kvh*g + i % g; `rows` counts them.  Everything below works on tokens: qtok is this
  // lane's token, tok_lo / tok_hi the first / last token of the wave's 32 rows.
  const int rows = p.pack ? p.m * p.g : p.m;
  const int row0 = tile * BM;
  const int rows_end = min(rows, row0 + BM);
  const int rb = wave % RB, kpar = wave / RB;  // row block; which half of every tile (KB == 1)
  const int kw0 = (KB == 1) ? 32 * kpar : 0;   // first key of the wave's part of a tile
  const int qblk0 = row0 + rb * 32;
  const int l32_ = lane & 31;
  const int qidx = min(qblk0 + l32_, rows - 1);
  const bool row_valid = qblk0 + l32_ < rows;
  const int qtok = p.pack ? qidx / p.g : qidx;
  const int qhead = p.pack ? head + qidx % p.g : head;
  const int tok_lo = p.pack ? qblk0 / p.g : qblk0;
  const int tok_hi = p.pack ? (min(qblk0 + 31, rows - 1)) / p.g : min(qblk0 + 31, rows - 1);
  const int tile_tok_end = p.pack ? (rows_end - 1) / p.g + 1 : rows_end;  // one past the tile's last token
  // This workgroup's key range, seen as a cache of its own: rows [k_lo, k_lo + n_) with the causal
  // offset shifted accordingly (negative when the range starts past a row's last visible key).
  const int k_lo = split * p.chunk;
  const int n_ = min(p.n - k_lo, p.chunk);
  const int offset_ = p.offset - k_lo;
  const int n_vis = min(n_, tile_tok_end + offset_);  // keys any row of this tile can see
  const int J = (n_vis + kTileN - 1) / kTileN;        // 64-key tiles of the workgroup
  const size_t q_row_bytes = (size_t)p.H * kRowBytes;
  const int kv_row_bytes = p.Hkv * kRowBytes;
  const char *kbase = p.k + (size_t)k_lo * kv_row_bytes + (size_t)kvh * kRowBytes;
  const char *vbase = p.v + (size_t)k_lo * kv_row_bytes + (size_t)kvh * kRowBytes;

  WaveAttn<T, KB> w;
  w.init(lane, kVRegion, (KB == 1) ? kpar : 0);
  // tiles in which this wave's keys hold at least one visible key
  const int Jw = (qblk0 < rows) ? max(0, min(J, (min(n_, tok_hi + offset_ + 1) - kw0 + kTileN - 1) / kTileN)) : 0;
  float *part_o = nullptr, *part_ml = nullptr;
  if (p.num_splits > 1) {
    const size_t slot = ((size_t)split * p.m + qtok) * p.H + qhead;
    part_o = p.ws_o + slot * kHeadDim;
    part_ml = p.ws_ml + slot * 2;
    if (J <= 0) {  // workgroup-uniform: no row of this tile sees a key of this range
      store_partial(w, part_o, part_ml, row_valid);
      return;
    }
  }
  w.load_q(p.q + (size_t)qtok * q_row_bytes + (size_t)qhead * kRowBytes);

  DirectLoader<NW, NT> ld;
  ld.init(wave, lane, kv_row_bytes, n_);
  // K runs one tile ahead of V: S(j+1) = K(j+1) Q^T is issued together with the softmax of
  // tile j, so K tile t is fetched SUB+1 iterations and V tile t SUB iterations before use.
#pragma unroll
  for (int u = 0; u <= SUB; ++u)
#pragma unroll
    for (int sl = 0; sl < PER; ++sl) {
      ld.template issue<false>(kbase, min(u, J - 1), (u % NSLOT) * kTileBytes, sl);
      if (u < SUB) ld.template issue<true>(vbase, min(u, J - 1), kVRegion + u * kTileBytes, sl);
    }
  w.pin_q();  // the Q fragments are in registers from here on
  ld.wait_all();
  lds_barrier();

  f32x16_t sa[KB], sb[KB];  // scores of the current / the next tile, roles alternate
  if (Jw > 0) w.qk(lds, 0, sa);

  auto tile_step = [&](int j, int slot, f32x16_t (&s_cur)[KB], f32x16_t (&s_nxt)[KB]) {
    const int kslot = (slot + SUB + 1) % NSLOT, vslot = (slot + SUB) % NSLOT;  // fetched now
    const int jk = min(j + SUB + 1, J - 1), jv = min(j + SUB, J - 1);
    if (j < Jw) {
      const int key0 = j * kTileN + kw0;
      if ((key0 + kWaveKeys - 1 > tok_lo + offset_) || (key0 + kWaveKeys > n_))
        w.mask(s_cur, key0, qtok, offset_, n_);
      // In the 8-wave kernel a burst of loads would stall every wave behind the texture addresser's
      // queue: one load every 8 * KB / PER MFMAs instead.  The 4-wave kernels run where a step is
      // short against a memory round trip, and issue a phase's loads beside its first MFMAs
      // (S=2560: 61.0 -> 59.1 us, S=3072: 76.3 -> 75.0 us; the 8-wave kernel loses 0.7 % that way).
      // (Paired waves, KB == 1, run short sequences, where a step is shorter than a memory round
      // trip: there all loads of a step go out with its first MFMAs.)
      auto k_hook = [&](int i) {
#pragma unroll
        for (int r = 0; r < PER; ++r) {
          if (KB == 1) {
            if (i == r) ld.template issue<false>(kbase, jk, kslot * kTileBytes, r);
            if (i == PER + r) ld.template issue<true>(vbase, jv, kVRegion + vslot * kTileBytes, r);
          } else if (i == (NW == 4 ? r : (8 * KB / PER) * r + 1)) {
            ld.template issue<false>(kbase, jk, kslot * kTileBytes, r);
          }
        }
      };
      // The MFMAs of S(j+1) overlap the softmax of tile j: the first ones run beside the row
      // maximum chain, the rest -- and the MFMAs of P.V -- beside the exponentials.  (For the
      // wave's last tile the result is not used: one surplus pass instead of a branch that
      // would separate these MFMAs from the instructions they overlap with.)
      const int koff = ((slot + 1) % NSLOT) * kTileBytes;
      w.template qk<0, kSplitKK>(lds, koff, s_nxt, k_hook);
      const float neg_ms = w.row_max(s_cur, p.scale_log2e);
      w.template qk<kSplitKK, 8>(lds, koff, s_nxt, k_hook);
      w.l_run += w.probabilities(s_cur, p.scale_log2e, neg_ms);
      w.pv(lds, slot * kTileBytes, [&](int i) {
#pragma unroll
        for (int r = 0; r < PER; ++r)
          if (KB != 1 && i == (NW == 4 ? r : (8 * KB / PER) * r + 1))
            ld.template issue<true>(vbase, jv, kVRegion + vslot * kTileBytes, r);
      });
    } else {
#pragma unroll
      for (int sl = 0; sl < PER; ++sl) {
        ld.template issue<false>(kbase, jk, kslot * kTileBytes, sl);
        ld.template issue<true>(vbase, jv, kVRegion + vslot * kTileBytes, sl);
      }
    }
  };

  for (int jb = 0; jb < J; jb += NSLOT) {
#pragma unroll
    for (int st = 0; st < 2; ++st) {
#pragma unroll
      for (int u = 0; u < SUB; ++u) {
        const int slot = st * SUB + u;  // compile-time after unrolling
        if (slot % 2 == 0)
          tile_step(jb + slot, slot, sa, sb);
        else
          tile_step(jb + slot, slot, sb, sa);
      }
      ld.wait_all();
      lds_barrier();
      if (st == 0 && jb + SUB >= J) break;  // workgroup-uniform: the second stage holds nothing
    }
  }
  // every wave is past the last barrier of the loop: nobody reads the K/V tiles any more
  if (KB == 1) {
    // the two waves of a row block: the second hands its state over (behind the RB output
    // staging regions of 8 KiB), the first folds it in and stores
    float *pair = reinterpret_cast<float *>(lds + RB * 32 * kRowBytes) + (size_t)rb * 66 * 64;
    if (kpar == 1) w.export_state(pair);
    __syncthreads();
    if (kpar == 1) return;
    w.import_state(pair, p.scale_log2e);
  }
  if (p.num_splits > 1)  // (packed rows exist in split mode only)
    store_partial(w, part_o, part_ml, row_valid);
  else
    w.store(lds + rb * 32 * kRowBytes, p.out + (size_t)qblk0 * q_row_bytes + (size_t)head * kRowBytes,
            q_row_bytes, p.m - qblk0);
#ifdef LLMHIP_BENCH
  if (p.clock_probe && blockIdx.x == 0 && tid == 0) {
    p.clock_probe[0] = __builtin_amdgcn_s_memtime() - clk0;
    p.clock_probe[1] = __builtin_amdgcn_s_memrealtime() - ref0;
  }
#endif
}

// Folds the key-range partials of the output rows with the log-sum-exp rule.  256 threads handle 8
// (row, head) slots, 32 threads (4 dims each) per slot; grid = ceil(m * H / 8).
template <typename T>
__global__ __launch_bounds__(256) void prefill_combine_kernel(PrefillParams p) {
  using E = Elem<T>;
  const size_t stride = (size_t)p.m * p.H;  // slots per split
  const size_t slot = (size_t)blockIdx.x * 8 + (threadIdx.x >> 5);
  const int d4 = threadIdx.x & 31;
  if (slot >= stride) return;
  // One pass, four key ranges per round: all loads of a round are issued before any is used, and the
  // running reference maximum moves between rounds (a pass for the maximum first would be one memory
  // round trip per key range).
  const int S = p.num_splits;
  float M = -INFINITY, L = 0.0f;
  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
  for (int s0 = 0; s0 < S; s0 += 4) {
    float mv[4], lv[4];
    f32x4_t ov[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const size_t at = (size_t)min(s0 + j, S - 1) * stride + slot;
      mv[j] = p.ws_ml[at * 2];
      lv[j] = p.ws_ml[at * 2 + 1];
      ov[j] = *reinterpret_cast<const f32x4_t *>(p.ws_o + at * kHeadDim + 4 * d4);
    }
    float Mn = M;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (s0 + j < S) Mn = fmaxf(Mn, mv[j]);
    const float M_use = (Mn == -INFINITY) ? 0.0f : Mn;
    const float resc = fast_exp2((M - M_use) * p.scale_log2e);  // 0 on the first round (M = -inf)
    L *= resc;
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] *= resc;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      // exp2(-inf) = 0 for an empty range
      const float wt = (s0 + j < S) ? fast_exp2((mv[j] - M_use) * p.scale_log2e) : 0.0f;
      L += wt * lv[j];
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] += wt * ov[j][i];
    }
    M = Mn;
  }
  const float inv = (L > 0.0f) ? 1.0f / L : 0.0f;
  u32x2_t w;
  w[0] = E::pack2(acc[0] * inv, acc[1] * inv);
  w[1] = E::pack2(acc[2] * inv, acc[3] * inv);
  *reinterpret_cast<u32x2_t *>(p.out + slot * kRowBytes + d4 * 8) = w;
}

// The same fold for few output rows and many key ranges (a short chunk over a very long cache): one
// (row, head) slot per workgroup, its key ranges dealt to 8 groups of 32 threads (group sg takes ranges
// sg, sg + 8, ..., four per round), the groups merged through LDS -- the slots alone would not fill
// the chip and every thread would walk all ranges.  grid = m * H.
template <typename T>
__global__ __launch_bounds__(256) void prefill_combine_wide_kernel(PrefillParams p) {
  using E = Elem<T>;
  __shared__ float red_m[8], red_l[8];
  __shared__ f32x4_t red_o[8][32];
  const size_t stride = (size_t)p.m * p.H, slot = blockIdx.x;
  const int sg = threadIdx.x >> 5, d4 = threadIdx.x & 31;
  const int S = p.num_splits;
  float M = -INFINITY, L = 0.0f;
  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
  for (int s0 = sg; s0 < S; s0 += 32) {
    float mv[4], lv[4];
    f32x4_t ov[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const size_t at = (size_t)min(s0 + 8 * j, S - 1) * stride + slot;
      mv[j] = p.ws_ml[at * 2];
      lv[j] = p.ws_ml[at * 2 + 1];
      ov[j] = *reinterpret_cast<const f32x4_t *>(p.ws_o + at * kHeadDim + 4 * d4);
    }
    float Mn = M;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (s0 + 8 * j < S) Mn = fmaxf(Mn, mv[j]);
    const float M_use = (Mn == -INFINITY) ? 0.0f : Mn;
    const float resc = fast_exp2((M - M_use) * p.scale_log2e);
    L *= resc;
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] *= resc;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float wt = (s0 + 8 * j < S) ? fast_exp2((mv[j] - M_use) * p.scale_log2e) : 0.0f;
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
    const float wt = fast_exp2((red_m[g8] - Mt_use) * p.scale_log2e);  // 0 for a group without ranges (-inf)
    Lt += wt * red_l[g8];
    const f32x4_t o = red_o[g8][d4];
#pragma unroll
    for (int i = 0; i < 4; ++i) tot[i] += wt * o[i];
  }
  const float inv = (Lt > 0.0f) ? 1.0f / Lt : 0.0f;
  u32x2_t w;
  w[0] = E::pack2(tot[0] * inv, tot[1] * inv);
  w[1] = E::pack2(tot[2] * inv, tot[3] * inv);
  *reinterpret_cast<u32x2_t *>(p.out + slot * kRowBytes + d4 * 8) = w;
}

template <typename T, int NW, int KB = 2>
static hipError_t launch_prefill_t(const PrefillParams &p0, hipStream_t stream) {
  PrefillParams p = p0;
  constexpr int BM = 16 * NW * KB;
  constexpr int NT = 64 * NW;
  p.num_q_tiles = (p.m + BM - 1) / BM;
  if (p.pack) p.num_q_tiles = (p.m * p.g + BM - 1) / BM;
  const int T_ = p.num_q_tiles;
  int grid;
  const int S_ = p.num_splits;
  if (p.pack) {
    p.sched_mode = 0;
    p.sched_a = 0;
    grid = T_ * p.Hkv * S_;
  } else if (p.Hkv <= 8 && 8 % p.Hkv == 0) {
    p.sched_mode = 1;
    p.sched_a = 8 / p.Hkv;
    const int per_kvh = p.g * T_ * S_;
    grid = 8 * ((per_kvh + p.sched_a - 1) / p.sched_a);
  } else if (p.Hkv % 8 == 0) {
    p.sched_mode = 2;
    p.sched_a = (p.Hkv / 8) * p.g;
    grid = 8 * p.sched_a * T_ * S_;
  } else {
    p.sched_mode = 0;
    p.sched_a = 0;
    grid = T_ * p.H * S_;
  }
  const size_t lds_bytes = (NW == 8 ? 2 : 1) * 4 * kTileBytes;
  // packed rows, one tile per kv head: every K/V tile is read by one workgroup only (KB == 2 there)
  const bool nt = KB == 2 && p.pack && T_ == 1;
  void (*kern)(PrefillParams) = flash_prefill_kernel<T, NW, KB, false>;
  if (nt) kern = flash_prefill_kernel<T, NW, KB, (KB == 2)>;
  // the opt-in for more than 64 KiB of dynamic LDS is per device: once per device and kernel
  static std::atomic<uint64_t> attr_done_both[2];
  std::atomic<uint64_t> &attr_done = attr_done_both[nt ? 1 : 0];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const uint64_t bit = 1ull << (dev & 63);
  if (!(attr_done.load(std::memory_order_acquire) & bit)) {
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (e != hipSuccess) return e;
    attr_done.fetch_or(bit, std::memory_order_release);
  }
  hipLaunchKernelGGL(kern, dim3(grid), dim3(NT), lds_bytes, stream, p);
  e = hipGetLastError();
  if (e != hipSuccess || p.num_splits == 1) return e;
  const size_t slots = (size_t)p.m * p.H;
  if (slots <= 2048 && p.num_splits >= 8)
    hipLaunchKernelGGL(prefill_combine_wide_kernel<T>, dim3((unsigned)slots), dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL(prefill_combine_kernel<T>, dim3((unsigned)((slots + 7) / 8)), dim3(256), 0, stream, p);
  return hipGetLastError();
}

// Compute units of the current device (the kernel choice and the split counts aim at them); 256 when
// no device can be asked.
int device_compute_units() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  int cus = cached[dev].load(std::memory_order_relaxed);
  if (cus <= 0) {
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
    cached[dev].store(cus, std::memory_order_relaxed);
  }
  return cus;
}

// Kernel and key-range split for one call.
// 256-row workgroups (one per CU) or 128-row ones (two per CU)?  The 256-row kernel has the
// cheaper step (K/V tiles shared by twice the rows) but coarser work items: with fewer than
// about one and a half of them per CU the heavy-first list packs badly (the second round is
// mostly idle) and the 128-row kernel wins.  Measured at H=28, bf16, 256 CUs (128-row / 256-row,
// us): S=2560 64/73, S=3072 82/88, S=3584 111/107, S=4096 139/131, S=5120 201/194, S=8192 452/438.
// Key-range split: a chunk of few query rows over a long cache (keys >= 8 x rows) makes too few
// workgroups to fill the chip; its key range is cut so that about one (256-row kernel) or two
// (128-row kernel) workgroups per CU exist, each with at least 1024 keys.  Square causal prefill is
// never split: the fp32 partials would cost more HBM traffic than K and V themselves.
struct PrefillPlan {
  bool rows256, pack;
  bool pair;  // two waves per row block, each on one 32-key half of every tile (short sequences)
  bool rows64;  // with pair: 64-row workgroups of 4 waves, two per CU, instead of 128 rows and 8 waves
  int num_splits, chunk;
};
static PrefillPlan plan_prefill(int m, int n, int offset, int g, int Hkv, int cus) {
  PrefillPlan pl;
  const int H = g * Hkv;
  const long long wg256 = (long long)((m + 255) / 256) * H;
  pl.rows256 = 2 * wg256 >= 3LL * cus;
  pl.pack = false;
  // up to two 128-row workgroups per CU: the launch waits for the serial chain of the waves with
  // the most keys, so two waves share every row block (measured at H=28, bf16, 256 CUs, 4-wave /
  // paired 8-wave workgroups, us: S=1024 22.6/20.2, S=1536 32.8/27.9, S=2048 45.6/42.1,
  // S=2560 60.8/64.6, S=3072 76.3/86.0)
  const long long wg128 = (long long)((m + 127) / 128) * H;
  pl.pair = !pl.rows256 && wg128 <= 2LL * cus;
  // Up to about 1.2 such workgroups per CU, halves of them (64 rows, 4 waves, two resident per CU) finish
  // sooner: the heavy tiles meet less competition for their SIMDs (128-row / 64-row, us: S=256
  // 10.5/8.6, S=512 13.6/11.5, S=1024 20.2/17.8, S=1280 25.4/23.9, S=1408 27.9/27.5, S=1536 28.0/29.4)
  pl.rows64 = pl.pair && 5 * wg128 <= 6LL * cus;
  pl.num_splits = 1;
  pl.chunk = 0x7fffffc0;
  const long long n_vis = ((long long)m + offset < n) ? (long long)m + offset : n;  // keys the last row sees
  if (n_vis < 256) pl.pair = pl.rows64 = false;
  if (pl.rows256 || n_vis < 8LL * m || n_vis < 2048) return pl;
  pl.pair = pl.rows64 = false;
  // Split mode.  A chunk shorter than a 128-row tile packs the g query heads of a kv head into the
  // rows of one tile (K and V of the kv head are then read once, not g times).
  pl.pack = g > 1 && m < 128;
  const long long rows = pl.pack ? (long long)m * g : m;  // rows per head (per kv head when packed)
  const long long groups = pl.pack ? Hkv : H;
  pl.rows256 = rows >= 192;  // enough rows to use most of a 256-row workgroup
  const long long wgs = (pl.rows256 ? (rows + 255) / 256 : (rows + 127) / 128) * groups;
  const long long want_wgs = pl.rows256 ? cus : 2LL * cus;  // one round of workgroups, not one and a bit
  long long splits = want_wgs / wgs;
  if (splits > n_vis / 1024) splits = n_vis / 1024;
  // at most 64 key ranges, 128 where one or two workgroups per range would otherwise leave half the chip
  // idle (two kv heads, 131072 keys, 16 tokens: 48.6 -> 37.5 us; with four kv heads 128 ranges are slower)
  const long long max_splits = wgs <= 2 ? kMaxPrefillSplits : kMaxPrefillSplits / 2;
  if (splits > max_splits) splits = max_splits;
  if (splits <= 1) {
    pl.pack = false;
    pl.rows256 = false;
    pl.pair = wg128 <= 2LL * cus;
    pl.rows64 = 5 * wg128 <= 6LL * cus;
    return pl;
  }
  long long chunk = (n_vis + splits - 1) / splits;
  chunk = (chunk + 127) / 128 * 128;
  pl.chunk = (int)chunk;
  pl.num_splits = (int)((n_vis + chunk - 1) / chunk);  // no empty trailing range
  return pl;
}

size_t flash_prefill_workspace_bytes(int m, int n, int offset, int group_size, int kv_head_num) {
  const int H = group_size * kv_head_num;
  const PrefillPlan pl = plan_prefill(m, n, offset, group_size, kv_head_num, device_compute_units());
  if (pl.num_splits <= 1) return 0;
  return (size_t)pl.num_splits * m * H * (kHeadDim + 2) * sizeof(float);
}

#ifdef LLMHIP_BENCH
hipError_t launch_flash_prefill(void *out, const void *q, const void *k, const void *v, int m,
                                int n, int offset, int group_size, int kv_head_num, int dt,
                                hipStream_t stream, void *workspace, void *clock_probe) {
  PrefillParams p;
  p.clock_probe = static_cast<unsigned long long *>(clock_probe);
#else
hipError_t launch_flash_prefill(void *out, const void *q, const void *k, const void *v, int m,
                                int n, int offset, int group_size, int kv_head_num, int dt,
                                hipStream_t stream, void *workspace) {
  PrefillParams p;
#endif
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
  PrefillPlan pl = plan_prefill(m, n, offset, group_size, kv_head_num, device_compute_units());
  if (pl.num_splits > 1 && !workspace) {  // no scratch offered: run unsplit (and unpacked)
    pl.num_splits = 1;
    pl.chunk = 0x7fffffc0;
    pl.pack = false;
    pl.rows256 = false;
    pl.rows64 = false;
  }
  p.pack = pl.pack ? 1 : 0;
  p.num_splits = pl.num_splits;
  p.chunk = pl.chunk;
  p.ws_o = static_cast<float *>(workspace);
  p.ws_ml = p.ws_o ? p.ws_o + (size_t)pl.num_splits * m * p.H * kHeadDim : nullptr;
  const bool f16 = dt == kDtFloat16;
  if (pl.rows256) return f16 ? launch_prefill_t<_Float16, 8>(p, stream) : launch_prefill_t<__bf16, 8>(p, stream);
  if (pl.pair && pl.rows64)
    return f16 ? launch_prefill_t<_Float16, 4, 1>(p, stream) : launch_prefill_t<__bf16, 4, 1>(p, stream);
  if (pl.pair) return f16 ? launch_prefill_t<_Float16, 8, 1>(p, stream) : launch_prefill_t<__bf16, 8, 1>(p, stream);
  return f16 ? launch_prefill_t<_Float16, 4>(p, stream) : launch_prefill_t<__bf16, 4>(p, stream);
}

}  // namespace LLMHIP_NS
