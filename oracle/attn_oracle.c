/*
 * attn_oracle.c -- CPU restatement of the llm_simple attention hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the parity checker for the HIP
 * kernels: it may be called from tests/, from __graft_entry__.smoke() and from
 * the cpu_baseline leg of bench.py, and from nowhere else.  Nothing in the
 * shipped library links or loads it.
 *
 * Every function restates, in plain C with no third-party dependency, the
 * arithmetic of a reference function (cited as path:line under the reference
 * tree).  The reference's own sources cannot be built in this image (they need
 * Eigen, Boost, spdlog, nlohmann-json, gtest and the Ascend ACL headers), so
 * this restatement is pinned by closed forms, invariants, library routines and
 * brute force in tests/test_oracle_*.py instead of by running the reference.
 *
 * Pin status of each exported function:
 *   orc_f32_to_f16 / orc_f16_to_f32 / orc_f32_to_bf16 / orc_bf16_to_f32
 *       pinned: exhaustive 2^16 round trips + numpy.float16 / torch.bfloat16.
 *   orc_init_freq_cis      pinned: float64 closed form, row 0 == (1,0).
 *   orc_rope               pinned: complex multiplication in float64, norm
 *                          preservation, composition, neox==interleaved under
 *                          the fixed permutation.
 *   orc_kv_append          pinned: canary bytes, byte identity.
 *   orc_attention_f32 / orc_attention_layer
 *                          pinned for MHA: textbook SDPA (torch, fp64), fp64
 *                          brute force, softmax invariants.
 *                          The three rounding points of orc_attention_layer
 *                          (scores after the scale, probabilities after the
 *                          division, output) are pinned by hand-derived bit
 *                          patterns on 2..11-key cases with exact dot products
 *                          (tests/test_oracle_layer_rounding.py): a chain that
 *                          drops one, moves the probability rounding before
 *                          the division or rounds to the other 16-bit type
 *                          misses at least one of them.
 *                          GQA head mapping (kv = h / group_size) and the bf16
 *                          variant have no reference CPU code and no reference
 *                          test: PARITY UNPINNED against the reference at that
 *                          point; pinned only against the HF repeat_kv
 *                          convention (repeat_interleave on K/V).
 *   orc_matmul_bias        pinned: numpy float64 matmul + bias within one
 *                          step of the storage type, identity weight, zero
 *                          input (output == rounded bias), row/column
 *                          permutation equivariance.
 *   orc_add                pinned: numpy float32 add + the pinned rounding.
 *
 * Build: see oracle/Makefile (gcc -O3 -ffp-contract=off -fopenmp).
 * -ffp-contract=off keeps a*b-c*d as two roundings + one, exactly what the
 * HIP RoPE kernel does with explicit non-fused intrinsics, so RoPE parity can
 * be asserted bit-exact.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* Data type numbering of the reference (prebuild/defs.hpp:8-18). */
enum { ORC_DT_FLOAT16 = 4, ORC_DT_BFLOAT16 = 5 };

/* ---------------------------------------------------------------- */
/* storage type conversions                                          */
/* ---------------------------------------------------------------- */

static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* fp32 -> bf16, restating src/util.cpp:33-72 step by step (split sign /
 * exponent / 24-bit significand with the hidden one, round the low 16 bits to
 * nearest-even, carry into the exponent, saturate the exponent at 0xFF).
 * Like the reference it does not special-case NaN or subnormals. */
uint16_t orc_f32_to_bf16(uint32_t bits) {
  const uint32_t sign = (bits >> 31) & 1u;
  const uint32_t exponent = (bits >> 23) & 0xFFu;
  const uint32_t sig24 = (bits & 0x007FFFFFu) | 0x00800000u;
  const uint32_t hi = (sig24 >> 16) & 0xFFu;
  const uint32_t lo = sig24 & 0xFFFFu;
  uint32_t r = hi;
  if (lo > 0x8000u) r += 1;
  else if (lo == 0x8000u && (hi & 1u)) r += 1;
  uint32_t e = exponent;
  if (r > 0xFFu) { e += 1; r = 0x80u; }
  if (e > 0xFFu) e = 0xFFu;
  return (uint16_t)((sign << 15) | (e << 7) | (r & 0x7Fu));
}

float orc_bf16_to_f32(uint16_t h) { return bits_f32(((uint32_t)h) << 16); }

/* fp32 -> fp16 round-to-nearest-even with subnormals, inf and NaN; the
 * semantics of Eigen's cast<Eigen::half>() used at
 * src/llama2_layer_cpu.cpp:218-219, :675, :275-279 and
 * tests/flash_attn_test.cpp:91-92. */
uint16_t orc_f32_to_f16(float f) {
  uint32_t x = f32_bits(f);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t ax = x & 0x7FFFFFFFu;
  if (ax >= 0x7F800000u) /* inf / nan */
    return (uint16_t)(sign | 0x7C00u | ((ax > 0x7F800000u) ? 0x200u : 0u));
  if (ax >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u); /* rounds to inf */
  if (ax < 0x38800000u) { /* result is subnormal or zero */
    if (ax < 0x33000000u) return (uint16_t)sign; /* < 2^-25 -> 0 */
    int e = (int)(ax >> 23);
    uint32_t sig = (ax & 0x7FFFFFu) | 0x800000u;
    int shift = 126 - e; /* 14..24 */
    uint32_t q = sig >> shift;
    uint32_t rem = sig & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q += 1;
    return (uint16_t)(sign | q);
  }
  uint32_t e = (ax >> 23) - 112u;
  uint32_t m = ax & 0x7FFFFFu;
  uint32_t q = (e << 10) | (m >> 13);
  uint32_t rem = m & 0x1FFFu;
  if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) q += 1;
  return (uint16_t)(sign | q);
}

float orc_f16_to_f32(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t e = (h >> 10) & 0x1Fu;
  uint32_t m = h & 0x3FFu;
  if (e == 0) {
    if (m == 0) return bits_f32(sign);
    float v = (float)m * (1.0f / 16777216.0f); /* m * 2^-24 */
    return sign ? -v : v;
  }
  if (e == 31) return bits_f32(sign | 0x7F800000u | (m << 13));
  return bits_f32(sign | ((e + 112u) << 23) | (m << 13));
}

static inline float load_t(const uint16_t *p, int dt) {
  return dt == ORC_DT_BFLOAT16 ? orc_bf16_to_f32(*p) : orc_f16_to_f32(*p);
}
static inline uint16_t round_t(float f, int dt) {
  return dt == ORC_DT_BFLOAT16 ? orc_f32_to_bf16(f32_bits(f)) : orc_f32_to_f16(f);
}

void orc_round_array(uint16_t *out, const float *in, int64_t count, int dt) {
  for (int64_t i = 0; i < count; ++i) out[i] = round_t(in[i], dt);
}
void orc_widen_array(float *out, const uint16_t *in, int64_t count, int dt) {
  for (int64_t i = 0; i < count; ++i) out[i] = load_t(in + i, dt);
}

/* ---------------------------------------------------------------- */
/* rotary table                                                      */
/* ---------------------------------------------------------------- */

/* freq_cis[max_seq_len][head_dim/2][2] = (cos, sin) of t * theta^(-2i/hd).
 * use_powf == 0: src/model_base.cpp:27-83 (inverse frequency through double
 *   pow, angle and cos/sin in fp32, and for DT_BFLOAT16 every entry rounded to
 *   bf16 and widened back, :59-66).
 * use_powf != 0: the test twin tests/npu_op_test_util.cpp:109-142 (powf, no
 *   bf16 rounding whatever dt says). */
void orc_init_freq_cis(float *freq_cis, int head_dim, int max_seq_len, float theta,
                       int dt, int use_powf) {
  int freq_len = head_dim / 2;
  float *freq = (float *)malloc(sizeof(float) * (size_t)freq_len);
  for (int i = 0; i < freq_len; ++i) {
    if (use_powf)
      freq[i] = 1.0f / powf(theta, (float)(i * 2) / (float)head_dim);
    else
      freq[i] = (float)(1.0f / pow((double)theta, (double)(i * 2) / (double)head_dim));
  }
  for (int t = 0; t < max_seq_len; ++t) {
    for (int j = 0; j < freq_len; ++j) {
      float angle = (float)t * freq[j];
      size_t o = ((size_t)t * freq_len + j) * 2;
      freq_cis[o] = cosf(angle);
      freq_cis[o + 1] = sinf(angle);
    }
  }
  if (!use_powf && dt == ORC_DT_BFLOAT16) {
    size_t total = (size_t)freq_len * max_seq_len * 2;
    for (size_t i = 0; i < total; ++i)
      freq_cis[i] = orc_bf16_to_f32(orc_f32_to_bf16(f32_bits(freq_cis[i])));
  }
  free(freq);
}

/* ---------------------------------------------------------------- */
/* RoPE                                                              */
/* ---------------------------------------------------------------- */

/* Rotate one tensor x[cur_size][n_heads][head_dim] by rows
 * start_pos .. start_pos+cur_size-1 of the table.  Arithmetic of
 * src/llama2_layer_cpu.cpp:835-856 (widen, (a*c - b*d, a*d + b*c) in fp32,
 * one rounding to the storage type, :858-859) with the start_pos offset the
 * device entry and every test golden use
 * (tests/rope_single_layer_test.cpp:78-97, tests/npu_operator_test.cpp:1005-1026)
 * and the neox pairing (f, f+hd/2) of tests/rope_single_layer_test.cpp:86-91.
 * `out` may alias `in`. */
void orc_rope(uint16_t *out, const uint16_t *in, const float *freq_cis, int start_pos,
              int cur_size, int n_heads, int head_dim, int is_neox, int dt) {
  int freq_len = head_dim / 2;
  for (int s = 0; s < cur_size; ++s) {
    const float *tab = freq_cis + (size_t)(s + start_pos) * freq_len * 2;
    for (int h = 0; h < n_heads; ++h) {
      size_t base = ((size_t)s * n_heads + h) * head_dim;
      for (int f = 0; f < freq_len; ++f) {
        float fc = tab[2 * f], fd = tab[2 * f + 1];
        int ia = is_neox ? f : 2 * f;
        int ib = is_neox ? f + freq_len : 2 * f + 1;
        float a = load_t(in + base + ia, dt);
        float b = load_t(in + base + ib, dt);
        float ra = a * fc - b * fd;
        float rb = a * fd + b * fc;
        out[base + ia] = round_t(ra, dt);
        out[base + ib] = round_t(rb, dt);
      }
    }
  }
}

/* ---------------------------------------------------------------- */
/* KV-cache append                                                   */
/* ---------------------------------------------------------------- */

/* cache[prev_pos : prev_pos+cur_size, :] = src, a byte copy of
 * cur_size*row_elems 16-bit elements at element offset prev_pos*row_elems
 * (src/llama2_layer_npu.cpp:325-339, :830-844; CPU slice-assign
 * src/llama2_layer_cpu.cpp:140-161). */
void orc_kv_append(uint16_t *cache, const uint16_t *src, int prev_pos, int cur_size,
                   int row_elems) {
  memcpy(cache + (size_t)prev_pos * row_elems, src,
         (size_t)cur_size * row_elems * sizeof(uint16_t));
}

/* ---------------------------------------------------------------- */
/* attention                                                         */
/* ---------------------------------------------------------------- */

/* Shared body.  q[batch][m][H][hd], k/v[batch][kv_seq_stride rows][Hkv][hd]
 * with n valid rows, out token-major [batch][m][H*hd].
 *   layer_style != 0: src/llama2_layer_cpu.cpp:175-296 -- scores
 *     (dot + mask) * scale in fp32 then rounded to T (:212-219), softmax in
 *     fp32 over the rounded scores then rounded to T (:647-677), P*V in fp32
 *     then rounded to T (:272-280).  out16 receives T.
 *   layer_style == 0: tests/flash_attn_test.cpp:106-192 -- the same chain
 *     with no intermediate rounding; out32 receives fp32.
 * Mask rule col > row + offset => -inf, added before the scale
 * (src/llama2_layer_cpu.cpp:687-701, tests/flash_attn_test.cpp:124-145).
 * q head h reads kv head h / group_size (HF repeat_kv convention; for
 * group_size == 1 this is the reference MHA path exactly). */
static void attention_body(uint16_t *out16, float *out32, const uint16_t *q,
                           const uint16_t *k, const uint16_t *v, int batch, int m, int n,
                           int offset, int group_size, int kv_head_num, int head_dim,
                           int64_t kv_seq_stride, int dt, int layer_style) {
  const int H = group_size * kv_head_num;
  const float scale = 1.0f / sqrtf((float)head_dim);
  const int64_t jobs = (int64_t)batch * H;
#pragma omp parallel
  {
    float *sc = (float *)malloc(sizeof(float) * (size_t)n);
    float *qf = (float *)malloc(sizeof(float) * (size_t)head_dim);
    float *acc = (float *)malloc(sizeof(float) * (size_t)head_dim);
    /* the reference widens whole tensors to fp32 before contracting
     * (src/llama2_layer_cpu.cpp:186-193); do the same per (sequence, head) */
    float *kf = (float *)malloc(sizeof(float) * (size_t)n * head_dim);
    float *vf = (float *)malloc(sizeof(float) * (size_t)n * head_dim);
#pragma omp for schedule(dynamic, 1)
    for (int64_t job = 0; job < jobs; ++job) {
      int b = (int)(job / H), h = (int)(job % H);
      int kvh = h / group_size;
      const size_t kv_row = (size_t)kv_head_num * head_dim;
      const uint16_t *kb = k + ((size_t)b * kv_seq_stride * kv_head_num + kvh) * head_dim;
      const uint16_t *vb = v + ((size_t)b * kv_seq_stride * kv_head_num + kvh) * head_dim;
      for (int c = 0; c < n; ++c)
        for (int d = 0; d < head_dim; ++d) {
          kf[(size_t)c * head_dim + d] = load_t(kb + (size_t)c * kv_row + d, dt);
          vf[(size_t)c * head_dim + d] = load_t(vb + (size_t)c * kv_row + d, dt);
        }
      for (int r = 0; r < m; ++r) {
        const uint16_t *qr = q + (((size_t)b * m + r) * H + h) * head_dim;
        for (int d = 0; d < head_dim; ++d) qf[d] = load_t(qr + d, dt);
        /* columns c > r + offset carry -inf: exp gives exactly 0 and they
         * change neither max nor sum, so they are skipped, not computed */
        int64_t vis64 = (int64_t)r + offset + 1;
        int nvis = vis64 < n ? (int)vis64 : n;
        float mx = -INFINITY;
        for (int c = 0; c < nvis; ++c) {
          const float *kr = kf + (size_t)c * head_dim;
          /* fp32 accumulation in 8 interleaved partial sums (Eigen's blocked
           * contraction order is not recoverable; any fp32 order is within
           * the tolerance) */
          float p8[8] = {0, 0, 0, 0, 0, 0, 0, 0};
          int d = 0;
          for (; d + 8 <= head_dim; d += 8)
            for (int j = 0; j < 8; ++j) p8[j] += qf[d + j] * kr[d + j];
          for (; d < head_dim; ++d) p8[0] += qf[d] * kr[d];
          float dot = ((p8[0] + p8[4]) + (p8[1] + p8[5])) + ((p8[2] + p8[6]) + (p8[3] + p8[7]));
          float s = dot * scale;
          if (layer_style) { uint16_t t = round_t(s, dt); s = load_t(&t, dt); }
          sc[c] = s;
          if (s > mx) mx = s;
        }
        float sum = 0.0f;
        for (int c = 0; c < nvis; ++c) { sc[c] = expf(sc[c] - mx); sum += sc[c]; }
        for (int d = 0; d < head_dim; ++d) acc[d] = 0.0f;
        for (int c = 0; c < nvis; ++c) {
          float p = sc[c] / sum;
          if (layer_style) { uint16_t t = round_t(p, dt); p = load_t(&t, dt); }
          const float *vr = vf + (size_t)c * head_dim;
          for (int d = 0; d < head_dim; ++d) acc[d] += p * vr[d];
        }
        size_t o = (((size_t)b * m + r) * H + h) * head_dim;
        if (layer_style)
          for (int d = 0; d < head_dim; ++d) out16[o + d] = round_t(acc[d], dt);
        else
          for (int d = 0; d < head_dim; ++d) out32[o + d] = acc[d];
      }
    }
    free(sc); free(qf); free(acc); free(kf); free(vf);
  }
}

void orc_attention_layer(uint16_t *out, const uint16_t *q, const uint16_t *k,
                         const uint16_t *v, int batch, int m, int n, int offset,
                         int group_size, int kv_head_num, int head_dim,
                         int64_t kv_seq_stride, int dt, int n_threads) {
#ifdef _OPENMP
  if (n_threads > 0) omp_set_num_threads(n_threads);
#endif
  attention_body(out, NULL, q, k, v, batch, m, n, offset, group_size, kv_head_num,
                 head_dim, kv_seq_stride, dt, 1);
}

void orc_attention_f32(float *out, const uint16_t *q, const uint16_t *k, const uint16_t *v,
                       int batch, int m, int n, int offset, int group_size,
                       int kv_head_num, int head_dim, int64_t kv_seq_stride, int dt,
                       int n_threads) {
#ifdef _OPENMP
  if (n_threads > 0) omp_set_num_threads(n_threads);
#endif
  attention_body(NULL, out, q, k, v, batch, m, n, offset, group_size, kv_head_num,
                 head_dim, kv_seq_stride, dt, 0);
}

/* ---------------------------------------------------------------- */
/* projections either side of the attention block                    */
/* ---------------------------------------------------------------- */

/* out[m][n] = round_T(sum_k lhs[m][k] * w[n][k] + bias[n]): the golden of
 * tests/gemm_test.cpp:138-149 (fp32 contraction, fp32 bias broadcast over the
 * rows, one cast to T).  w is W[n][k] row-major, i.e. the transpose of the
 * [k][n] right-hand side the reference test builds before it repacks it into the
 * Ascend nz layout (tests/gemm_test.cpp:88-101).  bias may be NULL
 * (npu_matmul_nz_layer).  The order of the fp32 summation inside Eigen's
 * contraction is not specified; eight interleaved partial sums are used. */
void orc_matmul_bias(uint16_t *out, const uint16_t *lhs, const uint16_t *w, const float *bias,
                     int m, int n, int k, int dt, int n_threads) {
  float *wf = (float *)malloc((size_t)n * k * sizeof(float));
  float *xf = (float *)malloc((size_t)m * k * sizeof(float));
  orc_widen_array(wf, w, (int64_t)n * k, dt);
  orc_widen_array(xf, lhs, (int64_t)m * k, dt);
#ifdef _OPENMP
  if (n_threads <= 0) n_threads = omp_get_max_threads();
#pragma omp parallel for num_threads(n_threads) schedule(static)
#endif
  for (int i = 0; i < m; ++i) {
    const float *x = xf + (size_t)i * k;
    for (int j = 0; j < n; ++j) {
      const float *wr = wf + (size_t)j * k;
      float p[8] = {0, 0, 0, 0, 0, 0, 0, 0};
      int c = 0;
      for (; c + 8 <= k; c += 8)
        for (int e = 0; e < 8; ++e) p[e] += x[c + e] * wr[c + e];
      for (; c < k; ++c) p[c & 7] += x[c] * wr[c];
      float acc = ((p[0] + p[1]) + (p[2] + p[3])) + ((p[4] + p[5]) + (p[6] + p[7]));
      if (bias) acc += bias[j];
      out[(size_t)i * n + j] = round_t(acc, dt);
    }
  }
  (void)n_threads;
  free(wf);
  free(xf);
}

/* out[i] = round_T(float(lhs[i]) + float(rhs[i])): the residual add after o_proj
 * (npu_add_layer, src/llama2_layer_npu.cpp:900-901). */
void orc_add(uint16_t *out, const uint16_t *lhs, const uint16_t *rhs, int64_t count, int dt) {
  for (int64_t i = 0; i < count; ++i) out[i] = round_t(load_t(lhs + i, dt) + load_t(rhs + i, dt), dt);
}

/* Comparison rule of the reference's tests (tests/npu_op_test_util.cpp:33-48):
 * an element fails only when BOTH the absolute and the relative error exceed
 * their bound.  Returns the number of failing elements and the max abs error. */
int64_t orc_all_close(const float *a, const float *b, int64_t count, float abs_err,
                      float rel_err, float *max_abs_out) {
  int64_t bad = 0;
  float mx = 0.0f;
  for (int64_t i = 0; i < count; ++i) {
    float d = fabsf(a[i] - b[i]);
    float big = fmaxf(fabsf(a[i]), fabsf(b[i]));
    if (d > mx) mx = d;
    if (d > abs_err && d / big > rel_err) bad++;
  }
  if (max_abs_out) *max_abs_out = mx;
  return bad;
}

int orc_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
