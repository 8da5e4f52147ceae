/*
 * asan_check.c -- sanitizer driver of the CPU oracle (test infrastructure).
 *
 * Built with -fsanitize=address,undefined together with attn_oracle.c by
 * `make -C oracle asan`; runs every exported function once on small, exactly
 * sized heap buffers so that any out-of-bounds access, misaligned access or
 * undefined arithmetic in the restatement aborts the run.  The shapes cover
 * the ragged cases of the parity tests: m != n, offset > 0, n < m + offset,
 * group_size > 1, a KV stride larger than n, batch > 1.
 */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

uint16_t orc_f32_to_bf16(uint32_t bits);
float orc_bf16_to_f32(uint16_t h);
uint16_t orc_f32_to_f16(float f);
float orc_f16_to_f32(uint16_t h);
void orc_round_array(uint16_t *out, const float *in, int64_t count, int dt);
void orc_widen_array(float *out, const uint16_t *in, int64_t count, int dt);
void orc_init_freq_cis(float *freq_cis, int head_dim, int max_seq_len, float theta, int dt, int use_powf);
void orc_rope(uint16_t *out, const uint16_t *in, const float *freq_cis, int start_pos, int cur_size,
              int n_heads, int head_dim, int is_neox, int dt);
void orc_kv_append(uint16_t *cache, const uint16_t *src, int prev_pos, int cur_size, int row_elems);
void orc_attention_layer(uint16_t *out, const uint16_t *q, const uint16_t *k, const uint16_t *v, int batch,
                         int m, int n, int offset, int group_size, int kv_head_num, int head_dim,
                         int64_t kv_seq_stride, int dt, int n_threads);
void orc_attention_f32(float *out, const uint16_t *q, const uint16_t *k, const uint16_t *v, int batch, int m,
                       int n, int offset, int group_size, int kv_head_num, int head_dim,
                       int64_t kv_seq_stride, int dt, int n_threads);
void orc_matmul_bias(uint16_t *out, const uint16_t *lhs, const uint16_t *w, const float *bias, int m, int n,
                     int k, int dt, int n_threads);
void orc_add(uint16_t *out, const uint16_t *lhs, const uint16_t *rhs, int64_t count, int dt);
int64_t orc_all_close(const float *a, const float *b, int64_t count, float abs_err, float rel_err,
                      float *max_abs_out);
int orc_max_threads(void);

static uint64_t rng_state = 0x9E3779B97F4A7C15ull;
static float uniform_pm1(void) {
  rng_state = rng_state * 6364136223846793005ull + 1442695040888963407ull;
  return (float)((rng_state >> 40) & 0xFFFF) / 32768.0f - 1.0f;
}
static uint16_t *random_bits(size_t count, int dt) {
  float *f = (float *)malloc(count * sizeof(float));
  uint16_t *b = (uint16_t *)malloc(count * sizeof(uint16_t));
  for (size_t i = 0; i < count; ++i) f[i] = 2.0f * uniform_pm1();
  orc_round_array(b, f, (int64_t)count, dt);
  free(f);
  return b;
}

int main(void) {
  const int hd = 128;
  int checks = 0;
  for (int dt = 4; dt <= 5; ++dt) {
    /* conversions over every 16-bit pattern */
    for (uint32_t h = 0; h < 65536; ++h) {
      volatile float a = orc_f16_to_f32((uint16_t)h), b = orc_bf16_to_f32((uint16_t)h);
      (void)orc_f32_to_f16(a);
      union { float f; uint32_t u; } cv;
      cv.f = b;
      (void)orc_f32_to_bf16(cv.u);
    }
    /* table, RoPE at the last rows of the table, append at the last rows of the cache */
    const int max_seq = 37, heads = 3, kvh = 1, cur = 5, start = max_seq - cur;
    float *tab = (float *)malloc(sizeof(float) * (size_t)max_seq * hd);
    orc_init_freq_cis(tab, hd, max_seq, 1e6f, dt, 0);
    orc_init_freq_cis(tab, hd, max_seq, 10000.0f, dt, 1);
    uint16_t *x = random_bits((size_t)cur * heads * hd, dt);
    uint16_t *xr = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)cur * heads * hd);
    orc_rope(xr, x, tab, start, cur, heads, hd, 0, dt);
    orc_rope(x, x, tab, start, cur, heads, hd, 1, dt); /* in place */
    uint16_t *cache = (uint16_t *)calloc((size_t)max_seq * kvh * hd, sizeof(uint16_t));
    uint16_t *src = random_bits((size_t)cur * kvh * hd, dt);
    orc_kv_append(cache, src, start, cur, kvh * hd);
    free(tab); free(x); free(xr); free(cache); free(src);
    /* attention: (batch, m, n, offset, g, Hkv, stride) */
    const int cases[][7] = {{1, 1, 1, 0, 1, 1, 1},   {1, 4, 4, 0, 1, 2, 4},   {1, 3, 7, 4, 2, 2, 9},
                            {2, 1, 33, 32, 6, 1, 40}, {1, 9, 10, 5, 2, 1, 10}, {3, 5, 6, 3, 1, 3, 6}};
    for (size_t c = 0; c < sizeof(cases) / sizeof(cases[0]); ++c) {
      const int B = cases[c][0], m = cases[c][1], n = cases[c][2], off = cases[c][3], g = cases[c][4],
                Hkv = cases[c][5], stride = cases[c][6];
      const int H = g * Hkv;
      uint16_t *q = random_bits((size_t)B * m * H * hd, dt);
      /* exactly the rows the contract allows to be read: the last sequence ends at row n */
      const size_t kv_count = ((size_t)(B - 1) * stride + n) * Hkv * hd;
      uint16_t *k = random_bits(kv_count, dt), *v = random_bits(kv_count, dt);
      uint16_t *o16 = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)B * m * H * hd);
      float *o32 = (float *)malloc(sizeof(float) * (size_t)B * m * H * hd);
      float *w32 = (float *)malloc(sizeof(float) * (size_t)B * m * H * hd);
      for (int threads = 1; threads <= 2; ++threads) {
        orc_attention_layer(o16, q, k, v, B, m, n, off, g, Hkv, hd, stride, dt, threads);
        orc_attention_f32(o32, q, k, v, B, m, n, off, g, Hkv, hd, stride, dt, threads);
      }
      orc_widen_array(w32, o16, (int64_t)B * m * H * hd, dt);
      float mx = 0.0f;
      (void)orc_all_close(w32, o32, (int64_t)B * m * H * hd, 1e-3f, 1e-3f, &mx);
      if (!(mx < 0.05f)) {
        fprintf(stderr, "asan_check: layer-style and fp32 attention differ by %g\n", mx);
        return 1;
      }
      ++checks;
      free(q); free(k); free(v); free(o16); free(o32); free(w32);
    }
    /* projection with and without bias, residual add */
    const int m = 3, n = 16, kk = 32;
    uint16_t *lhs = random_bits((size_t)m * kk, dt), *w = random_bits((size_t)n * kk, dt);
    float *bias = (float *)malloc(sizeof(float) * n);
    for (int i = 0; i < n; ++i) bias[i] = 0.02f * uniform_pm1();
    uint16_t *out = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)m * n);
    orc_matmul_bias(out, lhs, w, bias, m, n, kk, dt, 1);
    orc_matmul_bias(out, lhs, w, NULL, m, n, kk, dt, 2);
    orc_add(out, out, out, (int64_t)m * n, dt);
    free(lhs); free(w); free(bias); free(out);
    ++checks;
  }
  (void)orc_max_threads();
  printf("asan_check: %d checks, no sanitizer report\n", checks);
  return 0;
}
