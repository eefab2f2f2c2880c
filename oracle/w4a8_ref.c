/* TEST INFRASTRUCTURE -- the CPU oracle of the W4A8-iu8 decoder-linear path.
 *
 * This file is a checker. Only the test-suite, the smoke check and the benchmark's
 * cpu_baseline leg may build, load or call it; no product code links or imports it.
 *
 * It restates, in plain C on the host, the arithmetic contract the reference writes
 * down for its int4/int8-weight x int8-activation GEMM (paths relative to the
 * reference tree, under crates/saber-kernels/):
 *
 *   Q1  per-token int8 law ........ hip/macaq_i8.h:1-13, hip/mxfp4_hadi8.hip:21-58
 *   Q2  A-tiled byte order ........ hip/macaq_iu8.hip:8-10, hip/mxfp4_hadi8.hip:55
 *   G1  exact int32 accumulate .... hip/macaq_iu8.hip:12-24
 *   G3  epilogue .................. hip/macaq_iu8.hip:20-24,41-50
 *   M1  router softmax/top-k ...... hip/moe_route.hip:43-57,108-175
 *   M2  expert-major sort + tiles . src/moe.rs:691-708,798-865, hip/moe_route.hip:176-284
 *   M4  SiLU*up + requant ......... hip/mxfp4_hadi8.hip:118-146 (Hadamard left out)
 *   M5  weighted combine .......... hip/moe_route.hip:287-329
 *   bf16 rounding ................. crates/saber-cpux/src/lib.rs:82-90
 *
 * The reference's own CPU twin (saber-cpux) is Rust and implements a different
 * (MXFP4 x e4m3) law, and the reference holds no golden vector for this path, so
 * what pins each function is stated where the tests check it (tests/test_oracle_*.py):
 * IEEE identities recomputed in float64, int64 matrix products, exhaustive bf16
 * sweeps against torch's rounding, brute-force sorts.  M4 calls libm expf(), the
 * one function that is not IEEE-specified: "parity unpinned" beyond the exhaustive
 * on-device comparison of all 65,536 bf16 inputs.  The same holds for the bf16
 * sigmoid of the attention gate; gdn_norm's f32 silu gate is "parity unpinned"
 * beyond a 2-ulp bound against the card's own table, and the two norms' rsqrtf
 * (an approximate device instruction) is restated as IEEE 1/sqrt.
 *
 * Structure follows saber-cpux: a scalar law (gemm_*_ref), a vectorised multi-thread
 * body (gemm_fast: 16-column tiles as the work unit, lib.rs:280-303; threads pinned
 * one per core, src/bin/cpux_bench.rs:85-92) and a twin test that the two agree.
 *
 * Build: see oracle/Makefile (gcc -O2 -ffp-contract=off; no -ffast-math).
 */
#define _GNU_SOURCE
#include <math.h>
#include <pthread.h>
#include <sched.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <immintrin.h>


/* ------------------------------------------------------------------ bf16 */

/* fp32 -> bf16 bits, round to nearest even (saber-cpux/src/lib.rs:82-90). */
uint16_t w4a8_bf16_rne(float x) {
  uint32_t u;
  memcpy(&u, &x, 4);
  if (x != x) return (uint16_t)((u >> 16) | 0x40);
  return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

float w4a8_bf16_f32(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* ------------------------------------------------------------------ Q1: int8 law */

/* One row: amax over |x| (order-free max), sc = max(amax/127, 1e-30) with an IEEE
 * divide, q = rint(clamp(x/sc, -127, 127)) in round-half-even
 * (hip/macaq_i8.h:10-13; hip/mxfp4_hadi8.hip:26-45). */
void w4a8_quant_row(const float *x, int K, int8_t *q, float *scale) {
  float amax = 0.f;
  for (int k = 0; k < K; ++k) amax = fmaxf(amax, fabsf(x[k]));
  volatile float scv = amax / 127.f; /* volatile: one rounding, no reassociation */
  const float sc = fmaxf(scv, 1e-30f);
  *scale = sc;
  for (int k = 0; k < K; ++k) {
    volatile float d = x[k] / sc;
    const float y = fminf(fmaxf(d, -127.f), 127.f);
    q[k] = (int8_t)(int)nearbyintf(y); /* default rounding mode = to nearest even */
  }
}

/* M rows of bf16 activations -> row-major int8 codes [M,K] + f32 scale [M]. */
void w4a8_quant_bf16(const uint16_t *x, int M, int K, int8_t *q, float *scale) {
  float *row = (float *)malloc(sizeof(float) * (size_t)K);
  for (int m = 0; m < M; ++m) {
    for (int k = 0; k < K; ++k) row[k] = w4a8_bf16_f32(x[(size_t)m * K + k]);
    w4a8_quant_row(row, K, q + (size_t)m * K, scale + m);
  }
  free(row);
}

/* ------------------------------------------------------------------ Q2 and weight orders */

/* Byte address of activation (m,k) in the reference's gfx12 A-tiled order
 * (hip/macaq_iu8.hip:8-10): 256-byte fragments of 16 rows x 16 k. */
uint64_t w4a8_a_tiled_gfx12(uint32_t m, uint32_t k, uint32_t K) {
  return ((uint64_t)(m >> 4) * (K / 16) + (k >> 4)) * 256 + ((m & 15) + 16 * ((k >> 3) & 1)) * 8 + (k & 7);
}

/* Byte address and nibble (0 = low) of weight (n,k) in the reference's gfx12 W4
 * fragment order (hip/macaq_iu8.hip:12-15): 128-byte fragments (nt,kk); lane l's
 * dword holds, in byte b, W[nt*16 + l%16][kk*16 + (l/16)*8 + b] low and k+4 high. */
uint64_t w4a8_w4_frag_gfx12(uint32_t n, uint32_t k, uint32_t K, uint32_t *nibble) {
  const uint32_t nt = n >> 4, kk = k >> 4, r = k & 15;
  const uint32_t half = r >> 3, j = r & 7; /* half selects lane group l/16 */
  const uint32_t lane = (n & 15) + 16 * half;
  *nibble = j >> 2;
  return ((uint64_t)nt * (K / 16) + kk) * 128 + lane * 4 + (j & 3);
}

/* The export's canonical W4 form: row-major [N][K/2], low nibble = even k
 * (crates/saber-model/src/graph.rs:2591-2592). Returns the signed code in [-8,7]. */
static inline int w4_get(const uint8_t *w4, int n, int k, int K) {
  const uint8_t b = w4[(size_t)n * (K / 2) + (k >> 1)];
  const int v = (k & 1) ? (b >> 4) : (b & 15);
  return v >= 8 ? v - 16 : v;
}

/* ------------------------------------------------------------------ G1: the scalar law */

/* S[m,n] = sum_k a[m,k] * w[n,k], exact int32, k in order (order is not numerics:
 * int32 adds are associative). A row-major int8 [M,K]; W4 canonical nibbles. */
void w4a8_gemm_w4_ref(const int8_t *A, const uint8_t *W4, int M, int N, int K, int32_t *S) {
  for (int m = 0; m < M; ++m)
    for (int n = 0; n < N; ++n) {
      int32_t s = 0;
      for (int k = 0; k < K; ++k) s += (int32_t)A[(size_t)m * K + k] * w4_get(W4, n, k, K);
      S[(size_t)m * N + n] = s;
    }
}

/* Same with int8 per-row weights W8 row-major [N,K] in [-127,127]. */
void w4a8_gemm_w8_ref(const int8_t *A, const int8_t *W8, int M, int N, int K, int32_t *S) {
  for (int m = 0; m < M; ++m)
    for (int n = 0; n < N; ++n) {
      int32_t s = 0;
      for (int k = 0; k < K; ++k) s += (int32_t)A[(size_t)m * K + k] * (int32_t)W8[(size_t)n * K + k];
      S[(size_t)m * N + n] = s;
    }
}

/* ------------------------------------------------------------------ G3: epilogue */

/* acc is the reference's accumulator: 16*S for W4 (the nibble is unpacked to the
 * int8 16*w, hip/macaq_iu8.hip:14-15), S for W8.
 * y = bf16_rne( (f32(acc) * as) * (w8 ? ws : ws * 0.0625f) ), every `*` one f32
 * multiply (hip/macaq_iu8.hip:20-24,41-50). */
uint16_t w4a8_epilogue(int32_t acc, float a_scale, float w_scale, int w8) {
  volatile float wsu = w8 ? w_scale : w_scale * 0.0625f;
  volatile float t = (float)acc * a_scale;
  volatile float y = t * wsu;
  return w4a8_bf16_rne(y);
}

/* C[m,n] for a whole S matrix; S holds sum a*w (W4: multiplied by 16 here). */
void w4a8_epilogue_all(const int32_t *S, const float *as, const float *ws, int M, int N, int w8, uint16_t *C) {
  for (int m = 0; m < M; ++m)
    for (int n = 0; n < N; ++n) {
      const int32_t acc = w8 ? S[(size_t)m * N + n] : S[(size_t)m * N + n] * 16;
      C[(size_t)m * N + n] = w4a8_epilogue(acc, as[m], ws[n], w8);
    }
}

/* ------------------------------------------------------------------ the fast body */

typedef struct {
  const int8_t *A;
  const uint8_t *W; /* W4 canonical nibbles, or int8 rows when w8 */
  int M, N, K, w8;
  int32_t *S;
  int tile_lo, tile_hi; /* 16-column tiles [lo,hi) */
  int core;             /* >= 0: pin to this core */
  int isa;              /* 0 scalar, 1 avx2, 2 avx512-vnni */
} gemm_job;

static void unpack_row(const gemm_job *j, int n, int8_t *dst) {
  if (j->w8) {
    memcpy(dst, j->W + (size_t)n * j->K, (size_t)j->K);
    return;
  }
  const uint8_t *src = j->W + (size_t)n * (j->K / 2);
  for (int b = 0; b < j->K / 2; ++b) {
    const uint8_t v = src[b];
    dst[2 * b] = (int8_t)((int8_t)(v << 4) >> 4);
    dst[2 * b + 1] = (int8_t)((int8_t)v >> 4);
  }
}

__attribute__((target("avx2"))) static int32_t dot_avx2(const int8_t *a, const int8_t *w, int K) {
  __m256i acc = _mm256_setzero_si256();
  for (int k = 0; k < K; k += 16) {
    const __m256i av = _mm256_cvtepi8_epi16(_mm_loadu_si128((const __m128i *)(a + k)));
    const __m256i wv = _mm256_cvtepi8_epi16(_mm_loadu_si128((const __m128i *)(w + k)));
    acc = _mm256_add_epi32(acc, _mm256_madd_epi16(av, wv));
  }
  __m128i s = _mm_add_epi32(_mm256_castsi256_si128(acc), _mm256_extracti128_si256(acc, 1));
  s = _mm_add_epi32(s, _mm_shuffle_epi32(s, 0x4E));
  s = _mm_add_epi32(s, _mm_shuffle_epi32(s, 0xB1));
  return _mm_cvtsi128_si32(s);
}

/* 16 columns at once against one activation row: sum (a+128)*w with vpdpbusd, the
 * 128*sum(w) bias removed afterwards (exact: |sum| < 2^31 for K <= 32768). */
__attribute__((target("avx512f,avx512bw,avx512vnni"))) static void tile_vnni(const int8_t *a, const int8_t *wt,
                                                                               const int32_t *wsum, int K,
                                                                               int32_t *out) {
  __m512i acc[16];
  for (int c = 0; c < 16; ++c) acc[c] = _mm512_setzero_si512();
  const __m512i bias = _mm512_set1_epi8((char)0x80);
  for (int k = 0; k < K; k += 64) {
    const __m512i au = _mm512_xor_si512(_mm512_loadu_si512((const void *)(a + k)), bias); /* a + 128 as u8 */
    for (int c = 0; c < 16; ++c)
      acc[c] = _mm512_dpbusd_epi32(acc[c], au, _mm512_loadu_si512((const void *)(wt + (size_t)c * K + k)));
  }
  for (int c = 0; c < 16; ++c) out[c] = _mm512_reduce_add_epi32(acc[c]) - 128 * wsum[c];
}

static void *gemm_worker(void *p) {
  gemm_job *j = (gemm_job *)p;
  if (j->core >= 0) {
    cpu_set_t set;
    CPU_ZERO(&set);
    CPU_SET(j->core, &set);
    pthread_setaffinity_np(pthread_self(), sizeof(set), &set);
  }
  const int K = j->K;
  int8_t *wt = (int8_t *)aligned_alloc(64, (size_t)16 * K);
  int32_t wsum[16];
  for (int t = j->tile_lo; t < j->tile_hi; ++t) {
    for (int c = 0; c < 16; ++c) {
      unpack_row(j, t * 16 + c, wt + (size_t)c * K);
      int32_t s = 0;
      for (int k = 0; k < K; ++k) s += wt[(size_t)c * K + k];
      wsum[c] = s;
    }
    for (int m = 0; m < j->M; ++m) {
      const int8_t *a = j->A + (size_t)m * K;
      int32_t *out = j->S + (size_t)m * j->N + t * 16;
      if (j->isa == 2 && K % 64 == 0) {
        tile_vnni(a, wt, wsum, K, out);
      } else if (j->isa >= 1 && K % 16 == 0) {
        for (int c = 0; c < 16; ++c) out[c] = dot_avx2(a, wt + (size_t)c * K, K);
      } else {
        for (int c = 0; c < 16; ++c) {
          int32_t s = 0;
          for (int k = 0; k < K; ++k) s += (int32_t)a[k] * wt[(size_t)c * K + k];
          out[c] = s;
        }
      }
    }
  }
  free(wt);
  return NULL;
}

/* 0 scalar, 1 AVX2, 2 AVX-512 VNNI -- detected at run time (cf. has_avx512,
 * saber-cpux/src/lib.rs:322-336). */
int w4a8_isa(void) {
  __builtin_cpu_init();
  if (__builtin_cpu_supports("avx512f") && __builtin_cpu_supports("avx512bw") && __builtin_cpu_supports("avx512vnni"))
    return 2;
  if (__builtin_cpu_supports("avx2")) return 1;
  return 0;
}

/* The vectorised, threaded body. S = sum a*w for columns of tiles [tile_lo,tile_hi)
 * (16 columns each; other columns untouched). threads >= 1; pin != 0 pins thread i
 * to core i. isa < 0 = best available. Returns the isa used. */
int w4a8_gemm_fast(const int8_t *A, const uint8_t *W, int M, int N, int K, int w8, int32_t *S, int tile_lo,
                   int tile_hi, int threads, int pin, int isa) {
  const int best = w4a8_isa();
  if (isa < 0 || isa > best) isa = best;
  if (threads < 1) threads = 1;
  const int tiles = tile_hi - tile_lo;
  if (threads > tiles) threads = tiles > 0 ? tiles : 1;
  gemm_job *jobs = (gemm_job *)calloc((size_t)threads, sizeof(gemm_job));
  pthread_t *th = (pthread_t *)calloc((size_t)threads, sizeof(pthread_t));
  for (int i = 0; i < threads; ++i) {
    gemm_job j = {A, W, M, N, K, w8, S, tile_lo + (int)((long)tiles * i / threads),
                  tile_lo + (int)((long)tiles * (i + 1) / threads), pin ? i : -1, isa};
    jobs[i] = j;
  }
  for (int i = 1; i < threads; ++i) pthread_create(&th[i], NULL, gemm_worker, &jobs[i]);
  gemm_worker(&jobs[0]);
  for (int i = 1; i < threads; ++i) pthread_join(th[i], NULL);
  free(jobs);
  free(th);
  return isa;
}

/* The whole dense linear on the CPU: quantise bf16 rows, GEMM (fast body), epilogue.
 * Outputs that are NULL are skipped. This is what bench.py's cpu_baseline leg times. */
int w4a8_linear(const uint16_t *X, const uint8_t *W, const float *ws, int M, int N, int K, int w8, int8_t *q,
                float *as, int32_t *S, uint16_t *C, int threads, int pin) {
  w4a8_quant_bf16(X, M, K, q, as);
  const int isa = w4a8_gemm_fast(q, W, M, N, K, w8, S, 0, N / 16, threads, pin, -1);
  if (C) w4a8_epilogue_all(S, as, ws, M, N, w8, C);
  return isa;
}

/* ------------------------------------------------------------------ M1: router */

static float bits_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* e^x for x <= 0 from IEEE mul/add/rint/ldexp only (hip/moe_route.hip:43-57). */
float w4a8_exp_nonpos(float x) {
  if (!(x > -80.f)) return 0.f;
  volatile float t;
  t = x * bits_f32(0x3FB8AA3Bu);
  const float n = nearbyintf(t);
  t = n * bits_f32(0x3F317200u);
  volatile float r = x - t;
  t = n * bits_f32(0x35BFBE8Eu);
  r = r - t;
  static const uint32_t c[5] = {0x3AB60B61u, 0x3C088889u, 0x3D2AAAABu, 0x3E2AAAABu, 0x3F000000u};
  volatile float p = bits_f32(0x39500D01u);
  for (int i = 0; i < 5; ++i) {
    t = p * r;
    p = t + bits_f32(c[i]);
  }
  t = p * r;
  p = t + 1.f;
  t = p * r;
  p = t + 1.f;
  return ldexpf(p, (int)n);
}

/* Softmax (f32) -> top-k by repeated argmax, the LOWER expert id wins a tie ->
 * renormalise w = p * (1 / (sel > 0 ? sel : 1)), sel summed in k order
 * (hip/moe_route.hip:108-175).  The reference fixes the summation tree for 512
 * experts on a wave32: 16 consecutive experts are summed in index order, then the
 * E/16 group sums are combined by an xor butterfly (strides E/32 ... 1).  The same
 * tree is used here for any E that is 16 * a power of two.
 * logits bf16 [T,E] -> ids i32 [T,topk], w f32 [T,topk]. Returns 0, or -1 on a bad E. */
int w4a8_route(const uint16_t *logits, int T, int E, int topk, int32_t *ids, float *w) {
  const int G = E / 16;
  if (E % 16 || G < 1 || (G & (G - 1)) || topk > E) return -1;
  float *p = (float *)malloc(sizeof(float) * (size_t)E);
  float *g = (float *)malloc(sizeof(float) * (size_t)G);
  float *g2 = (float *)malloc(sizeof(float) * (size_t)G);
  for (int t = 0; t < T; ++t) {
    float mx = w4a8_bf16_f32(logits[(size_t)t * E]);
    for (int e = 0; e < E; ++e) {
      p[e] = w4a8_bf16_f32(logits[(size_t)t * E + e]);
      mx = fmaxf(mx, p[e]);
    }
    for (int l = 0; l < G; ++l) {
      volatile float s = 0.f;
      for (int j = 0; j < 16; ++j) {
        volatile float d = p[l * 16 + j] - mx;
        p[l * 16 + j] = w4a8_exp_nonpos(d);
        s = s + p[l * 16 + j];
      }
      g[l] = s;
    }
    for (int o = G / 2; o; o >>= 1) {
      for (int l = 0; l < G; ++l) {
        volatile float s = g[l] + g[l ^ o];
        g2[l] = s;
      }
      memcpy(g, g2, sizeof(float) * (size_t)G);
    }
    volatile float inv = 1.f / g[0];
    for (int e = 0; e < E; ++e) {
      volatile float q = p[e] * inv;
      p[e] = isfinite(q) ? q : 0.f;
    }
    volatile float sel = 0.f;
    for (int k = 0; k < topk; ++k) {
      int bi = 0;
      float bv = p[0];
      for (int e = 1; e < E; ++e)
        if (p[e] > bv) {
          bv = p[e];
          bi = e;
        }
      p[bi] = -1.f;
      ids[(size_t)t * topk + k] = bi;
      w[(size_t)t * topk + k] = bv;
      sel = sel + bv;
    }
    volatile float scale = 1.f / (sel > 0.f ? sel : 1.f);
    for (int k = 0; k < topk; ++k) {
      volatile float v = w[(size_t)t * topk + k] * scale;
      w[(size_t)t * topk + k] = v;
    }
  }
  free(p);
  free(g);
  free(g2);
  return 0;
}

/* ------------------------------------------------------------------ M2: sort + tiles */

/* Worst-case rows / tiles (src/moe.rs:691-708), no shared expert. */
uint32_t w4a8_rows_cap(uint32_t tokens, uint32_t topk, uint32_t e_loc) {
  const uint32_t r = tokens * topk;
  return r + 15u * (r < e_loc ? r : e_loc);
}
uint32_t w4a8_tiles_cap(uint32_t tokens, uint32_t topk, uint32_t e_loc, uint32_t tile_blocks) {
  const uint32_t r = tokens * topk;
  return (r < e_loc ? r : e_loc) + r / (16u * tile_blocks) + 1u;
}

/* Expert-major layout of the routes (src/moe.rs:798-865): every expert's routes in
 * token (route-index) order at rows off[e].., off = exclusive scan of ceil(cnt/16)*16;
 * tiles of 16*tile_blocks rows, never mixing experts. Arrays sized by the caps above;
 * row_tok pad rows = -1. meta[0] = tiles, meta[1] = rows. */
void w4a8_sort_layout(const int32_t *ids, int T, int topk, int E, int tile_blocks, int32_t *row_tok,
                      int32_t *route_pos, int32_t *tile_expert, int32_t *tile_row0, int32_t *tile_rows,
                      int32_t *expert_cnt, int32_t *meta) {
  int32_t *off = (int32_t *)calloc((size_t)E, sizeof(int32_t));
  int32_t *fill = (int32_t *)calloc((size_t)E, sizeof(int32_t));
  memset(expert_cnt, 0, sizeof(int32_t) * (size_t)E);
  for (int r = 0; r < T * topk; ++r) expert_cnt[ids[r]]++;
  int32_t rows = 0;
  for (int e = 0; e < E; ++e) {
    off[e] = rows;
    rows += (expert_cnt[e] + 15) / 16 * 16;
  }
  for (int r = 0; r < rows; ++r) row_tok[r] = -1;
  for (int r = 0; r < T * topk; ++r) {
    const int e = ids[r];
    const int p = off[e] + fill[e]++;
    row_tok[p] = r / topk;
    route_pos[r] = p;
  }
  const int tr = 16 * tile_blocks;
  int nt = 0;
  for (int e = 0; e < E; ++e)
    for (int j = 0; j * tr < expert_cnt[e]; ++j) {
      tile_expert[nt] = e;
      tile_row0[nt] = off[e] + j * tr;
      tile_rows[nt] = expert_cnt[e] - j * tr < tr ? expert_cnt[e] - j * tr : tr;
      ++nt;
    }
  meta[0] = nt;
  meta[1] = rows;
  free(off);
  free(fill);
}

/* ------------------------------------------------------------------ M4: SiLU * up + requant */

/* bf16 silu for one bf16 input: bf16( x / (1 + expf(-x)) ) (hip/mxfp4_hadi8.hip:139). */
uint16_t w4a8_silu_bf16(uint16_t xb) {
  const float x = w4a8_bf16_f32(xb);
  volatile float e = expf(-x);
  volatile float d = 1.f + e;
  volatile float s = x / d;
  return w4a8_bf16_rne(s);
}

/* One row: gu = [gate(I) | up(I)] bf16 -> p = bf16(bf16(silu(gate)) * up) -> Q1 over p
 * (hip/mxfp4_hadi8.hip:136-146 without the Hadamard). Optionally returns p. */
void w4a8_silu_mul_quant_row(const uint16_t *gu, int I, int8_t *q, float *scale, uint16_t *p_out) {
  float *p = (float *)malloc(sizeof(float) * (size_t)I);
  for (int i = 0; i < I; ++i) {
    const float t = w4a8_bf16_f32(w4a8_silu_bf16(gu[i]));
    volatile float m = t * w4a8_bf16_f32(gu[I + i]);
    const uint16_t pb = w4a8_bf16_rne(m);
    if (p_out) p_out[i] = pb;
    p[i] = w4a8_bf16_f32(pb);
  }
  w4a8_quant_row(p, I, q, scale);
  free(p);
}

/* ------------------------------------------------------------------ M5: combine */

/* out[t] = bf16( sum_{k in top-k order} w[t,k] * f32(Y[pos(t,k)]) ), f32 adds in k
 * order starting from 0, each product rounded before the add, one bf16 rounding
 * (hip/moe_route.hip:287-329). */
void w4a8_combine(const uint16_t *Y, const float *topk_w, const int32_t *route_pos, int T, int topk, int H,
                  uint16_t *out) {
  for (int t = 0; t < T; ++t)
    for (int h = 0; h < H; ++h) {
      volatile float acc = 0.f;
      for (int k = 0; k < topk; ++k) {
        const int p = route_pos[(size_t)t * topk + k];
        if (p < 0) continue;
        volatile float pr = topk_w[(size_t)t * topk + k] * w4a8_bf16_f32(Y[(size_t)p * H + h]);
        acc = acc + pr;
      }
      out[(size_t)t * H + h] = w4a8_bf16_rne(acc);
    }
}

/* sigmoid(g) of the shared expert's gate (hip/moe_route.hip:59-63): e = exp(-|g|) by the router's
 * IEEE-only exp, then 1 / (1 + e) for g >= 0 and e / (1 + e) below, IEEE divides. */
float w4a8_sigmoid(float g) {
  volatile float e = w4a8_exp_nonpos(-fabsf(g));
  volatile float d = 1.f + e;
  volatile float r = g >= 0.f ? 1.f / d : e / d;
  return r;
}

/* The combine of a layer with a shared expert (hip/moe_route.hip:299-321): the routes' sum as in
 * w4a8_combine, then + sigmoid(f32(sgate[t])) * f32(Y[sh0 + t]) (the product rounded before the add),
 * one bf16 rounding. sh0 < 0 or sgate NULL: the plain combine. */
void w4a8_combine_shared(const uint16_t *Y, const float *topk_w, const int32_t *route_pos, const uint16_t *sgate, int sh0,
                         int T, int topk, int H, uint16_t *out) {
  const int shared = sh0 >= 0 && sgate != NULL;
  for (int t = 0; t < T; ++t) {
    const float sg = shared ? w4a8_sigmoid(w4a8_bf16_f32(sgate[t])) : 0.f;
    for (int h = 0; h < H; ++h) {
      volatile float acc = 0.f;
      for (int k = 0; k < topk; ++k) {
        const int p = route_pos[(size_t)t * topk + k];
        if (p < 0) continue;
        volatile float pr = topk_w[(size_t)t * topk + k] * w4a8_bf16_f32(Y[(size_t)p * H + h]);
        acc = acc + pr;
      }
      if (shared) {
        volatile float pr = sg * w4a8_bf16_f32(Y[(size_t)(sh0 + t) * H + h]);
        acc = acc + pr;
      }
      out[(size_t)t * H + h] = w4a8_bf16_rne(acc);
    }
  }
}

/* ------------------------------------------------------------------ the MoE layer end to end */

/* Flash-Next-style expert layer under the iu8 law, one expert at a time (the grouped
 * tile schedule is not numerics).  x bf16 [T,H]; per expert e: gate_up W4 canonical
 * [2I,H] at Wgu + e*(2I*H/2), scales wsgu + e*2I; down W4 [H,I] at Wdn + e*(H*I/2),
 * scales wsdn + e*H.  row_tok / expert_cnt / route_pos come from w4a8_sort_layout.
 * Writes Y (expert-major rows, bf16 [rows,H], pad rows zero) and out bf16 [T,H].
 * Optional taps (may be NULL): gu_out bf16 [rows,2I], q2_out int8 [rows,I] row-major,
 * s2_out f32 [rows]. */
void w4a8_moe_layer(const uint16_t *x, int T, int H, int I, int E, int topk, const float *topk_w,
                    const int32_t *route_pos, const int32_t *row_tok, const int32_t *expert_cnt, int rows,
                    const uint8_t *Wgu, const float *wsgu, const uint8_t *Wdn, const float *wsdn, uint16_t *Y,
                    uint16_t *out, uint16_t *gu_out, int8_t *q2_out, float *s2_out, int threads) {
  int8_t *q1 = (int8_t *)malloc((size_t)T * H);
  float *s1 = (float *)malloc(sizeof(float) * (size_t)T);
  w4a8_quant_bf16(x, T, H, q1, s1);
  int cmax = 1;
  for (int e = 0; e < E; ++e) cmax = expert_cnt[e] > cmax ? expert_cnt[e] : cmax;
  int8_t *qa = (int8_t *)malloc((size_t)cmax * H);
  float *sa = (float *)malloc(sizeof(float) * (size_t)cmax);
  int32_t *S1 = (int32_t *)malloc(sizeof(int32_t) * (size_t)cmax * 2 * I);
  int32_t *S2 = (int32_t *)malloc(sizeof(int32_t) * (size_t)cmax * H);
  uint16_t *gu = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)cmax * 2 * I);
  int8_t *q2 = (int8_t *)malloc((size_t)cmax * I);
  float *s2 = (float *)malloc(sizeof(float) * (size_t)cmax);
  memset(Y, 0, sizeof(uint16_t) * (size_t)rows * H);
  int off = 0;
  for (int e = 0; e < E; ++e) {
    const int c = expert_cnt[e];
    if (!c) continue;
    for (int i = 0; i < c; ++i) {
      const int t = row_tok[off + i];
      memcpy(qa + (size_t)i * H, q1 + (size_t)t * H, (size_t)H);
      sa[i] = s1[t];
    }
    w4a8_gemm_fast(qa, Wgu + (size_t)e * I * H, c, 2 * I, H, 0, S1, 0, 2 * I / 16, threads, 0, -1);
    w4a8_epilogue_all(S1, sa, wsgu + (size_t)e * 2 * I, c, 2 * I, 0, gu);
    for (int i = 0; i < c; ++i) w4a8_silu_mul_quant_row(gu + (size_t)i * 2 * I, I, q2 + (size_t)i * I, s2 + i, NULL);
    w4a8_gemm_fast(q2, Wdn + (size_t)e * H * (I / 2), c, H, I, 0, S2, 0, H / 16, threads, 0, -1);
    w4a8_epilogue_all(S2, s2, wsdn + (size_t)e * H, c, H, 0, Y + (size_t)off * H);
    if (gu_out) memcpy(gu_out + (size_t)off * 2 * I, gu, sizeof(uint16_t) * (size_t)c * 2 * I);
    if (q2_out) memcpy(q2_out + (size_t)off * I, q2, (size_t)c * I);
    if (s2_out) memcpy(s2_out + off, s2, sizeof(float) * (size_t)c);
    off += (c + 15) / 16 * 16;
  }
  w4a8_combine(Y, topk_w, route_pos, T, topk, H, out);
  free(q1); free(s1); free(qa); free(sa); free(S1); free(S2); free(gu); free(q2); free(s2);
}

/* ------------------------------------------------------------------ Q3: Hadamard-basis producers */

/* The activation transform of the `*_hadi8_*` producers (hip/macaq_had.h:1-19, 47-83), on one
 * 32-block: u = v * t (one f32 multiply each), the unnormalised Sylvester butterfly over element
 * bits 0, 1, 2, 3, 4 in that order, each stage (lo, hi) -> (lo + hi, lo - hi) in f32, then one f32
 * multiply by (float)(1/sqrt(32)) = 0x3E3504F3. In place. */
void w4a8_had32_block(float *v, const float *t) {
  for (int e = 0; e < 32; ++e) {
    volatile float u = v[e] * t[e];
    v[e] = u;
  }
  for (int s = 1; s < 32; s <<= 1)
    for (int e = 0; e < 32; ++e) {
      if (e & s) continue;
      volatile float lo = v[e], hi = v[e | s];
      volatile float a = lo + hi, b = lo - hi;
      v[e] = a;
      v[e | s] = b;
    }
  const float inv = bits_f32(0x3E3504F3u);
  for (int e = 0; e < 32; ++e) {
    volatile float r = v[e] * inv;
    v[e] = r;
  }
}

/* Rows of f32 values (K a multiple of 32) -> transformed rows. */
void w4a8_had32_rows(float *v, const float *t, int M, int K) {
  for (int m = 0; m < M; ++m)
    for (int b = 0; b < K; b += 32) w4a8_had32_block(v + (size_t)m * K + b, t + b);
}

/* quant_hadi8: bf16 row -> had32 -> Q1. */
void w4a8_quant_had_row(const uint16_t *x, const float *t, int K, int8_t *q, float *scale) {
  float *v = (float *)malloc(sizeof(float) * (size_t)K);
  for (int k = 0; k < K; ++k) v[k] = w4a8_bf16_f32(x[k]);
  w4a8_had32_rows(v, t, 1, K);
  w4a8_quant_row(v, K, q, scale);
  free(v);
}

/* silu_mul_quant_hadi8 (hip/mxfp4_hadi8.hip:117-146): p = bf16(bf16(silu(g)) * u), had32, Q1. */
void w4a8_silu_mul_quant_had_row(const uint16_t *gu, const float *t, int I, int8_t *q, float *scale) {
  float *p = (float *)malloc(sizeof(float) * (size_t)I);
  for (int i = 0; i < I; ++i) {
    const float s = w4a8_bf16_f32(w4a8_silu_bf16(gu[i]));
    volatile float m = s * w4a8_bf16_f32(gu[I + i]);
    p[i] = w4a8_bf16_f32(w4a8_bf16_rne(m));
  }
  w4a8_had32_rows(p, t, 1, I);
  w4a8_quant_row(p, I, q, scale);
  free(p);
}

/* add_rms_quant_hadi8 (hip/mxfp4_hadi8.hip:60-115), one row, as a workgroup of T threads computes
 * it: v = f32(y) + f32(res); res_out = bf16(v); the sum of squares accumulates per thread with fma
 * over its 8-element groups g = tid + i*T in order, then the reference's trees: shfl_down 16, 8, 4, 2,
 * 1 inside each 32 lanes, then shfl_down T/64 ... 1 over the T/32 partials. inv = 1 / sqrt(ssq / K +
 * eps) with IEEE sqrt and divide (the reference calls the device's approximate rsqrtf, which no
 * host can restate: parity unpinned against the reference's hardware for this one function).
 * out = bf16((v * inv) * (f32(w) + 1)), had32, Q1. */
void w4a8_add_rms_quant_had_row(const uint16_t *y, const uint16_t *res, const uint16_t *w, const float *t, int K,
                                float eps, int T, int8_t *q, float *scale, uint16_t *res_out) {
  float *v = (float *)malloc(sizeof(float) * (size_t)K);
  float *part = (float *)calloc((size_t)T, sizeof(float));
  const int KV = K >> 3;
  for (int k = 0; k < K; ++k) {
    volatile float s = w4a8_bf16_f32(y[k]) + w4a8_bf16_f32(res[k]);
    v[k] = s;
    res_out[k] = w4a8_bf16_rne(s);
  }
  for (int tid = 0; tid < T; ++tid) {
    float ssq = 0.f;
    for (int g = tid; g < KV; g += T)
      for (int j = 0; j < 8; ++j) ssq = fmaf(v[g * 8 + j], v[g * 8 + j], ssq);
    part[tid] = ssq;
  }
  float wave[64];
  for (int wv = 0; wv < T / 32; ++wv) {
    float l[32];
    memcpy(l, part + wv * 32, sizeof l);
    for (int o = 16; o; o >>= 1)
      for (int i = 0; i < o; ++i) {
        volatile float s = l[i] + l[i + o];
        l[i] = s;
      }
    wave[wv] = l[0];
  }
  for (int o = T / 64; o; o >>= 1)
    for (int i = 0; i < o; ++i) {
      volatile float s = wave[i] + wave[i + o];
      wave[i] = s;
    }
  volatile float mean = wave[0] / (float)K;
  volatile float me = mean + eps;
  volatile float rt = sqrtf(me);
  volatile float inv = 1.f / rt;
  for (int k = 0; k < K; ++k) {
    volatile float a = v[k] * inv;
    volatile float wp = w4a8_bf16_f32(w[k]) + 1.f;
    volatile float b = a * wp;
    v[k] = w4a8_bf16_f32(w4a8_bf16_rne(b));
  }
  w4a8_had32_rows(v, t, 1, K);
  w4a8_quant_row(v, K, q, scale);
  free(part);
  free(v);
}

/* f32 silu of a bf16 input, z / (1 + expf(-z)), left unrounded: gdn_norm's gate
 * (hip/mxfp4_hadi8.hip:180-182). expf is the host's libm here and the device's own on a card, so a
 * checker that wants bit parity passes the device's table of all 65,536 values instead. */
float w4a8_silu_f32(uint16_t zb) {
  const float z = w4a8_bf16_f32(zb);
  volatile float e = expf(-z);
  volatile float d = 1.f + e;
  volatile float s = z / d;
  return s;
}
void w4a8_silu_f32_table(float *out) {
  for (int i = 0; i < 65536; ++i) out[i] = w4a8_silu_f32((uint16_t)i);
}

/* bf16( 1 / (1 + expf(-g)) ) for one bf16 input (hip/attn_glue_hadi8.hip:49). */
uint16_t w4a8_sigmoid_bf16(uint16_t gb) {
  const float g = w4a8_bf16_f32(gb);
  volatile float e = expf(-g);
  volatile float d = 1.f + e;
  volatile float s = 1.f / d;
  return w4a8_bf16_rne(s);
}

/* gdn_norm_quant_hadi8 (hip/mxfp4_hadi8.hip:148-186), one row of N = heads * 128 elements. Per
 * 128-element head, as its 16 lanes compute it: each lane's 8 elements give ssq = x1*x1, then
 * fma(x0, x0, ssq), then fma over x2..x7; the 16 lane sums meet in the xor butterfly 8, 4, 2, 1
 * (every lane ends with the same bits, additions being commutative). inv = 1 / sqrt(ssq * (1/128)
 * + eps) with IEEE sqrt and divide (the reference calls the device's approximate rsqrtf: parity
 * unpinned against the reference's hardware for that one function). out = bf16(((x * inv) * w[j])
 * * silu_f32(z)), had32, Q1. `silu_tab`: 65,536 f32 indexed by z's bits, or NULL for libm. */
void w4a8_gdn_norm_quant_had_row(const uint16_t *x, const uint16_t *z, const uint16_t *w, const float *t,
                                 const float *silu_tab, int N, float eps, int8_t *q, float *scale) {
  float *v = (float *)malloc(sizeof(float) * (size_t)N);
  for (int h = 0; h < N; h += 128) {
    float lane[16];
    for (int l = 0; l < 16; ++l) {
      const uint16_t *xl = x + h + l * 8;
      const float x0 = w4a8_bf16_f32(xl[0]), x1 = w4a8_bf16_f32(xl[1]);
      volatile float s = x1 * x1;
      float ssq = fmaf(x0, x0, s);
      for (int j = 2; j < 8; ++j) ssq = fmaf(w4a8_bf16_f32(xl[j]), w4a8_bf16_f32(xl[j]), ssq);
      lane[l] = ssq;
    }
    for (int o = 8; o; o >>= 1) {
      float nx[16];
      for (int l = 0; l < 16; ++l) {
        volatile float s = lane[l] + lane[l ^ o];
        nx[l] = s;
      }
      memcpy(lane, nx, sizeof nx);
    }
    volatile float mean = lane[0] * (1.f / 128.f);
    volatile float me = mean + eps;
    volatile float rt = sqrtf(me);
    volatile float inv = 1.f / rt;
    for (int j = 0; j < 128; ++j) {
      const float sg = silu_tab ? silu_tab[z[h + j]] : w4a8_silu_f32(z[h + j]);
      volatile float a = w4a8_bf16_f32(x[h + j]) * inv;
      volatile float b = a * w4a8_bf16_f32(w[j]);
      volatile float c = b * sg;
      v[h + j] = w4a8_bf16_f32(w4a8_bf16_rne(c));
    }
  }
  w4a8_had32_rows(v, t, 1, N);
  w4a8_quant_row(v, N, q, scale);
  free(v);
}

/* attn_gate_quant_hadi8 (hip/attn_glue_hadi8.hip:23-79), one row: `gate` is the row of the
 * projection's [q | gate] block, head h's gate values at h*2*hd + hd; p = bf16(core * bf16(sigmoid
 * (gate))), had32, Q1. */
void w4a8_attn_gate_quant_had_row(const uint16_t *core, const uint16_t *gate, const float *t, int n, int hd,
                                  int8_t *q, float *scale) {
  float *v = (float *)malloc(sizeof(float) * (size_t)n);
  for (int e = 0; e < n; ++e) {
    const int h = e / hd, o = e - h * hd;
    const float sig = w4a8_bf16_f32(w4a8_sigmoid_bf16(gate[(size_t)h * 2 * hd + hd + o]));
    volatile float p = w4a8_bf16_f32(core[e]) * sig;
    v[e] = w4a8_bf16_f32(w4a8_bf16_rne(p));
  }
  w4a8_had32_rows(v, t, 1, n);
  w4a8_quant_row(v, n, q, scale);
  free(v);
}
