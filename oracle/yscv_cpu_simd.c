/*
 * TEST / BENCHMARK INFRASTRUCTURE ONLY -- restatement of the reference's
 * runtime-dispatched x86 SIMD kernels, used to time "the reference's CPU path"
 * beside the GPU numbers.  Never linked into the shipped library.
 *
 * Each kernel restates the vector algorithm (same lane width, same reduction
 * points, same FMA use) of the Rust function it cites, so its speed and its
 * rounding behaviour are those of the reference's dispatch path:
 *   packed_int4_gemv_avx512   crates/yscv-kernels/src/ops/int4_matmul.rs:243-307
 *   packed_int4_gemv_avx2     crates/yscv-kernels/src/ops/int4_matmul.rs:170-229
 *   packed_int4_gemm_avx2     crates/yscv-kernels/src/ops/int4_matmul.rs:439-489
 *   int8_matmul_avx512_vnni   crates/yscv-kernels/src/ops/int8_matmul.rs:2100-2159
 *     (+ _blocked MR4xNR16    crates/yscv-kernels/src/ops/int8_matmul.rs:1850-1925)
 * The dispatchers follow int4_matmul.rs:310-377, :548-605 and the shape gates
 * of int8_matmul.rs:2114-2124.  The reference runs these single-threaded; the
 * `_mt` entry points add an N-row (int4) / M-row-block (int8) OpenMP partition
 * that the reference does not have for MatMul, and are labelled as such by the
 * benchmark.
 *
 * Checked against the scalar restatement in yscv_oracle.c: bitwise for int8,
 * within the reference's own test tolerances (1e-4 GEMV, 1e-3 GEMM) for int4.
 */
#include <immintrin.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define SIMD_API __attribute__((visibility("default")))

/* scalar kernels live in yscv_oracle.c */
void orc_packed_int4_gemv_scalar(const uint8_t *, const float *, const float *, float *, size_t,
                                 size_t, size_t);
void orc_packed_int4_gemm_scalar(const uint8_t *, const float *, const float *, float *, size_t,
                                 size_t, size_t, size_t);
void orc_int8_matmul_scalar(const int8_t *, const int8_t *, size_t, size_t, size_t, int32_t *);
void orc_transpose_b(const int8_t *, size_t, size_t, int8_t *);
int8_t orc_unpack_low(uint8_t);
int8_t orc_unpack_high(uint8_t);

static int has_avx512bw(void) {
  return __builtin_cpu_supports("avx512f") && __builtin_cpu_supports("avx512bw");
}
static int has_avx512vnni(void) { return has_avx512bw() && __builtin_cpu_supports("avx512vnni"); }
static int has_avx2fma(void) {
  return __builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma");
}

/* 0 scalar, 1 avx2, 2 avx512 -- what the int4 GEMV dispatcher would pick for g. */
SIMD_API int simd_int4_gemv_path(size_t group_size) {
  if (has_avx512bw() && group_size % 32 == 0) return 2;
  if (has_avx2fma() && group_size % 16 == 0) return 1;
  return 0;
}
SIMD_API int simd_int4_gemm_path(size_t group_size) {
  if (has_avx2fma() && group_size % 8 == 0 && group_size <= 256) return 1;
  return 0;
}
/* 0 scalar, 3 avx512-vnni */
SIMD_API int simd_int8_path(void) { return has_avx512vnni() ? 3 : 0; }

/* ---- int4 GEMV, AVX-512 ---------------------------------------------------- */
__attribute__((target("avx512f,avx512bw,avx512vl,avx2,fma"))) static void
int4_gemv_avx512(const uint8_t *w, const float *scales, const float *x, float *out, size_t row0,
                 size_t row1, size_t k, size_t g) {
  size_t groups = k / g;
  size_t blocks = g / 32;
  const __m512i idx_even = _mm512_setr_epi32(0, 2, 4, 6, 8, 10, 12, 14, 16, 18, 20, 22, 24, 26, 28, 30);
  const __m512i idx_odd = _mm512_setr_epi32(1, 3, 5, 7, 9, 11, 13, 15, 17, 19, 21, 23, 25, 27, 29, 31);
  for (size_t row = row0; row < row1; row++) {
    const uint8_t *rb = w + row * k / 2;
    const float *rs = scales + row * groups;
    __m512 acc_total = _mm512_setzero_ps();
    for (size_t gi = 0; gi < groups; gi++) {
      __m512 scale_v = _mm512_set1_ps(rs[gi]);
      __m512 group_acc = _mm512_setzero_ps();
      for (size_t blk = 0; blk < blocks; blk++) {
        size_t byte_off = gi * g / 2 + blk * 16;
        size_t act_off = gi * g + blk * 32;
        __m128i packed = _mm_loadu_si128((const __m128i *)(rb + byte_off));
        __m256i p16 = _mm256_cvtepu8_epi16(packed);
        __m256i lo = _mm256_srai_epi16(_mm256_slli_epi16(p16, 12), 12);
        __m256i hi = _mm256_srai_epi16(_mm256_slli_epi16(p16, 8), 12);
        __m512 lo_f = _mm512_cvtepi32_ps(_mm512_cvtepi16_epi32(lo));
        __m512 hi_f = _mm512_cvtepi32_ps(_mm512_cvtepi16_epi32(hi));
        __m512 a0 = _mm512_loadu_ps(x + act_off);
        __m512 a1 = _mm512_loadu_ps(x + act_off + 16);
        __m512 a_even = _mm512_permutex2var_ps(a0, idx_even, a1);
        __m512 a_odd = _mm512_permutex2var_ps(a0, idx_odd, a1);
        group_acc = _mm512_fmadd_ps(lo_f, a_even, group_acc);
        group_acc = _mm512_fmadd_ps(hi_f, a_odd, group_acc);
      }
      acc_total = _mm512_fmadd_ps(group_acc, scale_v, acc_total);
    }
    out[row] = _mm512_reduce_add_ps(acc_total);
  }
}

/* ---- int4 GEMV, AVX2 --------------------------------------------------------- */
__attribute__((target("avx2,fma"))) static void int4_gemv_avx2(const uint8_t *w,
                                                                const float *scales,
                                                                const float *x, float *out,
                                                                size_t row0, size_t row1,
                                                                size_t k, size_t g) {
  size_t groups = k / g;
  for (size_t row = row0; row < row1; row++) {
    const uint8_t *rb = w + row * k / 2;
    const float *rs = scales + row * groups;
    float acc = 0.0f;
    for (size_t gi = 0; gi < groups; gi++) {
      size_t byte_base = gi * g / 2, act_base = gi * g;
      __m256 group_acc = _mm256_setzero_ps();
      size_t i = 0;
      while (i + 8 <= g / 2) {
        float inter[16];
        for (int j = 0; j < 8; j++) {
          uint8_t byte = rb[byte_base + i + j];
          inter[2 * j] = (float)orc_unpack_low(byte);
          inter[2 * j + 1] = (float)orc_unpack_high(byte);
        }
        const float *as = x + act_base + 2 * i;
        group_acc = _mm256_fmadd_ps(_mm256_loadu_ps(inter), _mm256_loadu_ps(as), group_acc);
        group_acc = _mm256_fmadd_ps(_mm256_loadu_ps(inter + 8), _mm256_loadu_ps(as + 8), group_acc);
        i += 8;
      }
      float buf[8];
      _mm256_storeu_ps(buf, group_acc);
      float total = 0.0f;
      for (int j = 0; j < 8; j++) total += buf[j];
      while (i < g / 2) {
        uint8_t byte = rb[byte_base + i];
        total += (float)orc_unpack_low(byte) * x[act_base + 2 * i];
        total += (float)orc_unpack_high(byte) * x[act_base + 2 * i + 1];
        i++;
      }
      acc += rs[gi] * total;
    }
    out[row] = acc;
  }
}

/* packed_int4_gemv_dispatch, rows [row0,row1) */
static void int4_gemv_rows(const uint8_t *w, const float *s, const float *x, float *out,
                           size_t row0, size_t row1, size_t k, size_t g) {
  int path = simd_int4_gemv_path(g);
  if (path == 2)
    int4_gemv_avx512(w, s, x, out, row0, row1, k, g);
  else if (path == 1)
    int4_gemv_avx2(w, s, x, out, row0, row1, k, g);
  else
    orc_packed_int4_gemv_scalar(w + row0 * k / 2, s + row0 * (k / g), x, out + row0, row1 - row0,
                                k, g);
}

SIMD_API void simd_packed_int4_gemv_dispatch(const uint8_t *w, const float *s, const float *x,
                                             float *out, size_t m_w, size_t k, size_t g) {
  int4_gemv_rows(w, s, x, out, 0, m_w, k, g);
}

SIMD_API void simd_packed_int4_gemv_dispatch_mt(const uint8_t *w, const float *s, const float *x,
                                                float *out, size_t m_w, size_t k, size_t g,
                                                int threads) {
  size_t chunk = (m_w + (size_t)threads - 1) / (size_t)threads;
#pragma omp parallel for num_threads(threads) schedule(static)
  for (int t = 0; t < threads; t++) {
    size_t r0 = (size_t)t * chunk, r1 = r0 + chunk;
    if (r1 > m_w) r1 = m_w;
    if (r0 < r1) int4_gemv_rows(w, s, x, out, r0, r1, k, g);
  }
}

/* ---- int4 GEMM, AVX2 (the widest GEMM variant the reference has) -------------- */
__attribute__((target("avx2,fma"))) static void int4_gemm_avx2_rows(
    const uint8_t *w, const float *scales, const float *x, float *out, size_t m, size_t n,
    size_t n0, size_t n1, size_t k, size_t g) {
  size_t groups = k / g;
  float unpacked[256];
  for (size_t nn = n0; nn < n1; nn++) {
    const uint8_t *rb = w + nn * k / 2;
    const float *rs = scales + nn * groups;
    for (size_t gi = 0; gi < groups; gi++) {
      float scale = rs[gi];
      size_t byte_base = gi * g / 2, act_base = gi * g;
      for (size_t i = 0; i < g / 2; i++) {
        uint8_t byte = rb[byte_base + i];
        unpacked[2 * i] = (float)orc_unpack_low(byte);
        unpacked[2 * i + 1] = (float)orc_unpack_high(byte);
      }
      for (size_t mi = 0; mi < m; mi++) {
        const float *ar = x + mi * k + act_base;
        __m256 acc = _mm256_setzero_ps();
        size_t j = 0;
        while (j + 8 <= g) {
          acc = _mm256_fmadd_ps(_mm256_loadu_ps(unpacked + j), _mm256_loadu_ps(ar + j), acc);
          j += 8;
        }
        float buf[8];
        _mm256_storeu_ps(buf, acc);
        float sum = 0.0f;
        for (int t = 0; t < 8; t++) sum += buf[t];
        while (j < g) {
          sum += unpacked[j] * ar[j];
          j++;
        }
        out[mi * n + nn] += scale * sum;
      }
    }
  }
}

SIMD_API void simd_packed_int4_gemm_dispatch(const uint8_t *w, const float *s, const float *x,
                                             float *out, size_t m, size_t n, size_t k, size_t g) {
  if (simd_int4_gemm_path(g) == 1) {
    memset(out, 0, sizeof(float) * m * n);
    int4_gemm_avx2_rows(w, s, x, out, m, n, 0, n, k, g);
  } else {
    orc_packed_int4_gemm_scalar(w, s, x, out, m, n, k, g);
  }
}

SIMD_API void simd_packed_int4_gemm_dispatch_mt(const uint8_t *w, const float *s, const float *x,
                                                float *out, size_t m, size_t n, size_t k,
                                                size_t g, int threads) {
  if (simd_int4_gemm_path(g) != 1) {
    orc_packed_int4_gemm_scalar(w, s, x, out, m, n, k, g);
    return;
  }
  memset(out, 0, sizeof(float) * m * n);
  size_t chunk = (n + (size_t)threads - 1) / (size_t)threads;
#pragma omp parallel for num_threads(threads) schedule(static)
  for (int t = 0; t < threads; t++) {
    size_t r0 = (size_t)t * chunk, r1 = r0 + chunk;
    if (r1 > n) r1 = n;
    if (r0 < r1) int4_gemm_avx2_rows(w, s, x, out, m, n, r0, r1, k, g);
  }
}

/* ---- int8 GEMM, AVX-512-VNNI ------------------------------------------------- */
/* pack_b_vnni_4x16, int8_matmul.rs:1815-1835 */
static int8_t *pack_b_vnni_4x16(const int8_t *b, size_t k, size_t n, size_t *k4_full_out) {
  size_t k4_full = (k / 4) * 4, groups = k4_full / 4, n_panels = n / 16;
  int8_t *bp = (int8_t *)malloc(n_panels * groups * 64 + 64);
  for (size_t jp = 0; jp < n_panels; jp++)
    for (size_t g = 0; g < groups; g++)
      for (size_t c = 0; c < 16; c++)
        for (size_t r = 0; r < 4; r++)
          bp[jp * groups * 64 + g * 64 + c * 4 + r] = b[(g * 4 + r) * n + jp * 16 + c];
  *k4_full_out = k4_full;
  return bp;
}

__attribute__((target("avx512f,avx512bw,avx512vl,avx512vnni"))) static void
int8_vnni_blocked_rows(const int8_t *a, const int8_t *b, const int8_t *bp, const int32_t *col_sum,
                       size_t k4_full, size_t m0, size_t m1, size_t k, size_t n, int32_t *out) {
  size_t groups = k4_full / 4, n_panels = n / 16;
  const __m512i bias_xor = _mm512_set1_epi8((char)-128);
  for (size_t ib = m0; ib < m1; ib += 4) {
    for (size_t jp = 0; jp < n_panels; jp++) {
      __m512i a0 = _mm512_setzero_si512(), a1 = a0, a2 = a0, a3 = a0;
      const int8_t *panel = bp + jp * groups * 64;
      for (size_t g = 0; g < groups; g++) {
        __m512i bv = _mm512_loadu_si512((const void *)(panel + g * 64));
        size_t k_idx = g * 4;
        int32_t p0, p1, p2, p3;
        memcpy(&p0, a + ib * k + k_idx, 4);
        memcpy(&p1, a + (ib + 1) * k + k_idx, 4);
        memcpy(&p2, a + (ib + 2) * k + k_idx, 4);
        memcpy(&p3, a + (ib + 3) * k + k_idx, 4);
        a0 = _mm512_dpbusd_epi32(a0, _mm512_xor_si512(_mm512_set1_epi32(p0), bias_xor), bv);
        a1 = _mm512_dpbusd_epi32(a1, _mm512_xor_si512(_mm512_set1_epi32(p1), bias_xor), bv);
        a2 = _mm512_dpbusd_epi32(a2, _mm512_xor_si512(_mm512_set1_epi32(p2), bias_xor), bv);
        a3 = _mm512_dpbusd_epi32(a3, _mm512_xor_si512(_mm512_set1_epi32(p3), bias_xor), bv);
      }
      int32_t buf[4][16];
      _mm512_storeu_si512((void *)buf[0], a0);
      _mm512_storeu_si512((void *)buf[1], a1);
      _mm512_storeu_si512((void *)buf[2], a2);
      _mm512_storeu_si512((void *)buf[3], a3);
      for (size_t r = 0; r < 4; r++)
        for (size_t c = 0; c < 16; c++) {
          size_t n_idx = jp * 16 + c;
          int32_t v = buf[r][c] - 128 * col_sum[n_idx];
          for (size_t kk = k4_full; kk < k; kk++)
            v += (int32_t)a[(ib + r) * k + kk] * (int32_t)b[kk * n + n_idx];
          out[(ib + r) * n + n_idx] = v;
        }
    }
  }
}

/* simple transposed-B kernel, int8_matmul.rs:2125-2158 / :2176-2207 */
__attribute__((target("avx512f,avx512bw,avx512vl,avx512vnni"))) static void
int8_vnni_bt_rows(const int8_t *a, const int8_t *bt, const int32_t *col_sum, size_t m0, size_t m1,
                  size_t k, size_t n, int32_t *out) {
  const __m512i bias128 = _mm512_set1_epi8((char)-128);
  for (size_t i = m0; i < m1; i++) {
    for (size_t j = 0; j < n; j++) {
      __m512i acc = _mm512_setzero_si512();
      size_t kk = 0;
      while (kk + 64 <= k) {
        __m512i av = _mm512_loadu_si512((const void *)(a + i * k + kk));
        __m512i bv = _mm512_loadu_si512((const void *)(bt + j * k + kk));
        acc = _mm512_dpbusd_epi32(acc, _mm512_xor_si512(av, bias128), bv);
        kk += 64;
      }
      int32_t tail = _mm512_reduce_add_epi32(acc) - 128 * col_sum[j];
      while (kk < k) {
        tail += (int32_t)a[i * k + kk] * (int32_t)bt[j * k + kk];
        kk++;
      }
      out[i * n + j] = tail;
    }
  }
}

static int blocked_gate(size_t m, size_t k, size_t n) {
  /* MR8 gate (k >= 8000 && n <= 2048) is not restated: no BASELINE shape reaches it. */
  return m >= 4 && m % 4 == 0 && n % 16 == 0 && k >= 4 && (k * n <= 1000000 || n >= 16384);
}

/*
 * Prepacked handle = what pack_i8_b_for_matmul builds once at load time
 * (int8_matmul.rs:163-191): B transposed, the VNNI 4x16 panel and its column sums.
 */
typedef struct {
  size_t k, n, k4_full;
  int8_t *bt;
  int8_t *bp;          /* NULL unless n % 16 == 0 && k >= 4 */
  int32_t *col_sum_bp; /* over [0,k4_full) */
  int32_t *col_sum_bt; /* over [0,(k/64)*64) */
} simd_packed_i8b;

SIMD_API simd_packed_i8b *simd_pack_i8_b_for_matmul(const int8_t *b, size_t k, size_t n) {
  simd_packed_i8b *p = (simd_packed_i8b *)calloc(1, sizeof(*p));
  p->k = k;
  p->n = n;
  p->bt = (int8_t *)malloc(k * n + 64);
  orc_transpose_b(b, k, n, p->bt);
  if (n % 16 == 0 && k >= 4) {
    p->bp = pack_b_vnni_4x16(b, k, n, &p->k4_full);
    p->col_sum_bp = (int32_t *)malloc(sizeof(int32_t) * n);
    for (size_t j = 0; j < n; j++) {
      int32_t s = 0;
      for (size_t kk = 0; kk < p->k4_full; kk++) s += b[kk * n + j];
      p->col_sum_bp[j] = s;
    }
  }
  return p;
}
SIMD_API void simd_packed_i8b_free(simd_packed_i8b *p) {
  if (!p) return;
  free(p->bt);
  free(p->bp);
  free(p->col_sum_bp);
  free(p->col_sum_bt);
  free(p);
}

/* int8_matmul_prepacked_dispatch (int8_matmul.rs:2420-2425 -> :2163-2208).  The
 * simple kernel recomputes its column sums on every call, as the reference does. */
static void int8_prepacked_rows(const int8_t *a, const simd_packed_i8b *p, const int8_t *b_kn,
                                size_t m_total, size_t m0, size_t m1, int32_t *out,
                                const int32_t *col_sum_bt) {
  size_t k = p->k, n = p->n;
  if (p->bp && blocked_gate(m_total, k, n)) {
    /* K tail of the blocked kernel reads B in [k][n] order; the reference's
       prepacked variant reads it from bt -- same values. */
    int8_vnni_blocked_rows(a, b_kn, p->bp, p->col_sum_bp, p->k4_full, m0, m1, k, n, out);
    return;
  }
  int8_vnni_bt_rows(a, p->bt, col_sum_bt, m0, m1, k, n, out);
}

static int32_t *bt_col_sums(const simd_packed_i8b *p) {
  size_t k = p->k, n = p->n, k_vnni = (k / 64) * 64;
  int32_t *cs = (int32_t *)malloc(sizeof(int32_t) * n);
  for (size_t j = 0; j < n; j++) {
    int32_t s = 0;
    for (size_t kk = 0; kk < k_vnni; kk++) s += p->bt[j * k + kk];
    cs[j] = s;
  }
  return cs;
}

/* b_kn: the original [k][n] matrix (only read for the <=3-element K tail of the blocked kernel). */
SIMD_API void simd_int8_matmul_prepacked_dispatch(const int8_t *a, const simd_packed_i8b *p,
                                                  const int8_t *b_kn, size_t m, int32_t *out) {
  if (simd_int8_path() != 3) {
    orc_int8_matmul_scalar(a, b_kn, m, p->k, p->n, out);
    return;
  }
  int32_t *cs = bt_col_sums(p);
  int8_prepacked_rows(a, p, b_kn, m, 0, m, out, cs);
  free(cs);
}

/* M-row-block partition as crates/yscv-onnx/src/runner/conv/quantized.rs:410-445 does for
 * QLinearConv; not present in the reference for MatMul. */
SIMD_API void simd_int8_matmul_prepacked_dispatch_mt(const int8_t *a, const simd_packed_i8b *p,
                                                     const int8_t *b_kn, size_t m, int32_t *out,
                                                     int threads) {
  if (simd_int8_path() != 3) {
    orc_int8_matmul_scalar(a, b_kn, m, p->k, p->n, out);
    return;
  }
  int32_t *cs = bt_col_sums(p);
  size_t blocks = (m + 3) / 4;
  size_t per = (blocks + (size_t)threads - 1) / (size_t)threads;
#pragma omp parallel for num_threads(threads) schedule(static)
  for (int t = 0; t < threads; t++) {
    size_t m0 = (size_t)t * per * 4, m1 = m0 + per * 4;
    if (m1 > m) m1 = m;
    if (m0 < m1) int8_prepacked_rows(a, p, b_kn, m, m0, m1, out, cs);
  }
  free(cs);
}

/* int8_matmul_dispatch (int8_matmul.rs:2407-2413 -> :2100-2159): packs B on every call. */
SIMD_API void simd_int8_matmul_dispatch(const int8_t *a, const int8_t *b, size_t m, size_t k,
                                        size_t n, int32_t *out) {
  if (simd_int8_path() != 3) {
    orc_int8_matmul_scalar(a, b, m, k, n, out);
    return;
  }
  if (blocked_gate(m, k, n)) {
    /* int8_matmul_avx512_vnni_blocked packs the 4x16 panel and its column sums per call */
    size_t k4_full;
    int8_t *bp = pack_b_vnni_4x16(b, k, n, &k4_full);
    int32_t *cs = (int32_t *)malloc(sizeof(int32_t) * n);
    for (size_t j = 0; j < n; j++) {
      int32_t s = 0;
      for (size_t kk = 0; kk < k4_full; kk++) s += b[kk * n + j];
      cs[j] = s;
    }
    int8_vnni_blocked_rows(a, b, bp, cs, k4_full, 0, m, k, n, out);
    free(cs);
    free(bp);
    return;
  }
  /* simple path: transpose B and sum its columns per call */
  int8_t *bt = (int8_t *)malloc(k * n + 64);
  orc_transpose_b(b, k, n, bt);
  size_t k_vnni = (k / 64) * 64;
  int32_t *cs = (int32_t *)malloc(sizeof(int32_t) * n);
  for (size_t j = 0; j < n; j++) {
    int32_t s = 0;
    for (size_t kk = 0; kk < k_vnni; kk++) s += bt[j * k + kk];
    cs[j] = s;
  }
  int8_vnni_bt_rows(a, bt, cs, 0, m, k, n, out);
  free(cs);
  free(bt);
}

SIMD_API int simd_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
