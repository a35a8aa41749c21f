/*
 * galois_oracle.c -- CPU restatement of the galois Q4_0 hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing shipped by the product may link, load or
 * call this file: it is the checker for the HIP kernels and the timed CPU
 * baseline.  Every function cites the reference file:line it restates
 * (paths relative to the szuwgh/galois tree).
 *
 * Parity status (what pins each function -- the reference's own tests hold no
 * golden vectors for this path, so all pins come from closed forms, invariants
 * and independent numpy/scipy restatements in tests/test_oracle_*.py):
 *   orc_f32_to_f16 / orc_f16_to_f32 .... exhaustive vs numpy float16 (IEEE RNE)
 *   orc_dequantize_row_q4_0 ............ hand-built blocks + brute force over nibbles x scales
 *   orc_quantize_row_q4_0 .............. canonical ggml definition (the reference's
 *                                        from_f32 is todo!(), src/ggml_quants.rs:198-200):
 *                                        hand-derived byte vectors, invariants, and an
 *                                        independent vectorised numpy implementation.
 *                                        Tie/truncation rules are pinned only by the published
 *                                        ggml definition: PARITY UNPINNED against galois itself.
 *   orc_quantize_row_q8_0 .............. hand-derived blocks, round-half-away cases, numpy twin
 *   orc_vec_dot_q4_0_q8_0_{scalar,avx2}  integer part exact vs numpy int64; avx2 == scalar up to
 *                                        f32 summation order
 *   orc_mul_mat_q4_0_f32 (dequant, f64)  numpy float64 matmul of the dequantized matrix; unit
 *                                        vectors; all-0x88 weights
 *   orc_cpu_mul_mat_q4_0_f32 ........... equals per-element orc_vec_dot on Q8_0 rows (structure
 *                                        only; it is the timing baseline, not the parity oracle)
 *   orc_rms_norm_f32 / orc_mul_f32 ..... closed form in numpy float64; constant-row case
 *   orc_rope_f32 ....................... closed form; pos=0 identity; norm preservation; additivity
 *   orc_soft_max_f32 ................... scipy.special.softmax in float64; row sums; -inf mask
 *   orc_add/scale/silu/cpy/get_rows .... numpy closed forms (transpose / astype(float16) / row gather)
 */
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#if defined(__AVX2__) && defined(__FMA__)
#include <immintrin.h>
#define ORC_HAVE_AVX2 1
#else
#define ORC_HAVE_AVX2 0
#endif

#define QK4_0 32
#define QK8_0 32

/* src/ggml_quants.rs:140-145 (#[repr(C)] BlockQ4_0) and
 * galois-kernels/src/matmul.cu:19-23 (block_q4_0): f16 scale then 16 nibble bytes. */
typedef struct {
    uint16_t d;
    uint8_t qs[QK4_0 / 2];
} orc_block_q4_0;

/* src/ggml_quants.rs:721-726 (BlockQ8_0): f16 scale then 32 signed bytes. */
typedef struct {
    uint16_t d;
    int8_t qs[QK8_0];
} orc_block_q8_0;

_Static_assert(sizeof(orc_block_q4_0) == 18, "Q4_0 block is 18 bytes");
_Static_assert(sizeof(orc_block_q8_0) == 34, "Q8_0 block is 34 bytes");

int orc_sizeof_block_q4_0(void) { return (int)sizeof(orc_block_q4_0); }
int orc_sizeof_block_q8_0(void) { return (int)sizeof(orc_block_q8_0); }
int orc_have_avx2(void) { return ORC_HAVE_AVX2; }

/* ------------------------------------------------------------------------- */
/* f16 <-> f32.  The reference uses the `half` crate (Cargo.toml:13):        */
/* f16::from_f32 is IEEE round-to-nearest-even, to_f32 is exact              */
/* (src/ggml_quants.rs:162,215,758).  Software version, no F16C needed.      */
/* ------------------------------------------------------------------------- */
static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    if (exp == 0) {
        if (man == 0) return bits_f32(sign);
        /* subnormal: value = man * 2^-24 */
        float v = (float)man * 5.9604644775390625e-8f;
        return sign ? -v : v;
    }
    if (exp == 31) return bits_f32(sign | 0x7F800000u | (man << 13));
    return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

uint16_t orc_f32_to_f16(float f) {
    uint32_t x = f32_bits(f);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t ax = x & 0x7FFFFFFFu;
    if (ax >= 0x7F800000u) { /* inf / nan */
        if (ax > 0x7F800000u) return (uint16_t)(sign | 0x7E00u | ((ax >> 13) & 0x3FFu));
        return (uint16_t)(sign | 0x7C00u);
    }
    if (ax >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u); /* rounds to >= 65520 -> inf */
    if (ax < 0x38800000u) {                                    /* below 2^-14: subnormal half */
        if (ax < 0x33000000u) return sign;                     /* < 2^-25 -> 0 (2^-25 itself ties to even = 0) */
        uint32_t e = ax >> 23;
        uint32_t m = (ax & 0x7FFFFFu) | 0x800000u;             /* 24-bit significand */
        uint32_t shift = 126u - e;                             /* result = m >> shift, in units of 2^-24 */
        uint32_t q = m >> shift;
        uint32_t rem = m & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1u);
        if (rem > half || (rem == half && (q & 1u))) q++;
        return (uint16_t)(sign | q);
    }
    uint32_t e = (ax >> 23) - 112u;
    uint32_t m = ax & 0x7FFFFFu;
    uint32_t q = (e << 10) | (m >> 13);
    uint32_t rem = m & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) q++;
    return (uint16_t)(sign | q);
}

void orc_f16_to_f32_row(const uint16_t *h, float *f, int64_t n) {
    for (int64_t i = 0; i < n; i++) f[i] = orc_f16_to_f32(h[i]);
}
void orc_f32_to_f16_row(const float *f, uint16_t *h, int64_t n) {
    for (int64_t i = 0; i < n; i++) h[i] = orc_f32_to_f16(f[i]);
}

/* ------------------------------------------------------------------------- */
/* Q4_0                                                                      */
/* ------------------------------------------------------------------------- */

/* Canonical ggml quantize_row_q4_0.  galois leaves BlockQ4_0::from_f32 as
 * todo!() (src/ggml_quants.rs:198-200); the layout it must produce is fixed by
 * to_f32 (src/ggml_quants.rs:209-228).  Per block: the element of largest
 * magnitude (first wins) keeps its sign, d = max / -8, id = 1/d (0 if d == 0)
 * from the unrounded f32 d, q = min(15, (int8)(x*id + 8.5)). */
void orc_quantize_row_q4_0(const float *x, void *vy, int64_t k) {
    orc_block_q4_0 *y = (orc_block_q4_0 *)vy;
    const int64_t nb = k / QK4_0;
    for (int64_t i = 0; i < nb; i++) {
        float amax = 0.0f, max = 0.0f;
        for (int j = 0; j < QK4_0; j++) {
            const float v = x[i * QK4_0 + j];
            if (amax < fabsf(v)) { amax = fabsf(v); max = v; }
        }
        const float d = max / -8.0f;
        const float id = d != 0.0f ? 1.0f / d : 0.0f;
        y[i].d = orc_f32_to_f16(d);
        for (int j = 0; j < QK4_0 / 2; j++) {
            const float x0 = x[i * QK4_0 + j] * id;
            const float x1 = x[i * QK4_0 + QK4_0 / 2 + j] * id;
            int8_t q0 = (int8_t)(x0 + 8.5f);
            int8_t q1 = (int8_t)(x1 + 8.5f);
            const uint8_t u0 = (uint8_t)(q0 < 15 ? q0 : 15);
            const uint8_t u1 = (uint8_t)(q1 < 15 ? q1 : 15);
            y[i].qs[j] = (uint8_t)(u0 | (u1 << 4));
        }
    }
}

/* BlockQ4_0::to_f32, src/ggml_quants.rs:209-228 (device twin dequantize_q4_0,
 * galois-kernels/src/matmul.cu:25-43): weight j = low nibble of qs[j], weight
 * j+16 = high nibble; value = (nibble - 8) * f32(d). */
void orc_dequantize_row_q4_0(const void *vx, float *y, int64_t k) {
    const orc_block_q4_0 *x = (const orc_block_q4_0 *)vx;
    const int64_t nb = k / QK4_0;
    for (int64_t i = 0; i < nb; i++) {
        const float d = orc_f16_to_f32(x[i].d);
        for (int j = 0; j < QK4_0 / 2; j++) {
            const int lo = (x[i].qs[j] & 0x0F) - 8;
            const int hi = (x[i].qs[j] >> 4) - 8;
            y[i * QK4_0 + j] = (float)lo * d;
            y[i * QK4_0 + j + QK4_0 / 2] = (float)hi * d;
        }
    }
}

/* ------------------------------------------------------------------------- */
/* Q8_0 activations + the reference CPU dot                                  */
/* ------------------------------------------------------------------------- */

/* BlockQ8_0::from_f32, src/ggml_quants.rs:736-764: d = amax/127 (f32),
 * id = 1/d from the unrounded d, q = f32::round (half away from zero). */
void orc_quantize_row_q8_0(const float *x, void *vy, int64_t k) {
    orc_block_q8_0 *y = (orc_block_q8_0 *)vy;
    const int64_t nb = k / QK8_0;
    for (int64_t i = 0; i < nb; i++) {
        float amax = 0.0f;
        for (int j = 0; j < QK8_0; j++) amax = fmaxf(amax, fabsf(x[i * QK8_0 + j]));
        const float d = amax / 127.0f;
        const float id = d != 0.0f ? 1.0f / d : 0.0f;
        y[i].d = orc_f32_to_f16(d);
        for (int j = 0; j < QK8_0; j++) y[i].qs[j] = (int8_t)roundf(x[i * QK8_0 + j] * id);
    }
}

/* BlockQ4_0::vec_dot_unopt, src/ggml_quants.rs:174-191. */
float orc_vec_dot_q4_0_q8_0_scalar(int64_t n, const void *vx, const void *vy) {
    const orc_block_q4_0 *x = (const orc_block_q4_0 *)vx;
    const orc_block_q8_0 *y = (const orc_block_q8_0 *)vy;
    const int64_t nb = n / QK8_0;
    float sumf = 0.0f;
    for (int64_t i = 0; i < nb; i++) {
        int sumi = 0;
        for (int j = 0; j < QK8_0 / 2; j++) {
            const int v0 = (x[i].qs[j] & 0x0F) - 8;
            const int v1 = (x[i].qs[j] >> 4) - 8;
            sumi += v0 * y[i].qs[j] + v1 * y[i].qs[j + QK8_0 / 2];
        }
        sumf += (float)sumi * orc_f16_to_f32(x[i].d) * orc_f16_to_f32(y[i].d);
    }
    return sumf;
}

#if ORC_HAVE_AVX2
/* BlockQ4_0::vec_dot_q8_0 (AVX2), src/ggml_quants.rs:156-172, with its helpers
 * bytes_from_nibbles_32 (:78-83), mul_sum_i8_pairs_float (:86-90),
 * mul_sum_us8_pairs_float (:63-66), sum_i16_pairs_float (:56-60) and
 * hsum_float_8 (:69-75): same intrinsic sequence, same accumulation order. */
static inline float orc_hsum8(__m256 v) {
    __m128 r = _mm256_extractf128_ps(v, 1);
    r = _mm_add_ps(r, _mm256_castps256_ps128(v));
    r = _mm_add_ps(r, _mm_movehl_ps(r, r));
    r = _mm_add_ss(r, _mm_movehdup_ps(r));
    return _mm_cvtss_f32(r);
}
float orc_vec_dot_q4_0_q8_0_avx2(int64_t n, const void *vx, const void *vy) {
    const orc_block_q4_0 *x = (const orc_block_q4_0 *)vx;
    const orc_block_q8_0 *y = (const orc_block_q8_0 *)vy;
    const int64_t nb = n / QK8_0;
    const __m256i lowmask = _mm256_set1_epi8(0x0F);
    const __m256i eight = _mm256_set1_epi8(8);
    const __m256i ones16 = _mm256_set1_epi16(1);
    __m256 acc = _mm256_setzero_ps();
    for (int64_t i = 0; i < nb; i++) {
        const __m256 d = _mm256_set1_ps(orc_f16_to_f32(x[i].d) * orc_f16_to_f32(y[i].d));
        const __m128i raw = _mm_loadu_si128((const __m128i *)x[i].qs);
        __m256i bx = _mm256_insertf128_si256(_mm256_castsi128_si256(raw), _mm_srli_epi16(raw, 4), 1);
        bx = _mm256_sub_epi8(_mm256_and_si256(lowmask, bx), eight);
        const __m256i by = _mm256_loadu_si256((const __m256i *)y[i].qs);
        const __m256i ax = _mm256_sign_epi8(bx, bx);
        const __m256i sy = _mm256_sign_epi8(by, bx);
        const __m256i dot16 = _mm256_maddubs_epi16(ax, sy);
        const __m256 q = _mm256_cvtepi32_ps(_mm256_madd_epi16(ones16, dot16));
        acc = _mm256_fmadd_ps(d, q, acc);
    }
    return orc_hsum8(acc);
}
#else
float orc_vec_dot_q4_0_q8_0_avx2(int64_t n, const void *vx, const void *vy) {
    return orc_vec_dot_q4_0_q8_0_scalar(n, vx, vy);
}
#endif

/* QuantType::vec_dot dispatch, src/ggml_quants.rs:202-207: AVX when built with it. */
static inline float orc_vec_dot(int64_t n, const void *x, const void *y) {
#if ORC_HAVE_AVX2
    return orc_vec_dot_q4_0_q8_0_avx2(n, x, y);
#else
    return orc_vec_dot_q4_0_q8_0_scalar(n, x, y);
#endif
}

/* ------------------------------------------------------------------------- */
/* Parity oracle for the matmul: dequant-then-dot, f64 accumulation.         */
/* Semantics of dequantize_mul_mat_vec_q4_0 (galois-kernels/src/matmul.cu:   */
/* 45-117): dst[row] = sum_col (q-8)*d * y[col]; M>1 is the same contraction */
/* per activation row with dst[m*N + n] (matmul.cu:359, src/op.rs:1534-1544).*/
/* ------------------------------------------------------------------------- */
typedef struct {
    const orc_block_q4_0 *W;
    const float *X;
    float *Y;
    int64_t K, N, M, n0, n1;
} orc_mm_job;

static void *orc_mm_worker(void *p) {
    orc_mm_job *j = (orc_mm_job *)p;
    const int64_t nb = j->K / QK4_0;
    float *wrow = (float *)malloc(sizeof(float) * (size_t)j->K);
    for (int64_t n = j->n0; n < j->n1; n++) {
        orc_dequantize_row_q4_0(j->W + n * nb, wrow, j->K);
        for (int64_t m = 0; m < j->M; m++) {
            const float *x = j->X + m * j->K;
            double acc = 0.0;
            for (int64_t k = 0; k < j->K; k++) acc += (double)wrow[k] * (double)x[k];
            j->Y[m * j->N + n] = (float)acc;
        }
    }
    free(wrow);
    return NULL;
}

void orc_mul_mat_q4_0_f32(const void *W, const float *X, float *Y, int64_t K, int64_t N,
                          int64_t M, int nthreads) {
    if (nthreads < 1) nthreads = 1;
    if (nthreads > 64) nthreads = 64;
    pthread_t th[64];
    orc_mm_job jobs[64];
    const int64_t per = (N + nthreads - 1) / nthreads;
    for (int t = 0; t < nthreads; t++) {
        int64_t n0 = per * t, n1 = n0 + per;
        if (n0 > N) n0 = N;
        if (n1 > N) n1 = N;
        jobs[t] = (orc_mm_job){(const orc_block_q4_0 *)W, X, Y, K, N, M, n0, n1};
        pthread_create(&th[t], NULL, orc_mm_worker, &jobs[t]);
    }
    for (int t = 0; t < nthreads; t++) pthread_join(th[t], NULL);
}

/* ------------------------------------------------------------------------- */
/* The reference CPU op MatMul::f_q_f32_f32 (src/op.rs:1383-1598): the timed */
/* baseline.  (i) every activation row -> Q8_0 (:1397-1420); (ii) `nth` tasks */
/* split the larger of (weight rows, activation rows) (:1487-1511; the        */
/* reference hard-codes nth = 4 at :1438); (iii) 16x16 blocked loops calling  */
/* vec_dot per output (:1512-1548).  2-D operands only (ne2 = ne3 = 1).       */
/* ------------------------------------------------------------------------- */
typedef struct {
    const orc_block_q4_0 *W;
    const orc_block_q8_0 *Xq;
    float *Y;
    int64_t K, N, M;
    int64_t ir0_lo, ir0_hi, ir1_lo, ir1_hi;
} orc_cpu_job;

static void *orc_cpu_worker(void *p) {
    orc_cpu_job *j = (orc_cpu_job *)p;
    const int64_t nb = j->K / QK8_0;
    const int64_t blck0 = 16, blck1 = 16;
    for (int64_t iir1 = j->ir1_lo; iir1 < j->ir1_hi; iir1 += blck1) {
        for (int64_t iir0 = j->ir0_lo; iir0 < j->ir0_hi; iir0 += blck0) {
            const int64_t e1 = iir1 + blck1 < j->ir1_hi ? iir1 + blck1 : j->ir1_hi;
            const int64_t e0 = iir0 + blck0 < j->ir0_hi ? iir0 + blck0 : j->ir0_hi;
            for (int64_t ir1 = iir1; ir1 < e1; ir1++) {
                const orc_block_q8_0 *xcol = j->Xq + ir1 * nb;
                float *d = j->Y + ir1 * j->N;
                for (int64_t ir0 = iir0; ir0 < e0; ir0++)
                    d[ir0] = orc_vec_dot(j->K, j->W + ir0 * nb, xcol);
            }
        }
    }
    return NULL;
}

void orc_cpu_mul_mat_q4_0_f32(const void *W, const float *X, float *Y, int64_t K, int64_t N,
                              int64_t M, int nth) {
    if (nth < 1) nth = 1;
    if (nth > 512) nth = 512;
    const int64_t nb = K / QK8_0;
    orc_block_q8_0 *Xq = (orc_block_q8_0 *)malloc(sizeof(orc_block_q8_0) * (size_t)(nb * M));
    for (int64_t m = 0; m < M; m++) orc_quantize_row_q8_0(X + m * K, Xq + m * nb, K);

    pthread_t *th = (pthread_t *)malloc(sizeof(pthread_t) * (size_t)nth);
    orc_cpu_job *jobs = (orc_cpu_job *)malloc(sizeof(orc_cpu_job) * (size_t)nth);
    const int64_t nr0 = N, nr1 = M;
    const int64_t nth0 = nr0 > nr1 ? nth : 1;
    const int64_t nth1 = nr0 > nr1 ? 1 : nth;
    const int64_t dr0 = (nr0 + nth0 - 1) / nth0;
    const int64_t dr1 = (nr1 + nth1 - 1) / nth1;
    for (int ith = 0; ith < nth; ith++) {
        const int64_t ith0 = ith % nth0, ith1 = ith / nth0;
        int64_t a0 = dr0 * ith0, a1 = a0 + dr0, b0 = dr1 * ith1, b1 = b0 + dr1;
        if (a0 > nr0) a0 = nr0;
        if (a1 > nr0) a1 = nr0;
        if (b0 > nr1) b0 = nr1;
        if (b1 > nr1) b1 = nr1;
        jobs[ith] = (orc_cpu_job){(const orc_block_q4_0 *)W, Xq, Y, K, N, M, a0, a1, b0, b1};
        pthread_create(&th[ith], NULL, orc_cpu_worker, &jobs[ith]);
    }
    for (int ith = 0; ith < nth; ith++) pthread_join(th[ith], NULL);
    free(jobs);
    free(th);
    free(Xq);
}

/* ------------------------------------------------------------------------- */
/* Row ops                                                                   */
/* ------------------------------------------------------------------------- */

/* rms_norm_f32, galois-kernels/src/rms_norm.cu:13-49 (CPU twin f32::rms_norm,
 * src/lib.rs:594-604): y = x * rsqrt(mean(x^2) + eps), no weight.  f64 inside. */
void orc_rms_norm_f32(const float *x, float *y, int64_t ncols, int64_t nrows, float eps) {
    for (int64_t r = 0; r < nrows; r++) {
        const float *xr = x + r * ncols;
        double ss = 0.0;
        for (int64_t c = 0; c < ncols; c++) ss += (double)xr[c] * (double)xr[c];
        const double scale = 1.0 / sqrt(ss / (double)ncols + (double)eps);
        for (int64_t c = 0; c < ncols; c++) y[r * ncols + c] = (float)((double)xr[c] * scale);
    }
}

/* mul_f32 / add_f32 row broadcast, galois-kernels/src/mul.cu:3-12, add.cu:3-12:
 * dst[i] = x[i] (op) y[i % ky]. */
void orc_mul_f32(const float *x, const float *y, float *dst, int64_t kx, int64_t ky) {
    for (int64_t i = 0; i < kx; i++) dst[i] = x[i] * y[i % ky];
}
void orc_add_f32(const float *x, const float *y, float *dst, int64_t kx, int64_t ky) {
    for (int64_t i = 0; i < kx; i++) dst[i] = x[i] + y[i % ky];
}
/* scale_f32, galois-kernels/src/scale.cu:1-11. */
void orc_scale_f32(const float *x, float *dst, float scale, int64_t k) {
    for (int64_t i = 0; i < k; i++) dst[i] = scale * x[i];
}
/* silu_f32, galois-kernels/src/unary.cu:1-10: x / (1 + exp(-x)), f64 inside. */
void orc_silu_f32(const float *x, float *dst, int64_t k) {
    for (int64_t i = 0; i < k; i++) dst[i] = (float)((double)x[i] / (1.0 + exp(-(double)x[i])));
}

/* rope_f32, galois-kernels/src/rope.cu:3-28 with the launcher's parameters
 * (src/cuda.rs:1300-1356): adjacent pairs, theta = pos[row / p_delta_rows] *
 * freq_scale * theta_scale^(col/2).  theta_scale is the f32 the launcher
 * computes (freq_base^(-2/n_dims), src/cuda.rs:1327); angles in f64. */
void orc_rope_f32(const float *x, float *dst, int64_t ncols, int64_t nrows, const int32_t *pos,
                  float freq_scale, int64_t p_delta_rows, float theta_scale) {
    for (int64_t r = 0; r < nrows; r++) {
        const double p0 = (double)pos[r / p_delta_rows] * (double)freq_scale;
        for (int64_t c = 0; c < ncols; c += 2) {
            const double theta = p0 * pow((double)theta_scale, (double)(c / 2));
            const double s = sin(theta), co = cos(theta);
            const double x0 = x[r * ncols + c], x1 = x[r * ncols + c + 1];
            dst[r * ncols + c] = (float)(x0 * co - x1 * s);
            dst[r * ncols + c + 1] = (float)(x0 * s + x1 * co);
        }
    }
}

/* soft_max_f32, galois-kernels/src/softmax.cu:3-48 (f32 expf semantics; the CPU
 * twin src/lib.rs:564-592 goes through an f16 exp table and is NOT the oracle):
 * -inf inputs give exactly 0 (src/lib.rs:573-576).  f64 inside. */
void orc_soft_max_f32(const float *x, float *dst, int64_t ncols, int64_t nrows) {
    for (int64_t r = 0; r < nrows; r++) {
        const float *xr = x + r * ncols;
        float mx = -INFINITY;
        for (int64_t c = 0; c < ncols; c++) mx = xr[c] > mx ? xr[c] : mx;
        double sum = 0.0;
        for (int64_t c = 0; c < ncols; c++)
            if (xr[c] != -INFINITY) sum += exp((double)xr[c] - (double)mx);
        for (int64_t c = 0; c < ncols; c++)
            dst[r * ncols + c] =
                xr[c] == -INFINITY ? 0.0f : (float)(exp((double)xr[c] - (double)mx) / sum);
    }
}

/* Causal variant = soft_max_f32 over a row whose columns > n_past + (row %
 * rows_per_head) are -inf (the reference has no mask op; its softmax treats
 * -inf as masked, src/lib.rs:573-576, softmax.cu:26-32). */
void orc_soft_max_causal_f32(const float *x, float *dst, int64_t ncols, int64_t rows_per_head,
                             int64_t nrows, int64_t n_past) {
    float *tmp = (float *)malloc(sizeof(float) * (size_t)ncols);
    for (int64_t r = 0; r < nrows; r++) {
        const int64_t last = n_past + (r % rows_per_head);
        for (int64_t c = 0; c < ncols; c++) tmp[c] = c <= last ? x[r * ncols + c] : -INFINITY;
        orc_soft_max_f32(tmp, dst + r * ncols, ncols, 1);
    }
    free(tmp);
}

/* Batched f32 x f32 matmul with galois shape conventions (the reference leaves it
 * todo!(), src/op.rs:1624-1662, src/cuda.rs:867-879): a = [ne00=K, ne01=N, ne02],
 * b = [K, M, ne12], dst = [N, M, ne12]; a is broadcast over ne12/ne02 like the
 * quantized path (src/op.rs:1473-1483).  Element strides (in floats) are given
 * for dims 1 and 2 of a so permuted K/V-cache views work.  f64 accumulate. */
void orc_mul_mat_f32(const float *a, const float *b, float *dst, int64_t K, int64_t N, int64_t M,
                     int64_t ne02, int64_t ne12, int64_t a_s0, int64_t a_s1, int64_t a_s2) {
    const int64_t r2 = ne12 / ne02;
    for (int64_t i2 = 0; i2 < ne12; i2++) {
        const float *ab = a + (i2 / r2) * a_s2;
        for (int64_t m = 0; m < M; m++)
            for (int64_t n = 0; n < N; n++) {
                double acc = 0.0;
                for (int64_t k = 0; k < K; k++)
                    acc += (double)ab[n * a_s1 + k * a_s0] * (double)b[(i2 * M + m) * K + k];
                dst[(i2 * M + m) * N + n] = (float)acc;
            }
    }
}

/* cpy_f32_f32 / cpy_f32_f16, galois-kernels/src/cpy.cu:79-156: element i of the [ne00, ne01, *]
 * source (byte strides nb00..nb02) goes to element i of the [ne10, ne11, *] destination
 * (byte strides nb10..nb12); f16 destination rounds to nearest even. */
void orc_cpy_f32(const void *cx, void *cdst, int dst_is_f16, int64_t ne, int64_t ne00, int64_t ne01, int64_t nb00,
                 int64_t nb01, int64_t nb02, int64_t ne10, int64_t ne11, int64_t nb10, int64_t nb11, int64_t nb12) {
    for (int64_t i = 0; i < ne; i++) {
        const int64_t i02 = i / (ne00 * ne01), i01 = (i - i02 * ne01 * ne00) / ne00;
        const int64_t i00 = i - i02 * ne01 * ne00 - i01 * ne00;
        const int64_t i12 = i / (ne10 * ne11), i11 = (i - i12 * ne10 * ne11) / ne10;
        const int64_t i10 = i - i12 * ne10 * ne11 - i11 * ne10;
        float v;
        memcpy(&v, (const char *)cx + i00 * nb00 + i01 * nb01 + i02 * nb02, 4);
        char *d = (char *)cdst + i10 * nb10 + i11 * nb11 + i12 * nb12;
        if (dst_is_f16) {
            const uint16_t h = orc_f32_to_f16(v);
            memcpy(d, &h, 2);
        } else {
            memcpy(d, &v, 4);
        }
    }
}

/* GetRows::f_q_x_f32, src/op.rs:2546-2571: dst row i = to_f32(table row ids[i]). */
void orc_get_rows_q4_0(const void *table, const int32_t *ids, float *dst, int64_t ncols, int64_t nr) {
    const int64_t row_bytes = ncols / QK4_0 * (int64_t)sizeof(orc_block_q4_0);
    for (int64_t i = 0; i < nr; i++)
        orc_dequantize_row_q4_0((const char *)table + ids[i] * row_bytes, dst + i * ncols, ncols);
}
