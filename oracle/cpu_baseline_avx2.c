/*
 * cpu_baseline_avx2.c -- the x86 forms of Frink's Q4_K CPU path, for the timed CPU baseline.
 *
 * TEST INFRASTRUCTURE ONLY (see frink_oracle.h).  The scalar functions in frink_oracle.c are the
 * checker; these are what is TIMED beside the GPU, because they are what the reference runs on an
 * x86 host with AVX2 + FMA:
 *   - the integer decode dot, crates/frink-quant/src/lib.rs:1245-1306 (dot_q4_k_q8_avx2 and its
 *     madd_i8_avx2): integers exact, float order that of the scalar form -- tests hold it bit-equal
 *     to fo_dot_q4_k_q8k;
 *   - the f32 decode dot, the reference's x86 default for decode
 *     (crates/frink-core/src/weight_matrix.rs:2044-2048 -> crates/frink-quant/src/lib.rs:1411-1466,
 *     fma_affine8 :1385-1398, hsum256_ps :1359-1369).  Eight-lane partial sums: not the scalar form's
 *     summation order.  No vector of the reference pins it ("parity unpinned"); tests hold it to
 *     the scalar f32 dot within fp32 reassociation, and nothing but the timing uses it;
 *   - the batched shape (M activation rows): the same integer dot, weight row outermost so that a
 *     row's 2.3 KB stay in L1 across the activations (the role the reference's 8-row repack plays,
 *     crates/frink-quant/src/repack/q4_kx8.rs:342-420; the repack itself is not restated).
 * Rows are partitioned over OpenMP threads as the reference's rayon row partition does
 * (weight_matrix.rs:2031-2048).  Compiled for AVX2+FMA by function attribute; every entry point
 * returns -1 on a host without them.
 */
#include "frink_oracle.h"

#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#if defined(__x86_64__)
#include <immintrin.h>

#define Q4_K_BYTES 144
#define QK_K 256
#define AVX2 __attribute__((target("avx2,fma")))

AVX2 static inline int32_t hsum_i32(__m256i v) {
    __m128i s = _mm_add_epi32(_mm256_castsi256_si128(v), _mm256_extracti128_si256(v, 1));
    s = _mm_add_epi32(s, _mm_shuffle_epi32(s, 0x4e));
    s = _mm_add_epi32(s, _mm_shuffle_epi32(s, 0xb1));
    return _mm_cvtsi128_si32(s);
}
/* lib.rs:1295-1306 */
AVX2 static inline int32_t madd_i8(__m256i w, __m256i a) {
    __m256i w_lo = _mm256_cvtepi8_epi16(_mm256_castsi256_si128(w));
    __m256i w_hi = _mm256_cvtepi8_epi16(_mm256_extracti128_si256(w, 1));
    __m256i a_lo = _mm256_cvtepi8_epi16(_mm256_castsi256_si128(a));
    __m256i a_hi = _mm256_cvtepi8_epi16(_mm256_extracti128_si256(a, 1));
    return hsum_i32(_mm256_add_epi32(_mm256_madd_epi16(w_lo, a_lo), _mm256_madd_epi16(w_hi, a_hi)));
}

/* lib.rs:1245-1293 */
AVX2 static float dot_q4_k_q8k_avx2(const uint8_t *row, size_t nb, const int8_t *q, const float *dact,
                                    const int16_t *bsums_all) {
    const __m256i low_mask = _mm256_set1_epi8(0x0f);
    float acc = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * Q4_K_BYTES;
        uint16_t hd, hm;
        memcpy(&hd, blk, 2);
        memcpy(&hm, blk + 2, 2);
        const float d = fo_f16_to_f32(hd), dmin = fo_f16_to_f32(hm);
        const uint8_t *scales = blk + 4, *qs = blk + 16;
        const float da = dact[b];
        const int8_t *q8 = q + b * QK_K;
        const int16_t *bsums = bsums_all + b * 16;
        int32_t sum_min = 0;
        for (int i = 0; i < 8; i++) {
            uint8_t sc, m;
            fo_q4_k_scale_min(i, scales, &sc, &m);
            sum_min += (int32_t)m * ((int32_t)bsums[2 * i] + (int32_t)bsums[2 * i + 1]);
        }
        acc -= dmin * da * (float)sum_min;
        for (int p = 0; p < 4; p++) {
            uint8_t sc1, sc2, m_;
            fo_q4_k_scale_min(2 * p, scales, &sc1, &m_);
            fo_q4_k_scale_min(2 * p + 1, scales, &sc2, &m_);
            const __m256i packed = _mm256_loadu_si256((const __m256i *)(qs + 32 * p));
            const __m256i lo = _mm256_and_si256(packed, low_mask);
            const __m256i hi = _mm256_and_si256(_mm256_srli_epi16(packed, 4), low_mask);
            const __m256i a0 = _mm256_loadu_si256((const __m256i *)(q8 + 64 * p));
            const __m256i a1 = _mm256_loadu_si256((const __m256i *)(q8 + 64 * p + 32));
            const int32_t isum1 = madd_i8(lo, a0), isum2 = madd_i8(hi, a1);
            acc += d * da * ((float)sc1 * (float)isum1 + (float)sc2 * (float)isum2);
        }
    }
    return acc;
}

/* lib.rs:1359-1369 */
AVX2 static inline float hsum256_ps(__m256 v) {
    const __m128 hi = _mm256_extractf128_ps(v, 1), lo = _mm256_castps256_ps128(v);
    const __m128 sum128 = _mm_add_ps(hi, lo);
    const __m128 shuf = _mm_movehdup_ps(sum128);
    const __m128 sums = _mm_add_ps(sum128, shuf);
    const __m128 shuf2 = _mm_movehl_ps(shuf, sums);
    return _mm_cvtss_f32(_mm_add_ss(sums, shuf2));
}
/* lib.rs:1385-1398 */
AVX2 static inline __m256 fma_affine8(__m128i part, float d, float min, const float *x, __m256 acc) {
    const __m256 f = _mm256_cvtepi32_ps(_mm256_cvtepu8_epi32(part));
    const __m256 weight = _mm256_fmsub_ps(f, _mm256_set1_ps(d), _mm256_set1_ps(min));
    return _mm256_fmadd_ps(weight, _mm256_loadu_ps(x), acc);
}
/* lib.rs:1411-1466 */
AVX2 static float dot_q4_k_f32_avx2(const uint8_t *row, size_t nb, const float *x) {
    const __m128i low_mask = _mm_set1_epi8(0x0f);
    float acc = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * Q4_K_BYTES;
        uint16_t hd, hm;
        memcpy(&hd, blk, 2);
        memcpy(&hm, blk + 2, 2);
        const float d = fo_f16_to_f32(hd), dmin = fo_f16_to_f32(hm);
        const uint8_t *scales = blk + 4, *qs = blk + 16;
        const float *xb = x + b * QK_K;
        for (int p = 0; p < 4; p++) {
            uint8_t sc1, m1, sc2, m2;
            fo_q4_k_scale_min(2 * p, scales, &sc1, &m1);
            fo_q4_k_scale_min(2 * p + 1, scales, &sc2, &m2);
            const float d1 = d * (float)sc1, min1 = dmin * (float)m1;
            const float d2 = d * (float)sc2, min2 = dmin * (float)m2;
            __m256 lo_acc = _mm256_setzero_ps(), hi_acc = _mm256_setzero_ps();
            for (int g = 0; g < 2; g++) {
                const __m128i raw16 = _mm_loadu_si128((const __m128i *)(qs + 32 * p + 16 * g));
                const __m128i lo_nib = _mm_and_si128(raw16, low_mask);
                const __m128i hi_nib = _mm_and_si128(_mm_srli_epi16(raw16, 4), low_mask);
                lo_acc = fma_affine8(lo_nib, d1, min1, xb + 64 * p + 16 * g, lo_acc);
                lo_acc = fma_affine8(_mm_srli_si128(lo_nib, 8), d1, min1, xb + 64 * p + 16 * g + 8, lo_acc);
                hi_acc = fma_affine8(hi_nib, d2, min2, xb + 64 * p + 32 + 16 * g, hi_acc);
                hi_acc = fma_affine8(_mm_srli_si128(hi_nib, 8), d2, min2, xb + 64 * p + 32 + 16 * g + 8, hi_acc);
            }
            acc += hsum256_ps(lo_acc) + hsum256_ps(hi_acc);
        }
    }
    return acc;
}

static int have(void) { return __builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma"); }

AVX2 int fo_avx2_gemv_q4_k_f32(const uint8_t *w, size_t rows, size_t cols, const float *x, float *y, int threads) {
    if (!have() || cols % QK_K) return -1;
    const size_t nb = cols / QK_K;
    if (threads < 1) threads = 1;
#pragma omp parallel for schedule(static) num_threads(threads)
    for (long r = 0; r < (long)rows; r++) y[r] = dot_q4_k_f32_avx2(w + (size_t)r * nb * Q4_K_BYTES, nb, x);
    return 0;
}

/* y[b][r] for `batch` activation rows: each quantized once (Q8_K), then row-outer integer dots */
AVX2 int fo_avx2_gemm_q4_k_q8k(const uint8_t *w, size_t rows, size_t cols, const float *x, size_t batch, float *y,
                               int threads) {
    if (!have() || cols % QK_K) return -1;
    const size_t nb = cols / QK_K;
    if (threads < 1) threads = 1;
    int8_t *q = (int8_t *)malloc(batch * cols);
    float *d = (float *)malloc(batch * nb * sizeof(float));
    int16_t *bs = (int16_t *)malloc(batch * nb * 16 * sizeof(int16_t));
    if (!q || !d || !bs) {
        free(q), free(d), free(bs);
        return -2;
    }
#pragma omp parallel for schedule(static) num_threads(threads)
    for (long b = 0; b < (long)batch; b++)
        fo_quantize_q8_k(x + (size_t)b * cols, cols, q + (size_t)b * cols, d + (size_t)b * nb, bs + (size_t)b * nb * 16);
#pragma omp parallel for schedule(static) num_threads(threads)
    for (long r = 0; r < (long)rows; r++) {
        const uint8_t *row = w + (size_t)r * nb * Q4_K_BYTES;
        for (size_t b = 0; b < batch; b++)
            y[b * rows + (size_t)r] = dot_q4_k_q8k_avx2(row, nb, q + b * cols, d + b * nb, bs + b * nb * 16);
    }
    free(q), free(d), free(bs);
    return 0;
}

#else /* not x86-64 */

int fo_avx2_gemv_q4_k_f32(const uint8_t *w, size_t rows, size_t cols, const float *x, float *y, int threads) {
    (void)w, (void)rows, (void)cols, (void)x, (void)y, (void)threads;
    return -1;
}
int fo_avx2_gemm_q4_k_q8k(const uint8_t *w, size_t rows, size_t cols, const float *x, size_t batch, float *y,
                          int threads) {
    (void)w, (void)rows, (void)cols, (void)x, (void)batch, (void)y, (void)threads;
    return -1;
}

#endif
