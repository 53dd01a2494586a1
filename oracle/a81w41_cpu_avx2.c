/*
 * TEST INFRASTRUCTURE ONLY -- AVX2 + OpenMP port of the reference's CPU path,
 * used as the timed CPU baseline next to the GPU numbers.  It keeps the
 * reference's blocking and scheduling: one OpenMP task per 8-column group
 * (dynamic schedule), the K loop over 64-wide super-blocks in order, the GEMM's
 * 6-row M tile (quantized_gemx_kernels.cc:129-193, :364-582) and the serial
 * quantizer (:693-911).  Every lane performs the same IEEE operations in the
 * same order as the scalar oracle, so the two agree bit for bit (checked in
 * tests/test_oracle_avx2.py).  Integer dots follow mul_sum_us8_pairs_acc_int32x8
 * (lib.h:45-55), whose branch is picked by the compiler flags: dpbusd with
 * AVX512-VNNI + VL or with AVX-VNNI, else maddubs+madd (the products cannot
 * saturate there: 2*15*127 < 32767).  The Makefile builds one library per
 * branch from this file; oracle/ora.py loads the best one the host CPU runs.
 */
#include <immintrin.h>
#include <omp.h>
#include <stdint.h>
#include <string.h>

#include "a81w41_oracle.h"

int avx_max_threads(void) { return omp_get_max_threads(); }

static inline __m256i dot_u8s8_acc(__m256i acc, __m256i u, __m256i s) {
#if defined(__AVX512VNNI__) && defined(__AVX512VL__)
    return _mm256_dpbusd_epi32(acc, u, s);
#elif defined(__AVXVNNI__)
    return _mm256_dpbusd_avx_epi32(acc, u, s);
#else
    return _mm256_add_epi32(acc, _mm256_madd_epi16(_mm256_maddubs_epi16(u, s), _mm256_set1_epi16(1)));
#endif
}

/* Which branch of lib.h:45-55 this build of the file takes. */
const char *avx_dot_branch(void) {
#if defined(__AVX512VNNI__) && defined(__AVX512VL__)
    return "avx512-vnni dpbusd";
#elif defined(__AVXVNNI__)
    return "avx-vnni dpbusd";
#else
    return "avx2 maddubs+madd";
#endif
}

static inline int hsum_i32(__m256i v) {
    __m128i s = _mm_add_epi32(_mm256_castsi256_si128(v), _mm256_extracti128_si256(v, 1));
    s = _mm_add_epi32(s, _mm_unpackhi_epi64(s, s));
    s = _mm_add_epi32(s, _mm_shuffle_epi32(s, 0xb1));
    return _mm_cvtsi128_si32(s);
}

static inline float hmax_ps(__m256 v) {
    __m128 m = _mm_max_ps(_mm256_castps256_ps128(v), _mm256_extractf128_ps(v, 1));
    m = _mm_max_ps(m, _mm_movehl_ps(m, m));
    m = _mm_max_ss(m, _mm_movehdup_ps(m));
    return _mm_cvtss_f32(m);
}

/* One 32-block -> 32 int8 in natural order; returns d, *ssum = d * float(sum q). */
static inline float quant32(const float *x, int8_t *q, float *ssum) {
    const __m256 sign = _mm256_set1_ps(-0.0f);
    __m256 v[4];
    __m256 amax = _mm256_setzero_ps();
    for (int i = 0; i < 4; i++) {
        v[i] = _mm256_loadu_ps(x + 8 * i);
        amax = _mm256_max_ps(amax, _mm256_andnot_ps(sign, v[i]));
    }
    const float mx = hmax_ps(amax);
    const float d = mx / 127.f;
    const float id = (mx != 0.0f) ? 127.f / mx : 0.0f;
    const __m256 mul = _mm256_set1_ps(id);
    __m256i r[4];
    __m256i tot = _mm256_setzero_si256();
    for (int i = 0; i < 4; i++) {
        r[i] = _mm256_cvtps_epi32(_mm256_round_ps(_mm256_mul_ps(v[i], mul), _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC));
        tot = _mm256_add_epi32(tot, r[i]);
    }
    *ssum = d * (float)hsum_i32(tot);
    __m256i p01 = _mm256_packs_epi32(r[0], r[1]);
    __m256i p23 = _mm256_packs_epi32(r[2], r[3]);
    __m256i b = _mm256_packs_epi16(p01, p23);
    b = _mm256_permutevar8x32_epi32(b, _mm256_setr_epi32(0, 4, 1, 5, 2, 6, 3, 7));
    _mm256_storeu_si256((__m256i *)q, b);
    return d;
}

void avx_quantize_row_q8_1_repack_fp16(const float *x, void *vy, int64_t k) {
    ora_q8_repack_1x2_fp16 *y = (ora_q8_repack_1x2_fp16 *)vy;
    for (int64_t i = 0; i < k / 64; i++) {
        float sl, sh;
        const float d1 = quant32(x + 64 * i, y[i].q_low, &sl);
        const float d2 = quant32(x + 64 * i + 32, y[i].q_high, &sh);
        y[i].s_low = _cvtss_sh(d1, 0);
        y[i].s_high = _cvtss_sh(d2, 0);
        y[i].scaled_sum_low = _cvtss_sh(sl, 0);
        y[i].scaled_sum_high = _cvtss_sh(sh, 0);
    }
}

void avx_quantize_row_q8_1_repack_fp32(const float *x, void *vy, int64_t k) {
    ora_q8_repack_1x2_fp32 *y = (ora_q8_repack_1x2_fp32 *)vy;
    for (int64_t i = 0; i < k / 64; i++) {
        float sl, sh;
        y[i].s_low = quant32(x + 64 * i, y[i].q_low, &sl);
        y[i].s_high = quant32(x + 64 * i + 32, y[i].q_high, &sh);
        y[i].scaled_sum_low = sl;
        y[i].scaled_sum_high = sh;
    }
}

static inline void unpack_block(const uint8_t *q_coupled, __m256i *lo, __m256i *hi) {
    const __m256i mask = _mm256_set1_epi8(0x0f);
    for (int p = 0; p < 8; p++) {
        const __m256i c = _mm256_loadu_si256((const __m256i *)(q_coupled + 32 * p));
        lo[p] = _mm256_and_si256(c, mask);
        hi[p] = _mm256_and_si256(_mm256_srli_epi16(c, 4), mask);
    }
}

void avx_gemv_repack_A81W41_fp16(const void *A_repack, const void *B_repack, float *C, int M, int N,
                                 int K, int nthreads) {
    (void)M;
    const ora_q8_repack_1x2_fp16 *A = (const ora_q8_repack_1x2_fp16 *)A_repack;
    const ora_q4_repack_2x8_fp16 *B = (const ora_q4_repack_2x8_fp16 *)B_repack;
    const int nb_k = K / 64, nb_n = N / 8;
#pragma omp parallel for schedule(dynamic) num_threads(nthreads)
    for (int g = 0; g < nb_n; g++) {
        __m256 acc = _mm256_setzero_ps();
        for (int sb = 0; sb < nb_k; sb++) {
            const ora_q4_repack_2x8_fp16 *b = B + (size_t)g * nb_k + sb;
            __m256i lo[8], hi[8];
            unpack_block(b->q_coupled, lo, hi);
            __m256i il = _mm256_setzero_si256(), ih = _mm256_setzero_si256();
            int32_t ql[8], qh[8];
            memcpy(ql, A[sb].q_low, 32);
            memcpy(qh, A[sb].q_high, 32);
            for (int p = 0; p < 8; p++) {
                il = dot_u8s8_acc(il, lo[p], _mm256_set1_epi32(ql[p]));
                ih = dot_u8s8_acc(ih, hi[p], _mm256_set1_epi32(qh[p]));
            }
            const __m256 dl = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)b->s_low));
            const __m256 dh = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)b->s_high));
            const __m256 ml = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)b->min_low));
            const __m256 mh = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)b->min_high));
            const __m256 al = _mm256_cvtph_ps(_mm_set1_epi16((short)A[sb].s_low));
            const __m256 ah = _mm256_cvtph_ps(_mm_set1_epi16((short)A[sb].s_high));
            const __m256 sl = _mm256_cvtph_ps(_mm_set1_epi16((short)A[sb].scaled_sum_low));
            const __m256 sh = _mm256_cvtph_ps(_mm_set1_epi16((short)A[sb].scaled_sum_high));
            acc = _mm256_fmadd_ps(_mm256_cvtepi32_ps(il), _mm256_mul_ps(al, dl), acc);
            acc = _mm256_fmadd_ps(_mm256_cvtepi32_ps(ih), _mm256_mul_ps(ah, dh), acc);
            acc = _mm256_fmadd_ps(ml, sl, acc);
            acc = _mm256_fmadd_ps(mh, sh, acc);
        }
        _mm256_storeu_ps(C + 8 * g, acc);
    }
}

#define MR 6 /* the reference's M tile, quantized_gemx_kernels.cc:367 */

void avx_gemm_repack_A81W41_fp32(const void *A_repack, const void *B_repack, float *C, int M, int N,
                                 int K, int nthreads) {
    const ora_q8_repack_1x2_fp32 *A = (const ora_q8_repack_1x2_fp32 *)A_repack;
    const ora_q4_repack_2x8_fp32 *B = (const ora_q4_repack_2x8_fp32 *)B_repack;
    const int nb_k = K / 64, nb_n = N / 8;
#pragma omp parallel for schedule(dynamic) num_threads(nthreads)
    for (int g = 0; g < nb_n; g++) {
        for (int i0 = 0; i0 < M; i0 += MR) {
            const int rows = (M - i0 < MR) ? M - i0 : MR;
            const ora_q8_repack_1x2_fp32 *a[MR];
            for (int r = 0; r < MR; r++) /* rows past M alias the last valid row; never stored */
                a[r] = A + (size_t)((r < rows) ? i0 + r : i0 + rows - 1) * nb_k;
            __m256 acc[MR];
            for (int r = 0; r < MR; r++) acc[r] = _mm256_setzero_ps();
            for (int sb = 0; sb < nb_k; sb++) {
                const ora_q4_repack_2x8_fp32 *b = B + (size_t)g * nb_k + sb;
                __m256i lo[8], hi[8];
                unpack_block(b->q_coupled, lo, hi);
                const __m256 dl = _mm256_loadu_ps(b->s_low), dh = _mm256_loadu_ps(b->s_high);
                const __m256 ml = _mm256_loadu_ps(b->min_low), mh = _mm256_loadu_ps(b->min_high);
                for (int r = 0; r < MR; r++) {
                    const ora_q8_repack_1x2_fp32 *ar = a[r] + sb;
                    int32_t ql[8], qh[8];
                    memcpy(ql, ar->q_low, 32);
                    memcpy(qh, ar->q_high, 32);
                    __m256i il = _mm256_setzero_si256(), ih = _mm256_setzero_si256();
                    for (int p = 0; p < 8; p++) {
                        il = dot_u8s8_acc(il, lo[p], _mm256_set1_epi32(ql[p]));
                        ih = dot_u8s8_acc(ih, hi[p], _mm256_set1_epi32(qh[p]));
                    }
                    acc[r] = _mm256_fmadd_ps(_mm256_cvtepi32_ps(il), _mm256_mul_ps(_mm256_set1_ps(ar->s_low), dl), acc[r]);
                    acc[r] = _mm256_fmadd_ps(_mm256_cvtepi32_ps(ih), _mm256_mul_ps(_mm256_set1_ps(ar->s_high), dh), acc[r]);
                    acc[r] = _mm256_fmadd_ps(ml, _mm256_set1_ps(ar->scaled_sum_low), acc[r]);
                    acc[r] = _mm256_fmadd_ps(mh, _mm256_set1_ps(ar->scaled_sum_high), acc[r]);
                }
            }
            for (int r = 0; r < rows; r++) _mm256_storeu_ps(C + (size_t)(i0 + r) * N + 8 * g, acc[r]);
        }
    }
}
