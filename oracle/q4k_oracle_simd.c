/*
 * q4k_oracle_simd.c -- AVX2 + pthreads restatement of the reference's x86
 * batched-row kernel, used ONLY as the timed CPU baseline beside the GPU
 * numbers (and cross-checked against the scalar oracle in the tests).
 * TEST INFRASTRUCTURE ONLY (see q4k_oracle.h).
 *
 * Follows core/src/llm/matmul/kquant_batched_kernels.h:406-549 (one Q4_K row
 * against up to 16 Q8_K rows, nibbles and scales decoded once per block) and
 * the thread partition of core/src/llm/matmul/gemv_exec.cpp:376-380
 * (rows [ith*ceil(N/nth), ...) per thread, one thread quantizes first).
 * fp32 order = ORC_ORDER_AVX2 of the scalar oracle, bit for bit.
 *
 * Built a second time with -mavx512vnni -mavx512vl (liboracle_simd_vnni.so): the block product then is the
 * reference's VNNI kernel's, _mm256_dpbusd_epi32 on the nibbles and the codes and a 32-bit multiply by the scale
 * (ComputeMoEQ4KQ8KBatchedRowVnni, core/src/backend/cpu_backend_moe_raw_batched.inl:562-616).  Lane i of its eight
 * sums holds the same four products of every 32-weight sub-block as the AVX2 form's, so the results are the same
 * bits; it is the build the CPU baseline is timed with where the host has the instructions.
 */
#define _GNU_SOURCE
#include "q4k_oracle.h"

#include <immintrin.h>
#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

#define SIMD_TILE_M 16

static inline float half_to_float(uint16_t h) { return _cvtsh_ss(h); }

static inline float hsum8(__m256 v) {
    __m128 r = _mm_add_ps(_mm256_extractf128_ps(v, 1), _mm256_castps256_ps128(v));
    r = _mm_add_ps(r, _mm_movehl_ps(r, r));
    r = _mm_add_ss(r, _mm_movehdup_ps(r));
    return _mm_cvtss_f32(r);
}

static inline void unpack_scales(const uint8_t packed[12], uint8_t sc[8], uint8_t mn[8]) {
    uint32_t w[3];
    memcpy(w, packed, 12);
    const uint32_t s_lo = w[0] & 0x3f3f3f3fu, m_lo = w[1] & 0x3f3f3f3fu;
    const uint32_t s_hi = (w[2] & 0x0f0f0f0fu) | (((w[0] >> 6) & 0x03030303u) << 4);
    const uint32_t m_hi = ((w[2] >> 4) & 0x0f0f0f0fu) | (((w[1] >> 6) & 0x03030303u) << 4);
    memcpy(sc, &s_lo, 4);
    memcpy(sc + 4, &s_hi, 4);
    memcpy(mn, &m_lo, 4);
    memcpy(mn + 4, &m_hi, 4);
}

/* One weight row against m <= 16 activation rows. */
static void row_times_tile(const orc_block_q4k* w, int64_t nb, const uint8_t* q8, size_t q8_row_bytes, int m,
                           float* out) {
    float acc[SIMD_TILE_M] = {0};
    const __m256i nib = _mm256_set1_epi8(0x0f);
    for (int64_t b = 0; b < nb; ++b) {
        uint8_t sc[8], mn[8];
        unpack_scales(w[b].scales, sc, mn);
        __m256i lo[4], hi[4], slo[4], shi[4];
#if defined(__AVX512VNNI__) && defined(__AVX512VL__)
        __m256i slo32[4], shi32[4];
        for (int c = 0; c < 4; ++c) slo32[c] = _mm256_set1_epi32(sc[2 * c]), shi32[c] = _mm256_set1_epi32(sc[2 * c + 1]);
#endif
        for (int c = 0; c < 4; ++c) {
            const __m256i bytes = _mm256_loadu_si256((const __m256i*)(w[b].qs + 32 * c));
            lo[c] = _mm256_and_si256(bytes, nib);
            hi[c] = _mm256_and_si256(_mm256_srli_epi16(bytes, 4), nib);
            slo[c] = _mm256_set1_epi16(sc[2 * c]);
            shi[c] = _mm256_set1_epi16(sc[2 * c + 1]);
            (void)slo[c], (void)shi[c];  /* the VNNI build multiplies by the 32-bit copies */
        }
        const float wd = half_to_float(w[b].d), wm = half_to_float(w[b].dmin);
        for (int t = 0; t < m; ++t) {
            const orc_block_q8k* y = (const orc_block_q8k*)(q8 + (size_t)t * q8_row_bytes) + b;
            int32_t md = 0;
            for (int j = 0; j < 16; ++j) md += (int32_t)y->bsums[j] * (int32_t)mn[j >> 1];
            __m256i sum = _mm256_setzero_si256();
            for (int c = 0; c < 4; ++c) {
                const __m256i ya = _mm256_loadu_si256((const __m256i*)(y->qs + 64 * c));
                const __m256i yb = _mm256_loadu_si256((const __m256i*)(y->qs + 64 * c + 32));
#if defined(__AVX512VNNI__) && defined(__AVX512VL__)
                const __m256i pa = _mm256_mullo_epi32(_mm256_dpbusd_epi32(_mm256_setzero_si256(), lo[c], ya), slo32[c]);
                const __m256i pb = _mm256_mullo_epi32(_mm256_dpbusd_epi32(_mm256_setzero_si256(), hi[c], yb), shi32[c]);
#else
                const __m256i pa = _mm256_madd_epi16(slo[c], _mm256_maddubs_epi16(lo[c], ya));
                const __m256i pb = _mm256_madd_epi16(shi[c], _mm256_maddubs_epi16(hi[c], yb));
#endif
                sum = _mm256_add_epi32(sum, _mm256_add_epi32(pa, pb));
            }
            const float d = wd * y->d;
            const float dm = -wm * y->d;
            const float term = d * hsum8(_mm256_cvtepi32_ps(sum)) + dm * (float)md;
            acc[t] += term;
        }
    }
    memcpy(out, acc, sizeof(float) * (size_t)m);
}

/* 2: this build multiplies with AVX-512 VNNI (256-bit), 1: with AVX2. */
int orc_simd_isa(void) {
#if defined(__AVX512VNNI__) && defined(__AVX512VL__)
    return 2;
#else
    return 1;
#endif
}

typedef struct {
    const uint8_t* w;
    int64_t rows, cols;
    size_t row_bytes;
    const uint8_t* q8;
    size_t q8_row_bytes;
    int64_t n;
    float* out;
    int64_t ldo;
    int ith, nth;
} job_t;

static void* worker(void* arg) {
    const job_t* j = (const job_t*)arg;
    const int64_t per = (j->rows + j->nth - 1) / j->nth;
    const int64_t r0 = per * j->ith;
    const int64_t r1 = r0 + per < j->rows ? r0 + per : j->rows;
    const int64_t nb = j->cols / ORC_QK_K;
    float tile[SIMD_TILE_M];
    for (int64_t r = r0; r < r1; ++r) {
        const orc_block_q4k* wr = (const orc_block_q4k*)(j->w + (size_t)r * j->row_bytes);
        for (int64_t m0 = 0; m0 < j->n; m0 += SIMD_TILE_M) {
            const int m = (int)(j->n - m0 < SIMD_TILE_M ? j->n - m0 : SIMD_TILE_M);
            row_times_tile(wr, nb, j->q8 + (size_t)m0 * j->q8_row_bytes, j->q8_row_bytes, m, tile);
            for (int t = 0; t < m; ++t) j->out[(m0 + t) * j->ldo + r] = tile[t];
        }
    }
    return NULL;
}

/* out[m*ldo + r] = W[r] . q8[m], rows split over `threads` pthreads. */
int orc_simd_mul_mat_q4k_q8k(const void* w, int64_t rows, int64_t cols, size_t row_bytes, const void* q8, int64_t n,
                             size_t q8_row_bytes, float* out, int64_t ldo, int threads) {
    if (!w || !q8 || !out || rows <= 0 || n <= 0 || cols <= 0 || cols % ORC_QK_K || threads < 1 || threads > 256)
        return -1;
    pthread_t tid[256];
    job_t jobs[256];
    for (int i = 0; i < threads; ++i) {
        jobs[i] = (job_t){(const uint8_t*)w, rows, cols, row_bytes, (const uint8_t*)q8, q8_row_bytes, n, out, ldo, i,
                          threads};
        if (i > 0 && pthread_create(&tid[i], NULL, worker, &jobs[i]) != 0) return -2;
    }
    worker(&jobs[0]);
    for (int i = 1; i < threads; ++i) pthread_join(tid[i], NULL);
    return 0;
}

/* Grouped (expert-routed) variant for the MoE baseline: `count` independent
 * (matrix, activation row) pairs, one output row of `rows` floats each. */
int orc_simd_mul_mat_id_q4k_q8k(const void* const* w_list, const void* const* q8_list, int64_t count, int64_t rows,
                                int64_t cols, size_t row_bytes, float* out, int64_t ldo, int threads) {
    for (int64_t i = 0; i < count; ++i) {
        const int rc = orc_simd_mul_mat_q4k_q8k(w_list[i], rows, cols, row_bytes, q8_list[i], 1,
                                                (size_t)(cols / ORC_QK_K) * sizeof(orc_block_q8k), out + i * ldo, ldo,
                                                threads);
        if (rc) return rc;
    }
    return 0;
}

/* Dense SwiGLU FFN on host cores: quantize (scalar oracle), gate and up rows split over the
 * threads, SiLU-gate, re-quantize, down rows split over the threads.  Timed as the CPU baseline of
 * the FFN-shaped workload; equals orc_ffn_swiglu_q4k(..., ORC_ORDER_AVX2, ...) bit for bit. */
int orc_simd_ffn_swiglu_q4k(const void* gate, const void* up, const void* down, int64_t hidden, int64_t inter,
                            const float* x, int64_t n, float* y, int threads, int silu_mode) {
    if (!gate || !up || !down || !x || !y || hidden % ORC_QK_K || inter % ORC_QK_K || n <= 0) return -1;
    const size_t wrow_in = (size_t)(hidden / ORC_QK_K) * sizeof(orc_block_q4k);
    const size_t wrow_mid = (size_t)(inter / ORC_QK_K) * sizeof(orc_block_q4k);
    const size_t q8_in = (size_t)(hidden / ORC_QK_K) * sizeof(orc_block_q8k);
    const size_t q8_mid = (size_t)(inter / ORC_QK_K) * sizeof(orc_block_q8k);
    uint8_t* xq = (uint8_t*)malloc(q8_in * (size_t)n);
    uint8_t* hq = (uint8_t*)malloc(q8_mid * (size_t)n);
    float* g = (float*)malloc(sizeof(float) * (size_t)n * (size_t)inter * 2);
    int rc = (xq && hq && g) ? 0 : -2;
    if (rc == 0) {
        float* u = g + (size_t)n * (size_t)inter;
        orc_quantize_rows_q8k(x, n, hidden, xq, hidden);
        rc = orc_simd_mul_mat_q4k_q8k(gate, inter, hidden, wrow_in, xq, n, q8_in, g, inter, threads);
        if (rc == 0) rc = orc_simd_mul_mat_q4k_q8k(up, inter, hidden, wrow_in, xq, n, q8_in, u, inter, threads);
        if (rc == 0) {
            for (int64_t i = 0; i < n * inter; ++i) g[i] = orc_silu_mul(g[i], u[i], silu_mode);
            orc_quantize_rows_q8k(g, n, inter, hq, inter);
            rc = orc_simd_mul_mat_q4k_q8k(down, hidden, inter, wrow_mid, hq, n, q8_mid, y, hidden, threads);
        }
    }
    free(xq);
    free(hq);
    free(g);
    return rc;
}
