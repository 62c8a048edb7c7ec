/*
 * q5k_oracle.c -- CPU restatement of the reference's Q5_K x Q8_K dot product.
 * TEST INFRASTRUCTURE ONLY (see q4k_oracle.h): nothing that ships links against it.
 *
 * block_q5_K = block_q4_K plus one high bit per weight (core/src/kernels/hwy/hwy_moe_quant.cc:36-45:
 * fp16 d, fp16 dmin, scales[12], qh[32], qs[128]; 176 bytes).  Element l of sub-block s takes bit s of
 * qh[l] as its fifth bit (hwy_moe_quant.cc:177-200), so the codes are 0..31; scales, mins, the two
 * integer sums and the fp32 update are those of Q4_K (DotKQ8KImpl<MoEQ5KBlock, true>,
 * hwy_moe_quant.cc:145-258).
 *
 * Pins (tests/test_oracle_pins.py): layout sizeof/offsetof; a block whose qh is zero gives exactly the
 * Q4_K sums of the same fields; setting every qh bit adds 16 * scale_s * (sum of the sub-block's codes)
 * -- a closed form through bsums; brute-force int64 triple loop; dequantize-then-double dot within 1e-4.
 */
#include <math.h>
#include <stddef.h>
#include <string.h>

#include "q4k_oracle.h"

typedef struct {
    uint16_t d;
    uint16_t dmin;
    uint8_t scales[12];
    uint8_t qh[ORC_QK_K / 8];
    uint8_t qs[ORC_QK_K / 2];
} orc_block_q5k;

_Static_assert(sizeof(orc_block_q5k) == 176, "block_q5_K is 176 bytes");
_Static_assert(offsetof(orc_block_q5k, qh) == 16 && offsetof(orc_block_q5k, qs) == 48, "block_q5_K field offsets");

size_t orc_q5k_block_bytes(void) { return sizeof(orc_block_q5k); }

/* element e = 32*s + l of the block: nibble as in Q4_K, fifth bit = bit s of qh[l] */
static inline int q5_element(const orc_block_q5k* w, int e) {
    const int chunk = e >> 6, within = e & 63, l = e & 31, s = e >> 5;
    const uint8_t byte = w->qs[32 * chunk + l];
    const int nib = within < 32 ? (byte & 15) : (byte >> 4);
    return nib + (((w->qh[l] >> s) & 1) << 4);
}

void orc_q5k_block_sums(const void* w_block, const void* q8_block, int32_t* dot_scaled, int32_t* min_dot) {
    const orc_block_q5k* w = (const orc_block_q5k*)w_block;
    const orc_block_q8k* y = (const orc_block_q8k*)q8_block;
    uint8_t sc[8], mn[8];
    orc_q4k_scales_kmask(w->scales, sc, mn);
    int32_t acc = 0;
    for (int s = 0; s < 8; ++s) {
        int32_t sub = 0;
        for (int l = 0; l < 32; ++l) sub += q5_element(w, 32 * s + l) * (int32_t)y->qs[32 * s + l];
        acc += (int32_t)sc[s] * sub;
    }
    int32_t md = 0;
    for (int j = 0; j < 16; ++j) md += (int32_t)y->bsums[j] * (int32_t)mn[j >> 1];
    if (dot_scaled) *dot_scaled = acc;
    if (min_dot) *min_dot = md;
}

int orc_q5k_matrix_block_sums(const void* w, int64_t rows, int64_t cols, size_t row_bytes, const void* q8, int64_t n,
                              size_t q8_row_bytes, int32_t* dot_scaled, int32_t* min_dot) {
    if (!w || !q8 || rows < 0 || n < 0 || cols <= 0 || cols % ORC_QK_K) return -1;
    const int64_t nb = cols / ORC_QK_K;
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t m = 0; m < n; ++m)
            for (int64_t b = 0; b < nb; ++b) {
                const size_t idx = ((size_t)r * (size_t)n + (size_t)m) * (size_t)nb + (size_t)b;
                orc_q5k_block_sums((const uint8_t*)w + (size_t)r * row_bytes + (size_t)b * sizeof(orc_block_q5k),
                                   (const uint8_t*)q8 + (size_t)m * q8_row_bytes + (size_t)b * sizeof(orc_block_q8k),
                                   dot_scaled ? dot_scaled + idx : NULL, min_dot ? min_dot + idx : NULL);
            }
    return 0;
}

/* Row dot.  order 0 (Highway, the only Q5_K kernel the reference has): eight int32 lanes (lane j = elements
 * 4j..4j+3 of every sub-block, scaled), converted and summed as a pairwise tree, then
 * sumf += d*block_dot; sumf -= dmin*min_dot (hwy_moe_quant.cc:228-253).  order 3: the plain per-block
 * form d*dot - dmin*min added to the total (core/src/llm/matmul/kquant_batched_kernels.h:299-301). */
float orc_dot_q5k_q8k(const void* w_row, const void* q8_row, int64_t cols, int order) {
    const orc_block_q5k* w = (const orc_block_q5k*)w_row;
    const orc_block_q8k* y = (const orc_block_q8k*)q8_row;
    float total = 0.0f;
    for (int64_t b = 0; b < cols / ORC_QK_K; ++b) {
        uint8_t sc[8], mn[8];
        orc_q4k_scales_kmask(w[b].scales, sc, mn);
        int32_t md = 0;
        for (int j = 0; j < 16; ++j) md += (int32_t)y[b].bsums[j] * (int32_t)mn[j >> 1];
        const float yd = y[b].d;
        const float d = orc_fp16_to_fp32(w[b].d) * yd, dm = orc_fp16_to_fp32(w[b].dmin) * yd;
        if (order == ORC_ORDER_HWY) {
            int32_t lane[8] = {0};
            for (int s = 0; s < 8; ++s)
                for (int j = 0; j < 8; ++j) {
                    int32_t acc = 0;
                    for (int i = 0; i < 4; ++i) {
                        const int e = 32 * s + 4 * j + i;
                        acc += q5_element(w + b, e) * (int32_t)y[b].qs[e];
                    }
                    lane[j] += (int32_t)sc[s] * acc;
                }
            float f[8];
            for (int j = 0; j < 8; ++j) f[j] = (float)lane[j];
            const float block_dot = ((f[0] + f[4]) + (f[2] + f[6])) + ((f[1] + f[5]) + (f[3] + f[7]));
            total += d * block_dot;
            total -= dm * (float)md;
        } else {
            int32_t ds = 0;
            orc_q5k_block_sums(w + b, y + b, &ds, NULL);
            const float t = d * (float)ds - dm * (float)md;
            total += t;
        }
    }
    return total;
}

/* dequantize both sides, multiply-accumulate in double (the reference's slow check,
 * core/tests/moe/test_moe_ops.cpp:170-201) */
double orc_dot_dequant_q5k_f64(const void* w_row, const void* q8_row, int64_t cols, int magnitude) {
    const orc_block_q5k* w = (const orc_block_q5k*)w_row;
    const orc_block_q8k* y = (const orc_block_q8k*)q8_row;
    double acc = 0.0;
    for (int64_t b = 0; b < cols / ORC_QK_K; ++b) {
        uint8_t sc[8], mn[8];
        orc_q4k_scales_indexed(w[b].scales, sc, mn);
        const double wd = orc_fp16_to_fp32(w[b].d), wm = orc_fp16_to_fp32(w[b].dmin);
        for (int e = 0; e < ORC_QK_K; ++e) {
            const int s = e >> 5;
            const double wv = wd * sc[s] * q5_element(w + b, e) - wm * mn[s];
            const double xv = (double)y[b].d * y[b].qs[e];
            acc += magnitude ? fabs(wd * sc[s] * q5_element(w + b, e) * xv) + fabs(wm * mn[s] * xv) : wv * xv;
        }
    }
    return acc;
}

int orc_mul_mat_q5k_q8k(const void* w, int64_t rows, int64_t cols, size_t row_bytes, const void* q8, int64_t n,
                        size_t q8_row_bytes, float* out, int64_t ldo, int order) {
    if (!w || !q8 || !out || rows < 0 || n < 0 || cols <= 0 || cols % ORC_QK_K) return -1;
    for (int64_t m = 0; m < n; ++m)
        for (int64_t r = 0; r < rows; ++r)
            out[m * ldo + r] = orc_dot_q5k_q8k((const uint8_t*)w + (size_t)r * row_bytes,
                                               (const uint8_t*)q8 + (size_t)m * q8_row_bytes, cols, order);
    return 0;
}
