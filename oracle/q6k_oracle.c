/*
 * q6k_oracle.c -- CPU restatement of the reference's Q6_K x Q8_K dot product.
 * TEST INFRASTRUCTURE ONLY (see q4k_oracle.h): nothing that ships links against it.
 *
 * block_q6_K (core/src/llm/matmul/q6_small_batch.h:13-24): ql[128] low nibbles, qh[64] top two bits,
 * scales[16] signed bytes (one per 16 weights), fp16 d; 210 bytes, d at offset 208.  Element
 * e = 128 j + 32 z + l (j < 2, z < 4, l < 32) is
 *     q = (z < 2 ? ql[64 j + 32 (z & 1) + l] & 15 : ql[64 j + 32 (z & 1) + l] >> 4) | ((qh[32 j + l] >> 2 z) & 3) << 4
 * with weight value d * scales[e / 16] * (q - 32)  (q6_small_batch.h:56-76: q[0..3] are z = 0..3, the scale pair of
 * group z is scales[8 j + 2 z], scales[8 j + 2 z + 1], and maddubs(q, v) - maddubs(32, v) is sum (q - 32) v).
 * One integer per super-block: isum = sum_g scales[g] * sum_{i in g} (q_i - 32) * y_i; fp32: one fused
 * multiply-add per block, acc = fma(y.d * fp16(d), float(.), acc) (q6_small_batch.h:84-86).
 *
 * Pins (tests/test_oracle_pins.py): layout sizeof/offsetof; single-element placement (one non-zero code and one
 * non-zero activation contribute scale * (q - 32) * y at exactly that element); q = 32 everywhere gives 0, q = 0
 * gives -32 * sum_g scale_g * bsums_g (closed form through bsums); int64 brute force over an independent numpy
 * decode; both fp32 orders against the dequantize-then-double dot.
 */
#include <math.h>
#include <stddef.h>
#include <string.h>

#include "q4k_oracle.h"

typedef struct {
    uint8_t ql[ORC_QK_K / 2];
    uint8_t qh[ORC_QK_K / 4];
    int8_t scales[ORC_QK_K / 16];
    uint16_t d;
} orc_block_q6k;

_Static_assert(sizeof(orc_block_q6k) == 210, "block_q6_K is 210 bytes");
_Static_assert(offsetof(orc_block_q6k, qh) == 128 && offsetof(orc_block_q6k, scales) == 192 && offsetof(orc_block_q6k, d) == 208,
               "block_q6_K field offsets");

size_t orc_q6k_block_bytes(void) { return sizeof(orc_block_q6k); }

/* unsigned 6-bit code of element e (the weight is d * scale * (code - 32)) */
static inline int q6_code(const orc_block_q6k* w, int e) {
    const int j = e >> 7, z = (e >> 5) & 3, l = e & 31;
    const uint8_t lo = w->ql[64 * j + 32 * (z & 1) + l];
    const int nib = z < 2 ? (lo & 15) : (lo >> 4);
    return nib | (((w->qh[32 * j + l] >> (2 * z)) & 3) << 4);
}

int32_t orc_q6k_block_sum(const void* w_block, const void* q8_block) {
    const orc_block_q6k* w = (const orc_block_q6k*)w_block;
    const orc_block_q8k* y = (const orc_block_q8k*)q8_block;
    int32_t acc = 0;
    for (int g = 0; g < 16; ++g) {
        int32_t sub = 0;
        for (int i = 0; i < 16; ++i) sub += (q6_code(w, 16 * g + i) - 32) * (int32_t)y->qs[16 * g + i];
        acc += (int32_t)w->scales[g] * sub;
    }
    return acc;
}

int orc_q6k_matrix_block_sums(const void* w, int64_t rows, int64_t cols, size_t row_bytes, const void* q8, int64_t n,
                              size_t q8_row_bytes, int32_t* isum) {
    if (!w || !q8 || !isum || rows < 0 || n < 0 || cols <= 0 || cols % ORC_QK_K) return -1;
    const int64_t nb = cols / ORC_QK_K;
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t m = 0; m < n; ++m)
            for (int64_t b = 0; b < nb; ++b)
                isum[((size_t)r * (size_t)n + (size_t)m) * (size_t)nb + (size_t)b] =
                    orc_q6k_block_sum((const uint8_t*)w + (size_t)r * row_bytes + (size_t)b * sizeof(orc_block_q6k),
                                      (const uint8_t*)q8 + (size_t)m * q8_row_bytes + (size_t)b * sizeof(orc_block_q8k));
    return 0;
}

/* Row dot.  order 0 (the reference's kernel, q6_small_batch.h:50-92): eight int32 lanes per block -- lane i of a
 * 32-element group holds scale * (elements 4i..4i+3), groups added lane-wise -- each fused into its own fp32
 * accumulator, acc_i = fma(y.d * fp16(d), float(lane_i), acc_i); at the end ((a0+a4)+(a2+a6)) + ((a1+a5)+(a3+a7)).
 * Any other order: the plain per-block form, total = fma(y.d * fp16(d), float(isum), total). */
float orc_dot_q6k_q8k(const void* w_row, const void* q8_row, int64_t cols, int order) {
    const orc_block_q6k* w = (const orc_block_q6k*)w_row;
    const orc_block_q8k* y = (const orc_block_q8k*)q8_row;
    float lanes[8] = {0};
    float total = 0.0f;
    for (int64_t b = 0; b < cols / ORC_QK_K; ++b) {
        const float scale = y[b].d * orc_fp16_to_fp32(w[b].d);
        if (order == ORC_ORDER_HWY) {
            int32_t lane[8] = {0};
            for (int grp = 0; grp < 8; ++grp)  /* 32-element group (j, z) */
                for (int i = 0; i < 8; ++i) {
                    int32_t four = 0;
                    for (int k = 0; k < 4; ++k) {
                        const int e = 32 * grp + 4 * i + k;
                        four += (q6_code(w + b, e) - 32) * (int32_t)y[b].qs[e];
                    }
                    lane[i] += (int32_t)w[b].scales[2 * grp + (i >> 2)] * four;
                }
            for (int i = 0; i < 8; ++i) lanes[i] = fmaf(scale, (float)lane[i], lanes[i]);
        } else {
            total = fmaf(scale, (float)orc_q6k_block_sum(w + b, y + b), total);
        }
    }
    if (order == ORC_ORDER_HWY) {
        const float r0 = lanes[0] + lanes[4], r1 = lanes[1] + lanes[5], r2 = lanes[2] + lanes[6], r3 = lanes[3] + lanes[7];
        return (r0 + r2) + (r1 + r3);
    }
    return total;
}

/* dequantize both sides, multiply-accumulate in double; magnitude != 0: sum of |terms| instead */
double orc_dot_dequant_q6k_f64(const void* w_row, const void* q8_row, int64_t cols, int magnitude) {
    const orc_block_q6k* w = (const orc_block_q6k*)w_row;
    const orc_block_q8k* y = (const orc_block_q8k*)q8_row;
    double acc = 0.0;
    for (int64_t b = 0; b < cols / ORC_QK_K; ++b) {
        const double wd = orc_fp16_to_fp32(w[b].d);
        for (int e = 0; e < ORC_QK_K; ++e) {
            const double t = wd * w[b].scales[e >> 4] * (q6_code(w + b, e) - 32) * ((double)y[b].d * y[b].qs[e]);
            acc += magnitude ? fabs(t) : t;
        }
    }
    return acc;
}

int orc_mul_mat_q6k_q8k(const void* w, int64_t rows, int64_t cols, size_t row_bytes, const void* q8, int64_t n,
                        size_t q8_row_bytes, float* out, int64_t ldo, int order) {
    if (!w || !q8 || !out || rows < 0 || n < 0 || cols <= 0 || cols % ORC_QK_K) return -1;
    for (int64_t m = 0; m < n; ++m)
        for (int64_t r = 0; r < rows; ++r)
            out[m * ldo + r] = orc_dot_q6k_q8k((const uint8_t*)w + (size_t)r * row_bytes,
                                               (const uint8_t*)q8 + (size_t)m * q8_row_bytes, cols, order);
    return 0;
}
