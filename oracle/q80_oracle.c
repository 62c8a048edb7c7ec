/*
 * q80_oracle.c -- CPU restatement of the reference's Q8_0 x Q8_0 small-batch dot product.
 * TEST INFRASTRUCTURE ONLY (see q4k_oracle.h): nothing that ships links against it.
 *
 * Block (core/src/llm/matmul/q8_small_batch.h:9-14): fp16 d, int8 qs[32]; 34 bytes, qs at offset 2.  A weight is
 * d * qs[i].  The reference multiplies Q8_0 weights with activations quantized to Q8_0 as well (vec_dot_type of
 * Q8_0 is Q8_0, core/src/llm/matmul/batched_exec.cpp:630).
 *
 * Dot product (Q8SmallBatchDot4, core/src/llm/matmul/q8_small_batch.h:29-77): per 32-element block eight int32
 * lanes, lane i = sum of the products of elements 4i..4i+3; acc_i = fma(fp16(dx) * fp16(dy), float(lane_i), acc_i);
 * at the end ((a4+a0) + (a6+a2)) + ((a5+a1) + (a7+a3)) (:66-71).
 *
 * Activation quantizer: ggml's from_float for GGML_TYPE_Q8_0 (called at core/src/llm/matmul/gemv_exec.cpp:298,
 * core/src/llm/matmul/batched_exec.cpp:1364) lives in the ggml submodule, which is absent from the reference tree
 * (no pinned commit recorded).  PARITY UNPINNED: what is restated here is ggml's published algorithm in its two
 * forms -- variant 0, the x86 AVX2 path (d = amax / 127 stored as fp16; codes = round-half-even(x * (127 / amax)));
 * variant 1, the scalar reference (codes = roundf(x * (1 / d)), half away from zero).  The checks below hold for
 * either; no reference fixture tells them apart.
 *
 * Pins (tests/test_oracle_pins.py): layout sizeof/offsetof; integer block sums against an int64 numpy brute force
 * and closed forms; both fp32 orders against the dequantize-then-double dot; quantizer invariants (the extreme
 * element maps to +-127, every code within [-127, 127], d * q reconstructs x within d / 2, zero block -> zero
 * bytes, sign symmetry).
 */
#include <math.h>
#include <stddef.h>
#include <string.h>

#include "q4k_oracle.h"

#define ORC_Q80 32

typedef struct {
    uint16_t d;
    int8_t qs[ORC_Q80];
} orc_block_q80;

_Static_assert(sizeof(orc_block_q80) == 34, "Q8_0 block is 34 bytes");
_Static_assert(offsetof(orc_block_q80, qs) == 2, "Q8_0 codes follow the fp16 scale");

size_t orc_q80_block_bytes(void) { return sizeof(orc_block_q80); }

int orc_quantize_row_q80(const float* x, void* out, int64_t cols, int variant) {
    if (!x || !out || cols <= 0 || cols % ORC_Q80 || variant < 0 || variant > 1) return -1;
    orc_block_q80* y = (orc_block_q80*)out;
    for (int64_t b = 0; b < cols / ORC_Q80; ++b) {
        const float* v = x + b * ORC_Q80;
        float amax = 0.0f;
        for (int i = 0; i < ORC_Q80; ++i) {
            const float a = fabsf(v[i]);
            if (a > amax) amax = a;
        }
        const float d = amax / 127.0f;
        y[b].d = orc_fp32_to_fp16(d);
        for (int i = 0; i < ORC_Q80; ++i) {
            if (variant == 0) {
                const float id = amax != 0.0f ? 127.0f / amax : 0.0f;
                y[b].qs[i] = (int8_t)(int)nearbyintf(v[i] * id); /* default rounding mode: half to even */
            } else {
                const float id = d != 0.0f ? 1.0f / d : 0.0f;
                y[b].qs[i] = (int8_t)(int)roundf(v[i] * id);
            }
        }
    }
    return 0;
}

int orc_quantize_rows_q80(const float* x, int64_t n, int64_t ldx, void* out, int64_t cols, int variant) {
    if (n < 0 || ldx < cols) return -1;
    const size_t row_bytes = (size_t)(cols / ORC_Q80) * sizeof(orc_block_q80);
    for (int64_t m = 0; m < n; ++m)
        if (orc_quantize_row_q80(x + (size_t)m * (size_t)ldx, (uint8_t*)out + (size_t)m * row_bytes, cols, variant)) return -1;
    return 0;
}

static inline int32_t q80_block_sum(const orc_block_q80* w, const orc_block_q80* y) {
    int32_t s = 0;
    for (int i = 0; i < ORC_Q80; ++i) s += (int32_t)w->qs[i] * (int32_t)y->qs[i];
    return s;
}

/* isum[rows][n][cols / 32]: the integer every form of the kernel reaches before floating point. */
int orc_q80_matrix_block_sums(const void* w, int64_t rows, int64_t cols, size_t row_bytes, const void* q, int64_t n,
                              size_t q_row_bytes, int32_t* isum) {
    if (!w || !q || !isum || rows < 0 || n < 0 || cols <= 0 || cols % ORC_Q80) return -1;
    const int64_t nb = cols / ORC_Q80;
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t m = 0; m < n; ++m)
            for (int64_t b = 0; b < nb; ++b)
                isum[((size_t)r * (size_t)n + (size_t)m) * (size_t)nb + (size_t)b] =
                    q80_block_sum((const orc_block_q80*)((const uint8_t*)w + (size_t)r * row_bytes) + b,
                                  (const orc_block_q80*)((const uint8_t*)q + (size_t)m * q_row_bytes) + b);
    return 0;
}

/* order 0: the reference's eight-lane kernel; anything else: total = fma(dx * dy, float(block sum), total). */
float orc_dot_q80_q80(const void* w_row, const void* q_row, int64_t cols, int order) {
    const orc_block_q80* w = (const orc_block_q80*)w_row;
    const orc_block_q80* y = (const orc_block_q80*)q_row;
    float a[8] = {0};
    float total = 0.0f;
    for (int64_t b = 0; b < cols / ORC_Q80; ++b) {
        const float d = orc_fp16_to_fp32(w[b].d) * orc_fp16_to_fp32(y[b].d);
        if (order == ORC_ORDER_HWY) {
            for (int i = 0; i < 8; ++i) {
                int32_t lane = 0;
                for (int k = 0; k < 4; ++k) lane += (int32_t)w[b].qs[4 * i + k] * (int32_t)y[b].qs[4 * i + k];
                a[i] = fmaf(d, (float)lane, a[i]);
            }
        } else {
            total = fmaf(d, (float)q80_block_sum(w + b, y + b), total);
        }
    }
    if (order == ORC_ORDER_HWY) return ((a[4] + a[0]) + (a[6] + a[2])) + ((a[5] + a[1]) + (a[7] + a[3]));
    return total;
}

/* sum_i (dx qx_i) (dy qy_i) in double; magnitude: sum of the absolute values of the terms */
double orc_dot_dequant_q80_f64(const void* w_row, const void* q_row, int64_t cols, int magnitude) {
    const orc_block_q80* w = (const orc_block_q80*)w_row;
    const orc_block_q80* y = (const orc_block_q80*)q_row;
    double total = 0.0;
    for (int64_t b = 0; b < cols / ORC_Q80; ++b) {
        const double dx = (double)orc_fp16_to_fp32(w[b].d), dy = (double)orc_fp16_to_fp32(y[b].d);
        for (int i = 0; i < ORC_Q80; ++i) {
            const double t = (dx * (double)w[b].qs[i]) * (dy * (double)y[b].qs[i]);
            total += magnitude ? fabs(t) : t;
        }
    }
    return total;
}

int orc_mul_mat_q80_q80(const void* w, int64_t rows, int64_t cols, size_t row_bytes, const void* q, int64_t n,
                        size_t q_row_bytes, float* y, int64_t ldy, int order) {
    if (!w || !q || !y || rows < 0 || n < 0 || cols <= 0 || cols % ORC_Q80 || ldy < rows) return -1;
    for (int64_t m = 0; m < n; ++m)
        for (int64_t r = 0; r < rows; ++r)
            y[(size_t)m * (size_t)ldy + (size_t)r] = orc_dot_q80_q80((const uint8_t*)w + (size_t)r * row_bytes,
                                                                     (const uint8_t*)q + (size_t)m * q_row_bytes, cols, order);
    return 0;
}
