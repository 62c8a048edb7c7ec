/*
 * q4k_oracle.c -- scalar CPU restatement of DenseCore's Q4_K x Q8_K path.
 * TEST INFRASTRUCTURE ONLY (see q4k_oracle.h).  Build with
 *   gcc -O2 -ffp-contract=off -fno-fast-math
 * so that every fp32 operation below is a separately rounded IEEE operation
 * in exactly the written order.
 */
#include "q4k_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

_Static_assert(sizeof(orc_block_q4k) == 144, "block_q4_K must be 144 bytes (q4_rowpair.h:22)");
_Static_assert(offsetof(orc_block_q4k, qs) == 16, "block_q4_K qs offset (q4_rowpair.h:22)");
_Static_assert(sizeof(orc_block_q8k) == 292, "block_q8_K must be 292 bytes (q4_rowpair.h:23)");
_Static_assert(offsetof(orc_block_q8k, bsums) == 260, "block_q8_K bsums offset (q4_rowpair.h:23)");

/* ------------------------------------------------------------------ */
/* fp16 <-> fp32.  hwy_moe_quant.cc:55-81 decodes by field; this does  */
/* the same decode, written as a normalisation of the significand.     */
/* ------------------------------------------------------------------ */
float orc_fp16_to_fp32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h >> 15) << 31;
    uint32_t e = (h >> 10) & 31u;
    uint32_t m = h & 1023u;
    uint32_t bits;
    if (e == 31u) {
        bits = sign | 0x7f800000u | (m << 13); /* inf / nan keep payload */
    } else if (e != 0u) {
        bits = sign | ((e + 112u) << 23) | (m << 13);
    } else if (m == 0u) {
        bits = sign;
    } else {
        /* subnormal half: shift the significand up until the hidden bit appears */
        int shift = 0;
        while (!(m & 1024u)) {
            m <<= 1;
            ++shift;
        }
        bits = sign | ((uint32_t)(113 - shift) << 23) | ((m & 1023u) << 13);
    }
    float f;
    memcpy(&f, &bits, sizeof f);
    return f;
}

/* Round-to-nearest-even fp32 -> fp16; only the synthetic generators need it. */
uint16_t orc_fp32_to_fp16(float f) {
    uint32_t x;
    memcpy(&x, &f, sizeof x);
    const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    const uint32_t absx = x & 0x7fffffffu;
    if (absx >= 0x7f800000u) {
        return (uint16_t)(sign | 0x7c00u | (absx > 0x7f800000u ? 0x200u | ((absx >> 13) & 0x3ffu) : 0u));
    }
    if (absx >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (absx < 0x33000001u) { /* below half of the smallest subnormal */
        return sign;
    }
    int32_t e = (int32_t)(absx >> 23) - 127;
    uint32_t m = (absx & 0x7fffffu) | 0x800000u;
    int shift; /* number of low bits dropped from the 24-bit significand */
    uint32_t base;
    if (e >= -14) {
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
        m &= 0x7fffffu;
    } else {
        shift = 13 + (-14 - e);
        base = 0;
    }
    uint32_t q = m >> shift;
    const uint32_t rem = m & ((1u << shift) - 1u);
    const uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) {
        ++q;
    }
    return (uint16_t)(sign | (base + q)); /* a carry out of the mantissa bumps the exponent */
}

/* hwy_moe_quant.cc:83-88: adding 1.5*2^23 leaves round-to-nearest-even(v) in the low mantissa bits. */
int orc_nearest_int(float v) {
    const float shifted = v + 12582912.0f;
    int32_t bits;
    memcpy(&bits, &shifted, sizeof bits);
    return (bits & 0x007fffff) - 0x00400000;
}

/* ------------------------------------------------------------------ */
/* 6-bit scale / min unpacking, two independent formulations           */
/* ------------------------------------------------------------------ */
/* Word-parallel form (hwy_moe_quant.cc:90-101). */
void orc_q4k_scales_kmask(const uint8_t packed[12], uint8_t scales[8], uint8_t mins[8]) {
    uint32_t w[3];
    memcpy(w, packed, 12);
    const uint32_t lo6 = 0x3f3f3f3fu, lo4 = 0x0f0f0f0fu, lo2 = 0x03030303u;
    const uint32_t sc_lo = w[0] & lo6;                                    /* scales 0..3 */
    const uint32_t mn_lo = w[1] & lo6;                                    /* mins   0..3 */
    const uint32_t sc_hi = (w[2] & lo4) | (((w[0] >> 6) & lo2) << 4);     /* scales 4..7 */
    const uint32_t mn_hi = ((w[2] >> 4) & lo4) | (((w[1] >> 6) & lo2) << 4); /* mins 4..7 */
    memcpy(scales, &sc_lo, 4);
    memcpy(scales + 4, &sc_hi, 4);
    memcpy(mins, &mn_lo, 4);
    memcpy(mins + 4, &mn_hi, 4);
}

/* Per-index form (q4_rowpair.h:60-62). */
void orc_q4k_scales_indexed(const uint8_t packed[12], uint8_t scales[8], uint8_t mins[8]) {
    for (int g = 0; g < 8; ++g) {
        if (g < 4) {
            scales[g] = packed[g] & 63;
            mins[g] = packed[g + 4] & 63;
        } else {
            scales[g] = (uint8_t)((packed[g + 4] & 15) | ((packed[g - 4] >> 6) << 4));
            mins[g] = (uint8_t)((packed[g + 4] >> 4) | ((packed[g] >> 6) << 4));
        }
    }
}

/* ------------------------------------------------------------------ */
/* fast exp / SiLU flavours                                             */
/* ------------------------------------------------------------------ */
/* cpu_backend_internal.h:99-114 and native.cpp:287-301 (unfused Horner). */
float orc_fast_exp(float x) {
    if (x < -50.0f) x = -50.0f;
    if (x > 50.0f) x = 50.0f;
    const float y = x * 1.4426950408889634f;
    const int32_t i = (int32_t)floorf(y);
    const float f = y - (float)i;
    const float inner = 0.224494337302845f + f * 0.07944023841053369f;
    const float mid = 0.6960656421638072f + f * inner;
    const float p = 1.0f + f * mid;
    const int32_t ebits = (i + 127) << 23;
    float two_i;
    memcpy(&two_i, &ebits, sizeof two_i);
    return two_i * p;
}

/* hwy_fastexp.h:13-47 (vector) / :50-84 (scalar tail): same cubic with fused multiply-adds. */
float orc_fast_exp_fma(float x) {
    x = fmaxf(fminf(x, 50.0f), -50.0f);
    const float y = x * 1.4426950408889634f;
    const float fl = floorf(y);
    const float f = y - fl;
    float p = fmaf(f, 0.07944023841053369f, 0.224494337302845f);
    p = fmaf(f, p, 0.6960656421638072f);
    p = fmaf(f, p, 1.0f);
    const int32_t ebits = ((int32_t)fl + 127) << 23;
    float two_i;
    memcpy(&two_i, &ebits, sizeof two_i);
    return two_i * p;
}

float orc_silu_mul(float gate, float up, int silu_mode) {
    switch (silu_mode) {
    case ORC_SILU_FAST: /* cpu_backend_moe_raw_batched.inl:1672-1673 */
        return (gate / (1.0f + orc_fast_exp(-gate))) * up;
    case ORC_SILU_FAST_FMA: { /* hwy_activation.cc:163-166 */
        const float e = orc_fast_exp_fma(gate * -1.0f);
        const float sig = 1.0f / (1.0f + e);
        return (gate * sig) * up;
    }
    default: /* hwy_moe_quant.cc:377 */
        return (gate / (1.0f + expf(-gate))) * up;
    }
}

/* ------------------------------------------------------------------ */
/* Q8_K quantizer (hwy_moe_quant.cc:103-143)                            */
/* ------------------------------------------------------------------ */
static void quantize_block_q8k(const float* x, orc_block_q8k* y) {
    float best_abs = 0.0f, best = 0.0f;
    for (int j = 0; j < ORC_QK_K; ++j) {
        const float a = fabsf(x[j]);
        if (a > best_abs) { /* strict: the first of equal magnitudes wins and keeps its sign */
            best_abs = a;
            best = x[j];
        }
    }
    if (best_abs == 0.0f) {
        memset(y, 0, sizeof *y);
        return;
    }
    const float inv = -127.0f / best;
    for (int j = 0; j < ORC_QK_K; ++j) {
        const int q = orc_nearest_int(inv * x[j]);
        y->qs[j] = (int8_t)(q > 127 ? 127 : q);
    }
    for (int s = 0; s < ORC_QK_K / 16; ++s) {
        int acc = 0;
        for (int i = 0; i < 16; ++i) acc += y->qs[16 * s + i];
        y->bsums[s] = (int16_t)acc;
    }
    y->d = 1.0f / inv;
}

int orc_quantize_row_q8k(const float* x, void* q8_out, int64_t cols) {
    if (!x || !q8_out || cols <= 0 || cols % ORC_QK_K) return -1;
    orc_block_q8k* y = (orc_block_q8k*)q8_out;
    for (int64_t b = 0; b < cols / ORC_QK_K; ++b) quantize_block_q8k(x + b * ORC_QK_K, y + b);
    return 0;
}

int orc_quantize_rows_q8k(const float* x, int64_t n, int64_t ldx, void* q8_out, int64_t cols) {
    if (!x || !q8_out || n < 0 || cols <= 0 || cols % ORC_QK_K || ldx < cols) return -1;
    const size_t row_bytes = (size_t)(cols / ORC_QK_K) * sizeof(orc_block_q8k);
    for (int64_t r = 0; r < n; ++r) {
        orc_quantize_row_q8k(x + r * ldx, (uint8_t*)q8_out + (size_t)r * row_bytes, cols);
    }
    return 0;
}

/* ------------------------------------------------------------------ */
/* integer sums                                                         */
/* ------------------------------------------------------------------ */
/* Element e of a super-block: chunk c = e/64 holds 32 bytes; the low nibbles
 * are sub-block 2c, the high nibbles sub-block 2c+1
 * (kquant_batched_kernels.h:63-71). */
static inline int q4_element(const orc_block_q4k* w, int e) {
    const int chunk = e >> 6, within = e & 63;
    const uint8_t byte = w->qs[32 * chunk + (within & 31)];
    return within < 32 ? (byte & 15) : (byte >> 4);
}

/* Per-sub-block raw dots, split into `parts` equal slices of the 32 elements
 * (parts = 1, 8 slices of 4, or 8 residue classes mod 8 -- see callers). */
static void subblock_dots(const orc_block_q4k* w, const orc_block_q8k* y, int32_t sub[8]) {
    for (int g = 0; g < 8; ++g) {
        int32_t acc = 0;
        for (int i = 0; i < 32; ++i) acc += q4_element(w, 32 * g + i) * (int32_t)y->qs[32 * g + i];
        sub[g] = acc;
    }
}

static int32_t min_dot_of(const uint8_t mins[8], const orc_block_q8k* y) {
    int32_t acc = 0;
    for (int j = 0; j < 16; ++j) acc += (int32_t)y->bsums[j] * (int32_t)mins[j >> 1];
    return acc;
}

void orc_block_sums(const orc_block_q4k* w, const orc_block_q8k* y, int32_t* dot_scaled, int32_t* min_dot) {
    uint8_t sc[8], mn[8];
    int32_t sub[8];
    orc_q4k_scales_kmask(w->scales, sc, mn);
    subblock_dots(w, y, sub);
    int32_t acc = 0;
    for (int g = 0; g < 8; ++g) acc += (int32_t)sc[g] * sub[g];
    if (dot_scaled) *dot_scaled = acc;
    if (min_dot) *min_dot = min_dot_of(mn, y);
}

int orc_matrix_block_sums(const void* w, int64_t rows, int64_t cols, size_t row_bytes, const void* q8, int64_t n,
                          size_t q8_row_bytes, int32_t* dot_scaled, int32_t* min_dot) {
    if (!w || !q8 || rows < 0 || n < 0 || cols <= 0 || cols % ORC_QK_K) return -1;
    const int64_t nb = cols / ORC_QK_K;
    for (int64_t r = 0; r < rows; ++r) {
        const orc_block_q4k* wr = (const orc_block_q4k*)((const uint8_t*)w + (size_t)r * row_bytes);
        for (int64_t m = 0; m < n; ++m) {
            const orc_block_q8k* ym = (const orc_block_q8k*)((const uint8_t*)q8 + (size_t)m * q8_row_bytes);
            for (int64_t b = 0; b < nb; ++b) {
                const size_t idx = ((size_t)r * (size_t)n + (size_t)m) * (size_t)nb + (size_t)b;
                orc_block_sums(wr + b, ym + b, dot_scaled ? dot_scaled + idx : NULL, min_dot ? min_dot + idx : NULL);
            }
        }
    }
    return 0;
}

/* ------------------------------------------------------------------ */
/* row dot in the four fp32 orders                                      */
/* ------------------------------------------------------------------ */
/* Eight int32 lanes, lane l = sum over sub-blocks of scale * (elements 4l..4l+3
 * of the sub-block).  This is both the 256-bit Highway partition
 * (hwy_moe_quant.cc:228-247, SumOfMulQuadAccumulate on 32 bytes -> 8 lanes)
 * and the AVX2 one (maddubs pairs, then madd pairs: kquant_batched_kernels.h:529-537). */
static void lanes_quad(const orc_block_q4k* w, const orc_block_q8k* y, const uint8_t sc[8], int32_t lane[8]) {
    memset(lane, 0, 8 * sizeof(int32_t));
    for (int g = 0; g < 8; ++g) {
        for (int l = 0; l < 8; ++l) {
            int32_t acc = 0;
            for (int i = 0; i < 4; ++i) {
                const int e = 32 * g + 4 * l + i;
                acc += q4_element(w, e) * (int32_t)y->qs[e];
            }
            lane[l] += (int32_t)sc[g] * acc;
        }
    }
}

/* Eight int32 lanes, lane l = elements with index % 8 == l
 * (kquant_batched_kernels.h:99-108). */
static void lanes_mod8(const orc_block_q4k* w, const orc_block_q8k* y, const uint8_t sc[8], int32_t lane[8]) {
    memset(lane, 0, 8 * sizeof(int32_t));
    for (int g = 0; g < 8; ++g) {
        for (int i = 0; i < 32; ++i) {
            const int e = 32 * g + i;
            lane[i & 7] += (int32_t)sc[g] * ((int32_t)y->qs[e] * q4_element(w, e));
        }
    }
}

/* HSumFloat8 (kquant_batched_kernels.h:398-404): upper+lower halves, then
 * movehl, then the odd element.  Highway's 256-bit ReduceSum is taken to be
 * the same tree (Highway itself is absent from the reference tree). */
static float hsum8_tree(const int32_t lane[8]) {
    float v[8];
    for (int l = 0; l < 8; ++l) v[l] = (float)lane[l];
    const float a0 = v[4] + v[0], a1 = v[5] + v[1], a2 = v[6] + v[2], a3 = v[7] + v[3];
    const float b0 = a0 + a2, b1 = a1 + a3;
    return b0 + b1;
}

float orc_dot_q4k_q8k(const void* w_row, const void* q8_row, int64_t cols, int order) {
    const orc_block_q4k* w = (const orc_block_q4k*)w_row;
    const orc_block_q8k* y = (const orc_block_q8k*)q8_row;
    const int64_t nb = cols / ORC_QK_K;
    float total = 0.0f;
    float lane_acc[8] = {0};
    float min_acc = 0.0f;
    for (int64_t b = 0; b < nb; ++b) {
        uint8_t sc[8], mn[8];
        int32_t lane[8];
        orc_q4k_scales_kmask(w[b].scales, sc, mn);
        const int32_t md = min_dot_of(mn, y + b);
        const float wd = orc_fp16_to_fp32(w[b].d);
        const float wm = orc_fp16_to_fp32(w[b].dmin);
        const float yd = y[b].d;
        switch (order) {
        case ORC_ORDER_HWY: {
            lanes_quad(w + b, y + b, sc, lane);
            const float block_dot = hsum8_tree(lane);
            const float d = wd * yd;
            const float dm = wm * yd;
            total += d * block_dot;
            total -= dm * (float)md;
            break;
        }
        case ORC_ORDER_AVX2: {
            lanes_quad(w + b, y + b, sc, lane);
            const float d = wd * yd;
            const float dm = -wm * yd;
            const float t = d * hsum8_tree(lane) + dm * (float)md;
            total += t;
            break;
        }
        case ORC_ORDER_SCALAR: {
            lanes_mod8(w + b, y + b, sc, lane);
            const float d = wd * yd;
            const float dm = wm * yd;
            for (int l = 0; l < 8; ++l) lane_acc[l] += d * (float)lane[l];
            min_acc -= dm * (float)md;
            break;
        }
        default: { /* ORC_ORDER_DOTPROD */
            int32_t ds;
            orc_block_sums(w + b, y + b, &ds, NULL);
            const float d = wd * yd;
            const float dm = wm * yd;
            const float t = d * (float)ds - dm * (float)md;
            total += t;
            break;
        }
        }
    }
    if (order == ORC_ORDER_SCALAR) {
        total = min_acc;
        for (int l = 0; l < 8; ++l) total += lane_acc[l];
    }
    return total;
}

/* The reference's own slow check (tests/moe/test_moe_ops.cpp:170-201):
 * dequantize both sides, multiply-accumulate in double. */
double orc_dot_dequant_f64(const void* w_row, const void* q8_row, int64_t cols) {
    const orc_block_q4k* w = (const orc_block_q4k*)w_row;
    const orc_block_q8k* y = (const orc_block_q8k*)q8_row;
    double acc = 0.0;
    for (int64_t b = 0; b < cols / ORC_QK_K; ++b) {
        uint8_t sc[8], mn[8];
        orc_q4k_scales_indexed(w[b].scales, sc, mn);
        const double wd = orc_fp16_to_fp32(w[b].d), wm = orc_fp16_to_fp32(w[b].dmin);
        for (int e = 0; e < ORC_QK_K; ++e) {
            const int g = e >> 5;
            const double weight = wd * sc[g] * q4_element(w + b, e) - wm * mn[g];
            const double act = (double)y[b].d * (double)y[b].qs[e];
            acc += weight * act;
        }
    }
    return acc;
}

double orc_dot_magnitude_f64(const void* w_row, const void* q8_row, int64_t cols) {
    const orc_block_q4k* w = (const orc_block_q4k*)w_row;
    const orc_block_q8k* y = (const orc_block_q8k*)q8_row;
    double acc = 0.0;
    for (int64_t b = 0; b < cols / ORC_QK_K; ++b) {
        int32_t ds, md;
        orc_block_sums(w + b, y + b, &ds, &md);
        const double yd = y[b].d;
        acc += fabs((double)orc_fp16_to_fp32(w[b].d) * yd * ds) + fabs((double)orc_fp16_to_fp32(w[b].dmin) * yd * md);
    }
    return acc;
}

int orc_mul_mat_q4k_q8k(const void* w, int64_t rows, int64_t cols, size_t row_bytes, const void* q8, int64_t n,
                        size_t q8_row_bytes, float* out, int64_t ldo, int order) {
    if (!w || !q8 || !out || rows < 0 || n < 0 || cols <= 0 || cols % ORC_QK_K || ldo < rows) return -1;
    if (row_bytes < (size_t)(cols / ORC_QK_K) * sizeof(orc_block_q4k)) return -1;
    if (q8_row_bytes < (size_t)(cols / ORC_QK_K) * sizeof(orc_block_q8k)) return -1;
    for (int64_t m = 0; m < n; ++m) {
        const uint8_t* ym = (const uint8_t*)q8 + (size_t)m * q8_row_bytes;
        for (int64_t r = 0; r < rows; ++r) {
            out[m * ldo + r] = orc_dot_q4k_q8k((const uint8_t*)w + (size_t)r * row_bytes, ym, cols, order);
        }
    }
    return 0;
}

int orc_mul_mat_q4k_f32(const void* w, int64_t rows, int64_t cols, size_t row_bytes, const float* x, int64_t n,
                        int64_t ldx, float* out, int64_t ldo, int order) {
    if (!x || cols <= 0 || cols % ORC_QK_K || n < 0) return -1;
    const size_t q8_row_bytes = (size_t)(cols / ORC_QK_K) * sizeof(orc_block_q8k);
    void* q8 = malloc(q8_row_bytes * (size_t)(n > 0 ? n : 1));
    if (!q8) return -2;
    int rc = orc_quantize_rows_q8k(x, n, ldx, q8, cols);
    if (rc == 0) rc = orc_mul_mat_q4k_q8k(w, rows, cols, row_bytes, q8, n, q8_row_bytes, out, ldo, order);
    free(q8);
    return rc;
}

/* ------------------------------------------------------------------ */
/* fused gate/up + SwiGLU on one activation set (hwy_moe_quant.cc:359-380) */
/* ------------------------------------------------------------------ */
int orc_swiglu_mul_mat_q4k_f32(const void* gate, const void* up, int64_t inter, int64_t hidden, const float* x,
                               int64_t n, float* out, int order, int silu_mode) {
    if (!gate || !up || !x || !out || hidden <= 0 || hidden % ORC_QK_K || inter <= 0) return -1;
    const size_t wrow = (size_t)(hidden / ORC_QK_K) * sizeof(orc_block_q4k);
    float* u = (float*)malloc(sizeof(float) * (size_t)n * (size_t)inter);
    if (!u) return -2;
    int rc = orc_mul_mat_q4k_f32(gate, inter, hidden, wrow, x, n, hidden, out, inter, order);
    if (rc == 0) rc = orc_mul_mat_q4k_f32(up, inter, hidden, wrow, x, n, hidden, u, inter, order);
    for (int64_t i = 0; rc == 0 && i < n * inter; ++i) out[i] = orc_silu_mul(out[i], u[i], silu_mode);
    free(u);
    return rc;
}

/* ------------------------------------------------------------------ */
/* dense SwiGLU FFN                                                     */
/* ------------------------------------------------------------------ */
int orc_ffn_swiglu_q4k(const void* gate, const void* up, const void* down, int64_t hidden, int64_t inter,
                       const float* x, int64_t n, float* y, int order, int silu_mode, float* inter_out) {
    if (!gate || !up || !down || !x || !y || hidden <= 0 || inter <= 0 || hidden % ORC_QK_K || inter % ORC_QK_K)
        return -1;
    const size_t wrow_in = (size_t)(hidden / ORC_QK_K) * sizeof(orc_block_q4k);
    const size_t wrow_mid = (size_t)(inter / ORC_QK_K) * sizeof(orc_block_q4k);
    float* g = (float*)malloc(sizeof(float) * (size_t)n * (size_t)inter * 2);
    if (!g) return -2;
    float* u = g + (size_t)n * (size_t)inter;
    int rc = orc_mul_mat_q4k_f32(gate, inter, hidden, wrow_in, x, n, hidden, g, inter, order);
    if (rc == 0) rc = orc_mul_mat_q4k_f32(up, inter, hidden, wrow_in, x, n, hidden, u, inter, order);
    if (rc == 0) {
        for (int64_t i = 0; i < n * inter; ++i) g[i] = orc_silu_mul(g[i], u[i], silu_mode);
        if (inter_out) memcpy(inter_out, g, sizeof(float) * (size_t)n * (size_t)inter);
        rc = orc_mul_mat_q4k_f32(down, hidden, inter, wrow_mid, g, n, inter, y, hidden, order);
    }
    free(g);
    return rc;
}

/* ------------------------------------------------------------------ */
/* router                                                               */
/* ------------------------------------------------------------------ */
/* native.cpp:610-619: non-NaN before NaN, larger logit first, lower id on ties. */
static int candidate_precedes(float a, int32_t ia, float b, int32_t ib) {
    const int an = isnan(a), bn = isnan(b);
    if (an != bn) return !an;
    if (a > b) return 1;
    if (a < b) return 0;
    return ia < ib;
}

static void softmax_selected(const float* logits, int64_t n_experts, const int32_t* ids, int top_k, int mode,
                             float* weights) {
    if (mode == 0) { /* native.cpp:650-675 */
        float mx = -INFINITY;
        int all_finite = 1;
        for (int k = 0; k < top_k; ++k) {
            const float v = logits[ids[k]];
            all_finite = all_finite && isfinite(v);
            if (isfinite(v)) mx = fmaxf(mx, v);
        }
        float den = 0.0f;
        if (all_finite && isfinite(mx)) {
            for (int k = 0; k < top_k; ++k) {
                weights[k] = expf(logits[ids[k]] - mx);
                den += weights[k];
            }
        }
        if (!(den > 0.0f) || !isfinite(den)) {
            for (int k = 0; k < top_k; ++k) weights[k] = 1.0f / (float)top_k;
            return;
        }
        for (int k = 0; k < top_k; ++k) weights[k] /= den;
    } else if (mode == 1) { /* native.cpp:2321-2355 */
        float mx = -INFINITY;
        for (int k = 0; k < top_k; ++k) {
            if (ids[k] >= 0 && ids[k] < n_experts) mx = fmaxf(mx, logits[ids[k]]);
        }
        if (!isfinite(mx)) mx = 0.0f;
        float den = 0.0f;
        for (int k = 0; k < top_k; ++k) {
            float v = 0.0f;
            if (ids[k] >= 0 && ids[k] < n_experts) {
                v = expf(logits[ids[k]] - mx);
                den += v;
            }
            weights[k] = v;
        }
        den = fmaxf(den, 6.103515625e-5f);
        for (int k = 0; k < top_k; ++k) weights[k] /= den;
    } else { /* native.cpp:822-866 */
        float mx = -INFINITY;
        int valid = 0;
        for (int k = 0; k < top_k; ++k) {
            if (ids[k] >= 0 && ids[k] < n_experts && isfinite(logits[ids[k]])) mx = fmaxf(mx, logits[ids[k]]);
        }
        float den = 0.0f;
        for (int k = 0; k < top_k; ++k) {
            if (ids[k] >= 0 && ids[k] < n_experts) {
                ++valid;
                if (isfinite(logits[ids[k]]) && isfinite(mx)) den += expf(logits[ids[k]] - mx);
            }
        }
        const int uniform = !(den > 0.0f) || !isfinite(den);
        den = uniform ? 1.0f : fmaxf(den, 6.103515625e-5f);
        const float uni = valid > 0 ? 1.0f / (float)valid : 0.0f;
        for (int k = 0; k < top_k; ++k) {
            float v = 0.0f;
            if (ids[k] >= 0 && ids[k] < n_experts) {
                const float l = logits[ids[k]];
                v = (uniform || !isfinite(l) || !isfinite(mx)) ? uni : expf(l - mx) / den;
            }
            weights[k] = v;
        }
    }
}

int orc_route_topk(const float* logits, int64_t n_experts, int64_t n_tokens, int top_k, int weights_mode,
                   int32_t* ids, float* weights) {
    if (!logits || !ids || !weights || n_experts <= 0 || top_k <= 0 || top_k > n_experts || n_tokens < 0) return -1;
    for (int64_t t = 0; t < n_tokens; ++t) {
        const float* row = logits + t * n_experts;
        int32_t* sel = ids + t * top_k;
        int count = 0;
        /* insertion into a sorted list of at most top_k (native.cpp:628-645) */
        for (int32_t e = 0; e < n_experts; ++e) {
            int pos = count;
            while (pos > 0 && candidate_precedes(row[e], e, row[sel[pos - 1]], sel[pos - 1])) --pos;
            if (pos >= top_k) continue;
            const int last = count < top_k - 1 ? count : top_k - 1;
            for (int j = last; j > pos; --j) sel[j] = sel[j - 1];
            sel[pos] = e;
            if (count < top_k) ++count;
        }
        softmax_selected(row, n_experts, sel, top_k, weights_mode, weights + t * top_k);
    }
    return 0;
}

/* Routing weights of GIVEN ids (the down node resolves them from the raw logits itself):
 * native.cpp:2305-2357.  Ids outside [0, n_experts) get weight 0 and take no part in the max. */
int orc_route_weights_from_ids(const float* logits, int64_t n_experts, int64_t n_tokens, const int32_t* ids, int top_k,
                               float* weights) {
    if (!logits || !ids || !weights || n_experts <= 0 || top_k <= 0 || n_tokens < 0) return -1;
    for (int64_t t = 0; t < n_tokens; ++t) {
        const float* row = logits + t * n_experts;
        const int32_t* sel = ids + t * top_k;
        float* w = weights + t * top_k;
        float mx = -INFINITY;
        for (int k = 0; k < top_k; ++k)
            if (sel[k] >= 0 && sel[k] < n_experts && row[sel[k]] > mx) mx = row[sel[k]];
        if (!isfinite(mx)) mx = 0.0f;
        float den = 0.0f;
        for (int k = 0; k < top_k; ++k) {
            float v = 0.0f;
            if (sel[k] >= 0 && sel[k] < n_experts) {
                v = expf(row[sel[k]] - mx);
                den += v;
            }
            w[k] = v;
        }
        if (den < 6.103515625e-5f) den = 6.103515625e-5f;
        for (int k = 0; k < top_k; ++k) w[k] /= den;
    }
    return 0;
}

static int cmp_assignment(const void* pa, const void* pb) {
    const orc_assignment* a = (const orc_assignment*)pa;
    const orc_assignment* b = (const orc_assignment*)pb;
    if (a->expert != b->expert) return a->expert < b->expert ? -1 : 1;
    if (a->token != b->token) return a->token < b->token ? -1 : 1;
    if (a->k != b->k) return a->k < b->k ? -1 : 1;
    return 0;
}

/* native.cpp:1697-1733 */
int64_t orc_build_assignments(const int32_t* ids, int64_t n_tokens, int top_k, int64_t n_experts, orc_assignment* out) {
    int64_t count = 0;
    for (int64_t t = 0; t < n_tokens; ++t) {
        for (int k = 0; k < top_k; ++k) {
            const int32_t e = ids[t * top_k + k];
            if (e < 0 || e >= n_experts) continue;
            out[count].expert = e;
            out[count].token = (int32_t)t;
            out[count].k = k;
            ++count;
        }
    }
    qsort(out, (size_t)count, sizeof *out, cmp_assignment);
    return count;
}

/* ------------------------------------------------------------------ */
/* MoE layer                                                            */
/* ------------------------------------------------------------------ */
static float stable_sigmoid(float x) { /* fused_ops.cpp:451-458 */
    if (x >= 0.0f) {
        const float z = expf(-x);
        return 1.0f / (1.0f + z);
    }
    const float z = expf(x);
    return z / (1.0f + z);
}

/* One row product for any of the K-quant types a stack may have. */
float orc_dot_q5k_q8k(const void* w_row, const void* q8_row, int64_t cols, int order);
float orc_dot_q6k_q8k(const void* w_row, const void* q8_row, int64_t cols, int order);
float orc_dot_typed_q8k(int ggml_type, const void* w_row, const void* q8_row, int64_t cols, int order) {
    if (ggml_type == 13) return orc_dot_q5k_q8k(w_row, q8_row, cols, order);
    if (ggml_type == 14) return orc_dot_q6k_q8k(w_row, q8_row, cols, order);
    return orc_dot_q4k_q8k(w_row, q8_row, cols, order);
}
size_t orc_row_bytes_typed(int ggml_type, int64_t cols) {
    const size_t blocks = (size_t)(cols / ORC_QK_K);
    return blocks * (ggml_type == 13 ? 176u : ggml_type == 14 ? 210u : sizeof(orc_block_q4k));
}

int orc_ffn_swiglu_typed(int gu_type, int down_type, const void* gate, const void* up, const void* down, int64_t hidden,
                         int64_t inter, const float* x, int64_t n, float* y, int order, int silu_mode, float* inter_out) {
    if (!gate || !up || !down || !x || !y || hidden <= 0 || inter <= 0 || hidden % ORC_QK_K || inter % ORC_QK_K)
        return -1;
    const size_t wrow_in = orc_row_bytes_typed(gu_type, hidden), wrow_mid = orc_row_bytes_typed(down_type, inter);
    const size_t q8_in = (size_t)(hidden / ORC_QK_K) * sizeof(orc_block_q8k);
    const size_t q8_mid = (size_t)(inter / ORC_QK_K) * sizeof(orc_block_q8k);
    uint8_t* xq = (uint8_t*)malloc(q8_in > q8_mid ? q8_in : q8_mid);
    float* h = (float*)malloc(sizeof(float) * (size_t)inter);
    int rc = (xq && h) ? 0 : -2;
    for (int64_t m = 0; rc == 0 && m < n; ++m) {
        rc = orc_quantize_row_q8k(x + (size_t)m * hidden, xq, hidden);
        for (int64_t r = 0; rc == 0 && r < inter; ++r) {
            const float g = orc_dot_typed_q8k(gu_type, (const uint8_t*)gate + (size_t)r * wrow_in, xq, hidden, order);
            const float u = orc_dot_typed_q8k(gu_type, (const uint8_t*)up + (size_t)r * wrow_in, xq, hidden, order);
            h[r] = orc_silu_mul(g, u, silu_mode);
        }
        if (rc == 0 && inter_out) memcpy(inter_out + (size_t)m * inter, h, sizeof(float) * (size_t)inter);
        if (rc == 0) rc = orc_quantize_row_q8k(h, xq, inter);
        for (int64_t r = 0; rc == 0 && r < hidden; ++r)
            y[(size_t)m * hidden + r] = orc_dot_typed_q8k(down_type, (const uint8_t*)down + (size_t)r * wrow_mid, xq, inter, order);
    }
    free(xq);
    free(h);
    return rc;
}

/* hidden[t][k][r] = silu(gate_e[r] . q8(x[t])) * (up_e[r] . q8(x[t])), e = ids[t][k]
 * (native.cpp:4306-4342 / hwy_moe_quant.cc:359-380; raw_batched.inl:1629-1698 for n > 4).
 * Entries whose id is outside [0, n_experts) are left untouched. */
int orc_moe_gateup_swiglu(const orc_moe_weights* w, const float* x, const int32_t* ids, int64_t n_tokens, int order,
                          int silu_mode, float* hidden) {
    if (!w || !x || !ids || !hidden || w->hidden % ORC_QK_K) return -1;
    const int64_t H = w->hidden, I = w->inter;
    const int K = w->top_k;
    const size_t row_in = orc_row_bytes_typed(w->gu_type, H);
    const size_t exp_in = row_in * (size_t)I;
    const size_t q8_in = (size_t)(H / ORC_QK_K) * sizeof(orc_block_q8k);
    uint8_t* xq = (uint8_t*)malloc(q8_in * (size_t)n_tokens);
    if (!xq) return -2;
    int rc = orc_quantize_rows_q8k(x, n_tokens, H, xq, H);
    for (int64_t t = 0; rc == 0 && t < n_tokens; ++t) {
        for (int k = 0; k < K; ++k) {
            const int32_t e = ids[t * K + k];
            if (e < 0 || e >= w->n_experts) continue;
            const uint8_t* ge = (const uint8_t*)w->gate_exps + (size_t)e * exp_in;
            const uint8_t* ue = (const uint8_t*)w->up_exps + (size_t)e * exp_in;
            float* h = hidden + ((size_t)t * K + k) * (size_t)I;
            for (int64_t r = 0; r < I; ++r) {
                const float g = orc_dot_typed_q8k(w->gu_type, ge + (size_t)r * row_in, xq + (size_t)t * q8_in, H, order);
                const float u = orc_dot_typed_q8k(w->gu_type, ue + (size_t)r * row_in, xq + (size_t)t * q8_in, H, order);
                h[r] = orc_silu_mul(g, u, silu_mode);
            }
        }
    }
    free(xq);
    return rc;
}

/* y[t][r] = sum over routed experts of weights[t][k] * (down_e[r] . q8(hidden[t][k])).
 * accumulate_mode 0: per token, k = 0..top_k-1 in routing order (native.cpp:3233-3285);
 * accumulate_mode 1: expert-sorted assignment order (native.cpp:3152-3194). */
int orc_moe_down_weighted(const orc_moe_weights* w, const float* hidden, const int32_t* ids, const float* weights,
                          int64_t n_tokens, int order, int accumulate_mode, float* y) {
    if (!w || !hidden || !ids || !weights || !y || w->inter % ORC_QK_K) return -1;
    const int64_t H = w->hidden, I = w->inter, E = w->n_experts;
    const int K = w->top_k;
    const size_t row_mid = orc_row_bytes_typed(w->down_type, I);
    const size_t exp_mid = row_mid * (size_t)H;
    const size_t q8_mid = (size_t)(I / ORC_QK_K) * sizeof(orc_block_q8k);
    uint8_t* hq = (uint8_t*)malloc(q8_mid * (size_t)n_tokens * K);
    orc_assignment* asg = (orc_assignment*)malloc(sizeof(orc_assignment) * (size_t)n_tokens * K);
    if (!hq || !asg) {
        free(hq);
        free(asg);
        return -2;
    }
    orc_quantize_rows_q8k(hidden, n_tokens * K, I, hq, I);
    memset(y, 0, sizeof(float) * (size_t)n_tokens * (size_t)H);
    const int64_t cnt = orc_build_assignments(ids, n_tokens, K, E, asg);
    if (accumulate_mode == 0) { /* re-sort the valid entries into (token, k) order */
        int64_t c = 0;
        for (int64_t t = 0; t < n_tokens; ++t)
            for (int k = 0; k < K; ++k) {
                const int32_t e = ids[t * K + k];
                if (e < 0 || e >= E) continue;
                asg[c].expert = e;
                asg[c].token = (int32_t)t;
                asg[c].k = k;
                ++c;
            }
    }
    for (int64_t a = 0; a < cnt; ++a) {
        const float gw = weights[(size_t)asg[a].token * K + asg[a].k];
        if (gw == 0.0f) continue; /* native.cpp:3237 */
        const uint8_t* de = (const uint8_t*)w->down_exps + (size_t)asg[a].expert * exp_mid;
        const uint8_t* q = hq + ((size_t)asg[a].token * K + asg[a].k) * q8_mid;
        for (int64_t r = 0; r < H; ++r) {
            const float v = orc_dot_typed_q8k(w->down_type, de + (size_t)r * row_mid, q, I, order);
            y[(size_t)asg[a].token * H + r] += v * gw;
        }
    }
    free(hq);
    free(asg);
    return 0;
}

/* Shared expert: dense FFN (fast-exp SiLU on the contiguous dense path, fused_ops.cpp:342-343),
 * scaled by sigmoid(sh_gate_inp . x) (fused_ops.cpp:437-475), added to y (decoder.cpp:2600). */
int orc_moe_add_shared(const orc_moe_weights* w, const float* x, int64_t n_tokens, int order, float* y) {
    if (!w->sh_gate || !w->sh_up || !w->sh_down) return 0;
    const int64_t H = w->hidden, I = w->inter;
    float* sh = (float*)malloc(sizeof(float) * (size_t)n_tokens * (size_t)H);
    if (!sh) return -2;
    int rc = orc_ffn_swiglu_typed(w->sh_gu_type, w->sh_down_type, w->sh_gate, w->sh_up, w->sh_down, H, I, x, n_tokens, sh,
                                  order, ORC_SILU_FAST_FMA, NULL);
    for (int64_t t = 0; rc == 0 && t < n_tokens; ++t) {
        float scale = 1.0f;
        if (w->sh_gate_inp) {
            double acc = 0.0;
            for (int64_t c = 0; c < H; ++c) acc += (double)w->sh_gate_inp[c] * (double)x[t * H + c];
            scale = stable_sigmoid((float)acc);
        }
        for (int64_t r = 0; r < H; ++r) {
            const float s = sh[t * H + r] * scale;
            y[t * H + r] = y[t * H + r] + s;
        }
    }
    free(sh);
    return rc;
}

int orc_moe_layer(const orc_moe_weights* w, const float* x, const float* logits, int64_t n_tokens, float* y,
                  int order, int silu_mode, int weights_mode, int accumulate_mode, int32_t* ids_out,
                  float* weights_out, float* hidden_out) {
    if (!w || !x || !logits || !y || n_tokens <= 0 || w->hidden % ORC_QK_K || w->inter % ORC_QK_K || w->top_k <= 0)
        return -1;
    const int K = w->top_k;
    int32_t* ids = (int32_t*)malloc(sizeof(int32_t) * (size_t)n_tokens * K);
    float* wts = (float*)malloc(sizeof(float) * (size_t)n_tokens * K);
    float* hid = (float*)calloc((size_t)n_tokens * K * (size_t)w->inter, sizeof(float));
    int rc = (ids && wts && hid) ? 0 : -2;
    if (rc == 0) rc = orc_route_topk(logits, w->n_experts, n_tokens, K, weights_mode, ids, wts);
    if (rc == 0) rc = orc_moe_gateup_swiglu(w, x, ids, n_tokens, order, silu_mode, hid);
    if (rc == 0) rc = orc_moe_down_weighted(w, hid, ids, wts, n_tokens, order, accumulate_mode, y);
    if (rc == 0) rc = orc_moe_add_shared(w, x, n_tokens, order, y);
    if (rc == 0 && ids_out) memcpy(ids_out, ids, sizeof(int32_t) * (size_t)n_tokens * K);
    if (rc == 0 && weights_out) memcpy(weights_out, wts, sizeof(float) * (size_t)n_tokens * K);
    if (rc == 0 && hidden_out) memcpy(hidden_out, hid, sizeof(float) * (size_t)n_tokens * K * (size_t)w->inter);
    free(ids);
    free(wts);
    free(hid);
    return rc;
}
