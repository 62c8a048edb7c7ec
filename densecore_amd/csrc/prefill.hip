// Prefill GEMM for gfx950: C[M][N] = q8k(A[M][K]) . W_q4k[N][K]^T for M in the hundreds and above,
// where the work is arithmetic on the int8 matrix cores rather than weight streaming
// (RunQ4KRawBatchedDenseGemm, core/src/backend/cpu_backend_q4k_dense.cpp:57-101, behind
// CpuBackend::MatMulGgmlQuantizedTransB, core/src/backend/cpu_backend_quantized_matmul.cpp:150-175).
//
// The per-sub-block 6-bit scales are what keeps Q4_K off a plain int8 GEMM.  Here they are folded
// into the weight operand so that v_mfma_i32_16x16x64_i8 accumulates over the whole super-block:
//     scale = 8*s1 + s0  (two 3-bit digits)   ->   (s1*q4) and (s0*q4) both fit a signed byte (<= 105)
//     dot_scaled = 8 * sum_k (s1*q4)_k q8_k  +  sum_k (s0*q4)_k q8_k                  (exact, int32)
// and the min term runs on the matrix cores as well, from the sub-block sums of the codes
// bs_g = bsums[2g] + bsums[2g+1] = 128*h_g + l_g (h in [-32, 31], l in [0, 127]):
//     min_dot = sum_g min_g (128 h_g)  +  sum_g min_g l_g
// which is the reference's sum_j bsums[j] * min[j/2] (core/src/llm/matmul/kquant_batched_kernels.h:285-297).
// One v_mfma_f32_16x16x32_f16 forms it: the sixteen operands l_g, 128 h_g and the mins are integers of at most
// thirteen bits, exact as fp16; every product and every partial sum is an integer below 2^24, so the fp32 result
// is the integer min_dot itself -- the value (float)min_dot that the update needs, with nothing to combine or
// convert on the vector unit.
// Nine MFMAs per 16x16 output tile and super-block, no per-sub-block vector work; the fp32 update
//     acc += yd * (d * dot_scaled - dmin * min_dot)
// is done once per super-block, as every reference kernel does (three fp32 operations per output, five vector
// instructions with the digits' shift-add and one conversion; the reference's
// grouping (d*yd) * dot_scaled - (dmin*yd) * min_dot takes four, and the update is what the kernel's vector unit is
// busy with: 308 against 325 us at M = 2048; the two groupings differ in the last bits only).
//
//   grid      = (ceil(rowtiles / 8), ceil(m_tiles / 8)); workgroup = 4 wavefronts
//   workgroup = 128 weight rows x 128 activation rows; per super-block the 128 activation rows (37 KB
//               in the P-major layout below) are staged in LDS, double-buffered and requested one
//               super-block ahead with LDS-direct loads
//   wavefront = 2 weight tiles (32 rows) x the 8 activation tiles; it reads its weight tiles
//               straight from HBM in MFMA lane order and expands them in registers
//
// P-major activations (written by quantize_q8k_pmajor_kernel): [b][mt][4688 B], mt = m / 16:
//   [j 0..3][kq 0..3][tok 0..15][16 B]   codes: bytes 0..7 = sub-block ga(j), elements 8kq..8kq+7,
//                                        bytes 8..15 = sub-block gb(j), same elements, with
//                                        (ga, gb) = (0,2) (1,3) (4,6) (5,7) for j = 0..3 -- the pairs
//                                        that one 16-byte word of a weight tile holds per nibble half
//   [tok][32 B] at 4096                  fp16: l_0..l_7, then 128 h_0..128 h_7
//   [tok] fp32 at 4608                   block scale d
//   16 zero bytes at 4672                what the lanes of k-groups 2 and 3 feed the min MFMA
#include <hip/hip_ext.h>

#include "common.h"
#include "kernels.h"
#include "decode_tile.h"
#include "q8k_block.h"

namespace mq {

namespace {

constexpr int kPTileBytes = 4688;
constexpr int kPTileWords = kPTileBytes / 16;  // 293
constexpr int kPDigitOff = 4096, kPScaleOff = 4608, kPZeroOff = 4672;
constexpr int kMTilesPerGroup = 8;             // activation tiles (of 16 rows) per workgroup
constexpr int kMTilesSmall = 2;                // ... of an expert-grouped launch whose experts hold a dozen or two rows
constexpr int kMTilesMid = 4;                  // ... or three or four dozen

typedef unsigned short v2us __attribute__((ext_vector_type(2)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));

// four bytes (each <= 15) times a 3-bit digit, bytewise: two 16-bit products whose bytes do not carry into each
// other (15 * 7 < 256).  The digit is half H of `digits`, taken for both products (the operand-select bits of the
// packed multiply: no instruction of its own).
template <int H>
__device__ __forceinline__ uint32_t scale_bytes(uint32_t nibbles, uint32_t digits) {
    const v2us a = __builtin_bit_cast(v2us, nibbles);
    const v2us d = __builtin_bit_cast(v2us, digits);
    const v2us dd = H ? v2us{d.y, d.y} : v2us{d.x, d.x};
    return __builtin_bit_cast(uint32_t, (v2us)(a * dd));
}

// bytes i and i + 1 of `word` as two 16-bit numbers (one v_perm_b32: selector 0x0c yields a zero byte)
__device__ __forceinline__ uint32_t digit_pair(uint32_t word, int i) {
    return __builtin_amdgcn_perm(0u, word, 0x0c000c00u | (uint32_t)i | ((uint32_t)(i + 1) << 16));
}

struct WTile {
    v4i b5[4];         // Q5_K only: the fifth code bits times the whole 6-bit scale (16 * scale * bit is their share)
    v4i hi[4], lo[4];  // B operands of the four chunk pairs, scaled by the high / low scale digit
    v8h mins;          // B operand of the min MFMA: the eight mins as fp16, in every k-group
    float d, dmin;
};

// Q5: the codes are nibble + 16 * bit (bit s of the bytes of qh = fifth bit in sub-block s, core/src/kernels/hwy/hwy_moe_quant.cc:177-200);
// scale * code = scale * nibble + 16 * (scale * bit), and scale * bit <= 63 is a byte: a third MFMA chain.
template <bool Q5>
__device__ __forceinline__ void expand_tile(const v4u seg0, const v4u seg1, const v4u hdr, const v2u qh, int kq, WTile& t) {
    // 6-bit scales and mins (core/src/kernels/hwy/hwy_moe_quant.cc:90-101), four to a word
    const uint32_t sc03 = hdr.y & 0x3f3f3f3fu, mn03 = hdr.z & 0x3f3f3f3fu;
    const uint32_t sc47 = (hdr.w & 0x0f0f0f0fu) | (((hdr.y >> 6) & 0x03030303u) << 4);
    const uint32_t mn47 = ((hdr.w >> 4) & 0x0f0f0f0fu) | (((hdr.z >> 6) & 0x03030303u) << 4);
    const uint32_t s1_03 = (sc03 >> 3) & 0x07070707u, s0_03 = sc03 & 0x07070707u;
    const uint32_t s1_47 = (sc47 >> 3) & 0x07070707u, s0_47 = sc47 & 0x07070707u;
    const v4u seg[2] = {seg0, seg1};
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const uint32_t s1w = i ? s1_47 : s1_03, s0w = i ? s0_47 : s0_03;
        // sub-blocks 4i .. 4i+3 are bytes 0..3 of the digit words
        const uint32_t l0 = seg[i].x & 0x0f0f0f0fu, l1 = seg[i].y & 0x0f0f0f0fu;  // sub-block 4i
        const uint32_t l2 = seg[i].z & 0x0f0f0f0fu, l3 = seg[i].w & 0x0f0f0f0fu;  // sub-block 4i+2
        const uint32_t h0 = (seg[i].x >> 4) & 0x0f0f0f0fu, h1 = (seg[i].y >> 4) & 0x0f0f0f0fu;  // 4i+1
        const uint32_t h2 = (seg[i].z >> 4) & 0x0f0f0f0fu, h3 = (seg[i].w >> 4) & 0x0f0f0f0fu;  // 4i+3
        // digits of sub-blocks (4i, 4i+1) and (4i+2, 4i+3), two to a word
        const uint32_t ab1 = digit_pair(s1w, 0), ab0 = digit_pair(s0w, 0);
        const uint32_t ce1 = digit_pair(s1w, 2), ce0 = digit_pair(s0w, 2);
        t.hi[2 * i] = v4i{(int)scale_bytes<0>(l0, ab1), (int)scale_bytes<0>(l1, ab1), (int)scale_bytes<0>(l2, ce1),
                          (int)scale_bytes<0>(l3, ce1)};
        t.lo[2 * i] = v4i{(int)scale_bytes<0>(l0, ab0), (int)scale_bytes<0>(l1, ab0), (int)scale_bytes<0>(l2, ce0),
                          (int)scale_bytes<0>(l3, ce0)};
        t.hi[2 * i + 1] = v4i{(int)scale_bytes<1>(h0, ab1), (int)scale_bytes<1>(h1, ab1), (int)scale_bytes<1>(h2, ce1),
                              (int)scale_bytes<1>(h3, ce1)};
        t.lo[2 * i + 1] = v4i{(int)scale_bytes<1>(h0, ab0), (int)scale_bytes<1>(h1, ab0), (int)scale_bytes<1>(h2, ce0),
                              (int)scale_bytes<1>(h3, ce0)};
        if constexpr (Q5) {
            const uint32_t scw = i ? sc47 : sc03;
            const uint32_t abs_ = digit_pair(scw, 0), ces = digit_pair(scw, 2);  // whole scales of sub-blocks (4i, 4i+1), (4i+2, 4i+3)
            auto bits = [&](uint32_t word, int sb) { return (word >> sb) & 0x01010101u; };
            t.b5[2 * i] = v4i{(int)scale_bytes<0>(bits(qh.x, 4 * i), abs_), (int)scale_bytes<0>(bits(qh.y, 4 * i), abs_),
                              (int)scale_bytes<0>(bits(qh.x, 4 * i + 2), ces), (int)scale_bytes<0>(bits(qh.y, 4 * i + 2), ces)};
            t.b5[2 * i + 1] = v4i{(int)scale_bytes<1>(bits(qh.x, 4 * i + 1), abs_), (int)scale_bytes<1>(bits(qh.y, 4 * i + 1), abs_),
                                  (int)scale_bytes<1>(bits(qh.x, 4 * i + 3), ces), (int)scale_bytes<1>(bits(qh.y, 4 * i + 3), ces)};
        }
    }
    // byte -> fp16: 0x6400 | n is 1024 + n; two at a time
    const v2h bias = {(_Float16)1024.0f, (_Float16)1024.0f};
    const v2h m01 = __builtin_bit_cast(v2h, __builtin_amdgcn_perm(0x64006400u, mn03, 0x05010500u)) - bias;
    const v2h m23 = __builtin_bit_cast(v2h, __builtin_amdgcn_perm(0x64006400u, mn03, 0x05030502u)) - bias;
    const v2h m45 = __builtin_bit_cast(v2h, __builtin_amdgcn_perm(0x64006400u, mn47, 0x05010500u)) - bias;
    const v2h m67 = __builtin_bit_cast(v2h, __builtin_amdgcn_perm(0x64006400u, mn47, 0x05030502u)) - bias;
    t.mins = v8h{m01.x, m01.y, m23.x, m23.y, m45.x, m45.y, m67.x, m67.y};
    t.d = half_bits_to_float(hdr.x & 0xffffu);
    t.dmin = half_bits_to_float(hdr.x >> 16);
}

// ---- Q6_K on the matrix cores ---------------------------------------------------------------------------------
// weight = d * scale_g * (code - 32): sixteen signed 8-bit scales per super-block, one per 16 weights, six-bit codes
// (core/src/llm/matmul/q6_small_batch.h:13-92).  scale * (code - 32) reaches 4096, so both factors are cut in two:
//     scale + 128 = u = 16 u1 + u0   (u1, u0 in 0..15)          code - 32 = c = 8 c1 + c0   (c0 in 0..7, c1 in -4..3)
//     sum_g scale_g sum_i c_i q_i = 128 P11 + 16 P10 + 8 P01 + P00 - 128 R,
//     Pjk = sum_i (u_j c_k)_i q_i,  R = sum_i c_i q_i
// exactly, in int32: every byte u_j * c_k lies in [-60, 105] and c itself in [-32, 31] (the chain R multiplies
// 4 c, the tile's own bytes, and enters with -32).  Five chains of four K = 64 MFMAs per 16 x 16 outputs and
// super-block, no term from the activations' block sums, so the activation tiles are the Q4_K kernel's: the tile
// keeps each 64-byte run of low / high nibbles as two 32-weight sub-blocks (4 j + z and 4 j + z + 2 for the low and
// high nibbles of one byte), the pairs the P-major layout puts side by side.
// u_j * c1 for a signed c1 comes bytewise from the unsigned product with d1 = c1 + 4 = code >> 3:
//     u c1 = u d1 - 4 u,   ((u d1 | 0x80) - 4 u) ^ 0x80 per byte (u d1 <= 105 < 128, 4 u <= 60: no borrow).
struct WTile6 {
    v4i p11[4], p10[4], p01[4], p00[4], r4[4];
    float d;
};

__device__ __forceinline__ uint32_t signed_digit_bytes(uint32_t prod, uint32_t four_u) {
    return ((prod | 0x80808080u) - four_u) ^ 0x80808080u;
}

__device__ __forceinline__ void expand_tile6(const v4u ql0, const v4u ql1, const v4u qh, const v4u sc, uint32_t dw, int kq, WTile6& t) {
    const uint32_t scw[4] = {sc.x, sc.y, sc.z, sc.w};
    uint32_t u1w[4], u0w[4], f1w[4], f0w[4];  // digits of the sixteen scales, and four times the digits
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        const uint32_t u = scw[w] ^ 0x80808080u;  // scale + 128, bytewise
        u1w[w] = (u >> 4) & 0x0f0f0f0fu;
        u0w[w] = u & 0x0f0f0f0fu;
        f1w[w] = u1w[w] << 2;
        f0w[w] = u0w[w] << 2;
    }
    // weights 128 j + 32 z + l, l = 8 kq .. 8 kq + 7, have scale 8 j + 2 z + (kq >> 1): byte 2 (z & 1) + (kq >> 1) of
    // scale word 2 j + (z >> 1)
    const uint32_t sel = (uint32_t)(kq >> 1);
    const v4u qlw[2] = {ql0, ql1};
    const uint32_t qhw[4] = {qh.x, qh.y, qh.z, qh.w};
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
        for (int zp = 0; zp < 2; ++zp) {  // B operand jj = 2 j + zp: sub-blocks z = zp (dwords 0, 1) and z = zp + 2 (dwords 2, 3)
            const int jj = 2 * j + zp;
            const uint32_t k = 2u * (uint32_t)zp + sel;
            // the two sub-blocks' digits as 16-bit numbers side by side (low half: z = zp, high half: z = zp + 2)
            const uint32_t pick = 0x0c040c00u + k * 0x00010001u;
            const uint32_t d1p = __builtin_amdgcn_perm(u1w[2 * j + 1], u1w[2 * j], pick);
            const uint32_t d0p = __builtin_amdgcn_perm(u0w[2 * j + 1], u0w[2 * j], pick);
            const uint32_t spread = k * 0x01010101u;  // byte k in all four bytes
            const uint32_t f1[2] = {__builtin_amdgcn_perm(0u, f1w[2 * j], spread), __builtin_amdgcn_perm(0u, f1w[2 * j + 1], spread)};
            const uint32_t f0[2] = {__builtin_amdgcn_perm(0u, f0w[2 * j], spread), __builtin_amdgcn_perm(0u, f0w[2 * j + 1], spread)};
            const uint32_t src[2] = {zp ? qlw[j].z : qlw[j].x, zp ? qlw[j].w : qlw[j].y};
            uint32_t r4[4], p11[4], p10[4], p01[4], p00[4];
#pragma unroll
            for (int h = 0; h < 2; ++h) {      // h = 0: z = zp (low nibbles), h = 1: z = zp + 2 (high nibbles)
                const int z = zp + 2 * h;
#pragma unroll
                for (int i = 0; i < 2; ++i) {  // the lane's eight weights of the sub-block, four to a word
                    const uint32_t nib = (h ? src[i] >> 2 : src[i] << 2) & 0x3c3c3c3cu;
                    const uint32_t hi = qhw[2 * j + i];
                    const uint32_t top = (z == 3 ? hi : hi << (6 - 2 * z)) & 0xc0c0c0c0u;
                    const uint32_t b4 = top | nib;              // 4 (code - 32) as signed bytes
                    const uint32_t code4 = b4 ^ 0x80808080u;    // 4 code
                    const uint32_t d1 = (code4 >> 5) & 0x07070707u, c0 = (code4 >> 2) & 0x07070707u;
                    const int o = 2 * h + i;
                    r4[o] = b4;
                    if (h == 0) {
                        p10[o] = scale_bytes<0>(c0, d1p), p00[o] = scale_bytes<0>(c0, d0p);
                        p11[o] = signed_digit_bytes(scale_bytes<0>(d1, d1p), f1[0]);
                        p01[o] = signed_digit_bytes(scale_bytes<0>(d1, d0p), f0[0]);
                    } else {
                        p10[o] = scale_bytes<1>(c0, d1p), p00[o] = scale_bytes<1>(c0, d0p);
                        p11[o] = signed_digit_bytes(scale_bytes<1>(d1, d1p), f1[1]);
                        p01[o] = signed_digit_bytes(scale_bytes<1>(d1, d0p), f0[1]);
                    }
                }
            }
            t.r4[jj] = v4i{(int)r4[0], (int)r4[1], (int)r4[2], (int)r4[3]};
            t.p11[jj] = v4i{(int)p11[0], (int)p11[1], (int)p11[2], (int)p11[3]};
            t.p10[jj] = v4i{(int)p10[0], (int)p10[1], (int)p10[2], (int)p10[3]};
            t.p01[jj] = v4i{(int)p01[0], (int)p01[1], (int)p01[2], (int)p01[3]};
            t.p00[jj] = v4i{(int)p00[0], (int)p00[1], (int)p00[2], (int)p00[3]};
        }
    }
    t.d = half_bits_to_float(dw & 0xffffu);
}

// Q6_K the way compute_tile6 multiplies it (decode_tile.h), for activation tiles of sixteen rows: the B bytes are
// 4 * (code - 32), a scale per 16 weights.  Word jj = 2 j + zp of a P-major activation tile holds a lane's eight values
// of sub-block z = zp (bytes 0..7) and of z = zp + 2 (bytes 8..15) of half j, and the k-groups 0, 1 / 2, 3 of a K = 32
// MFMA over one of those runs are the two 16-weight scale groups of the sub-block: four MFMAs per word, each with the
// bytes of one group alone (the others' lanes zero), sixteen group sums per (row, token) and super-block, each times
// its scale in integers -- dot = sum_g scale_g * sum (code - 32) * q8 exactly (core/src/llm/matmul/q6_small_batch.h:56-83),
// carrying the bytes' factor 4.
struct WTile6G {
    long bg[4][4];  // [word jj][(z = zp, first 16), (zp, last 16), (zp + 2, first 16), (zp + 2, last 16)]
    int sg[4][4];   // their scales
    float d;
};

__device__ __forceinline__ long two_words(uint32_t lo, uint32_t hi) { return (long)(((uint64_t)hi << 32) | lo); }

__device__ __forceinline__ void expand_tile6g(const v4u ql0, const v4u ql1, const v4u qh, const v4u sc, uint32_t dw, int kq, WTile6G& t) {
    const uint32_t qlw[2][4] = {{ql0.x, ql0.y, ql0.z, ql0.w}, {ql1.x, ql1.y, ql1.z, ql1.w}};
    const uint32_t qhw[4] = {qh.x, qh.y, qh.z, qh.w};
    const uint32_t scw[4] = {sc.x, sc.y, sc.z, sc.w};
    const uint32_t keep_lo = kq < 2 ? 0xffffffffu : 0u, keep_hi = ~keep_lo;
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int zp = 0; zp < 2; ++zp) {
            const int jj = 2 * j + zp;
            uint32_t b4[2][2];  // [nibble side h][word i]: 4 * (code - 32) of z = zp + 2 h
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const int z = zp + 2 * h;
                    const uint32_t src = qlw[j][2 * zp + i];
                    const uint32_t nib = (h ? src >> 2 : src << 2) & 0x3c3c3c3cu;
                    const uint32_t hi = qhw[2 * j + i];
                    const uint32_t top = (z == 3 ? hi : hi << (6 - 2 * z)) & 0xc0c0c0c0u;
                    b4[h][i] = top | nib;
                }
            t.bg[jj][0] = two_words(b4[0][0] & keep_lo, b4[0][1] & keep_lo);
            t.bg[jj][1] = two_words(b4[0][0] & keep_hi, b4[0][1] & keep_hi);
            t.bg[jj][2] = two_words(b4[1][0] & keep_lo, b4[1][1] & keep_lo);
            t.bg[jj][3] = two_words(b4[1][0] & keep_hi, b4[1][1] & keep_hi);
            // group 8 j + 2 z + half: byte 2 (z & 1) + half of scale word 2 j + (z >> 1)
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    const int z = zp + 2 * h;
                    t.sg[jj][2 * h + half] = (int)(int8_t)((scw[2 * j + (z >> 1)] >> (8 * (2 * (z & 1) + half))) & 0xffu);
                }
        }
    t.d = half_bits_to_float(dw & 0xffffu);
}

// one activation tile of sixteen rows (its four words a[]) against the expanded tile: dot[i] += the lane's four
// (token 4 kq + i, weight row r) sums, times 4
template <bool kFenced = false>
__device__ __forceinline__ void mul_tile6g(const v4i (&a)[4], const WTile6G& w, int (&dot)[4]) {
    const v4i zero = {0, 0, 0, 0};
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
        // kFenced: the scheduler keeps each word's four MFMAs and their sums together instead of sixteen results in
        // flight (kernels with many accumulators: registers)
        if (kFenced && jj > 0) __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int gq = 0; gq < 4; ++gq) {
            const long a8 = gq < 2 ? two_words((uint32_t)a[jj].x, (uint32_t)a[jj].y) : two_words((uint32_t)a[jj].z, (uint32_t)a[jj].w);
            const v4i pg = __builtin_amdgcn_mfma_i32_16x16x32_i8(a8, w.bg[jj][gq], zero, 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 4; ++i) dot[i] += __mul24(pg[i], w.sg[jj][gq]);
        }
    }
}

typedef __attribute__((address_space(1))) const void* global_ptr_t;
typedef __attribute__((address_space(3))) void* lds_ptr_t;

// Requests the activation tiles of super-block b (copy_words 16-byte words, contiguous in HBM) straight
// into LDS with global_load_lds_dwordx4: lane l of a request writes its 16 bytes at base + 16*l, so a
// run of 64-word requests is a linear copy that never touches a register.  The instruction offset must
// stay 0 (the hardware adds it to the global address as well).
template <int MT>
__device__ __forceinline__ void request_a_tiles(const uint8_t* __restrict__ src, uint8_t* buf, int copy_words, int wave,
                                                int lane) {
    // Written as inline assembly on purpose: the compiler then does not know that LDS is written, and so does
    // not make every later LDS read wait for these requests (they fill the OTHER buffer).  The kernel waits
    // for them itself, with vmcnt(0) and a barrier, before the buffer is read.  M0 (the LDS base of the request)
    // is used by nothing else in this kernel.
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr_t)buf;
    constexpr int kRounds = (MT * kPTileWords + 255) / 256;  // 4 waves x 64 words a round: ten rounds for eight tiles of 293 words
#pragma unroll
    for (int j = 0; j < kRounds; ++j) {
        const int first = (j * 4 + wave) * 64;
        if (first + lane < copy_words) {
            const uint8_t* g = src + (size_t)(first + lane) * 16;
            const uint32_t dst = lds_base + (uint32_t)first * 16u;  // wave-uniform; lane l lands at dst + 16*l
            asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(g), "s"(dst) : "memory", "m0");
        }
    }
}

// kWTilesPerWave = 2: the 128 x 128 workgroup tile above.  1: 64 weight rows per workgroup, for launches whose
// 128-row workgroups would leave compute units without their two workgroups (M up to a few hundred).
// PAIR (two weight tiles per wavefront, Q4_K): the wavefront's two tiles are the SAME row tile of two matrices, gate
// (w) and up (w2), and what is stored is silu(gate) * up -- the two fp32 planes a gate launch and an up launch would
// write, and the pass that reads them back to form the product, never exist (for 2048 rows of a 4096 -> 14336 FFN that
// is 235 MB written and read).  The same accumulators, the same SiLU function on the same values: the same bits.
// MT: activation tiles (of 16 rows) a workgroup multiplies.  Eight for the dense product; the expert-grouped one also
// comes with two (items of 32 rows): with a dozen or two routed rows per expert a workgroup has one or two tiles, its
// accumulators for eight only cost registers and LDS -- and how many workgroups a compute unit holds is what hides the
// latency of a workgroup that walks eight super-blocks with a barrier each.
template <int kWTilesPerWave, int WT = kWtQ4, bool PAIR = false, int MT = kMTilesPerGroup>
__global__ void __launch_bounds__(256, 2) prefill_gemm_kernel(const uint8_t* __restrict__ w, int64_t rowtiles, int64_t rows,
                                                           int64_t nb, const uint8_t* __restrict__ ap, int64_t m_tiles,
                                                           int64_t n_tokens, float* __restrict__ y, int64_t ldy, int sb_split,
                                                           int64_t split_stride, const int32_t* __restrict__ plan,
                                                           int64_t expert_bytes, const int32_t* __restrict__ out_rows,
                                                           const uint8_t* __restrict__ w_shared,
                                                           const uint8_t* __restrict__ w2 = nullptr,
                                                           const uint8_t* __restrict__ w2_shared = nullptr, int silu_mode = 0) {
    static_assert(!PAIR || (kWTilesPerWave == 2 && WT == kWtQ4), "the pair form is the two-tile Q4_K kernel");
    extern __shared__ __align__(16) uint8_t a_lds[];  // two buffers of MT * kPTileBytes bytes
    constexpr int kBufBytes = MT * kPTileBytes;
    constexpr bool Q5 = WT == kWtQ5, Q6 = WT == kWtQ6;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, kq = lane >> 4;
    // Dense: workgroup column blockIdx.y takes the activation tiles 8 y .. 8 y + 7.  Expert-grouped (plan != null): it
    // takes item blockIdx.y of the plan -- an expert's weights and a run of up to eight tiles of that expert's rows.
    int64_t mt0 = (int64_t)blockIdx.y * MT;
    int mt_count = (int)(m_tiles - mt0 < MT ? m_tiles - mt0 : MT);
    if (plan) {
        const int item = blockIdx.y;
        if (item >= plan[0]) return;  // the whole workgroup, before any barrier
        const int expert = plan[4 + 3 * item];  // -1: the shared expert's rows
        w = expert < 0 ? w_shared : w + (size_t)expert * (size_t)expert_bytes;
        if constexpr (PAIR) {
            w2 = expert < 0 ? w2_shared : w2 + (size_t)expert * (size_t)expert_bytes;
            if (expert < 0) silu_mode = plan[3];  // the shared expert's rows: its own SiLU form
        }
        mt0 = plan[5 + 3 * item];
        mt_count = plan[6 + 3 * item];
    }
    const int64_t rt0 = ((int64_t)blockIdx.x * 4 + wave) * (PAIR ? 1 : kWTilesPerWave);
    // weight tiles past the end are replaced by the last valid one and simply not stored
    int64_t rt[kWTilesPerWave];
#pragma unroll
    for (int t = 0; t < kWTilesPerWave; ++t) rt[t] = rt0 + (PAIR ? 0 : t) < rowtiles ? rt0 + (PAIR ? 0 : t) : rowtiles - 1;

    float acc[kWTilesPerWave][MT][4];
#pragma unroll
    for (int t = 0; t < kWTilesPerWave; ++t)
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[t][m][i] = 0.0f;

    const int copy_words = mt_count * kPTileWords;
    // this lane's operand of the min MFMA: k-group 0 reads the l digits of token r, k-group 1 its 128 h digits, the others zeros
    const int digit_off = kq < 2 ? kPDigitOff + r * 32 + kq * 16 : kPZeroOff;
    const uint8_t* a_src = ap + (size_t)mt0 * kPTileBytes;           // + b * a_stride
    const size_t a_stride = (size_t)m_tiles * kPTileBytes;

    // Software pipeline over the super-blocks: while super-block b is multiplied, the activation tiles
    // of b+1 travel HBM/L2 -> LDS (other buffer) and this wave's weight tiles of b+1 travel into
    // registers.  One workgroup barrier per super-block.
    v4u seg0[kWTilesPerWave], seg1[kWTilesPerWave], hdr[kWTilesPerWave];
    v2u qh[kWTilesPerWave];
    v4u qh6[kWTilesPerWave];      // Q6_K: the top two bits of the codes; seg0 / seg1 hold its nibbles, hdr its sixteen scales
    uint32_t d6[kWTilesPerWave];  // Q6_K: fp16 d
    auto request_w = [&](int64_t b, int only = -1) {  // only >= 0: that tile alone
#pragma unroll
        for (int t = 0; t < kWTilesPerWave; ++t) {
            if (only >= 0 && t != only) continue;
            const uint8_t* tile = (PAIR && t == 1 ? w2 : w) + tile_offset(rt[t], b, nb, tile_stride<WT>());
            seg0[t] = load16(tile + lane * 16);
            seg1[t] = load16(tile + 1024 + lane * 16);
            if constexpr (Q6) {
                qh6[t] = load16(tile + kTile6HOff + lane * 16);
                hdr[t] = load16(tile + kTile6SOff + r * 16);
                d6[t] = *reinterpret_cast<const uint32_t*>(tile + kTile6DOff + r * 4);
            } else {
                hdr[t] = load16(tile + kTileQBytes + r * 16);
                if (Q5) qh[t] = *reinterpret_cast<const v2u*>(tile + kTileHBytes + lane * 8);
                else qh[t] = v2u{0u, 0u};
            }
        }
    };
    // K split over grid.z: this workgroup multiplies the super-blocks [b_begin, b_end) and writes its sums to
    // partial plane blockIdx.z (split_stride floats apart; the caller adds the planes in order)
    const int64_t b_begin = (int64_t)blockIdx.z * sb_split;
    const int64_t b_end = b_begin + sb_split < nb ? b_begin + sb_split : nb;
    y += (size_t)blockIdx.z * (size_t)split_stride;
    request_a_tiles<MT>(a_src + (size_t)b_begin * a_stride, a_lds + (b_begin & 1) * kBufBytes, copy_words, wave, lane);
    request_w(b_begin);

    for (int64_t b = b_begin; b < b_end; ++b) {
        // everything this thread requested for super-block b has landed ...
        __builtin_amdgcn_s_waitcnt(0 | (0x7 << 4) | (0xF << 8));  // vmcnt(0)
        // ... and after the barrier so has everybody else's share of the activation tiles; every wave
        // is also done reading the other buffer (super-block b-1), which the next requests overwrite
        __syncthreads();
        if constexpr (PAIR && MT <= 4) {
            // Few activation tiles: the two weight tiles are expanded and multiplied one after the other, so that one
            // expanded tile is live at a time (38 registers less: three wavefronts per SIMD instead of two, which is
            // what a launch of many short workgroups needs); the activation operands are read from LDS once per tile.
            if (b + 1 < b_end)
                request_a_tiles<MT>(a_src + (size_t)(b + 1) * a_stride, a_lds + ((b + 1) & 1) * kBufBytes, copy_words, wave, lane);
            const uint8_t* a_buf = a_lds + (b & 1) * kBufBytes;
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                WTile w1;
                expand_tile<false>(seg0[t], seg1[t], hdr[t], qh[t], kq, w1);
                if (b + 1 < b_end) request_w(b + 1, t);  // the raw tile's registers are free again
#pragma unroll
                for (int m = 0; m < MT; ++m) {
                    if (m < mt_count) {  // uniform over the workgroup
                        const uint8_t* at = a_buf + m * kPTileBytes;
                        v4i a[4];
#pragma unroll
                        for (int j = 0; j < 4; ++j) a[j] = *reinterpret_cast<const v4i*>(at + j * 1024 + lane * 16);
                        const float4 yd = *reinterpret_cast<const float4*>(at + kPScaleOff + kq * 16);
                        const float ydv[4] = {yd.x, yd.y, yd.z, yd.w};
                        const v8h dg = *reinterpret_cast<const v8h*>(at + digit_off);
                        const v4i zero = {0, 0, 0, 0};
                        const v4f zero_f = {0.0f, 0.0f, 0.0f, 0.0f};
                        v4i hi = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[0], w1.hi[0], zero, 0, 0, 0);
                        v4i lo = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[0], w1.lo[0], zero, 0, 0, 0);
                        const v4f mn = __builtin_amdgcn_mfma_f32_16x16x32_f16(dg, w1.mins, zero_f, 0, 0, 0);
#pragma unroll
                        for (int j = 1; j < 4; ++j) {
                            hi = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[j], w1.hi[j], hi, 0, 0, 0);
                            lo = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[j], w1.lo[j], lo, 0, 0, 0);
                        }
#pragma unroll
                        for (int i = 0; i < 4; ++i) {  // the arithmetic of the two-tiles-at-once form below
                            const int dot = hi[i] * 8 + lo[i];
                            const float v = __fmaf_rn(-w1.dmin, mn[i], __fmul_rn(w1.d, (float)dot));
                            acc[t][m][i] = __fmaf_rn(ydv[i], v, acc[t][m][i]);
                        }
                    }
                }
            }
            continue;
        }
        std::conditional_t<Q6, WTile6, WTile> wt[kWTilesPerWave];
#pragma unroll
        for (int t = 0; t < kWTilesPerWave; ++t) {
            if constexpr (Q6) expand_tile6(seg0[t], seg1[t], qh6[t], hdr[t], d6[t], kq, wt[t]);
            else expand_tile<Q5>(seg0[t], seg1[t], hdr[t], qh[t], kq, wt[t]);
        }
        if (b + 1 < b_end) {
            request_a_tiles<MT>(a_src + (size_t)(b + 1) * a_stride, a_lds + ((b + 1) & 1) * kBufBytes, copy_words, wave, lane);
            request_w(b + 1);
        }
        const uint8_t* a_buf = a_lds + (b & 1) * kBufBytes;

#pragma unroll
        for (int m = 0; m < MT; ++m) {
            if (m < mt_count) {  // uniform over the workgroup
                const uint8_t* at = a_buf + m * kPTileBytes;
                v4i a[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) a[j] = *reinterpret_cast<const v4i*>(at + j * 1024 + lane * 16);
                const float4 yd = *reinterpret_cast<const float4*>(at + kPScaleOff + kq * 16);
                const v4i zero = {0, 0, 0, 0};
                const float ydv[4] = {yd.x, yd.y, yd.z, yd.w};
                if constexpr (Q6) {
                    v4i p11[kWTilesPerWave], p10[kWTilesPerWave], p01[kWTilesPerWave], p00[kWTilesPerWave], r4[kWTilesPerWave];
#pragma unroll
                    for (int t = 0; t < kWTilesPerWave; ++t) {
                        p11[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[0], wt[t].p11[0], zero, 0, 0, 0);
                        p10[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[0], wt[t].p10[0], zero, 0, 0, 0);
                        p01[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[0], wt[t].p01[0], zero, 0, 0, 0);
                        p00[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[0], wt[t].p00[0], zero, 0, 0, 0);
                        r4[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[0], wt[t].r4[0], zero, 0, 0, 0);
                    }
#pragma unroll
                    for (int j = 1; j < 4; ++j)
#pragma unroll
                        for (int t = 0; t < kWTilesPerWave; ++t) {
                            p11[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[j], wt[t].p11[j], p11[t], 0, 0, 0);
                            p10[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[j], wt[t].p10[j], p10[t], 0, 0, 0);
                            p01[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[j], wt[t].p01[j], p01[t], 0, 0, 0);
                            p00[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[j], wt[t].p00[j], p00[t], 0, 0, 0);
                            r4[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[j], wt[t].r4[j], r4[t], 0, 0, 0);
                        }
#pragma unroll
                    for (int t = 0; t < kWTilesPerWave; ++t)
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            // sum_g scale_g sum (code - 32) q8, the integer of the reference's kernel, then its one fused
                            // multiply-add per block (core/src/llm/matmul/q6_small_batch.h:84-86)
                            const int isum = p11[t][i] * 128 + p10[t][i] * 16 + p01[t][i] * 8 + p00[t][i] - r4[t][i] * 32;
                            acc[t][m][i] = __fmaf_rn(__fmul_rn(ydv[i], wt[t].d), (float)isum, acc[t][m][i]);
                        }
                } else {
                    const v8h dg = *reinterpret_cast<const v8h*>(at + digit_off);
                    const v4f zero_f = {0.0f, 0.0f, 0.0f, 0.0f};
                    v4i hi[kWTilesPerWave], lo[kWTilesPerWave], fb[kWTilesPerWave];
                    v4f mn[kWTilesPerWave];
#pragma unroll
                    for (int t = 0; t < kWTilesPerWave; ++t) {
                        hi[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[0], wt[t].hi[0], zero, 0, 0, 0);
                        lo[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[0], wt[t].lo[0], zero, 0, 0, 0);
                        if (Q5) fb[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[0], wt[t].b5[0], zero, 0, 0, 0);
                        mn[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(dg, wt[t].mins, zero_f, 0, 0, 0);
                    }
#pragma unroll
                    for (int j = 1; j < 4; ++j)
#pragma unroll
                        for (int t = 0; t < kWTilesPerWave; ++t) {
                            hi[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[j], wt[t].hi[j], hi[t], 0, 0, 0);
                            lo[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[j], wt[t].lo[j], lo[t], 0, 0, 0);
                            if (Q5) fb[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[j], wt[t].b5[j], fb[t], 0, 0, 0);
                        }
#pragma unroll
                    for (int t = 0; t < kWTilesPerWave; ++t)
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            int dot = hi[t][i] * 8 + lo[t][i];
                            if (Q5) dot += fb[t][i] * 16;
                            // yd * (d * dot - dmin * min_dot): three fp32 operations per output and super-block
                            const float v = __fmaf_rn(-wt[t].dmin, mn[t][i], __fmul_rn(wt[t].d, (float)dot));
                            acc[t][m][i] = __fmaf_rn(ydv[i], v, acc[t][m][i]);
                        }
                }
            }
        }
    }

    if constexpr (PAIR) {  // one output per (token, row): silu(gate) * up
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[0][m][i] = silu_mul(acc[0][m][i], acc[1][m][i], silu_mode);
    }
    constexpr int kStoredTiles = PAIR ? 1 : kWTilesPerWave;
    if (out_rows) {  // grouped down product: row 16 (mt0 + m) + 4 kq + i of the plan goes to row out_rows[..] of y (-1: padding)
#pragma unroll
        for (int t = 0; t < kStoredTiles; ++t) {
            const int64_t row = (rt0 + t) * kTileRows + r;
            if (rt0 + t >= rowtiles || row >= rows) continue;
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                if (m >= mt_count) continue;
                const int4 dst = *reinterpret_cast<const int4*>(out_rows + (mt0 + m) * 16 + kq * 4);
                const int dsts[4] = {dst.x, dst.y, dst.z, dst.w};
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (dsts[i] >= 0) y[(size_t)dsts[i] * (size_t)ldy + row] = acc[t][m][i];
            }
        }
        return;
    }
    // Stores: lane (r, kq) holds weight row r of its tiles for the tokens 16 m + 4 kq + i.  One pointer per lane walks
    // down the token rows (an addition per store, no product).
    const int tok_left = (int)(n_tokens - mt0 * 16) - kq * 4;  // tokens from this lane's first one to the end
#pragma unroll
    for (int t = 0; t < kStoredTiles; ++t) {
        const int64_t row = (rt0 + t) * kTileRows + r;
        if (rt0 + t >= rowtiles || row >= rows) continue;
        float* yp = y + (mt0 * 16 + kq * 4) * ldy + row;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (m < mt_count && m * 16 + i < tok_left) *yp = acc[t][m][i];
                yp += ldy;
            }
            yp += 12 * ldy;
        }
    }
}

// ---- nine to sixteen activation rows against a streamed matrix ------------------------------------------------
// The decode kernels multiply a weight tile with EIGHT activation rows per MFMA (the sixteen operand rows hold a row's
// two sub-blocks of a 64-weight chunk side by side, the sub-block scales are applied on the vector unit); from nine rows
// they take two such token tiles per weight tile: 16 MFMAs and ~147 vector instructions.  This kernel multiplies the
// same rows as ONE tile of sixteen, the way prefill_gemm_kernel does (scale digits folded into the weight operand, the
// min term as one fp16 MFMA): 9 MFMAs and ~126 vector instructions per weight tile.  Everything else is
// dense_lds_kernel's (dense_lds.hip): eight wavefronts, WPR of them per row tile taking the super-blocks h, h + WPR, ...
// in ascending order, partial sums met in wave order, two register stages of raw weight tiles; the rows' quantized
// activations -- here P-major tiles -- are staged in LDS once per workgroup while the first weight tiles travel, or,
// where all super-blocks do not fit LDS (GA: the 14336 columns of an FFN's down projection), requested from global
// memory a stage ahead, beside the weight tile (six loads, all answered by the L2).  The integers of a (row, token,
// super-block) are the same and so is the fp32 update, (wd * yd) * dot - (wm * yd) * min_dot added to the running
// sum: the same bits as dense_lds_kernel and matmul_kernel.
// WT: Q4_K; Q5_K with a third MFMA chain for the fifth code bits times the whole scale (expand_tile<true>), the decode
// kernels' integers (scale * (nibble + 16 bit)) and update; Q6_K with the arithmetic of compute_tile6 carried over to
// tiles of sixteen (expand_tile6g, mul_tile6g above): sixteen K = 32 MFMAs per activation tile and super-block, one per
// 16-weight scale group, the group sums times their scales in integers, one fused multiply-add per super-block.
// LDS: [nb][4688] activation tiles (not GA), then the partial sums [8 / WPR][WPR - 1][NMAT][4][64].
// nb % WPR == 0 (host-checked): every wavefront has nb / WPR stages; FLOW 1: that count is odd (a single run); 0: even, a
// single run or runs of an even number of stages; 2: even, runs of an odd number of stages.
struct ATile16 {
    v4i a[4];   // the four 64-weight chunks of this lane's operand
    v4f yd;     // the Q8_K scales of rows 4 kq .. 4 kq + 3
    v8h dg;     // this lane's operand of the min MFMA (fp16 digits of the sub-block sums, or zeros)
};

// MT: activation tiles of sixteen rows (one, or two for 17 to 32 rows: the weight tile is expanded once for both, 18
// MFMAs and ~156 vector instructions against the 32 + 294 of two passes over two token tiles of eight each).  With two
// tiles the partial sums share LDS with the activation tiles (one more barrier before they are written).
template <int NMAT, int WPR, int FLOW, bool GA, int MT, int WT = kWtQ4>
__global__ void __launch_bounds__(512) skinny16_kernel(const Skinny16Args p) {
    constexpr bool ODD = FLOW == 1;  // (FLOW: the shape of the stage loop, below)
    constexpr int RPW = 8 / WPR;  // row tiles per workgroup
    constexpr bool Q5 = WT == kWtQ5, Q6 = WT == kWtQ6;
    constexpr int kStride = tile_stride<WT>();
    constexpr int kTileLoads = Q6 ? 5 : Q5 ? 4 : 3;  // requests of a weight tile (load_tile, load_tile6)
    constexpr bool kRedShares = MT > 1 && !GA;  // the partial sums reuse the activation tiles' LDS
    extern __shared__ __align__(16) uint8_t lds16[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15, kq = lane >> 4;
    const int nb = (int)p.nb;
    const int64_t rowtiles = (p.rows + 15) >> 4;
    const int pair = wave / WPR, h = wave % WPR;
    int64_t rt = (int64_t)blockIdx.x * RPW + pair;
    const bool dead = rt >= rowtiles;  // past the last row tile: stream the last one again and store nothing
    if (dead) rt = rowtiles - 1;
    float* red = reinterpret_cast<float*>(lds16 + ((GA || kRedShares) ? (size_t)0 : (size_t)nb * MT * kPTileBytes));  // (one run when the sums lie behind the tiles)

    const uint8_t* tiles[NMAT];
    tiles[0] = p.w0 + tile_offset(rt, 0, nb, kStride);
    if (NMAT == 2) tiles[1] = p.w1 + tile_offset(rt, 0, nb, kStride);
    const int cnt = nb / WPR;  // stages of this wavefront: super-blocks h, h + WPR, ...

    // lane (r, kq): weight row r of the tile, activation rows 4 kq .. 4 kq + 3 of every activation tile
    const int digit_off = kq < 2 ? kPDigitOff + r * 32 + kq * 16 : kPZeroOff;
    auto read_a = [&](ATile16& t, const uint8_t* at) {
#pragma unroll
        for (int j = 0; j < 4; ++j) t.a[j] = *reinterpret_cast<const v4i*>(at + j * 1024 + lane * 16);
        t.yd = *reinterpret_cast<const v4f*>(at + kPScaleOff + kq * 16);
        if constexpr (!Q6) t.dg = *reinterpret_cast<const v8h*>(at + digit_off);  // (Q6_K has no min term)
    };

    // ---- the activation tiles ([super-block][tile]) -> LDS: a linear copy, 1 KB per request, the wavefronts taking the
    // requests in turn.  Rows too long for LDS in one piece come in `ranges` runs of super-blocks, one run at a time:
    // stage i of every wavefront lies in run i / (cnt / ranges), so the wavefronts change runs together (cnt % ranges == 0,
    // host-checked).
    const int sb_per_range = nb / p.ranges, stages_per_range = cnt / p.ranges;
    auto stage_range = [&](int rg) {
        const uint32_t base = (uint32_t)(uintptr_t)(lds_ptr_t)lds16;
        const int words = sb_per_range * MT * kPTileWords;
        const uint8_t* src = p.ap + (size_t)rg * (size_t)words * 16;
        for (int c = wave; c * 64 < words; c += 8) {
            const int first = c * 64;
            if (first + lane < words) {
                const uint8_t* g = src + (size_t)(first + lane) * 16;
                const uint32_t dst = base + (uint32_t)first * 16u;
                asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(g), "s"(dst) : "memory", "m0");
            }
        }
    };
    if constexpr (!GA) stage_range(0);

    typename TileOf<WT>::Regs ring_t[2][NMAT];
    ATile16 ring_a[GA ? 2 : 1][GA ? MT : 1];
    auto issue = [&](auto st_c, int i) {  // only ever called for a stage that exists
        constexpr int st = decltype(st_c)::value;
        const int b = h + i * WPR;
        if constexpr (GA) {  // ahead of the tiles: they are needed first
#pragma unroll
            for (int t = 0; t < MT; ++t) read_a(ring_a[st][t], p.ap + ((size_t)b * MT + t) * kPTileBytes);
        }
#pragma unroll
        for (int m = 0; m < NMAT; ++m) load_tile_wt<WT>(ring_t[st][m], tiles[m] + (size_t)b * kStride, lane);
    };

    float acc[NMAT][MT][4];
#pragma unroll
    for (int m = 0; m < NMAT; ++m)
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[m][t][i] = 0.0f;

    int b_range0 = 0;  // first super-block of the run in LDS
    auto consume = [&](auto st_c, int i) {
        constexpr int st = decltype(st_c)::value;
        const int b = h + i * WPR;
        const v4i zero = {0, 0, 0, 0};
        const v4f zero_f = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int m = 0; m < NMAT; ++m) {
            // three and four tiles: the second matrix reads the activation tiles from LDS again instead of keeping the first
            // one's copies in registers (they would not fit)
            if (MT > 2 && m > 0) asm volatile("" ::: "memory");
            if constexpr (Q6) {
                const TileRegs6& tr = ring_t[st][m];
                WTile6G w6;
                expand_tile6g(tr.ql0, tr.ql1, tr.qh, tr.sc, tr.d, kq, w6);
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    if (MT > 2 && t > 0) asm volatile("" ::: "memory");  // a tile's LDS reads stay behind the tile before (registers)
                    ATile16 from_lds;
                    if constexpr (!GA) read_a(from_lds, lds16 + ((size_t)(b - b_range0) * MT + t) * kPTileBytes);
                    const ATile16& at = GA ? ring_a[GA ? st : 0][GA ? t : 0] : from_lds;
                    const float ydv[4] = {at.yd.x, at.yd.y, at.yd.z, at.yd.w};
                    int dot[4] = {0, 0, 0, 0};
                    mul_tile6g<(MT > 2)>(at.a, w6, dot);
#pragma unroll
                    for (int i2 = 0; i2 < 4; ++i2) {  // compute_tile6's update
                        const int isum = dot[i2] >> 2;  // the B bytes carried a factor 4
                        acc[m][t][i2] = __fmaf_rn(__fmul_rn(ydv[i2], w6.d), (float)isum, acc[m][t][i2]);
                    }
                }
            } else {
            WTile wt;
            expand_tile<Q5>(ring_t[st][m].q0, ring_t[st][m].q1, ring_t[st][m].hdr, Q5 ? ring_t[st][m].qh : v2u{0u, 0u}, kq, wt);
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                ATile16 from_lds;
                if constexpr (!GA) read_a(from_lds, lds16 + ((size_t)(b - b_range0) * MT + t) * kPTileBytes);
                const ATile16& at = GA ? ring_a[GA ? st : 0][GA ? t : 0] : from_lds;
                const float ydv[4] = {at.yd.x, at.yd.y, at.yd.z, at.yd.w};
                v4i hi = __builtin_amdgcn_mfma_i32_16x16x64_i8(at.a[0], wt.hi[0], zero, 0, 0, 0);
                v4i lo = __builtin_amdgcn_mfma_i32_16x16x64_i8(at.a[0], wt.lo[0], zero, 0, 0, 0);
                v4i fb = zero;  // Q5_K: the fifth code bits times the whole scale
                if constexpr (Q5) fb = __builtin_amdgcn_mfma_i32_16x16x64_i8(at.a[0], wt.b5[0], zero, 0, 0, 0);
                const v4f mn = __builtin_amdgcn_mfma_f32_16x16x32_f16(at.dg, wt.mins, zero_f, 0, 0, 0);
#pragma unroll
                for (int j = 1; j < 4; ++j) {
                    hi = __builtin_amdgcn_mfma_i32_16x16x64_i8(at.a[j], wt.hi[j], hi, 0, 0, 0);
                    lo = __builtin_amdgcn_mfma_i32_16x16x64_i8(at.a[j], wt.lo[j], lo, 0, 0, 0);
                    if constexpr (Q5) fb = __builtin_amdgcn_mfma_i32_16x16x64_i8(at.a[j], wt.b5[j], fb, 0, 0, 0);
                }
#pragma unroll
                for (int i2 = 0; i2 < 4; ++i2) {  // compute_tile's update (decode_tile.h); mn[i2] is the integer min_dot, exactly
                    int dot = hi[i2] * 8 + lo[i2];
                    if constexpr (Q5) dot += fb[i2] * 16;
                    const float d = __fmul_rn(wt.d, ydv[i2]);
                    const float dm = __fmul_rn(wt.dmin, ydv[i2]);
                    const float term = __fsub_rn(__fmul_rn(d, (float)dot), __fmul_rn(dm, mn[i2]));
                    acc[m][t][i2] = __fadd_rn(acc[m][t][i2], term);
                }
            }
            }
        }
    };

    // Two register stages, one in flight while the other is multiplied; written out for an even and for an odd number
    // of stages (an odd run is one stage followed by an even run with the stages' roles swapped), so that no request
    // is ever made for a stage that does not exist.
    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;
    const bool single = ODD && cnt == 1;  // wave-uniform
    issue(S0{}, 0);
    asm volatile("" ::: "memory");  // requests stay in stage order
    if (!single) {
        issue(S1{}, 1);
        asm volatile("" ::: "memory");
    }
    if constexpr (!GA) {
        // the LDS-direct copies are older than the tile requests: they have landed once at most those are outstanding
        if (single) asm volatile("s_waitcnt vmcnt(%0)" : : "n"(NMAT * kTileLoads) : "memory");
        else asm volatile("s_waitcnt vmcnt(%0)" : : "n"(2 * NMAT * kTileLoads) : "memory");
        __builtin_amdgcn_s_barrier();  // no fence: a fence would wait for the outstanding weight tiles as well
        asm volatile("" ::: "memory");
    }
    if constexpr (ODD) {
        consume(S0{}, 0);
        if (!single) {
            issue(S0{}, 2);  // cnt >= 3
            asm volatile("" ::: "memory");
            int i = 1;
            for (; i + 2 < cnt; i += 2) {
                consume(S1{}, i);
                issue(S1{}, i + 2);
                asm volatile("" ::: "memory");
                consume(S0{}, i + 1);
                issue(S0{}, i + 3);
                asm volatile("" ::: "memory");
            }
            consume(S1{}, i);
            consume(S0{}, i + 1);
        }
    } else {
        // The next run of super-blocks replaces the one in LDS once every wavefront has multiplied its last stage of it
        // (the weight tiles of the next run's first two stages are already on their way: they do not depend on LDS).
        if constexpr (FLOW == 0) {
            // A single run, or runs of an even number of stages: run by run, the change of runs between two inner loops
            // (a conditional change inside the pipelined loop, as below, costs the Q6_K forms their registers: 256 and
            // spills against 120-130).  The last pair of stages of the launch is peeled off: no request past the end.
            const int runs = GA ? 1 : p.ranges;
            int i = 0;
            for (int rg = 0; rg < runs; ++rg) {
                if (rg > 0) {  // wave-uniform, the same in every wavefront
                    __syncthreads();
                    stage_range(rg);
                    b_range0 = rg * sb_per_range;
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wavefront's share of the copy (and its two stages of weight tiles)
                    __syncthreads();
                }
                const int i_stop = (rg + 1) * (cnt / runs) - (rg == runs - 1 ? 2 : 0);
                for (; i < i_stop; i += 2) {
                    consume(S0{}, i);
                    issue(S0{}, i + 2);
                    asm volatile("" ::: "memory");
                    consume(S1{}, i + 1);
                    issue(S1{}, i + 3);
                    asm volatile("" ::: "memory");
                }
            }
            consume(S0{}, i);
            consume(S1{}, i + 1);
        } else {
            // FLOW == 2: runs of an odd number of stages begin at either stage of a pair
            auto next_range = [&](int i) {
                if (GA || p.ranges == 1 || i == 0 || i % stages_per_range) return;  // wave-uniform, the same i in every wavefront
                __syncthreads();
                const int rg = i / stages_per_range;
                stage_range(rg);
                b_range0 = rg * sb_per_range;
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wavefront's share of the copy (and its two stages of weight tiles)
                __syncthreads();
            };
            int i = 0;
            for (; i + 2 < cnt; i += 2) {
                next_range(i);
                consume(S0{}, i);
                issue(S0{}, i + 2);
                asm volatile("" ::: "memory");
                next_range(i + 1);
                consume(S1{}, i + 1);
                issue(S1{}, i + 3);
                asm volatile("" ::: "memory");
            }
            next_range(i);
            consume(S0{}, i);
            next_range(i + 1);
            consume(S1{}, i + 1);
        }
    }

    // ---- the WPR wavefronts of a row tile meet in wave order; the first one stores ----
    if (WPR > 1) {
        if (kRedShares) __syncthreads();  // every wavefront has read its last activation tile
        if (h > 0) {
#pragma unroll
            for (int m = 0; m < NMAT; ++m)
#pragma unroll
                for (int t = 0; t < MT; ++t)
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        red[(((((pair * (WPR - 1) + (h - 1)) * NMAT + m) * MT + t) * 4 + i) * 64) + lane] = acc[m][t][i];
        }
        __syncthreads();
    }
    if (h == 0 && !dead) {
        for (int wv = 1; wv < WPR; ++wv) {
#pragma unroll
            for (int m = 0; m < NMAT; ++m)
#pragma unroll
                for (int t = 0; t < MT; ++t)
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        acc[m][t][i] = __fadd_rn(acc[m][t][i], red[(((((pair * (WPR - 1) + (wv - 1)) * NMAT + m) * MT + t) * 4 + i) * 64) + lane]);
        }
        const int64_t row = rt * 16 + r;
        if (row < p.rows) {
#pragma unroll
            for (int t = 0; t < MT; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int tok = 16 * t + 4 * kq + i;
                    if (tok < p.n) {
                        float v = acc[0][t][i];
                        if (NMAT == 2) v = silu_mul(v, acc[NMAT - 1][t][i], p.silu_mode);
                        p.y[(size_t)tok * (size_t)p.ldy + (size_t)row] = v;
                    }
                }
        }
    }
}

// One workgroup per (tile of 16 activation rows, super-block): its four wavefronts quantize four rows each into an
// image of the tile in LDS, which then leaves as one run of 16-byte stores (a wavefront per row writing straight to
// the tile scattered its 256 bytes over 32 cache lines: 52 us for the 16384 gathered rows of a MoE block at 2048
// tokens).  Rows in [n, 16 * m_tiles) are written as zeros.
// kSwiglu: the row is silu(x) * x2 of two inputs (the gate and up products of an FFN), formed here instead of in a
// pass of its own; h_out, if given, receives it as fp32 as well.
// Expert-grouped forms: plan (tiles past plan[1] are skipped), row_src (row m of the tiles is row row_src[m] of x, -1:
// padding, zeros), h_rows (row m of the tiles is row h_rows[m] of h_out, -1: not written).
// kRowsPerWave: four (256 threads) in general; one (1024 threads, a wavefront per row) for launches of a few workgroups
// (sixteen rows: one workgroup per super-block), where the four rows one after the other are the launch's length.
template <bool kSwiglu, int kRowsPerWave = 4>
__global__ void __launch_bounds__(64 * 16 / kRowsPerWave) quantize_q8k_pmajor_kernel(const float* __restrict__ x, const float* __restrict__ x2,
                                                                  int silu_mode, float* __restrict__ h_out, int64_t ldh,
                                                                  int64_t n, int64_t ldx, int64_t nb, int64_t m_tiles,
                                                                  uint8_t* __restrict__ ap, const int32_t* __restrict__ plan,
                                                                  const int32_t* __restrict__ row_src,
                                                                  const int32_t* __restrict__ h_rows) {
    __shared__ __align__(16) uint8_t img[kPTileBytes];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t tile = blockIdx.x, b = blockIdx.y;
    if (plan && tile >= (int64_t)plan[1]) return;  // the whole workgroup, before the barrier
    if (plan && kSwiglu && tile >= (int64_t)plan[2]) silu_mode = plan[3];  // the shared expert's tiles: its own SiLU form
    constexpr int kThreads = 64 * 16 / kRowsPerWave;
    int64_t src[kRowsPerWave], hr[kRowsPerWave];
    float4 v[kRowsPerWave], u[kRowsPerWave];
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r) {
        const int64_t m = tile * 16 + wave * kRowsPerWave + r;
        src[r] = row_src ? row_src[m] : (m < n ? m : -1);
        hr[r] = h_rows ? h_rows[m] : src[r];
    }
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r) {  // all of the wavefront's rows are requested before any is worked on
        const int64_t from = src[r] >= 0 ? src[r] : 0;
        v[r] = *reinterpret_cast<const float4*>(x + from * ldx + b * kQK + lane * 4);
        if (kSwiglu) u[r] = *reinterpret_cast<const float4*>(x2 + from * ldx + b * kQK + lane * 4);
    }
    // elements 4*lane..4*lane+3: sub-block g = lane/8, elements 4*(lane%8).. of it
    const int g = lane >> 3;
    const int j = 2 * (g >> 2) + (g & 1), half = (g >> 1) & 1;
    const int kq = (lane & 7) >> 1;
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r) {
        const int tok = wave * kRowsPerWave + r;
        float e[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        if (src[r] >= 0) {  // wave-uniform
            e[0] = v[r].x, e[1] = v[r].y, e[2] = v[r].z, e[3] = v[r].w;
            if (kSwiglu) {
                e[0] = silu_mul(e[0], u[r].x, silu_mode), e[1] = silu_mul(e[1], u[r].y, silu_mode);
                e[2] = silu_mul(e[2], u[r].z, silu_mode), e[3] = silu_mul(e[3], u[r].w, silu_mode);
                if (h_out && hr[r] >= 0)
                    *reinterpret_cast<float4*>(h_out + hr[r] * ldh + b * kQK + lane * 4) = float4{e[0], e[1], e[2], e[3]};
            }
        }
        const Q8Lane q = quantize_block_q8k(e, lane);
        *reinterpret_cast<uint32_t*>(img + j * 1024 + (kq * 16 + tok) * 16 + half * 8 + (lane & 1) * 4) = q.packed;
        const int bs = q.bsum + __shfl_xor(q.bsum, 4, 64);  // codes 32g .. 32g+31
        if ((lane & 7) == 0) {  // bs = 128 h + l, both parts exact in fp16
            _Float16* digits = reinterpret_cast<_Float16*>(img + kPDigitOff + tok * 32);
            digits[g] = (_Float16)(float)(bs & 127);
            digits[8 + g] = (_Float16)(float)((bs >> 7) * 128);
        }
        if (lane == 0) *reinterpret_cast<float*>(img + kPScaleOff + tok * 4) = q.d;
    }
    if (tid < 4) *reinterpret_cast<uint32_t*>(img + kPZeroOff + tid * 4) = 0u;
    __syncthreads();
    v4u* dst = reinterpret_cast<v4u*>(ap + ((size_t)b * (size_t)m_tiles + (size_t)tile) * kPTileBytes);
    for (int i = tid; i < kPTileWords; i += kThreads) dst[i] = reinterpret_cast<const v4u*>(img)[i];
}

// The expert-grouped tiles of rows that repeat (a token is a row of top_k experts, and of the shared one): the distinct
// rows are quantized ONCE into tiles in their own order (quantize_q8k_pmajor_kernel on x as it is), and this kernel
// copies row row_src[m] of those tiles to row m of the plan's tiles -- sixteen 16-byte pieces of codes, two of digits
// and a scale per row and super-block, the same bytes the gathering quantizer writes (at top-8 it ran the block
// quantizer eight or nine times per token: 35 of the block's 406 us at 2048 tokens).  A workgroup per (tile,
// super-block); -1 in row_src: padding, zeros.
__global__ void __launch_bounds__(256) gather_pmajor_tiles_kernel(const uint8_t* __restrict__ ap_src, int64_t src_tiles,
                                                                  int64_t m_tiles, uint8_t* __restrict__ ap,
                                                                  const int32_t* __restrict__ plan,
                                                                  const int32_t* __restrict__ row_src) {
    const int tid = threadIdx.x;
    const int64_t tile = blockIdx.x, b = blockIdx.y;
    if (tile >= (int64_t)plan[1]) return;
    const uint8_t* from = ap_src + (size_t)b * (size_t)src_tiles * kPTileBytes;
    uint8_t* dst = ap + ((size_t)b * (size_t)m_tiles + (size_t)tile) * kPTileBytes;
    const int r = tid & 15, piece = tid >> 4;  // piece j * 4 + kq of row r: bytes j * 1024 + (kq * 16 + r) * 16
    const int t = row_src[tile * 16 + r];
    const uint8_t* st = from + (size_t)(t >= 0 ? t >> 4 : 0) * kPTileBytes;
    const int tr = t >= 0 ? (t & 15) : 0;
    const int j = piece >> 2, kq = piece & 3;
    v4u codes = *reinterpret_cast<const v4u*>(st + j * 1024 + (kq * 16 + tr) * 16);
    if (t < 0) codes = v4u{0u, 0u, 0u, 0u};
    *reinterpret_cast<v4u*>(dst + j * 1024 + (kq * 16 + r) * 16) = codes;
    if (tid < 32) {  // the row's sixteen fp16 digits: two pieces
        v4u d = *reinterpret_cast<const v4u*>(st + kPDigitOff + tr * 32 + piece * 16);
        if (t < 0) d = v4u{0u, 0u, 0u, 0u};
        *reinterpret_cast<v4u*>(dst + kPDigitOff + r * 32 + piece * 16) = d;
    } else if (tid < 48) {
        float sc = *reinterpret_cast<const float*>(st + kPScaleOff + tr * 4);
        if (t < 0) sc = 0.0f;
        *reinterpret_cast<float*>(dst + kPScaleOff + r * 4) = sc;
    } else if (tid < 52) {
        *reinterpret_cast<uint32_t*>(dst + kPZeroOff + (tid - 48) * 4) = 0u;
    }
}

// y[tok][row] = plane 0 + plane 1 + ... in that order; four rows per thread (rows % 4 == 0)
__global__ void __launch_bounds__(256) prefill_sum_planes_kernel(const float* __restrict__ part, int splits, int64_t n, int64_t rows,
                                                                 float* __restrict__ y, int64_t ldy) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;  // (token, group of four rows)
    const int64_t per_row = rows >> 2;
    if (i >= n * per_row) return;
    const int64_t tok = i / per_row, q = i - tok * per_row;
    const float4* src = reinterpret_cast<const float4*>(part + (size_t)tok * rows) + q;
    float4 acc = src[0];
    for (int z = 1; z < splits; ++z) {
        const float4 v = src[(size_t)z * (size_t)(n * per_row)];
        acc.x = __fadd_rn(acc.x, v.x), acc.y = __fadd_rn(acc.y, v.y), acc.z = __fadd_rn(acc.z, v.z), acc.w = __fadd_rn(acc.w, v.w);
    }
    float* dst = y + tok * ldy + q * 4;
    dst[0] = acc.x, dst[1] = acc.y, dst[2] = acc.z, dst[3] = acc.w;
}

// Workgroup shape and K split of a launch: 64-row workgroups while the 128-row ones would not give every compute
// unit one; K in `splits` runs of super-blocks while the launch would still leave workgroup slots empty (a
// workgroup walks its super-blocks one after the other, 2.2 us each: 4096 rows x 14336 columns at M = 128 are 64
// workgroups of 56 super-blocks, 115 us; in eight runs 37 us with the launch that adds the planes; at M = 256
// 119 -> 56 us in four runs, at M = 512 128 -> 100 us in two; 14336 x 4096 at M = 128: 40 -> 35 us in two).
struct PrefillShape {
    bool narrow;
    int splits, sb_split;
    unsigned row_wgs, groups;
};
PrefillShape prefill_shape(int64_t rows, int64_t nb, int64_t n, bool one_tile_per_wave = false) {
    const int64_t rowtiles = (rows + 15) / 16, m_tiles = (n + 15) / 16;
    PrefillShape ps;
    ps.groups = (unsigned)((m_tiles + kMTilesPerGroup - 1) / kMTilesPerGroup);
    // two workgroups fit a compute unit: while the 128-row workgroups would not even give every unit one, 64-row
    // ones fill the chip better (14336 rows on 256 units: up to M = 256; 52 -> 40 us at M = 128, 55 -> 51 at 256,
    // and 76 -> 79, 78 -> 91 at M = 384, 512, where the wide ones stay)
    ps.narrow = one_tile_per_wave || ((rowtiles + 7) / 8) * (int64_t)ps.groups <= (int64_t)compute_units();  // Q5_K, Q6_K: their operand sets only fit the registers of 64-row workgroups
    ps.row_wgs = (unsigned)(ps.narrow ? (rowtiles + 3) / 4 : (rowtiles + 7) / 8);
    const int64_t wgs = (int64_t)ps.row_wgs * ps.groups;
    int splits = (int)(2 * (int64_t)compute_units() / (wgs > 0 ? wgs : 1));
    if (splits > nb / 4) splits = (int)(nb / 4);  // at least four super-blocks per run
    if (splits < 1 || (rows & 3)) splits = 1;
    ps.sb_split = (int)((nb + splits - 1) / splits);
    ps.splits = (int)((nb + ps.sb_split - 1) / ps.sb_split);  // every run holds a super-block
    return ps;
}

// ---- expert-grouped GEMM: the plan ------------------------------------------------------------------------
// Every workgroup repeats the (short) prefix sums over the groups and then takes its share of the items and rows:
// each row costs two dependent reads of the entry lists, so one workgroup alone needs 29 us for 2048 tokens.
// From the expert groups of the routing (entries sorted by expert: group g holds the entries
// group_begin[g] .. group_begin[g + 1] - 1 of expert group_expert[g]) it lays the entries out in tiles of 16 rows, every
// group starting a new tile, and cuts every group's tiles into items of up to eight tiles, the unit a GEMM workgroup
// column multiplies.  plan: [0] items, [1] tiles, [4 + 3 i ..] = (expert, first tile, tiles) of item i; row_src[r] /
// out_row[r] for row r of the tiles: the token whose activations it holds and the row of the per-(token, slot) output
// it produces (token * slots + k), -1 for padding (src_per_slot: the activations are per (token, slot) rows too).
__global__ void __launch_bounds__(1024) moe_gemm_plan_kernel(const int32_t* __restrict__ n_groups, const int32_t* __restrict__ group_expert,
                                                             const int32_t* __restrict__ group_begin,
                                                             const int32_t* __restrict__ entry_token,
                                                             const int32_t* __restrict__ entry_k, int slots, int src_per_slot,
                                                             int groups_max, int sh_tokens, int sh_slot, int sh_silu_mode,
                                                             int32_t* __restrict__ plan, int32_t* __restrict__ row_src,
                                                             int32_t* __restrict__ out_row, int mt) {
    extern __shared__ int32_t plan_sh[];  // begin[g], tile0[g], item0[g]: groups_max + 2 each
    int32_t* begin = plan_sh;
    int32_t* tile0 = begin + groups_max + 2;
    int32_t* item0 = tile0 + groups_max + 2;
    const int tid = threadIdx.x, nt = blockDim.x;
    // sh_tokens > 0: one more group behind the routed ones, the shared expert with every token in order (expert -1,
    // output slot sh_slot); plan[2] = its first tile, plan[3] = its SiLU form
    const int ng_routed = *n_groups < groups_max ? *n_groups : groups_max;
    const int ng = ng_routed + (sh_tokens > 0 ? 1 : 0);
    for (int g = tid; g <= ng_routed; g += nt) begin[g] = group_begin[g];
    __syncthreads();
    if (tid == 0 && sh_tokens > 0) begin[ng] = begin[ng_routed] + sh_tokens;
    __syncthreads();
    if (tid < 64) {  // wavefront 0: exclusive prefix sums of tiles and items, lane l over a run of consecutive groups
        const int per = (ng + 63) / 64, g0 = tid * per;
        int tiles = 0, items = 0;
        for (int g = g0; g < g0 + per && g < ng; ++g) {
            const int t = (begin[g + 1] - begin[g] + 15) >> 4;
            tiles += t, items += (t + mt - 1) / mt;
        }
        int ts = tiles, is = items;  // inclusive scans across the lanes
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int a = __shfl_up(ts, d, 64), b = __shfl_up(is, d, 64);
            if (tid >= d) ts += a, is += b;
        }
        const int all_tiles = __shfl(ts, 63, 64), all_items = __shfl(is, 63, 64);
        ts -= tiles, is -= items;
        for (int g = g0; g < g0 + per && g < ng; ++g) {
            const int t = (begin[g + 1] - begin[g] + 15) >> 4;
            tile0[g] = ts, item0[g] = is;
            ts += t, is += (t + mt - 1) / mt;
        }
        if (tid == 0) {
            tile0[ng] = all_tiles, item0[ng] = all_items;
        }
    }
    __syncthreads();
    if (tid == 0 && blockIdx.x == 0)
        plan[0] = item0[ng], plan[1] = tile0[ng], plan[2] = sh_tokens > 0 ? tile0[ng_routed] : tile0[ng], plan[3] = sh_silu_mode;
    // the group of position q in a non-decreasing prefix array: the last g with first[g] <= q (empty groups cannot occur)
    auto group_of = [&](const int32_t* first, int q) {
        int lo = 0, hi = ng - 1;
        while (lo < hi) {
            const int mid = (lo + hi + 1) >> 1;
            if (first[mid] <= q) lo = mid;
            else hi = mid - 1;
        }
        return lo;
    };
    const int tiles = tile0[ng], items = item0[ng];
    const int first = blockIdx.x * nt + tid, step = gridDim.x * nt;
    for (int i = first; i < items; i += step) {
        const int g = group_of(item0, i);
        const int t_g = tile0[g + 1] - tile0[g], at = (i - item0[g]) * mt;
        plan[4 + 3 * i] = g < ng_routed ? group_expert[g] : -1;
        plan[5 + 3 * i] = tile0[g] + at;
        plan[6 + 3 * i] = t_g - at < mt ? t_g - at : mt;
    }
    for (int rr = first; rr < tiles * 16; rr += step) {
        const int g = group_of(tile0, rr >> 4);
        const int pos = rr - tile0[g] * 16;
        int src = -1, dst = -1;
        if (pos < begin[g + 1] - begin[g]) {
            if (g < ng_routed) {
                const int e = begin[g] + pos;
                src = entry_token[e];
                dst = src * slots + entry_k[e];
                if (src_per_slot) src = dst;  // the activations come per (token, slot) as well
            } else {
                src = pos;
                dst = pos * slots + sh_slot;
            }
        }
        row_src[rr] = src, out_row[rr] = dst;
    }
}

}  // namespace

// upper bounds: `entries` counts every row of the plan (the routed pairs and, with a shared expert, every token once
// more), groups_max every group (the experts, + 1 with a shared expert)
int64_t moe_gemm_tiles_max(int64_t entries, int64_t groups_max) { return (entries + 15) / 16 + groups_max; }
// (sized for the smallest items a plan may be cut into, so that the lists behind the items lie at one place whatever
// the item size of a launch)
int64_t moe_gemm_items_max(int64_t entries, int64_t groups_max) {  // a multiple of four: the row arrays behind the items stay 16-byte aligned
    return ((entries + 16 * kMTilesSmall - 1) / (16 * kMTilesSmall) + groups_max + 3) & ~(int64_t)3;
}
size_t moe_gemm_plan_ints(int64_t entries, int64_t groups_max) {
    return 4 + 3 * (size_t)moe_gemm_items_max(entries, groups_max) + 2 * 16 * (size_t)moe_gemm_tiles_max(entries, groups_max);
}

hipError_t launch_moe_gemm_plan(const int32_t* n_groups, const int32_t* group_expert, const int32_t* group_begin,
                                const int32_t* entry_token, const int32_t* entry_k, int slots, bool src_per_slot, int64_t entries,
                                int64_t groups_max, int64_t sh_tokens, int sh_silu_mode, int32_t* plan, hipStream_t stream, int mt) {
    if (groups_max > 4097 || (mt != kMTilesSmall && mt != kMTilesMid && mt != kMTilesPerGroup)) return hipErrorInvalidValue;
    int32_t* row_src = plan + 4 + 3 * moe_gemm_items_max(entries, groups_max);
    int32_t* out_row = row_src + 16 * moe_gemm_tiles_max(entries, groups_max);
    const int64_t rows_max = 16 * moe_gemm_tiles_max(entries, groups_max);
    const unsigned wgs = (unsigned)(rows_max / 1024 < 1 ? 1 : (rows_max / 1024 > 64 ? 64 : rows_max / 1024));
    MQ_LAUNCH(moe_gemm_plan_kernel, dim3(wgs), dim3(1024), 3 * (size_t)(groups_max + 2) * sizeof(int32_t), stream, n_groups,
                       group_expert, group_begin, entry_token, entry_k, slots, src_per_slot ? 1 : 0, (int)groups_max, (int)sh_tokens,
                       slots - 1, sh_silu_mode, plan, row_src, out_row, mt);
    return hipGetLastError();
}

// Rows of the plan's tiles in the P-major layout: gathered from x by the plan's row list (swiglu == false), or
// silu(gate) * up of two planes that already are in the plan's row order (swiglu == true; h_out, if given, receives
// those rows as fp32 at their per-(token, slot) places).
hipError_t launch_quantize_q8k_pmajor_grouped(const float* x, const float* x2, bool swiglu, int silu_mode, int64_t ldx, int64_t k,
                                              int64_t entries, int64_t groups_max, const int32_t* plan, uint8_t* ap, float* h_out,
                                              int64_t ldh, hipStream_t stream, int64_t distinct_rows, uint8_t* ap_rows) {
    const int64_t nb = k / kQK, m_tiles = moe_gemm_tiles_max(entries, groups_max);
    if (m_tiles == 0 || nb == 0) return hipSuccess;
    if (nb > 65535 || m_tiles >= (int64_t)1 << 31) return hipErrorInvalidValue;
    const int32_t* row_src = plan + 4 + 3 * moe_gemm_items_max(entries, groups_max);
    if (!swiglu && ap_rows && distinct_rows > 0) {
        // the plan's rows repeat the distinct_rows rows of x: quantize those once, then copy them to their places
        hipError_t e = launch_quantize_q8k_pmajor(x, distinct_rows, ldx, k, ap_rows, stream);
        if (e != hipSuccess) return e;
        MQ_LAUNCH(gather_pmajor_tiles_kernel, dim3((unsigned)m_tiles, (unsigned)nb), dim3(256), 0, stream, (const uint8_t*)ap_rows,
                  (distinct_rows + 15) / 16, m_tiles, ap, plan, row_src);
        return hipGetLastError();
    }
    if (swiglu) {
        MQ_LAUNCH(quantize_q8k_pmajor_kernel<true>, dim3((unsigned)m_tiles, (unsigned)nb), dim3(256), 0, stream, x, x2, silu_mode,
                           h_out, ldh, m_tiles * 16, ldx, nb, m_tiles, ap, plan, (const int32_t*)nullptr,
                           row_src + 16 * m_tiles);
    } else {
        MQ_LAUNCH(quantize_q8k_pmajor_kernel<false>, dim3((unsigned)m_tiles, (unsigned)nb), dim3(256), 0, stream, x,
                           (const float*)nullptr, 0, (float*)nullptr, (int64_t)0, m_tiles * 16, ldx, nb, m_tiles, ap, plan, row_src,
                           (const int32_t*)nullptr);
    }
    return hipGetLastError();
}

// y = the plan's tiles . W_expert^T per item.  scatter == false: y [tiles * 16][ldy] in the plan's row order;
// true: row out_row[r] of y (the per-(token, slot) rows of the down product).
int moe_gemm_item_tiles(int64_t entries, int64_t groups) {
    // An expert with more rows than an item takes several items, each of which expands the expert's weights again; an
    // item larger than its expert's rows holds accumulators and LDS for tiles that do not exist, and a compute unit
    // then holds fewer workgroups.  MoE block of 256 + 1 experts, top-8, 2048 x 512, items of 2 / 4 / 8 tiles: 162 / 172 /
    // 209 us at 384 tokens (13 rows per expert), 173 / 181 / 219 at 512, 195 / 203 / 239 at 768, 236 / 224 / 260 at 1024
    // (36 rows), 315 / 276 / 311 at 1536, 385 / 356 / 364 at 2048 (72 rows), 686 / 612 / 615 at 4096.
    if (groups <= 0) return kMTilesPerGroup;
    return entries <= 30 * groups ? kMTilesSmall : entries <= 160 * groups ? kMTilesMid : kMTilesPerGroup;
}

hipError_t launch_prefill_gemm_grouped(const uint8_t* w, int wtype, int64_t expert_bytes, const uint8_t* w_shared, int64_t rows,
                                       int64_t nb, const uint8_t* ap, int64_t entries, int64_t groups_max, const int32_t* plan,
                                       bool scatter, float* y, int64_t ldy, hipStream_t stream, int mt) {
    if (wtype != kTypeQ4K && wtype != kTypeQ5K && wtype != kTypeQ6K) return hipErrorInvalidValue;
    if (mt != kMTilesSmall && mt != kMTilesMid && mt != kMTilesPerGroup) return hipErrorInvalidValue;
    const int64_t rowtiles = (rows + 15) / 16, m_tiles = moe_gemm_tiles_max(entries, groups_max);
    const int64_t items = moe_gemm_items_max(entries, groups_max);
    if (rowtiles == 0 || items == 0) return hipSuccess;
    if (items > 65535) return hipErrorInvalidValue;
    static bool raised = false;
    if (!raised) {
        for (const void* k : {reinterpret_cast<const void*>(&prefill_gemm_kernel<1>), reinterpret_cast<const void*>(&prefill_gemm_kernel<2>),
                              reinterpret_cast<const void*>(&prefill_gemm_kernel<1, kWtQ5>), reinterpret_cast<const void*>(&prefill_gemm_kernel<1, kWtQ6>)}) {
            hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * kMTilesPerGroup * kPTileBytes);
            if (e != hipSuccess) return e;
        }
        raised = true;
    }
    const int32_t* out_row = scatter ? plan + 4 + 3 * items + 16 * m_tiles : nullptr;
    const dim3 narrow((unsigned)((rowtiles + 3) / 4), (unsigned)items), wide((unsigned)((rowtiles + 7) / 8), (unsigned)items);
#define MQ_GROUPED(KW, WT_, MT_, GRID)                                                                                             \
    MQ_LAUNCH((prefill_gemm_kernel<KW, WT_, false, MT_>), GRID, dim3(256), 2 * MT_ * kPTileBytes, stream, w, rowtiles, rows, nb, ap, \
              m_tiles, m_tiles * 16, y, ldy, (int)nb, (int64_t)0, plan, expert_bytes, out_row, w_shared, (const uint8_t*)nullptr,  \
              (const uint8_t*)nullptr, 0)
    if (mt == kMTilesSmall) {  // one weight tile per wavefront: few registers, several workgroups to a compute unit
        if (wtype == kTypeQ6K) MQ_GROUPED(1, kWtQ6, kMTilesSmall, narrow);
        else if (wtype == kTypeQ5K) MQ_GROUPED(1, kWtQ5, kMTilesSmall, narrow);
        else MQ_GROUPED(1, kWtQ4, kMTilesSmall, narrow);
    } else if (mt == kMTilesMid) {
        if (wtype == kTypeQ6K) MQ_GROUPED(1, kWtQ6, kMTilesMid, narrow);
        else if (wtype == kTypeQ5K) MQ_GROUPED(1, kWtQ5, kMTilesMid, narrow);
        else MQ_GROUPED(1, kWtQ4, kMTilesMid, narrow);
    } else if (wtype == kTypeQ6K) {
        MQ_GROUPED(1, kWtQ6, kMTilesPerGroup, narrow);
    } else if (wtype == kTypeQ5K) {
        MQ_GROUPED(1, kWtQ5, kMTilesPerGroup, narrow);
    } else {
        MQ_GROUPED(2, kWtQ4, kMTilesPerGroup, wide);
    }
#undef MQ_GROUPED
    return hipGetLastError();
}

// The pair form: h[tok][row] = silu(gate[row] . x[tok]) * (up[row] . x[tok]).  It has no K split (SiLU is not linear), so it
// applies where the two single launches would not split K either; Q4_K only (the other types' operand sets fill the
// registers with one tile per wavefront).
bool prefill_pair_applies(int wtype, int64_t rows, int64_t nb, int64_t n) {
    if (wtype != kTypeQ4K) return false;
    return prefill_shape(rows, nb, n, true).splits == 1;
}

hipError_t launch_prefill_gemm_pair(const uint8_t* gate, const uint8_t* up, int wtype, int64_t rows, int64_t nb, const uint8_t* ap,
                                    int64_t n, int silu_mode, float* h, int64_t ldh, hipStream_t stream) {
    const int64_t rowtiles = (rows + 15) / 16, m_tiles = (n + 15) / 16;
    if (rowtiles == 0 || m_tiles == 0) return hipSuccess;
    if (!prefill_pair_applies(wtype, rows, nb, n)) return hipErrorInvalidValue;
    const PrefillShape ps = prefill_shape(rows, nb, n, true);
    if (ps.groups > 65535u) return hipErrorInvalidValue;
    static bool raised = false;
    if (!raised) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&prefill_gemm_kernel<2, kWtQ4, true>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 2 * kMTilesPerGroup * kPTileBytes);
        if (e != hipSuccess) return e;
        raised = true;
    }
    MQ_LAUNCH((prefill_gemm_kernel<2, kWtQ4, true>), dim3(ps.row_wgs, ps.groups, 1u), dim3(256), 2 * kMTilesPerGroup * kPTileBytes, stream,
              gate, rowtiles, rows, nb, ap, m_tiles, n, h, ldh, (int)nb, (int64_t)0, (const int32_t*)nullptr, (int64_t)0,
              (const int32_t*)nullptr, (const uint8_t*)nullptr, up, (const uint8_t*)nullptr, silu_mode);
    return hipGetLastError();
}

// The expert-grouped pair form: scatter == false: h [tiles * 16][ldh] in the plan's row order; true: row out_row[r] of h.
hipError_t launch_prefill_gemm_grouped_pair(const uint8_t* gate, const uint8_t* up, int wtype, int64_t expert_bytes,
                                            const uint8_t* gate_shared, const uint8_t* up_shared, int64_t rows, int64_t nb,
                                            const uint8_t* ap, int64_t entries, int64_t groups_max, const int32_t* plan, bool scatter,
                                            int silu_mode, float* h, int64_t ldh, hipStream_t stream, int mt) {
    if (wtype != kTypeQ4K || (mt != kMTilesSmall && mt != kMTilesMid && mt != kMTilesPerGroup)) return hipErrorInvalidValue;
    const int64_t rowtiles = (rows + 15) / 16, m_tiles = moe_gemm_tiles_max(entries, groups_max);
    const int64_t items = moe_gemm_items_max(entries, groups_max);
    if (rowtiles == 0 || items == 0) return hipSuccess;
    if (items > 65535) return hipErrorInvalidValue;
    static bool raised = false;
    if (!raised) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&prefill_gemm_kernel<2, kWtQ4, true>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 2 * kMTilesPerGroup * kPTileBytes);
        if (e != hipSuccess) return e;
        raised = true;
    }
    const int32_t* out_row = scatter ? plan + 4 + 3 * items + 16 * m_tiles : nullptr;
    const dim3 grid((unsigned)((rowtiles + 3) / 4), (unsigned)items);
    if (mt == kMTilesSmall)
        MQ_LAUNCH((prefill_gemm_kernel<2, kWtQ4, true, kMTilesSmall>), grid, dim3(256), 2 * kMTilesSmall * kPTileBytes, stream, gate, rowtiles,
                  rows, nb, ap, m_tiles, m_tiles * 16, h, ldh, (int)nb, (int64_t)0, plan, expert_bytes, out_row, gate_shared, up, up_shared,
                  silu_mode);
    else if (mt == kMTilesMid)
        MQ_LAUNCH((prefill_gemm_kernel<2, kWtQ4, true, kMTilesMid>), grid, dim3(256), 2 * kMTilesMid * kPTileBytes, stream, gate, rowtiles,
                  rows, nb, ap, m_tiles, m_tiles * 16, h, ldh, (int)nb, (int64_t)0, plan, expert_bytes, out_row, gate_shared, up, up_shared,
                  silu_mode);
    else
        MQ_LAUNCH((prefill_gemm_kernel<2, kWtQ4, true>), grid, dim3(256), 2 * kMTilesPerGroup * kPTileBytes, stream, gate, rowtiles, rows, nb,
                  ap, m_tiles, m_tiles * 16, h, ldh, (int)nb, (int64_t)0, plan, expert_bytes, out_row, gate_shared, up, up_shared, silu_mode);
    return hipGetLastError();
}

size_t prefill_part_bytes(int64_t rows, int64_t nb, int64_t n, int wtype) {
    const PrefillShape ps = prefill_shape(rows, nb, n, wtype != kTypeQ4K);
    return ps.splits > 1 ? (size_t)ps.splits * (size_t)n * (size_t)rows * sizeof(float) : 0;
}

size_t pmajor_bytes(int64_t n, int64_t nb) { return (size_t)((n + 15) / 16) * (size_t)nb * kPTileBytes; }

hipError_t launch_quantize_q8k_pmajor(const float* x, int64_t n, int64_t ldx, int64_t k, uint8_t* ap,
                                      hipStream_t stream, const int32_t* plan) {
    const int64_t nb = k / kQK, m_tiles = (n + 15) / 16;
    if (m_tiles == 0 || nb == 0) return hipSuccess;
    if (nb > 65535 || m_tiles >= (int64_t)1 << 31) return hipErrorInvalidValue;
    if (m_tiles * nb <= 64 && !plan) {  // a few workgroups (sixteen rows of a decode-width product): a wavefront per row
        MQ_LAUNCH((quantize_q8k_pmajor_kernel<false, 1>), dim3((unsigned)m_tiles, (unsigned)nb), dim3(1024), 0, stream, x,
                  (const float*)nullptr, 0, (float*)nullptr, (int64_t)0, n, ldx, nb, m_tiles, ap, plan, (const int32_t*)nullptr,
                  (const int32_t*)nullptr);
        return hipGetLastError();
    }
    MQ_LAUNCH(quantize_q8k_pmajor_kernel<false>, dim3((unsigned)m_tiles, (unsigned)nb), dim3(256), 0, stream, x,
                       (const float*)nullptr, 0, (float*)nullptr, (int64_t)0, n, ldx, nb, m_tiles, ap, plan,
                       (const int32_t*)nullptr, (const int32_t*)nullptr);
    return hipGetLastError();
}

hipError_t launch_swiglu_quantize_q8k_pmajor(const float* gate, const float* up, int64_t n, int64_t ldx, int64_t k,
                                             int silu_mode, float* h_out, int64_t ldh, uint8_t* ap, hipStream_t stream) {
    const int64_t nb = k / kQK, m_tiles = (n + 15) / 16;
    if (m_tiles == 0 || nb == 0) return hipSuccess;
    if (nb > 65535 || m_tiles >= (int64_t)1 << 31) return hipErrorInvalidValue;
    MQ_LAUNCH(quantize_q8k_pmajor_kernel<true>, dim3((unsigned)m_tiles, (unsigned)nb), dim3(256), 0, stream, gate, up,
                       silu_mode, h_out, ldh, n, ldx, nb, m_tiles, ap, (const int32_t*)nullptr, (const int32_t*)nullptr,
                       (const int32_t*)nullptr);
    return hipGetLastError();
}

hipError_t launch_prefill_gemm(const uint8_t* w, int wtype, int64_t rows, int64_t nb, const uint8_t* ap, int64_t n, float* y,
                               int64_t ldy, float* part, hipStream_t stream) {
    const int64_t rowtiles = (rows + 15) / 16, m_tiles = (n + 15) / 16;
    if (rowtiles == 0 || m_tiles == 0) return hipSuccess;
    if (wtype != kTypeQ4K && wtype != kTypeQ5K && wtype != kTypeQ6K) return hipErrorInvalidValue;
    const PrefillShape ps = prefill_shape(rows, nb, n, wtype != kTypeQ4K);
    if (ps.groups > 65535u) return hipErrorInvalidValue;
    if (ps.splits > 1 && !part) return hipErrorInvalidValue;
    static bool raised = false;  // two activation buffers: more than the default 64 KB of dynamic LDS
    if (!raised) {
        for (const void* k : {reinterpret_cast<const void*>(&prefill_gemm_kernel<1>), reinterpret_cast<const void*>(&prefill_gemm_kernel<2>),
                              reinterpret_cast<const void*>(&prefill_gemm_kernel<1, kWtQ5>), reinterpret_cast<const void*>(&prefill_gemm_kernel<1, kWtQ6>)}) {
            hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * kMTilesPerGroup * kPTileBytes);
            if (e != hipSuccess) return e;
        }
        raised = true;
    }
    const bool split = ps.splits > 1;
    float* out = split ? part : y;
    const int64_t ld = split ? rows : ldy;
    const int64_t stride = split ? n * rows : 0;
    const dim3 grid(ps.row_wgs, ps.groups, (unsigned)ps.splits);
    if (wtype == kTypeQ6K) {
        MQ_LAUNCH((prefill_gemm_kernel<1, kWtQ6>), grid, dim3(256), 2 * kMTilesPerGroup * kPTileBytes, stream, w, rowtiles, rows, nb,
                           ap, m_tiles, n, out, ld, ps.sb_split, stride, (const int32_t*)nullptr, (int64_t)0, (const int32_t*)nullptr,
                           (const uint8_t*)nullptr);
    } else if (wtype == kTypeQ5K) {
        MQ_LAUNCH((prefill_gemm_kernel<1, kWtQ5>), grid, dim3(256), 2 * kMTilesPerGroup * kPTileBytes, stream, w, rowtiles, rows, nb,
                           ap, m_tiles, n, out, ld, ps.sb_split, stride, (const int32_t*)nullptr, (int64_t)0, (const int32_t*)nullptr,
                           (const uint8_t*)nullptr);
    } else if (ps.narrow) {
        MQ_LAUNCH(prefill_gemm_kernel<1>, grid, dim3(256), 2 * kMTilesPerGroup * kPTileBytes, stream, w, rowtiles, rows, nb,
                           ap, m_tiles, n, out, ld, ps.sb_split, stride, (const int32_t*)nullptr, (int64_t)0, (const int32_t*)nullptr,
                           (const uint8_t*)nullptr);
    } else {
        MQ_LAUNCH(prefill_gemm_kernel<2>, grid, dim3(256), 2 * kMTilesPerGroup * kPTileBytes, stream, w, rowtiles, rows, nb,
                           ap, m_tiles, n, out, ld, ps.sb_split, stride, (const int32_t*)nullptr, (int64_t)0, (const int32_t*)nullptr,
                           (const uint8_t*)nullptr);
    }
    if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
    if (split) {
        const int64_t units = n * (rows >> 2);
        MQ_LAUNCH(prefill_sum_planes_kernel, dim3((unsigned)((units + 255) / 256)), dim3(256), 0, stream, part, ps.splits, n,
                           rows, y, ldy);
    }
    return hipGetLastError();
}

// ---- skinny16 -------------------------------------------------------------------------------------------------
namespace {

constexpr size_t kSkinnyLdsMax = 160 * 1024;

size_t skinny16_red_bytes(int nmat, int wpr, int mt) { return (size_t)(8 / wpr) * (wpr - 1) * nmat * mt * 4 * 64 * sizeof(float); }
// LDS of the form with the rows' tiles in LDS, `ranges` runs of super-blocks one after the other: with one tile of
// sixteen the partial sums lie behind the tiles, with more they share the tiles' bytes
size_t skinny16_lds_bytes(int nmat, int wpr, int64_t nb, int mt, int ranges) {
    const size_t tiles = (size_t)(nb / ranges) * mt * kPTileBytes, red = skinny16_red_bytes(nmat, wpr, mt);
    return mt > 1 ? (tiles > red ? tiles : red) : tiles + red;
}
// Runs of super-blocks the rows' tiles need to pass through LDS (1, 2 or 4; every wavefront must have a whole number
// of stages per run), or 0: they do not fit that way.
int skinny16_ranges(int nmat, int wpr, int64_t nb, int mt) {
    for (int ranges = 1; ranges <= 4; ranges *= 2) {
        if (ranges > 1 && (mt == 1 || nb % ((int64_t)wpr * ranges))) break;
        if (skinny16_lds_bytes(nmat, wpr, nb, mt, ranges) <= kSkinnyLdsMax) return ranges;
    }
    return 0;
}

template <int NMAT, int WPR, int FLOW, bool GA, int MT, int WT>
hipError_t launch_skinny16_one(const Skinny16Args& a, int ranges, hipStream_t stream, hipEvent_t start, hipEvent_t stop) {
    const int64_t rowtiles = (a.rows + 15) / 16;
    const size_t lds = GA ? skinny16_red_bytes(NMAT, WPR, MT) : skinny16_lds_bytes(NMAT, WPR, a.nb, MT, ranges);
    auto* kernel = &skinny16_kernel<NMAT, WPR, FLOW, GA, MT, WT>;
    static bool raised = false;  // per instantiation; the attribute belongs to the function, not to a launch
    if (!raised) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)kSkinnyLdsMax);
        if (e != hipSuccess) return e;
        raised = true;
    }
    Skinny16Args b = a;
    b.ranges = GA ? 1 : ranges;
    constexpr int RPW = 8 / WPR;
    const dim3 grid((unsigned)((rowtiles + RPW - 1) / RPW));
    if (start && stop) hipExtLaunchKernelGGL(kernel, grid, dim3(512), lds, stream, start, stop, 0, b);
    else MQ_LAUNCH(kernel, grid, dim3(512), lds, stream, b);
    return hipGetLastError();
}

// MT <= 2: the rows' tiles in LDS (in runs if need be), else from global memory a stage ahead; three and four tiles only
// from LDS (read a stage ahead they do not fit the registers), an even number of stages per wavefront.
template <int NMAT, int WPR, int MT, int WT>
hipError_t launch_skinny16_form(const Skinny16Args& a, hipStream_t stream, hipEvent_t start, hipEvent_t stop) {
    const bool odd = ((a.nb / WPR) & 1) != 0;
    const int ranges = odd ? (skinny16_lds_bytes(NMAT, WPR, a.nb, MT, 1) <= kSkinnyLdsMax ? 1 : 0) : skinny16_ranges(NMAT, WPR, a.nb, MT);
    // (the forms left out below spill registers -- skinny16_applies knows them)
    if constexpr (WT == kWtQ6 && NMAT == 2 && WPR == 1) {
        return hipErrorInvalidValue;
    } else if constexpr (MT <= 2) {
        const bool ga = ranges != 1;  // (two tiles could also come in runs; read a stage ahead they cost no barrier)
        if constexpr (WT != kWtQ4 && NMAT == 2 && MT == 2) {  // two tiles of a Q5_K or Q6_K pair: not read a stage ahead
            if (ga) return hipErrorInvalidValue;
            if (odd) return launch_skinny16_one<NMAT, WPR, 1, false, MT, WT>(a, 1, stream, start, stop);
            return launch_skinny16_one<NMAT, WPR, 0, false, MT, WT>(a, 1, stream, start, stop);
        } else {
            if (odd) return ga ? launch_skinny16_one<NMAT, WPR, 1, true, MT, WT>(a, 1, stream, start, stop) : launch_skinny16_one<NMAT, WPR, 1, false, MT, WT>(a, 1, stream, start, stop);
            return ga ? launch_skinny16_one<NMAT, WPR, 0, true, MT, WT>(a, 1, stream, start, stop) : launch_skinny16_one<NMAT, WPR, 0, false, MT, WT>(a, 1, stream, start, stop);
        }
    } else if constexpr (WPR == 1 || (NMAT == 2 && MT == 4 && WPR == 8)) {
        return hipErrorInvalidValue;
    } else {
        if (ranges == 0) return hipErrorInvalidValue;
        if (odd) return launch_skinny16_one<NMAT, WPR, 1, false, MT, WT>(a, 1, stream, start, stop);  // (an odd stage count: one run only)
        if ((((a.nb / WPR) / ranges) & 1) == 0) return launch_skinny16_one<NMAT, WPR, 0, false, MT, WT>(a, ranges, stream, start, stop);
        if constexpr (WT == kWtQ6 || (WT == kWtQ5 && NMAT == 2 && MT == 4)) return hipErrorInvalidValue;  // (runs of an odd stage count)
        else return launch_skinny16_one<NMAT, WPR, 2, false, MT, WT>(a, ranges, stream, start, stop);
    }
}

template <int NMAT, int MT, int WT>
hipError_t launch_skinny16_wpr(const Skinny16Args& a, int wpr, hipStream_t stream, hipEvent_t start, hipEvent_t stop) {
    switch (wpr) {
        case 1: return launch_skinny16_form<NMAT, 1, MT, WT>(a, stream, start, stop);
        case 2: return launch_skinny16_form<NMAT, 2, MT, WT>(a, stream, start, stop);
        case 4: return launch_skinny16_form<NMAT, 4, MT, WT>(a, stream, start, stop);
        case 8: return launch_skinny16_form<NMAT, 8, MT, WT>(a, stream, start, stop);
    }
    return hipErrorInvalidValue;
}

template <int NMAT>
hipError_t launch_skinny16_tiles(const Skinny16Args& a, int wpr, hipStream_t stream, hipEvent_t start, hipEvent_t stop) {
    const int mt = (int)((a.n + 15) / 16);
    if (a.wtype == kTypeQ5K) {
        if (mt == 1) return launch_skinny16_wpr<NMAT, 1, kWtQ5>(a, wpr, stream, start, stop);
        if (mt == 2) return launch_skinny16_wpr<NMAT, 2, kWtQ5>(a, wpr, stream, start, stop);
        if (mt == 3) return launch_skinny16_wpr<NMAT, 3, kWtQ5>(a, wpr, stream, start, stop);
        if (mt == 4) return launch_skinny16_wpr<NMAT, 4, kWtQ5>(a, wpr, stream, start, stop);
        return hipErrorInvalidValue;
    }
    if (a.wtype == kTypeQ6K) {
        if (mt == 1) return launch_skinny16_wpr<NMAT, 1, kWtQ6>(a, wpr, stream, start, stop);
        if (mt == 2) return launch_skinny16_wpr<NMAT, 2, kWtQ6>(a, wpr, stream, start, stop);
        if (mt == 3) return launch_skinny16_wpr<NMAT, 3, kWtQ6>(a, wpr, stream, start, stop);
        if (mt == 4) return launch_skinny16_wpr<NMAT, 4, kWtQ6>(a, wpr, stream, start, stop);
        return hipErrorInvalidValue;
    }
    switch (mt) {
        case 1: return launch_skinny16_wpr<NMAT, 1, kWtQ4>(a, wpr, stream, start, stop);
        case 2: return launch_skinny16_wpr<NMAT, 2, kWtQ4>(a, wpr, stream, start, stop);
        case 3: return launch_skinny16_wpr<NMAT, 3, kWtQ4>(a, wpr, stream, start, stop);
        case 4: return launch_skinny16_wpr<NMAT, 4, kWtQ4>(a, wpr, stream, start, stop);
    }
    return hipErrorInvalidValue;
}

}  // namespace

// Whether a product of n rows (nine to 64) runs on skinny16_kernel: the wave split of the other decode kernels must be
// one of its own (a divisor of eight that divides the super-blocks of a row), and the form must be built
// (launch_skinny16_form returns an error for the others: those whose registers spill).
//   One and two tiles (up to 32 rows): always; the two tiles of a Q5_K or Q6_K gate/up pair only where they fit LDS in
//   one run; a Q6_K pair not with one wavefront per row tile.
//   Three and four tiles: not with one wavefront per row tile (more than 1,024 row tiles: the GEMM is faster from 33
//   rows -- 128256 x 4096 at 33 / 64 rows: 93 / 108 us against 102 / 126); the tiles must pass through LDS in at most four
//   runs of whole stages (in one run where a wavefront's stage count is odd); a pair of four tiles not with eight
//   wavefronts per row tile; in runs of an odd number of stages no Q6_K form and no Q5_K pair of four tiles.
bool skinny16_applies(int64_t nb, int64_t rowtiles, bool swiglu, int64_t n, int wtype) {
    const int wpr = dense_lds_wpr(nb, rowtiles);
    if (!wpr || nb % wpr || n < 1 || n > 64 || (wtype != kTypeQ4K && wtype != kTypeQ5K && wtype != kTypeQ6K)) return false;
    const int nmat = swiglu ? 2 : 1, mt = (int)((n + 15) / 16);
    if (wtype == kTypeQ6K && swiglu && wpr == 1) return false;
    if (mt <= 2) return !(wtype != kTypeQ4K && swiglu && mt == 2) || skinny16_lds_bytes(2, wpr, nb, 2, 1) <= kSkinnyLdsMax;
    if (wpr == 1 || (swiglu && mt == 4 && wpr == 8)) return false;
    if ((nb / wpr) & 1) return skinny16_lds_bytes(nmat, wpr, nb, mt, 1) <= kSkinnyLdsMax;  // an odd stage count: the tiles in one run
    const int ranges = skinny16_ranges(nmat, wpr, nb, mt);
    if (!ranges) return false;
    const bool odd_runs = (((nb / wpr) / ranges) & 1) != 0;
    return !odd_runs || !(wtype == kTypeQ6K || (wtype == kTypeQ5K && swiglu && mt == 4));
}

hipError_t launch_skinny16(const Skinny16Args& a, hipStream_t stream, hipEvent_t start, hipEvent_t stop) {
    if (a.rows <= 0 || a.nb <= 0 || a.n < 1 || a.n > 64 || !a.y || !a.w0 || !a.ap) return hipErrorInvalidValue;
    const int64_t rowtiles = (a.rows + 15) / 16;
    if (!skinny16_applies(a.nb, rowtiles, a.w1 != nullptr, a.n, a.wtype)) return hipErrorInvalidValue;
    const int wpr = dense_lds_wpr(a.nb, rowtiles);
    if (a.w1) return launch_skinny16_tiles<2>(a, wpr, stream, start, stop);
    return launch_skinny16_tiles<1>(a, wpr, stream, start, stop);
}

}  // namespace mq
