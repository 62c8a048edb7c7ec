// Per-tile arithmetic of the decode kernels: one 2304-byte weight tile (16 rows x one super-block) against
// up to 8 activation rows in the split-slot A-major layout (common.h).
#pragma once

#include <type_traits>

#include "common.h"

namespace mq {

#if defined(__HIPCC__)
typedef unsigned int v2u __attribute__((ext_vector_type(2)));

struct TileRegs {
    v4u q0, q1, hdr;
    v2u qh;  // Q5_K only: qh[8*kq .. 8*kq+7] of weight row lane%16 (bit s = fifth bit in sub-block s)
};

template <bool Q5 = false>
__device__ __forceinline__ void load_tile(TileRegs& t, const uint8_t* tile, int lane) {
    t.q0 = load_stream16(tile + lane * 16);
    t.q1 = load_stream16(tile + 1024 + lane * 16);
    t.hdr = load_stream16(tile + kTileQBytes + (lane & 15) * 16);
    if (Q5) t.qh = __builtin_nontemporal_load(reinterpret_cast<const v2u*>(tile + kTileHBytes + lane * 8));
}

template <int TT>
struct ARegs {
    v4u q[TT][4];    // [token tile][64-weight chunk]: this lane's 16 B of the split-slot A operand
    float yd[TT][2]; // Q8_K scales of the two activation rows this lane accumulates
};

// All loads are unconditional: the caller clamps the row of a dead slot to a live row of the same
// group, whose result is simply never stored.  Branch-free loads let the compiler count the
// outstanding requests exactly, which is what keeps the next tile in flight during the MFMAs.
template <int TT>
__device__ __forceinline__ void load_a(ARegs<TT>& a, const uint8_t* __restrict__ aq_blk, const float* __restrict__ ad_blk,
                                       const size_t (&a_off)[TT], const int (&d_idx)[TT][2]) {
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
#pragma unroll
        for (int c = 0; c < 4; ++c) a.q[tt][c] = load16(aq_blk + a_off[tt] + c * 1024);
#pragma unroll
        for (int j = 0; j < 2; ++j) a.yd[tt][j] = ad_blk[d_idx[tt][j]];
    }
}

// bit `s` of every byte of h, moved to bit 4 of that byte
__device__ __forceinline__ uint32_t fifth_bits(uint32_t h, int s) {
    return (s <= 4 ? h << (4 - s) : h >> (s - 4)) & 0x10101010u;
}

// J = 1: only the first of a lane's two activation rows is formed (a single activation row sits in row 0 of the
// operand: j = 1 would be work on a row that is never stored); the same bits for the row that is.
template <int TT, bool Q5 = false, int J = 2>
__device__ __forceinline__ void compute_tile(const TileRegs& t, const ARegs<TT>& a, float (&acc)[TT][2],
                                             int32_t (&dot_out)[TT][2], int32_t (&min_out)[TT][2]) {
    // 6-bit scale / min unpack, word-parallel (core/src/kernels/hwy/hwy_moe_quant.cc:90-101)
    const uint32_t w0 = t.hdr.y, w1 = t.hdr.z, w2 = t.hdr.w;
    const uint32_t sc[2] = {w0 & 0x3f3f3f3fu, (w2 & 0x0f0f0f0fu) | (((w0 >> 6) & 0x03030303u) << 4)};
    const uint32_t mn[2] = {w1 & 0x3f3f3f3fu, ((w2 >> 4) & 0x0f0f0f0fu) | (((w1 >> 6) & 0x03030303u) << 4)};
    const uint32_t qw[8] = {t.q0.x, t.q0.y, t.q0.z, t.q0.w, t.q1.x, t.q1.y, t.q1.z, t.q1.w};

    int32_t dot[TT][2];
    v4i mnd[TT];
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
        dot[tt][0] = dot[tt][1] = 0;
        mnd[tt] = v4i{0, 0, 0, 0};
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) {  // 64-weight chunk: sub-blocks 2c (low nibbles) and 2c+1 (high nibbles)
        const uint32_t qa = qw[2 * c], qb = qw[2 * c + 1];
        v4i b_q = {(int)(qa & 0x0f0f0f0fu), (int)(qb & 0x0f0f0f0fu), (int)((qa >> 4) & 0x0f0f0f0fu),
                   (int)((qb >> 4) & 0x0f0f0f0fu)};
        if (Q5) {  // codes 0..31: the fifth bit of sub-blocks 2c and 2c+1 (core/src/kernels/hwy/hwy_moe_quant.cc:177-200)
            b_q.x |= (int)fifth_bits(t.qh.x, 2 * c);
            b_q.y |= (int)fifth_bits(t.qh.y, 2 * c);
            b_q.z |= (int)fifth_bits(t.qh.x, 2 * c + 1);
            b_q.w |= (int)fifth_bits(t.qh.y, 2 * c + 1);
        }
        const int s_lo = (int)((sc[c >> 1] >> (16 * (c & 1))) & 0xffu);
        const int s_hi = (int)((sc[c >> 1] >> (16 * (c & 1) + 8)) & 0xffu);
        // v_perm_b32 replicates one byte of the unpacked mins into all four bytes of the operand
        const uint32_t m_lo = __builtin_amdgcn_perm(0u, mn[c >> 1], 0x01010101u * (uint32_t)(2 * (c & 1)));
        const uint32_t m_hi = __builtin_amdgcn_perm(0u, mn[c >> 1], 0x01010101u * (uint32_t)(2 * (c & 1) + 1));
        const v4i b_min = {(int)m_lo, (int)m_lo, (int)m_hi, (int)m_hi};
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
            const v4u av = a.q[tt][c];
            const v4i a16 = {(int)av.x, (int)av.y, (int)av.z, (int)av.w};
            const v4i zero = {0, 0, 0, 0};
            // p[0], p[2]: sub-block 2c of rows 2kq and 2kq+1;  p[1], p[3]: sub-block 2c+1
            const v4i p = __builtin_amdgcn_mfma_i32_16x16x64_i8(a16, b_q, zero, 0, 0, 0);
            dot[tt][0] += __mul24(p[0], s_lo) + __mul24(p[1], s_hi);
            if (J > 1) dot[tt][1] += __mul24(p[2], s_lo) + __mul24(p[3], s_hi);
            mnd[tt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a16, b_min, mnd[tt], 0, 0, 0);
        }
    }
    const float wd = half_bits_to_float(t.hdr.x & 0xffffu);
    const float wm = half_bits_to_float(t.hdr.x >> 16);
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
#pragma unroll
        for (int j = 0; j < J; ++j) {
            const int32_t md = mnd[tt][2 * j] + mnd[tt][2 * j + 1];
            const float d = __fmul_rn(wd, a.yd[tt][j]);
            const float dm = __fmul_rn(wm, a.yd[tt][j]);
            const float term = __fsub_rn(__fmul_rn(d, (float)dot[tt][j]), __fmul_rn(dm, (float)md));
            acc[tt][j] = __fadd_rn(acc[tt][j], term);
            dot_out[tt][j] = dot[tt][j];
            min_out[tt][j] = md;
        }
    }
}

// ---- Q6_K (tile layout in common.h) -------------------------------------------------------------------
struct TileRegs6 {
    v4u ql0, ql1;  // nibbles of the two 128-weight halves
    v4u qh;        // top bits: .x .y half 0, .z .w half 1 (bit 5 of every code already flipped)
    v4u sc;        // the row's 16 signed scales, byte g = scale of weights 16 g .. 16 g + 15
    uint32_t d;    // fp16 d in the low half
};

__device__ __forceinline__ void load_tile6(TileRegs6& t, const uint8_t* tile, int lane) {
    t.ql0 = load_stream16(tile + lane * 16);
    t.ql1 = load_stream16(tile + 1024 + lane * 16);
    t.qh = load_stream16(tile + kTile6HOff + lane * 16);
    t.sc = load_stream16(tile + kTile6SOff + (lane & 15) * 16);
    t.d = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(tile + kTile6DOff + (lane & 15) * 4));
}

// One Q6_K tile against up to 8 activation rows.  The B bytes are (six code bits) << 2, i.e. 4 * (code - 32) as a
// signed byte; scales apply per 16 weights, so every 64-weight chunk takes two MFMAs, one with the activations of
// k-groups 0..1 (weights 0..15 of each 32-wide half) and one with those of k-groups 2..3 (weights 16..31): the four
// sums that come out are the chunk's four 16-weight groups.  dot_out = sum_g scale_g * sum (code - 32) * q8 exactly
// (core/src/llm/matmul/q6_small_batch.h:56-83); fp32: acc = fma(d * yd, float(dot), acc) (:84-86).
template <int TT, int J = 2>
__device__ __forceinline__ void compute_tile6(const TileRegs6& t, const ARegs<TT>& a, float (&acc)[TT][2],
                                              int32_t (&dot_out)[TT][2], int32_t (&min_out)[TT][2], int lane) {
    const uint32_t keep_lo = (lane & 32) ? 0u : 0xffffffffu;  // k-groups 0 and 1
    const uint32_t keep_hi = ~keep_lo;
    const uint32_t qlw[8] = {t.ql0.x, t.ql0.y, t.ql0.z, t.ql0.w, t.ql1.x, t.ql1.y, t.ql1.z, t.ql1.w};
    const uint32_t qhw[4] = {t.qh.x, t.qh.y, t.qh.z, t.qh.w};
    const uint32_t scw[4] = {t.sc.x, t.sc.y, t.sc.z, t.sc.w};
    int32_t dot[TT][2];
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) dot[tt][0] = dot[tt][1] = 0;
#pragma unroll
    for (int c = 0; c < 4; ++c) {  // 64-weight chunk: half j = c / 2, nibble side hn = c % 2
        const int j = c >> 1, hn = c & 1;
        v4i b_q;
#pragma unroll
        for (int w = 0; w < 4; ++w) {  // dwords 0,1: first 32 weights of the chunk (z = 2 hn), dwords 2,3: z = 2 hn + 1
            const int z = 2 * hn + (w >> 1);
            const uint32_t nib = (hn ? qlw[4 * j + w] >> 2 : qlw[4 * j + w] << 2) & 0x3c3c3c3cu;
            const uint32_t hi = qhw[2 * j + (w & 1)];
            const uint32_t top = z == 3 ? hi : hi << (6 - 2 * z);
            b_q[w] = (int)((top & 0xc0c0c0c0u) | nib);
        }
        const int s0 = (int)(int8_t)(scw[c] & 0xffu), s1 = (int)(int8_t)((scw[c] >> 8) & 0xffu);
        const int s2 = (int)(int8_t)((scw[c] >> 16) & 0xffu), s3 = (int)(int8_t)(scw[c] >> 24);
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
            const v4u av = a.q[tt][c];
            const v4i a_lo = {(int)(av.x & keep_lo), (int)(av.y & keep_lo), (int)(av.z & keep_lo), (int)(av.w & keep_lo)};
            const v4i a_hi = {(int)(av.x & keep_hi), (int)(av.y & keep_hi), (int)(av.z & keep_hi), (int)(av.w & keep_hi)};
            const v4i zero = {0, 0, 0, 0};
            // p[0], p[2]: first 32-wide half of the chunk for rows 2kq and 2kq+1; p[1], p[3]: second half
            const v4i pl = __builtin_amdgcn_mfma_i32_16x16x64_i8(a_lo, b_q, zero, 0, 0, 0);
            const v4i ph = __builtin_amdgcn_mfma_i32_16x16x64_i8(a_hi, b_q, zero, 0, 0, 0);
            dot[tt][0] += __mul24(pl[0], s0) + __mul24(ph[0], s1) + __mul24(pl[1], s2) + __mul24(ph[1], s3);
            if (J > 1) dot[tt][1] += __mul24(pl[2], s0) + __mul24(ph[2], s1) + __mul24(pl[3], s2) + __mul24(ph[3], s3);
        }
    }
    const float wd = half_bits_to_float(t.d & 0xffffu);
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
#pragma unroll
        for (int j = 0; j < J; ++j) {
            const int32_t isum = dot[tt][j] >> 2;  // the B bytes carried a factor 4
            acc[tt][j] = __fmaf_rn(__fmul_rn(a.yd[tt][j], wd), (float)isum, acc[tt][j]);
            dot_out[tt][j] = isum;
            min_out[tt][j] = 0;
        }
    }
}

// ---- a ring of two register stages over `cnt` stages ---------------------------------------------------------------
// issue(slot, i) requests stage i into register slot `slot`; consume(slot, i) uses it.  `slot` arrives as a
// std::integral_constant so that it indexes register arrays at compile time.  While stage i is consumed exactly one
// further stage (i + 1) is in flight; stage i + 2 is requested as soon as slot i % 2 is free.  Stages go in pairs, so
// every iteration makes the same number of requests and the compiler's vmcnt immediates are exact; with an odd count
// issue() is called ONCE with i == cnt, past the end, and must then make the same loads from one fixed address in all
// lanes (a single cache line, answered by the L1), never a stage that does not exist.  Measured on the dense gate/up
// product (eight stages per wavefront): the old three- and four-deep rings padded their tails with two or three real
// tile requests per wavefront (a quarter more load instructions: 15.7 -> 13.3 us without them), and deeper rings
// make the wavefronts of a compute unit receive their first tiles one after the other instead of side by side.
// issue()'s third argument tells whether the request is one of the first two (std::true_type) or a refill inside
// the loop (std::false_type): a kernel whose stages alternate between two activation blocks keeps each block's
// operand in its slot and only asks for it the first time.
template <class Issue, class Consume>
__device__ __forceinline__ void ring2(int cnt, Issue issue, Consume consume) {
    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;
    if (cnt <= 0) return;
    issue(S0{}, 0, std::true_type{});
    asm volatile("" ::: "memory");  // requests stay in stage order (the scheduler would group them by base register)
    issue(S1{}, 1, std::true_type{});
    asm volatile("" ::: "memory");
    int i = 0;
    for (; i + 2 < cnt; i += 2) {
        consume(S0{}, i);
        issue(S0{}, i + 2, std::false_type{});
        asm volatile("" ::: "memory");
        consume(S1{}, i + 1);
        issue(S1{}, i + 3, std::false_type{});
        asm volatile("" ::: "memory");
    }
    consume(S0{}, i);
    if (i + 1 < cnt) consume(S1{}, i + 1);
}

// ---- one name per weight type ---------------------------------------------------------------------------
constexpr int kWtQ4 = 0, kWtQ5 = 1, kWtQ6 = 2;
template <int WT> struct TileOf { using Regs = TileRegs; };
template <> struct TileOf<kWtQ6> { using Regs = TileRegs6; };
template <int WT> constexpr int tile_stride() { return WT == kWtQ6 ? kTile6Bytes : WT == kWtQ5 ? kTile5Bytes : kTileBytes; }

template <int WT>
__device__ __forceinline__ void load_tile_wt(typename TileOf<WT>::Regs& t, const uint8_t* tile, int lane) {
    if constexpr (WT == kWtQ6) load_tile6(t, tile, lane);
    else load_tile<WT == kWtQ5>(t, tile, lane);
}
template <int TT, int WT, int J = 2>
__device__ __forceinline__ void compute_tile_wt(const typename TileOf<WT>::Regs& t, const ARegs<TT>& a, float (&acc)[TT][2],
                                                int32_t (&dot_out)[TT][2], int32_t (&min_out)[TT][2], int lane) {
    if constexpr (WT == kWtQ6) compute_tile6<TT, J>(t, a, acc, dot_out, min_out, lane);
    else compute_tile<TT, WT == kWtQ5, J>(t, a, acc, dot_out, min_out);
}

#endif

}  // namespace mq
