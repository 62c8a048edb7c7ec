// Per-tile arithmetic of the decode kernels: one 2304-byte weight tile (16 rows x one super-block) against
// up to 8 activation rows in the split-slot A-major layout (common.h).
#pragma once

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

template <int TT, bool Q5 = false>
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
            dot[tt][1] += __mul24(p[2], s_lo) + __mul24(p[3], s_hi);
            mnd[tt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a16, b_min, mnd[tt], 0, 0, 0);
        }
    }
    const float wd = half_bits_to_float(t.hdr.x & 0xffffu);
    const float wm = half_bits_to_float(t.hdr.x >> 16);
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
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

#endif

}  // namespace mq
