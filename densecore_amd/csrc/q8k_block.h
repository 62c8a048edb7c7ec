// Wave-level Q8_K quantization of one 256-value super-block, shared by the stand-alone quantizer
// and by the matmul epilogue that re-quantizes its own output.
//
// Bit-exact with the reference quantizer (core/src/kernels/hwy/hwy_moe_quant.cc:103-143):
//   * the extreme element is the FIRST one of largest magnitude and keeps its sign, so the
//     cross-lane arg-max breaks ties towards the lower index;
//   * iscale = -127/max and d = 1/iscale are correctly rounded divisions;
//   * iscale*x is rounded before the +1.5*2^23 add (no FMA contraction), which then yields
//     round-half-even in the low mantissa bits.
#pragma once

#include "common.h"
#include "decode_tile.h"

namespace mq {

#if defined(__HIPCC__)
__device__ __forceinline__ int nearest_int_rne(float v) {
    const float biased = __fadd_rn(v, 12582912.0f);
    return (__float_as_int(biased) & 0x007fffff) - 0x00400000;
}

struct Q8Lane {
    uint32_t packed;  // this lane's four int8 codes (elements 4*lane .. 4*lane+3)
    float d;          // block scale (same in every lane)
    int bsum;         // lanes 4j..4j+3: sum of codes 16j..16j+15
};

// Every lane of the wave passes elements 4*lane .. 4*lane+3 of the block.
__device__ __forceinline__ Q8Lane quantize_block_q8k(const float (&e)[4], int lane) {
    float best_abs = 0.0f, best = 0.0f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {  // strict >: the first of equal magnitudes stays
        const float a = fabsf(e[j]);
        if (a > best_abs) {
            best_abs = a;
            best = e[j];
        }
    }
    // Wave-wide: the largest magnitude (non-negative floats order like their bit patterns), then the first
    // lane that holds it -- lanes own ascending element ranges, so that is the first such element.
    const uint32_t top = wave_max_u32(__float_as_uint(best_abs));
    const unsigned long long holders = __ballot(__float_as_uint(best_abs) == top);
    const int first = __builtin_amdgcn_readfirstlane(__ffsll((long long)holders) - 1);
    best = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(best), first));
    best_abs = __uint_as_float(top);
    int q[4] = {0, 0, 0, 0};
    Q8Lane r;
    r.d = 0.0f;
    if (best_abs != 0.0f) {
        const float iscale = __fdiv_rn(-127.0f, best);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int v = nearest_int_rne(__fmul_rn(iscale, e[j]));
            q[j] = v > 127 ? 127 : v;
        }
        r.d = __fdiv_rn(1.0f, iscale);
    }
    r.packed = (uint32_t)(q[0] & 0xff) | ((uint32_t)(q[1] & 0xff) << 8) | ((uint32_t)(q[2] & 0xff) << 16) |
               ((uint32_t)(q[3] & 0xff) << 24);
    int s = q[0] + q[1] + q[2] + q[3];
    s += (int)dpp_u32<kDppXor1>((uint32_t)s);
    s += (int)dpp_u32<kDppXor2>((uint32_t)s);
    r.bsum = s;
    return r;
}

// Writes the lane's codes of activation row m, super-block b into the A-major layout (common.h).
__device__ __forceinline__ void store_amajor(uint8_t* aq, float* ad, int64_t m, int64_t b, int64_t nb, int lane,
                                             const Q8Lane& r) {
    // element 4*lane+j: sub-block g = lane/8, index in sub-block 4*(lane%8)+j.  The codes go to the
    // half of the row's slot that belongs to the sub-block's parity, zeros to the other half.
    const int g = lane >> 3, h = g & 1;
    const int kq = (lane & 7) >> 1;
    const size_t off = aq_offset(m, b, g >> 1, kq, h, nb) + (size_t)(lane & 1) * 4;
    *reinterpret_cast<uint32_t*>(aq + off + h * 8) = r.packed;
    *reinterpret_cast<uint32_t*>(aq + off + (1 - h) * 8) = 0u;
    if (lane == 0) ad[ad_index(m, b, nb)] = r.d;
}

// The A operand of one activation row quantized by this wavefront (row 0 of the tile; the other rows are dead):
// codes move from the quantizer's lanes into the split-slot operand with eight cross-lane reads per super-block.
// ACodes is the operand before the zeros of the dead rows are filled in: nine registers instead of eighteen for
// a kernel that quantizes ahead of the tiles it multiplies.
struct ACodes {
    uint32_t lo[4], hi[4];
    float d;
};

__device__ __forceinline__ void a_codes_from_lane_codes(ACodes& a, const Q8Lane& q, int lane) {
    const int slot = lane & 15, kq = lane >> 4;
    const int src = 8 * (slot & 1) + 2 * kq;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        a.lo[c] = (uint32_t)__shfl((int)q.packed, 16 * c + src, 64);
        a.hi[c] = (uint32_t)__shfl((int)q.packed, 16 * c + src + 1, 64);
    }
    a.d = q.d;
}

__device__ __forceinline__ void a_from_codes(ARegs<1>& a, const ACodes& s, int lane) {
    // Slot 0 holds the codes in its first half and zeros in the second, slot 1 the other way round (the lanes of odd
    // slots fetched the odd sub-block's codes).  Slots 2..15 belong to rows nobody stores, and every output row of
    // the product depends on its own operand row only: they take the same pattern by slot parity, which costs two
    // masks instead of a three-way choice per register.
    const uint32_t even = (lane & 1) ? 0u : 0xffffffffu, odd = ~even;
#pragma unroll
    for (int c = 0; c < 4; ++c) a.q[0][c] = v4u{s.lo[c] & even, s.hi[c] & even, s.lo[c] & odd, s.hi[c] & odd};
    a.yd[0][0] = s.d;
    a.yd[0][1] = 0.0f;
}

__device__ __forceinline__ void a_from_lane_codes(ARegs<1>& a, const Q8Lane& q, int lane) {
    ACodes s;
    a_codes_from_lane_codes(s, q, lane);
    a_from_codes(a, s, lane);
}

#endif

}  // namespace mq
