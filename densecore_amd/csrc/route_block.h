// Device helpers of the MoE router shared by the routing kernels and the fused decoder-layer kernel:
// the routing order, its 64-bit sort key, the three softmax variants and the shared-expert gate.
#pragma once

#include "common.h"

namespace mq {

#if defined(__HIPCC__)
// core/src/llm/moe/native.cpp:610-619: non-NaN before NaN, larger logit first, lower id on ties.
__device__ __forceinline__ bool precedes(float a, int ia, float b, int ib) {
    const bool an = isnan(a), bn = isnan(b);
    if (an != bn) return !an;
    if (a > b) return true;
    if (a < b) return false;
    return ia < ib;
}

// 64-bit sort key of a router candidate: larger key = earlier in the routing order.  High word:
// the logit mapped to an unsigned integer of the same order (NaN lowest, -0 folded into +0 because
// the reference compares with < and >); low word: ~id, so that equal logits order by lower id.
__device__ __forceinline__ unsigned long long route_key(float v, int id) {
    uint32_t hi;
    if (isnan(v)) {
        hi = 0u;
    } else {
        const uint32_t bits = __float_as_uint(v == 0.0f ? 0.0f : v);
        hi = (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
    }
    return ((unsigned long long)hi << 32) | (unsigned long long)(uint32_t)(~(uint32_t)id);
}

// The largest 64-bit key held by any lane, in every lane: the high words first, then the low words of the
// lanes that hold that high word (two 32-bit wave maxima instead of a 64-bit butterfly through LDS).
__device__ __forceinline__ unsigned long long wave_max_key(unsigned long long key) {
    const uint32_t hi = (uint32_t)(key >> 32), lo = (uint32_t)key;
    const uint32_t top_hi = wave_max_u32(hi);
    const uint32_t top_lo = wave_max_u32(hi == top_hi ? lo : 0u);
    return ((unsigned long long)top_hi << 32) | top_lo;
}

// softmax over the selected logits, summed in routing order (three reference variants)
__device__ __forceinline__ void route_weights(const float* l, int top_k, int mode, float* __restrict__ out) {
    float w[8];
    if (mode == 0) {  // core/src/llm/moe/native.cpp:650-675
        float mx = -INFINITY;
        bool all_finite = true;
        for (int k = 0; k < top_k; ++k) {
            all_finite = all_finite && isfinite(l[k]);
            if (isfinite(l[k])) mx = fmaxf(mx, l[k]);
        }
        float den = 0.0f;
        if (all_finite && isfinite(mx)) {
            for (int k = 0; k < top_k; ++k) {
                w[k] = expf(__fsub_rn(l[k], mx));
                den = __fadd_rn(den, w[k]);
            }
        }
        if (!(den > 0.0f) || !isfinite(den)) {
            for (int k = 0; k < top_k; ++k) out[k] = __fdiv_rn(1.0f, (float)top_k);
        } else {
            for (int k = 0; k < top_k; ++k) out[k] = __fdiv_rn(w[k], den);
        }
    } else if (mode == 1) {  // core/src/llm/moe/native.cpp:2321-2355
        float mx = -INFINITY;
        for (int k = 0; k < top_k; ++k) mx = fmaxf(mx, l[k]);
        if (!isfinite(mx)) mx = 0.0f;
        float den = 0.0f;
        for (int k = 0; k < top_k; ++k) {
            w[k] = expf(__fsub_rn(l[k], mx));
            den = __fadd_rn(den, w[k]);
        }
        den = fmaxf(den, 6.103515625e-5f);
        for (int k = 0; k < top_k; ++k) out[k] = __fdiv_rn(w[k], den);
    } else {  // core/src/llm/moe/native.cpp:822-866
        float mx = -INFINITY;
        for (int k = 0; k < top_k; ++k)
            if (isfinite(l[k])) mx = fmaxf(mx, l[k]);
        float den = 0.0f;
        for (int k = 0; k < top_k; ++k)
            if (isfinite(l[k]) && isfinite(mx)) den = __fadd_rn(den, expf(__fsub_rn(l[k], mx)));
        const bool uniform = !(den > 0.0f) || !isfinite(den);
        den = uniform ? 1.0f : fmaxf(den, 6.103515625e-5f);
        const float uni = __fdiv_rn(1.0f, (float)top_k);
        for (int k = 0; k < top_k; ++k)
            out[k] = (uniform || !isfinite(l[k]) || !isfinite(mx)) ? uni : __fdiv_rn(expf(__fsub_rn(l[k], mx)), den);
    }
}

// The logit behind a route_key (NaN comes back as a canonical NaN, -0 as +0: neither changes a weight).
__device__ __forceinline__ float route_key_logit(unsigned long long key) {
    const uint32_t hi = (uint32_t)(key >> 32);
    if (hi == 0u) return __int_as_float(0x7fc00000);
    return __uint_as_float((hi & 0x80000000u) ? (hi & 0x7fffffffu) : ~hi);
}

__device__ __forceinline__ float stable_sigmoid(float x) {  // core/src/llm/graph/fused_ops.cpp:451-458
    if (x >= 0.0f) {
        const float z = expf(-x);
        return __fdiv_rn(1.0f, __fadd_rn(1.0f, z));
    }
    const float z = expf(x);
    return __fdiv_rn(z, __fadd_rn(1.0f, z));
}

#endif

}  // namespace mq
