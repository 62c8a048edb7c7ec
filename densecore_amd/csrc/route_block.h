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

__device__ __forceinline__ float route_key_logit(unsigned long long key);

// ---- routing of one token by one wavefront ---------------------------------------------------------
// 32-bit order key of a logit: larger = earlier in the routing order, NaN = 1 (after every number), 0 = absent.
__device__ __forceinline__ uint32_t route_key32(float v) { return (uint32_t)(route_key(v, 0) >> 32) + 1u; }
__device__ __forceinline__ float route_key32_logit(uint32_t key) { return route_key_logit((unsigned long long)(key - 1u) << 32); }

// float maximum over lanes 0..7 (fmaxf semantics: a NaN operand is ignored), valid in lanes 0..7
__device__ __forceinline__ float max_first8(float x) {
    x = fmaxf(x, __uint_as_float(dpp_u32<kDppXor1>(__float_as_uint(x))));
    x = fmaxf(x, __uint_as_float(dpp_u32<kDppXor2>(__float_as_uint(x))));
    x = fmaxf(x, __uint_as_float(dpp_u32<kDppHalfMirror>(__float_as_uint(x))));
    return x;
}

// route_weights with lane k holding logit k (k < top_k <= 8): the same maxima, the same exponentials, the
// denominator summed in routing order by reading the lanes one after the other.  Returns lane k's weight.
__device__ __forceinline__ float route_weight_lane(float l, int lane, int top_k, int mode) {
    const bool in = lane < top_k;
    const bool fin = isfinite(l);
    const float uni = __fdiv_rn(1.0f, (float)top_k);
    float mx = max_first8(in && (mode == 1 || fin) ? l : -INFINITY);
    mx = __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(mx)));
    if (mode == 1 && !isfinite(mx)) mx = 0.0f;
    const bool all_finite = __ballot(in && !fin) == 0ull;
    const float w = expf(__fsub_rn(l, mx));
    // which slots enter the denominator
    bool counted;
    if (mode == 0) counted = in && all_finite && isfinite(mx);
    else if (mode == 1) counted = in;
    else counted = in && fin && isfinite(mx);
    const unsigned long long counted_mask = __ballot(counted);
    float den = 0.0f;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const float wk = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(w), k));
        if ((counted_mask >> k) & 1ull) den = __fadd_rn(den, wk);
    }
    if (mode == 0) return (!(den > 0.0f) || !isfinite(den)) ? uni : __fdiv_rn(w, den);
    if (mode == 1) return __fdiv_rn(w, fmaxf(den, 6.103515625e-5f));
    const bool uniform = !(den > 0.0f) || !isfinite(den);
    den = uniform ? 1.0f : fmaxf(den, 6.103515625e-5f);
    return (uniform || !fin || !isfinite(mx)) ? uni : __fdiv_rn(w, den);
}

// Stable top-k of one token (ComputeQwenNativeMoEStableTopK, core/src/llm/moe/native.cpp:610-645) and its
// weights.  Lane l owns the experts l, l + 64, ...: per round a wave-wide maximum of the 32-bit keys, the
// lowest expert id among the holders of that key (ballots, scanned in expert order), and the owner retires it.
// load(e) returns logit e.  Lanes k < top_k end up with expert k of the routing order and its logit
// (route_weight_lane turns those logits into the weights).
// The logits of one token, KPL per lane (lane l: experts l, l + 64, ...).  Every lane reads KPL of them (a lane past
// the end re-reads the last one): unconditional loads are requested together, not one round trip each.
template <int KPL, typename Load>
__device__ __forceinline__ void route_load_logits(Load load, int n_experts, int lane, float (&logit)[KPL]) {
#pragma unroll
    for (int i = 0; i < KPL; ++i) {
        const int e = lane + 64 * i;
        logit[i] = load(e < n_experts ? e : n_experts - 1);
    }
}

template <int KPL>
__device__ __forceinline__ void route_logits_wave(const float (&logit)[KPL], int n_experts, int top_k, int lane, int& id_out,
                                                  float& logit_out) {
    uint32_t key[KPL];
#pragma unroll
    for (int i = 0; i < KPL; ++i) key[i] = lane + 64 * i < n_experts ? route_key32(logit[i]) : 0u;
    float my_logit = 0.0f;
    int my_id = -1;
    for (int r = 0; r < top_k; ++r) {
        uint32_t best = key[0];
#pragma unroll
        for (int i = 1; i < KPL; ++i) best = key[i] > best ? key[i] : best;
        const uint32_t top = wave_max_u32(best);
        int id = -1;
#pragma unroll
        for (int i = 0; i < KPL; ++i) {
            const unsigned long long holders = __ballot(key[i] == top);
            if (id < 0 && holders != 0ull) id = 64 * i + __ffsll((long long)holders) - 1;
        }
#pragma unroll
        for (int i = 0; i < KPL; ++i)
            if (lane + 64 * i == id) key[i] = 0u;
        if (lane == r) {
            my_logit = route_key32_logit(top);
            my_id = id;
        }
    }
    id_out = my_id;
    logit_out = my_logit;
}

template <int KPL, typename Load>
__device__ __forceinline__ void route_token_wave(Load load, int n_experts, int top_k, int lane, int& id_out,
                                                 float& logit_out) {
    float logit[KPL];
    route_load_logits<KPL>(load, n_experts, lane, logit);
    route_logits_wave<KPL>(logit, n_experts, top_k, lane, id_out, logit_out);
}

// The same routing in one pass for the common case, for a wavefront that has LDS of its own (kRouteScratch 64-bit
// words, used by no other wavefront).  The smallest of the eight 8-lane group maxima is a key that at least eight
// keys reach, so the top_k <= 8 first experts of the routing order are among the keys >= it (typically one or two
// dozen of 256).  Those are packed into LDS as (key << 32 | ~id) -- larger = earlier in the routing order, never
// equal -- and every candidate counts the candidates ahead of it: its place in the routing order.  More than 64
// candidates (rows of equal logits) go the round-by-round way; ids and logits are the same either way.
constexpr int kRouteScratch = 72;
template <int KPL>
__device__ __forceinline__ void route_logits_wave_lds(const float (&logit)[KPL], int n_experts, int top_k, int lane, int& id_out,
                                                      float& logit_out, unsigned long long* scratch) {
    uint32_t key[KPL];
    uint32_t best = 0u;
#pragma unroll
    for (int i = 0; i < KPL; ++i) {
        key[i] = lane + 64 * i < n_experts ? route_key32(logit[i]) : 0u;
        best = key[i] > best ? key[i] : best;
    }
    uint32_t t;
    t = dpp_u32<kDppXor1>(best), best = t > best ? t : best;
    t = dpp_u32<kDppXor2>(best), best = t > best ? t : best;
    t = dpp_u32<kDppHalfMirror>(best), best = t > best ? t : best;  // the maximum of the lane's group of eight
    t = dpp_u32<kDppMirror>(best), best = t < best ? t : best;      // the smaller of two groups
    const uint32_t p0 = __builtin_amdgcn_readlane(best, 0), p1 = __builtin_amdgcn_readlane(best, 16);
    const uint32_t p2 = __builtin_amdgcn_readlane(best, 32), p3 = __builtin_amdgcn_readlane(best, 48);
    const uint32_t p01 = p0 < p1 ? p0 : p1, p23 = p2 < p3 ? p2 : p3;
    const uint32_t pivot = p01 < p23 ? p01 : p23;
    int total = 0;
    unsigned long long mask[KPL];
#pragma unroll
    for (int i = 0; i < KPL; ++i) {
        mask[i] = __ballot(key[i] >= pivot && key[i] != 0u);
        total += __popcll(mask[i]);
    }
    if (total > 64) {
        route_logits_wave<KPL>(logit, n_experts, top_k, lane, id_out, logit_out);
        return;
    }
    scratch[lane] = 0ull;  // an empty place is ahead of nobody
    int base = 0;
#pragma unroll
    for (int i = 0; i < KPL; ++i) {
        const int below = (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(mask[i] >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask[i], 0u));
        if ((mask[i] >> lane) & 1ull)
            scratch[base + below] = ((unsigned long long)key[i] << 32) | (unsigned long long)(uint32_t)(~(uint32_t)(lane + 64 * i));
        base += __popcll(mask[i]);
    }
    // one wavefront: its LDS accesses are carried out in program order, the fence keeps the compiler to that order
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    const unsigned long long mine = scratch[lane < total ? lane : 0];
    int rank = 0;
    for (int c = 0; c < total; c += 8) {  // eight candidates per round trip to LDS (all lanes read the same words)
        unsigned long long other[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) other[u] = scratch[c + u];
#pragma unroll
        for (int u = 0; u < 8; ++u) rank += other[u] > mine ? 1 : 0;
    }
    if (lane < total && rank < top_k) scratch[64 + rank] = mine;
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    id_out = -1;
    logit_out = 0.0f;
    if (lane < top_k) {
        const unsigned long long sel = scratch[64 + lane];
        id_out = (int)(~(uint32_t)sel);
        logit_out = route_key32_logit((uint32_t)(sel >> 32));
    }
}

template <int KPL, typename Load>
__device__ __forceinline__ void route_token_wave_lds(Load load, int n_experts, int top_k, int lane, int& id_out,
                                                     float& logit_out, unsigned long long* scratch) {
    float logit[KPL];
    route_load_logits<KPL>(load, n_experts, lane, logit);
    route_logits_wave_lds<KPL>(logit, n_experts, top_k, lane, id_out, logit_out, scratch);
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
