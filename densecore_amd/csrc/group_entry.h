// Which activation row and which output row an entry of an expert group stands for (expert-grouped launches).
#pragma once

#include "kernels.h"

namespace mq {

#if defined(__HIPCC__)
// Activation row and output row of entry e of the current group.
template <bool GROUPED>
__device__ __forceinline__ void entry_rows(const MatmulArgs& p, bool shared_group, int begin, int e, int& ar, int& yr) {
    if (!GROUPED) {
        ar = e;
        yr = e;
    } else if (shared_group) {
        ar = (begin + e) * p.sh_arow_stride + p.sh_arow_offset;
        yr = (begin + e) * p.sh_yrow_stride + p.sh_yrow_offset;
    } else {
        int tok, kk;
        if (p.direct_ids) {  // few tokens: the group is the one pair `begin` = (token, slot); e is always 0
            tok = begin / p.direct_top_k;  // wave-uniform
            kk = begin - tok * p.direct_top_k;
        } else {
            tok = p.entry_token[begin + e];
            kk = p.entry_k[begin + e];
        }
        ar = tok * p.a_tok_stride + kk * p.a_k_stride;
        yr = tok * p.y_tok_stride + kk * p.y_k_stride;
    }
}

// The same for N entries at once: the list reads of all of them are requested together (one entry at a time they
// are conditional loads, which go out one round trip after the other).
template <bool GROUPED, int N>
__device__ __forceinline__ void entry_rows_n(const MatmulArgs& p, bool shared_group, int begin, const int (&e)[N],
                                             int (&ar)[N], int (&yr)[N]) {
    if (!GROUPED || shared_group || p.direct_ids) {
#pragma unroll
        for (int i = 0; i < N; ++i) entry_rows<GROUPED>(p, shared_group, begin, e[i], ar[i], yr[i]);
    } else {
        int tok[N], kk[N];
#pragma unroll
        for (int i = 0; i < N; ++i) tok[i] = p.entry_token[begin + e[i]], kk[i] = p.entry_k[begin + e[i]];
#pragma unroll
        for (int i = 0; i < N; ++i) {
            ar[i] = tok[i] * p.a_tok_stride + kk[i] * p.a_k_stride;
            yr[i] = tok[i] * p.y_tok_stride + kk[i] * p.y_k_stride;
        }
    }
}

#endif

}  // namespace mq
