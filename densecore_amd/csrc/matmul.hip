// Q4_K x Q8_K matmul for decode widths on gfx950 (dense and expert-grouped).
//
// Work decomposition
//   workgroup = one 16-row tile of the weight matrix (two matrices when gate and up are fused),
//               all of K; its W wavefronts take the super-blocks b = w, w+W, ... so that the
//               workgroup as a whole streams one contiguous run of tiles.
//   wavefront = per super-block: three coalesced 16-byte-per-lane loads bring one 2304-byte tile
//               (16 rows x 256 weights) straight into MFMA operand order; the next tile is
//               requested before the current one is consumed.
//   arithmetic (per tile, up to 16 activation rows at once, independent of how many are live):
//       8 x v_mfma_i32_16x16x32_i8   one per 32-wide sub-block: sum q4*q8            (int32)
//       v_mad_i32_i24 with the 6-bit sub-block scale                 -> dot_scaled   (int32)
//       4 x v_mfma_i32_16x16x64_i8   6-bit mins broadcast as the B operand: sum min*q8 -> min_dot
//       fp32: acc += (d*yd)*dot_scaled - (dmin*yd)*min_dot   (core/src/llm/matmul/kquant_batched_kernels.h:299-301)
//   The two integers are exactly the reference's per-super-block sums; min_dot is formed from the
//   int8 codes instead of the 16 bsums, which is the same number because bsums[j] is by
//   construction the sum of codes 16j..16j+15 (core/src/kernels/hwy/hwy_moe_quant.cc:133-139).
//   epilogue: wave partials are added in wave order through LDS (deterministic), optional
//   silu(gate)*up, one store per (activation row, weight row).
//
// MFMA operand roles: A (M side) = 16 activation rows, B (N side) = 16 weight rows, so each lane's
// four accumulators belong to ONE weight row (lane%16) and it needs only that row's scales.
#include <cstdlib>

#include "common.h"
#include "kernels.h"

namespace mq {

namespace {

struct TileRegs {
    v4u q0, q1, hdr;
};

__device__ __forceinline__ void load_tile(TileRegs& t, const uint8_t* tile, int lane) {
    t.q0 = load_stream16(tile + lane * 16);
    t.q1 = load_stream16(tile + 1024 + lane * 16);
    t.hdr = load_stream16(tile + kTileQBytes + (lane & 15) * 16);
}

__device__ __forceinline__ long pack64(uint32_t lo, uint32_t hi) {
    return (long)(((uint64_t)hi << 32) | (uint64_t)lo);
}

template <int TT>
struct ARegs {
    v4u q[TT][4];    // [token tile][sub-block pair]: 16 B = 8 codes of sub-block 2gp, 8 of 2gp+1
    float yd[TT][4]; // Q8_K scale of the four activation rows this lane accumulates
};

// All loads are unconditional: the caller clamps the row of a dead slot to a live row of the same
// group, whose result is simply never stored.  Branch-free loads let the compiler count the
// outstanding requests exactly, which is what keeps the next tile in flight during the MFMAs.
template <int TT>
__device__ __forceinline__ void load_a(ARegs<TT>& a, const uint8_t* __restrict__ aq, const float* __restrict__ ad,
                                       const int (&arow)[TT], const int (&drow)[TT][4], int64_t b, int64_t nb,
                                       int kq) {
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
#pragma unroll
        for (int gp = 0; gp < 4; ++gp) a.q[tt][gp] = load16(aq + aq_offset(arow[tt], b, gp, kq, nb));
#pragma unroll
        for (int i = 0; i < 4; ++i) a.yd[tt][i] = ad[ad_index(drow[tt][i], b, nb)];
    }
}

template <int TT>
__device__ __forceinline__ void compute_tile(const TileRegs& t, const ARegs<TT>& a, float (&acc)[TT][4],
                                             int32_t (&dot_out)[TT][4], int32_t (&min_out)[TT][4]) {
    // 6-bit scale / min unpack, word-parallel (core/src/kernels/hwy/hwy_moe_quant.cc:90-101)
    const uint32_t w0 = t.hdr.y, w1 = t.hdr.z, w2 = t.hdr.w;
    const uint32_t sc[2] = {w0 & 0x3f3f3f3fu, (w2 & 0x0f0f0f0fu) | (((w0 >> 6) & 0x03030303u) << 4)};
    const uint32_t mn[2] = {w1 & 0x3f3f3f3fu, ((w2 >> 4) & 0x0f0f0f0fu) | (((w1 >> 6) & 0x03030303u) << 4)};
    const uint32_t qw[8] = {t.q0.x, t.q0.y, t.q0.z, t.q0.w, t.q1.x, t.q1.y, t.q1.z, t.q1.w};

    v4i dot[TT], mnd[TT];
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
        dot[tt] = v4i{0, 0, 0, 0};
        mnd[tt] = v4i{0, 0, 0, 0};
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) {  // 64-weight chunk: sub-blocks 2c (low nibbles) and 2c+1 (high nibbles)
        const uint32_t qa = qw[2 * c], qb = qw[2 * c + 1];
        const long b_lo = pack64(qa & 0x0f0f0f0fu, qb & 0x0f0f0f0fu);
        const long b_hi = pack64((qa >> 4) & 0x0f0f0f0fu, (qb >> 4) & 0x0f0f0f0fu);
        const int s_lo = (int)((sc[c >> 1] >> (16 * (c & 1))) & 0xffu);
        const int s_hi = (int)((sc[c >> 1] >> (16 * (c & 1) + 8)) & 0xffu);
        // v_perm_b32 replicates one byte of the unpacked mins into all four bytes of the operand
        const uint32_t m_lo = __builtin_amdgcn_perm(0u, mn[c >> 1], 0x01010101u * (uint32_t)(2 * (c & 1)));
        const uint32_t m_hi = __builtin_amdgcn_perm(0u, mn[c >> 1], 0x01010101u * (uint32_t)(2 * (c & 1) + 1));
        const v4i b_min = {(int)m_lo, (int)m_lo, (int)m_hi, (int)m_hi};
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
            const v4u av = a.q[tt][c];
            const v4i zero = {0, 0, 0, 0};
            const v4i p_lo = __builtin_amdgcn_mfma_i32_16x16x32_i8(pack64(av.x, av.y), b_lo, zero, 0, 0, 0);
            const v4i p_hi = __builtin_amdgcn_mfma_i32_16x16x32_i8(pack64(av.z, av.w), b_hi, zero, 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 4; ++i) dot[tt][i] += __mul24(p_lo[i], s_lo) + __mul24(p_hi[i], s_hi);
            const v4i a16 = {(int)av.x, (int)av.y, (int)av.z, (int)av.w};
            mnd[tt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a16, b_min, mnd[tt], 0, 0, 0);
        }
    }
    const float wd = half_bits_to_float(t.hdr.x & 0xffffu);
    const float wm = half_bits_to_float(t.hdr.x >> 16);
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float d = __fmul_rn(wd, a.yd[tt][i]);
            const float dm = __fmul_rn(wm, a.yd[tt][i]);
            const float term = __fsub_rn(__fmul_rn(d, (float)dot[tt][i]), __fmul_rn(dm, (float)mnd[tt][i]));
            acc[tt][i] = __fadd_rn(acc[tt][i], term);
            dot_out[tt][i] = dot[tt][i];
            min_out[tt][i] = mnd[tt][i];
        }
    }
}

// One workgroup: row tile blockIdx.x of group blockIdx.y (dense mode has a single group).
template <int NMAT, int TT, bool GROUPED, bool DEBUG>
__global__ void __launch_bounds__(512) matmul_kernel(const MatmulArgs p) {
    extern __shared__ float red[];  // [W][NMAT][TT][4][64]
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int n_waves = blockDim.x >> 6;
    const int slot = lane & 15;  // activation row within a token tile (A side), weight row (B side)
    const int kq = lane >> 4;
    const int64_t rt = blockIdx.x;
    const int64_t nb = p.nb;

    // ---- which activation rows does this workgroup see, and which weights ----
    const uint8_t* w[2] = {p.w0, p.w1};
    int count = (int)p.n;     // activation rows in this group
    int begin = 0;            // first entry (grouped mode)
    bool shared_group = false;
    int silu_mode = p.silu_mode;
    if (GROUPED) {
        const int ng = *p.n_groups;
        const int g = blockIdx.y;
        if (g < ng) {
            const size_t eoff = (size_t)p.group_expert[g] * p.expert_bytes;
            w[0] += eoff;
            if (NMAT == 2) w[1] += eoff;
            begin = p.group_begin[g];
            count = p.group_begin[g + 1] - begin;
        } else if (g == ng && p.sh_tokens > 0) {
            shared_group = true;
            w[0] = p.sh_w0;
            w[1] = p.sh_w1;
            count = p.sh_tokens;
            silu_mode = p.sh_silu_mode;
        } else {
            return;  // whole workgroup leaves together, before any barrier
        }
    }
    const uint8_t* tiles[NMAT];
#pragma unroll
    for (int m = 0; m < NMAT; ++m) tiles[m] = w[m] + tile_offset(rt, 0, nb);

    for (int chunk = 0; chunk < count; chunk += 16 * TT) {
        // activation-row / output-row indices of this lane's A slot and of its four D slots
        int arow[TT], drow[TT][4], yrow[TT][4];
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
            auto map = [&](int s, int& ar, int& yr) {
                const int e_raw = chunk + 16 * tt + s;
                const bool live = e_raw < count;
                const int e = live ? e_raw : count - 1;  // dead slot: read a live row, store nothing
                if (!GROUPED) {
                    ar = e;
                    yr = e;
                } else if (shared_group) {
                    ar = e * p.sh_arow_stride + p.sh_arow_offset;
                    yr = e * p.sh_yrow_stride + p.sh_yrow_offset;
                } else {
                    const int tok = p.entry_token[begin + e], kk = p.entry_k[begin + e];
                    ar = tok * p.a_tok_stride + kk * p.a_k_stride;
                    yr = tok * p.y_tok_stride + kk * p.y_k_stride;
                }
                if (!live) yr = -1;
            };
            int unused;
            map(slot, arow[tt], unused);
#pragma unroll
            for (int i = 0; i < 4; ++i) map(4 * kq + i, drow[tt][i], yrow[tt][i]);
        }

        float acc[NMAT][TT][4];
#pragma unroll
        for (int m = 0; m < NMAT; ++m)
#pragma unroll
            for (int tt = 0; tt < TT; ++tt)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[m][tt][i] = 0.0f;

        // Two register stages, ping-pong: while one tile's MFMAs run, the next tile's loads are in
        // flight.  The steady-state loop has no conditionals, so every wait counts exactly the
        // loads issued after the data it needs.
        if (wave < nb) {
            const int64_t cnt = (nb - wave + n_waves - 1) / n_waves;  // super-blocks of this wave
            TileRegs t0[NMAT], t1[NMAT];
            ARegs<TT> a0, a1;
            auto issue = [&](TileRegs(&t)[NMAT], ARegs<TT>& a, int64_t i) {
                const int64_t b = wave + i * n_waves;
#pragma unroll
                for (int m = 0; m < NMAT; ++m) load_tile(t[m], tiles[m] + (size_t)b * kTileBytes, lane);
                load_a<TT>(a, p.aq, p.ad, arow, drow, b, nb, kq);
            };
            auto consume = [&](const TileRegs(&t)[NMAT], const ARegs<TT>& a, int64_t i) {
                const int64_t b = wave + i * n_waves;
#pragma unroll
                for (int m = 0; m < NMAT; ++m) {
                    int32_t dsum[TT][4], msum[TT][4];
                    compute_tile<TT>(t[m], a, acc[m], dsum, msum);
                    if (DEBUG && p.dbg_dot) {
                        const int64_t row = rt * 16 + slot;
#pragma unroll
                        for (int tt = 0; tt < TT; ++tt)
#pragma unroll
                            for (int i2 = 0; i2 < 4; ++i2) {
                                if (yrow[tt][i2] >= 0 && row < p.rows) {
                                    const size_t idx = ((size_t)row * (size_t)p.n + (size_t)yrow[tt][i2]) * nb + b;
                                    p.dbg_dot[idx] = dsum[tt][i2];
                                    p.dbg_min[idx] = msum[tt][i2];
                                }
                            }
                    }
                }
            };
            issue(t0, a0, 0);
            int64_t i = 0;
            while (i + 2 < cnt) {
                issue(t1, a1, i + 1);
                consume(t0, a0, i);
                issue(t0, a0, i + 2);
                consume(t1, a1, i + 1);
                i += 2;
            }
            if (cnt - i == 2) {
                issue(t1, a1, i + 1);
                consume(t0, a0, i);
                consume(t1, a1, i + 1);
            } else {
                consume(t0, a0, i);
            }
        }

        // ---- cross-wave reduction in wave order, then the epilogue on wave 0 ----
        if (n_waves > 1) {
            if (wave > 0) {
#pragma unroll
                for (int m = 0; m < NMAT; ++m)
#pragma unroll
                    for (int tt = 0; tt < TT; ++tt)
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            red[((((wave - 1) * NMAT + m) * TT + tt) * 4 + i) * 64 + lane] = acc[m][tt][i];
            }
            __syncthreads();
        }
        if (wave == 0) {
            for (int wv = 1; wv < n_waves; ++wv) {
#pragma unroll
                for (int m = 0; m < NMAT; ++m)
#pragma unroll
                    for (int tt = 0; tt < TT; ++tt)
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            acc[m][tt][i] =
                                __fadd_rn(acc[m][tt][i], red[((((wv - 1) * NMAT + m) * TT + tt) * 4 + i) * 64 + lane]);
            }
            const int64_t row = rt * 16 + slot;
            if (row < p.rows) {
#pragma unroll
                for (int tt = 0; tt < TT; ++tt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        if (yrow[tt][i] >= 0) {
                            float v = acc[0][tt][i];
                            if (NMAT == 2) v = silu_mul(v, acc[1][tt][i], silu_mode);
                            p.y[(size_t)yrow[tt][i] * (size_t)p.ldy + (size_t)row] = v;
                        }
                    }
            }
        }
        if (n_waves > 1 && chunk + 16 * TT < count) __syncthreads();  // red[] is reused by the next chunk
    }
}

int pick_waves(int64_t nb, int64_t workgroups) {
    // Aim at ~4 waves per SIMD over the whole chip (256 CUs x 4 SIMDs), with waves that divide
    // the super-blocks of a row evenly where possible.
    const int64_t target = 4096;
    int64_t ideal = (target + workgroups - 1) / (workgroups > 0 ? workgroups : 1);
    if (ideal < 1) ideal = 1;
    if (ideal > 8) ideal = 8;
    if (ideal > nb) ideal = nb;
    for (int64_t w = ideal; w >= 1; --w) {
        if (nb % w == 0) return (int)w;
    }
    return 1;
}

template <int NMAT, int TT, bool GROUPED, bool DEBUG>
hipError_t launch_one(const MatmulArgs& a, int waves, dim3 grid, hipStream_t stream) {
    const size_t lds = waves > 1 ? (size_t)(waves - 1) * NMAT * TT * 4 * 64 * sizeof(float) : 0;
    hipLaunchKernelGGL((matmul_kernel<NMAT, TT, GROUPED, DEBUG>), grid, dim3(64 * waves), lds, stream, a);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_matmul(const MatmulArgs& a, hipStream_t stream) {
    if (a.rows <= 0 || a.nb <= 0) return hipErrorInvalidValue;
    const int64_t rowtiles = (a.rows + 15) / 16;
    const int nmat = a.swiglu ? 2 : 1;
    const bool debug = a.dbg_dot != nullptr;
    // widest activation group this launch can see decides the token-tile count
    const int64_t widest = a.grouped ? (a.n > a.sh_tokens ? a.n : a.sh_tokens) : a.n;
    const int tt = widest <= 16 ? 1 : (widest <= 32 ? 2 : 4);
    const int groups = a.grouped ? a.max_groups + (a.sh_tokens > 0 ? 1 : 0) : 1;
    // expected live groups: at most one per routed (token, k) pair
    int64_t live = a.grouped ? groups : 1;
    int waves = pick_waves(a.nb, rowtiles * live);
    if (const char* ev = getenv("MQ_WAVES")) waves = atoi(ev) > 0 ? atoi(ev) : waves;  // tuning knob
    while (waves > 1 && ((size_t)(waves - 1) * nmat * tt * 1024 > 64 * 1024 || a.nb % waves != 0)) --waves;
    const dim3 grid((unsigned)rowtiles, (unsigned)groups);

#define MQ_LAUNCH(NM, T)                                                              \
    do {                                                                              \
        if (a.grouped) return launch_one<NM, T, true, false>(a, waves, grid, stream); \
        if (debug) return launch_one<NM, T, false, true>(a, waves, grid, stream);     \
        return launch_one<NM, T, false, false>(a, waves, grid, stream);               \
    } while (0)

    if (nmat == 1) {
        if (tt == 1) MQ_LAUNCH(1, 1);
        if (tt == 2) MQ_LAUNCH(1, 2);
        MQ_LAUNCH(1, 4);
    } else {
        if (tt == 1) MQ_LAUNCH(2, 1);
        if (tt == 2) MQ_LAUNCH(2, 2);
        MQ_LAUNCH(2, 4);
    }
#undef MQ_LAUNCH
    return hipSuccess;
}

}  // namespace mq
