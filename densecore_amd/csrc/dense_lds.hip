// Dense Q4_K / Q5_K / Q6_K x Q8_K product for decode widths with the activations staged once per workgroup in LDS.
//
// matmul_kernel (matmul.hip) asks for its activation operand from global memory at every stage: six loads per
// stage and wavefront beside the three per weight tile, all answered by the L2 (every workgroup re-reads the whole
// quantized activation set).  Here a workgroup of eight wavefronts owns 8 / WPR consecutive row tiles, WPR
// wavefronts per row tile splitting the super-blocks exactly as matmul_kernel's do (wave h of a row tile takes
// super-blocks h, h + WPR, ...; partial sums meet in wave order), so the result has the same bits; but the
// quantized activations of all rows and super-blocks are brought into LDS once per workgroup while the first weight
// tiles travel, and every stage reads its operand from there:
//   * from the A-major workspace (the stand-alone quantizer ran before): 1 KB LDS-direct copies, no registers;
//   * XF: from the fp32 rows themselves -- the workgroup runs the block quantizer of quantize_q8k_kernel
//     (q8k_block.h: the same codes and scales) on all n x nb blocks, its eight wavefronts taking them in turn, and
//     writes the split-slot operand into LDS: no quantizer launch at all.  The fp32 rows are requested BEFORE the
//     weight tiles (loads return in order), the quantization then runs while the tiles travel.
// The weight stream is matmul_kernel's: three coalesced 16-byte-per-lane loads per 2304-byte tile, two register stages,
// no request past a wavefront's last super-block.
// cb_gemv_custom / cb_gemv_batched_custom quantize once and multiply on every thread
// (core/src/llm/matmul/gemv_exec.cpp:298-341, core/src/llm/matmul/batched_exec.cpp:1364-1444).
#include <hip/hip_ext.h>

#include "common.h"
#include "kernels.h"
#include "decode_tile.h"
#include "q8k_block.h"

namespace mq {

namespace {

typedef __attribute__((address_space(3))) void* lds_ptr_t;

template <int WT> constexpr int loads_per_tile() { return WT == kWtQ6 ? 5 : WT == kWtQ5 ? 4 : 3; }

// LDS: [TT][nb][4096] codes in the A-major split-slot order of common.h, [TT][nb][8] scales (padded to whole
// 256-byte chunks), then the partial sums of the wavefronts that do not store: [8 / WPR][WPR - 1][NMAT][TT][2][64].
// nb % WPR == 0 (host-checked): every wavefront has nb / WPR stages; ODD: that count is odd.
template <int NMAT, int TT, int WT, int J, int WPR, bool XF, bool ODD>
__global__ void __launch_bounds__(512) dense_lds_kernel(const DenseLdsArgs p) {
    constexpr int kTileStride = tile_stride<WT>();
    constexpr int RPW = 8 / WPR;  // row tiles per workgroup
    extern __shared__ __align__(16) uint8_t lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int slot = lane & 15, kq = lane >> 4;
    const int nb = (int)p.nb;
    const int64_t rowtiles = (p.rows + 15) >> 4;
    const int pair = wave / WPR, h = wave % WPR;
    int64_t rt = (int64_t)blockIdx.x * RPW + pair;
    const bool dead = rt >= rowtiles;  // a workgroup past the last row tile streams the last one again and stores nothing
    if (dead) rt = rowtiles - 1;

    uint8_t* a_lds = lds;
    const int d_floats = (TT * nb * 8 + 63) & ~63;
    float* d_lds = reinterpret_cast<float*>(lds + (size_t)TT * nb * 4096);
    float* red = d_lds + d_floats;

    const uint8_t* tiles[NMAT];
    tiles[0] = p.w0 + tile_offset(rt, 0, nb, kTileStride);
    if (NMAT == 2) tiles[1] = p.w1 + tile_offset(rt, 0, nb, kTileStride);
    const int cnt = nb / WPR;  // stages of this wavefront: super-blocks h, h + WPR, ...

    // ---- XF: request the fp32 rows first (they return before the weight tiles requested after them) ----
    // Item m * nb + b = super-block b of row m; wavefront w takes the items w, w + 8, ...: at most 64 items in all
    // (host-checked), eight per wavefront, so the whole phase is straight-line code whose waits count exactly.
    constexpr int kXBatch = 8;
    const int items = XF ? (int)p.n * nb : 0;
    float4 xv[XF ? kXBatch : 1];
    auto item_row = [&](int it) { return (it >= nb) + (it >= 2 * nb) + (it >= 3 * nb); };  // n <= 4
    if constexpr (XF) {
#pragma unroll
        for (int u = 0; u < kXBatch; ++u) {
            const int it = wave + 8 * u < items ? wave + 8 * u : 0;
            const int m = item_row(it), b = it - m * nb;
            xv[u] = *reinterpret_cast<const float4*>(p.xf + (size_t)m * p.ldx + (size_t)b * kQK + lane * 4);
        }
        asm volatile("" ::: "memory");  // these requests stay ahead of the tile requests
    } else {
        // ---- A-major workspace -> LDS: 1 KB chunks round the wavefronts, then the scales ----
        const uint32_t base = (uint32_t)(uintptr_t)(lds_ptr_t)a_lds;
        const int chunks = TT * nb * 4;
        for (int c = wave; c < chunks; c += 8) {
            const uint8_t* g = p.aq + (size_t)c * 1024 + lane * 16;
            const uint32_t dst = base + (uint32_t)c * 1024u;
            asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(g), "s"(dst) : "memory", "m0");
        }
        const uint32_t dbase = (uint32_t)(uintptr_t)(lds_ptr_t)d_lds;
        const int dchunks = d_floats / 64, d_live = TT * nb * 8;
        for (int c = wave; c < dchunks; c += 8) {
            const float* g = p.ad + (c * 64 + lane < d_live ? c * 64 + lane : 0);  // nothing is read past the workspace
            const uint32_t dst = dbase + (uint32_t)c * 256u;
            asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" : : "v"(g), "s"(dst) : "memory", "m0");
        }
    }

    typename TileOf<WT>::Regs ring_t[2][NMAT];
    auto issue = [&](auto st_c, int i) {  // only ever called for a stage that exists
        constexpr int st = decltype(st_c)::value;
        const int b = h + i * WPR;
#pragma unroll
        for (int m = 0; m < NMAT; ++m) load_tile_wt<WT>(ring_t[st][m], tiles[m] + (size_t)b * kTileStride, lane);
    };

    float acc[NMAT][TT][2];
#pragma unroll
    for (int m = 0; m < NMAT; ++m)
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) acc[m][tt][0] = acc[m][tt][1] = 0.0f;

    // operand of this lane: slot (activation row slot / 2, half slot % 2) of k-group kq; rows past n read row n - 1
    int a_lane_off[TT], d_off[TT][2];
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
        const int live = (int)p.n - 8 * tt < 8 ? (int)p.n - 8 * tt : 8;  // rows of this token tile (>= 1)
        const int r = (slot >> 1) < live ? (slot >> 1) : live - 1;
        a_lane_off[tt] = tt * nb * 4096 + kq * 256 + (2 * r + (slot & 1)) * 16;
#pragma unroll
        for (int j = 0; j < 2; ++j) d_off[tt][j] = tt * nb * 8 + ((2 * kq + j) < live ? 2 * kq + j : live - 1);
    }
    auto consume = [&](auto st_c, int i) {
        constexpr int st = decltype(st_c)::value;
        const int b = h + i * WPR;
        ARegs<TT> a;
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
#pragma unroll
            for (int c = 0; c < 4; ++c) a.q[tt][c] = *reinterpret_cast<const v4u*>(a_lds + (size_t)b * 4096 + c * 1024 + a_lane_off[tt]);
#pragma unroll
            for (int j = 0; j < 2; ++j) a.yd[tt][j] = d_lds[b * 8 + d_off[tt][j]];
        }
#pragma unroll
        for (int m = 0; m < NMAT; ++m) {
            int32_t dsum[TT][2], msum[TT][2];
            compute_tile_wt<TT, WT, J>(ring_t[st][m], a, acc[m], dsum, msum, lane);
        }
    };

    // Two register stages, one in flight while the other is multiplied.  The loop is written out for an even and for
    // an odd number of stages (an odd run is one stage followed by an even run with the stages' roles swapped), so
    // that every path has a fixed sequence of requests -- the waits count exactly -- and no request is ever made for
    // a stage that does not exist.
    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;
    const bool single = ODD && cnt == 1;  // wave-uniform
    issue(S0{}, 0);
    asm volatile("" ::: "memory");  // requests stay in stage order
    if (!single) {
        issue(S1{}, 1);
        asm volatile("" ::: "memory");
    }
    // ---- the activations are in LDS before anyone multiplies ----
    if constexpr (XF) {
#pragma unroll
        for (int u = 0; u < kXBatch; ++u) {
            const int it = wave + 8 * u;
            if (it < items) {  // wave-uniform
                const int m = item_row(it), b = it - m * nb;
                const float e[4] = {xv[u].x, xv[u].y, xv[u].z, xv[u].w};
                const Q8Lane r = quantize_block_q8k(e, lane);
                // as store_amajor (q8k_block.h), into LDS
                const int g = lane >> 3, hh = g & 1, kk = (lane & 7) >> 1;
                uint8_t* dst = a_lds + (size_t)b * 4096 + ((g >> 1) * 4 + kk) * 256 + (2 * m + hh) * 16 + (lane & 1) * 4;
                *reinterpret_cast<uint32_t*>(dst + hh * 8) = r.packed;
                *reinterpret_cast<uint32_t*>(dst + (1 - hh) * 8) = 0u;
                if (lane == 0) d_lds[b * 8 + m] = r.d;
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    } else {
        // the LDS-direct copies are older than the tile requests: they have landed once at most those are outstanding
        if (single) asm volatile("s_waitcnt vmcnt(%0)" : : "n"(NMAT * loads_per_tile<WT>()) : "memory");
        else asm volatile("s_waitcnt vmcnt(%0)" : : "n"(2 * NMAT * loads_per_tile<WT>()) : "memory");
    }
    __builtin_amdgcn_s_barrier();  // no fence here: a fence would wait for the outstanding weight tiles as well
    asm volatile("" ::: "memory");

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
        int i = 0;
        for (; i + 2 < cnt; i += 2) {
            consume(S0{}, i);
            issue(S0{}, i + 2);
            asm volatile("" ::: "memory");
            consume(S1{}, i + 1);
            issue(S1{}, i + 3);
            asm volatile("" ::: "memory");
        }
        consume(S0{}, i);
        consume(S1{}, i + 1);
    }

    // ---- the WPR wavefronts of a row tile meet in wave order; the first one stores ----
    if (WPR > 1) {
        if (h > 0) {
#pragma unroll
            for (int m = 0; m < NMAT; ++m)
#pragma unroll
                for (int tt = 0; tt < TT; ++tt)
#pragma unroll
                    for (int j = 0; j < J; ++j)
                        red[(((((pair * (WPR - 1) + (h - 1)) * NMAT + m) * TT + tt) * 2 + j) * 64) + lane] = acc[m][tt][j];
        }
        __syncthreads();
    }
    if (h == 0 && !dead) {
        for (int wv = 1; wv < WPR; ++wv) {
#pragma unroll
            for (int m = 0; m < NMAT; ++m)
#pragma unroll
                for (int tt = 0; tt < TT; ++tt)
#pragma unroll
                    for (int j = 0; j < J; ++j)
                        acc[m][tt][j] = __fadd_rn(acc[m][tt][j], red[(((((pair * (WPR - 1) + (wv - 1)) * NMAT + m) * TT + tt) * 2 + j) * 64) + lane]);
        }
        const int64_t row = rt * 16 + slot;
        if (row < p.rows) {
#pragma unroll
            for (int tt = 0; tt < TT; ++tt)
#pragma unroll
                for (int j = 0; j < J; ++j) {
                    const int tok = 8 * tt + 2 * kq + j;
                    if (tok < p.n) {
                        float v = acc[0][tt][j];
                        if (NMAT == 2) v = silu_mul(v, acc[NMAT - 1][tt][j], p.silu_mode);
                        p.y[(size_t)tok * (size_t)p.ldy + (size_t)row] = v;
                    }
                }
        }
    }
}

size_t lds_bytes(int nmat, int tt, int wpr, int64_t nb) {
    const size_t d_floats = (size_t)((tt * nb * 8 + 63) & ~63);
    return (size_t)tt * nb * 4096 + d_floats * 4 + (size_t)(8 / wpr) * (wpr - 1) * nmat * tt * 2 * 64 * 4;
}

template <int NMAT, int TT, int WT, int J, int WPR, bool XF, bool ODD>
hipError_t launch_odd(const DenseLdsArgs& a, hipStream_t stream, hipEvent_t start, hipEvent_t stop) {
    const int64_t rowtiles = (a.rows + 15) / 16;
    const size_t lds = lds_bytes(NMAT, TT, WPR, a.nb);
    auto* kernel = &dense_lds_kernel<NMAT, TT, WT, J, WPR, XF, ODD>;
    static bool raised = false;  // per instantiation; the attribute belongs to the function, not to a launch
    if (!raised) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
        raised = true;
    }
    constexpr int RPW = 8 / WPR;
    const dim3 grid((unsigned)((rowtiles + RPW - 1) / RPW));
    if (start && stop) hipExtLaunchKernelGGL(kernel, grid, dim3(512), lds, stream, start, stop, 0, a);
    else MQ_LAUNCH(kernel, grid, dim3(512), lds, stream, a);
    return hipGetLastError();
}

template <int NMAT, int TT, int WT, int J, int WPR, bool XF>
hipError_t launch_one(const DenseLdsArgs& a, hipStream_t stream, hipEvent_t start, hipEvent_t stop) {
    if ((a.nb / WPR) & 1) return launch_odd<NMAT, TT, WT, J, WPR, XF, true>(a, stream, start, stop);
    return launch_odd<NMAT, TT, WT, J, WPR, XF, false>(a, stream, start, stop);
}

template <int NMAT, int TT, int WT, int J, bool XF>
hipError_t launch_wpr(const DenseLdsArgs& a, int wpr, hipStream_t stream, hipEvent_t start, hipEvent_t stop) {
    switch (wpr) {
        case 1: return launch_one<NMAT, TT, WT, J, 1, XF>(a, stream, start, stop);
        case 2: return launch_one<NMAT, TT, WT, J, 2, XF>(a, stream, start, stop);
        case 4: return launch_one<NMAT, TT, WT, J, 4, XF>(a, stream, start, stop);
        case 8: return launch_one<NMAT, TT, WT, J, 8, XF>(a, stream, start, stop);
    }
    return hipErrorInvalidValue;
}

template <int NMAT, int WT>
hipError_t launch_shape(const DenseLdsArgs& a, int wpr, hipStream_t stream, hipEvent_t start, hipEvent_t stop) {
    if (a.n > 8) {
        if constexpr (WT == kWtQ4) {
            if (!a.xf) return launch_wpr<NMAT, 2, WT, 2, false>(a, wpr, stream, start, stop);
        }
        return hipErrorInvalidValue;
    }
    if (a.xf) {
        if (a.n == 1) return launch_wpr<NMAT, 1, WT, 1, true>(a, wpr, stream, start, stop);
        return launch_wpr<NMAT, 1, WT, 2, true>(a, wpr, stream, start, stop);
    }
    if (a.n == 1) return launch_wpr<NMAT, 1, WT, 1, false>(a, wpr, stream, start, stop);
    return launch_wpr<NMAT, 1, WT, 2, false>(a, wpr, stream, start, stop);
}

}  // namespace

// Wavefronts per row tile: what pick_waves gives matmul_kernel for the same matrix (so both kernels add a row's
// super-blocks in the same order), as a divisor of eight.
int dense_lds_wpr(int64_t nb, int64_t rowtiles) {
    const int w = pick_waves(nb, rowtiles);
    return (w == 1 || w == 2 || w == 4 || w == 8) ? w : 0;
}

bool dense_lds_applies(int64_t nb, int64_t rowtiles, int64_t n, bool swiglu, int wtype) {
    if (n < 1 || n > 16) return false;
    if (n > 8 && wtype != kTypeQ4K) return false;  // two token tiles of Q5_K / Q6_K do not fit the register file
    const int wpr = dense_lds_wpr(nb, rowtiles);
    if (!wpr || nb % wpr) return false;
    return lds_bytes(swiglu ? 2 : 1, n > 8 ? 2 : 1, wpr, nb) <= 160 * 1024;
}

hipError_t launch_dense_lds(const DenseLdsArgs& a, hipStream_t stream, hipEvent_t start, hipEvent_t stop) {
    if (a.rows <= 0 || a.nb <= 0 || a.n < 1 || a.n > 16 || !a.y || !a.w0) return hipErrorInvalidValue;
    const int64_t rowtiles = (a.rows + 15) / 16;
    if (!dense_lds_applies(a.nb, rowtiles, a.n, a.w1 != nullptr, a.wtype)) return hipErrorInvalidValue;
    if (a.xf ? ((reinterpret_cast<uintptr_t>(a.xf) & 15u) || (a.ldx & 3) || a.n > 4 || a.n * a.nb > 64) : (!a.aq || !a.ad)) return hipErrorInvalidValue;
    const int wpr = dense_lds_wpr(a.nb, rowtiles);
#define MQ_DL(NM)                                                                               \
    do {                                                                                        \
        if (a.wtype == kTypeQ6K) return launch_shape<NM, kWtQ6>(a, wpr, stream, start, stop);  \
        if (a.wtype == kTypeQ5K) return launch_shape<NM, kWtQ5>(a, wpr, stream, start, stop);  \
        if (a.wtype == kTypeQ4K) return launch_shape<NM, kWtQ4>(a, wpr, stream, start, stop);  \
        return hipErrorInvalidValue;                                                            \
    } while (0)
    if (a.w1) MQ_DL(2);
    MQ_DL(1);
#undef MQ_DL
}

}  // namespace mq
