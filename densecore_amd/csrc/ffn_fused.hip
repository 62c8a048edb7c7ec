// Dense SwiGLU FFN at decode width (n <= 8 rows) as ONE persistent launch on gfx950:
//     y = W_down . q8k( silu(W_gate . q8k(x)) * (W_up . q8k(x)) )
//
// Node by node this is four dependent launches (quantize, fused gate/up, quantize, down: the three
// smart_mul_mat calls plus cb_silu_mul_fused of core/src/llm/graph/decoder.cpp:2662-2730), and at these
// widths a third of the time is launch, ramp-up and drain.  Here one workgroup per compute unit stays resident
// and every wavefront runs ONE ring of weight-tile requests through both projections:
//
//   start     every workgroup quantizes x into its own LDS (compact codes, see load_a_compact) while its
//             first tiles travel
//   phase 1   gate/up row tiles spread over the workgroups; h = silu(gate) * up leaves with device-scope stores
//   barrier   device-wide (grid_sync.h).  The ring keeps requesting across it: the first down-projection tiles
//             of every wavefront are on their way or already in registers while the workgroups meet.
//   restage   every workgroup re-quantizes the rows of h into its LDS (device-scope loads)
//   phase 2   down row tiles spread over the workgroups; plain stores of y
//
// Arithmetic and summation order are those of the one-node kernels: a row tile is split over as many
// wavefronts as launch_matmul would give it (pick_waves), each of which adds its super-blocks in ascending
// order; the partial sums meet in wave order.  A workgroup of eight wavefronts therefore works on 8 / W row
// tiles at a time.  The result equals quantize + matmul + quantize + matmul bit for bit.
#include <hip/hip_ext.h>

#include "common.h"
#include "kernels.h"
#include "decode_tile.h"
#include "grid_sync.h"
#include "q8k_block.h"

namespace mq {

namespace {

constexpr int kWaves = 8;
constexpr int kThreads = kWaves * 64;
constexpr int kBatch = 8;  // super-blocks a wavefront has in flight while it quantizes rows into LDS

__device__ __forceinline__ void ld_dev4(float (&e)[4], const float* p) {
    const uint64_t lo = __hip_atomic_load(reinterpret_cast<const uint64_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const uint64_t hi = __hip_atomic_load(reinterpret_cast<const uint64_t*>(p) + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    e[0] = __uint_as_float((uint32_t)lo);
    e[1] = __uint_as_float((uint32_t)(lo >> 32));
    e[2] = __uint_as_float((uint32_t)hi);
    e[3] = __uint_as_float((uint32_t)(hi >> 32));
}

// Compact Q8_K codes in LDS: block (row t, super-block b) is 256 bytes at (t * nb + b) * 256, code e at byte
// ((e / 64) ^ (t & 3)) * 64 + e % 64 -- the 64-byte chunks of a block are permuted by the row so that the eight
// rows an MFMA reads side by side fall on different banks.  Scales: scales[t * nb + b].
struct LaneA {
    int row_off;  // t * nb * 256 + 32 h + 8 kq for this lane's M slot (row t = slot / 2, half h = slot % 2)
    int swz;      // t & 3
    uint32_t keep_lo, keep_hi;
    int d0, d1;   // scale rows of the two accumulators: min(2 kq + j, n - 1) * nb
};
__device__ __forceinline__ LaneA lane_a(int lane, int n, int nb) {
    const int slot = lane & 15, kq = lane >> 4;
    const int t = (slot >> 1) < n ? (slot >> 1) : n - 1;  // a dead slot reads the last live row; never stored
    const int h = slot & 1;
    LaneA la;
    la.row_off = t * nb * 256 + 32 * h + 8 * kq;
    la.swz = t & 3;
    la.keep_lo = h ? 0u : 0xffffffffu;
    la.keep_hi = ~la.keep_lo;
    la.d0 = (2 * kq < n ? 2 * kq : n - 1) * nb;
    la.d1 = (2 * kq + 1 < n ? 2 * kq + 1 : n - 1) * nb;
    return la;
}
// The split-slot A operand of super-block b (common.h): slot 2t = {codes of the even sub-block, 0 x 8},
// slot 2t+1 = {0 x 8, codes of the odd sub-block}.
__device__ __forceinline__ void load_a_compact(ARegs<1>& a, const uint8_t* codes, const float* scales, const LaneA& la, int b) {
    const uint8_t* base = codes + la.row_off + b * 256;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const v2u v = *reinterpret_cast<const v2u*>(base + ((c ^ la.swz) << 6));
        a.q[0][c] = v4u{v.x & la.keep_lo, v.y & la.keep_lo, v.x & la.keep_hi, v.y & la.keep_hi};
    }
    a.yd[0][0] = scales[la.d0 + b];
    a.yd[0][1] = scales[la.d1 + b];
}

// Q8_K of n rows x nb super-blocks of src (row stride ld) into the compact LDS layout, one wavefront per block,
// kBatch blocks of loads in flight per wavefront.  kCoherent: other workgroups wrote src during this launch.
template <bool kCoherent>
__device__ __forceinline__ void stage_rows(uint8_t* codes, float* scales, const float* src, int64_t ld, int n, int nb) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int blocks = n * nb;
    for (int base = wave; base < blocks; base += kWaves * kBatch) {
        float e[kBatch][4];
#pragma unroll
        for (int jj = 0; jj < kBatch; ++jj) {
            const int blk = base + kWaves * jj < blocks ? base + kWaves * jj : base;
            const int t = blk / nb, b = blk - t * nb;
            const float* at = src + (size_t)t * ld + (size_t)b * kQK + lane * 4;
            if (kCoherent) {
                ld_dev4(e[jj], at);
            } else {
                const float4 v = *reinterpret_cast<const float4*>(at);
                e[jj][0] = v.x, e[jj][1] = v.y, e[jj][2] = v.z, e[jj][3] = v.w;
            }
        }
#pragma unroll
        for (int jj = 0; jj < kBatch; ++jj) {
            const int blk = base + kWaves * jj;
            if (blk < blocks) {  // wave-uniform
                const int t = blk / nb, b = blk - t * nb;
                const Q8Lane r = quantize_block_q8k(e[jj], lane);
                *reinterpret_cast<uint32_t*>(codes + (size_t)blk * 256 + ((((lane >> 4) ^ (t & 3)) << 6) | ((lane & 15) << 2))) = r.packed;
                if (lane == 0) scales[blk] = r.d;
                (void)b;
            }
        }
    }
}

// How one projection is spread: W wavefronts per row tile, R = 8 / W row tiles per workgroup pass ("unit"),
// unit u of workgroup c covers row tiles ((c + u G) R .. +R-1).
struct Split {
    int w, r, grp, wv, per, tiles, units_mine;
    bool active;
};
__device__ __forceinline__ Split make_split(int waves_per_tile, int nb, int row_tiles, int wave) {
    Split s;
    s.w = waves_per_tile;
    s.r = kWaves / s.w;
    s.grp = wave / s.w;
    s.wv = wave - s.grp * s.w;
    s.active = s.grp < s.r;
    s.per = nb / s.w;
    s.tiles = row_tiles;
    const int units = (row_tiles + s.r - 1) / s.r;
    const int c = blockIdx.x, g = gridDim.x;
    s.units_mine = c < units ? (units - c + g - 1) / g : 0;
    return s;
}

template <int S>
__global__ void __launch_bounds__(kThreads) ffn_fused_kernel(const FfnFusedArgs p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int slot = lane & 15, kq = lane >> 4;
    const int n = p.n, nb_h = p.hidden / kQK, nb_i = p.inter / kQK;
    const int nb_max = nb_h > nb_i ? nb_h : nb_i;
    uint8_t* codes = lds_raw;
    float* scales = reinterpret_cast<float*>(lds_raw + (size_t)n * nb_max * 256);
    float* red = scales + n * nb_max;  // [2][kWaves][2][2][64]
    int* ok = reinterpret_cast<int*>(red + 2 * kWaves * 4 * 64);

    if (ld_dev(p.sync + 2 * kSyncLine) != 0u) return;  // an earlier launch abandoned a barrier: the state is unusable
    uint32_t my_gen = ld_dev(p.sync + kSyncLine);      // cannot move before this workgroup's own first arrival

    const int c = blockIdx.x, G = gridDim.x;
    const Split s1 = make_split(p.waves1, nb_h, p.inter / 16, wave);
    const Split s2 = make_split(p.waves2, nb_i, p.hidden / 16, wave);
    const int sp2 = (s2.per + 1) / 2;               // phase-2 stages per unit: two super-blocks each
    const int n1 = s1.units_mine * s1.per;          // phase-1 stages of every wavefront of this workgroup
    const int n1p = (n1 + S - 1) / S * S;           // padded so that phase 2 starts at ring slot 0
    const int total = n1p + s2.units_mine * sp2;

    // Ring of S stages of two weight tiles each (gate + up of one super-block, or two super-blocks of down).
    // Stage i lives in slot i % S.  Every request is issued whether or not the stage exists (a missing one
    // re-reads the first tile of the gate matrix), so that the waits can count.
    TileRegs ring[S][2];
    auto issue = [&](int st, int i) {
        const uint8_t* a0 = p.gate;
        const uint8_t* a1 = p.gate;
        if (i < n1) {
            const int u = i / s1.per, k = i - u * s1.per;
            const int rt = (c + u * G) * s1.r + s1.grp;
            if (s1.active && rt < s1.tiles) {
                const size_t off = tile_offset(rt, s1.wv + s1.w * k, nb_h);
                a0 = p.gate + off;
                a1 = p.up + off;
            }
        } else if (i >= n1p && i < total) {
            const int i2 = i - n1p;
            const int u = i2 / sp2, k = 2 * (i2 - u * sp2);
            const int rt = (c + u * G) * s2.r + s2.grp;
            if (s2.active && rt < s2.tiles) {
                a0 = p.down + tile_offset(rt, s2.wv + s2.w * k, nb_i);
                if (k + 1 < s2.per) a1 = p.down + tile_offset(rt, s2.wv + s2.w * (k + 1), nb_i);
            }
        }
        load_tile(ring[st][0], a0, lane);
        load_tile(ring[st][1], a1, lane);
    };
#pragma unroll
    for (int st = 0; st < S - 1; ++st) issue(st, st);

    stage_rows<false>(codes, scales, p.x, p.hidden, n, nb_h);
    __syncthreads();

    float acc[2][1][2] = {{{0.0f, 0.0f}}, {{0.0f, 0.0f}}};
    LaneA la = lane_a(lane, n, nb_h);

    // Partial sums of the W wavefronts of a row tile meet in wave order in the first of them (as in
    // matmul_kernel); red[] alternates between two halves so that a fast wavefront's next unit cannot overwrite
    // what a reducer still reads.
    auto reduce_unit = [&](const Split& s, int u, bool live, int nmat) {
        float* rb = red + (u & 1) * (kWaves * 4 * 64);
        if (s.w > 1) {
            if (live && s.wv > 0) {
                for (int m = 0; m < nmat; ++m)
#pragma unroll
                    for (int j = 0; j < 2; ++j) rb[((wave * 2 + m) * 2 + j) * 64 + lane] = acc[m][0][j];
            }
            __syncthreads();
            if (live && s.wv == 0) {
                for (int wv = 1; wv < s.w; ++wv)
                    for (int m = 0; m < nmat; ++m)
#pragma unroll
                        for (int j = 0; j < 2; ++j)
                            acc[m][0][j] = __fadd_rn(acc[m][0][j], rb[(((wave + wv) * 2 + m) * 2 + j) * 64 + lane]);
            }
        }
    };

    // ---- phase 1: gate/up + SwiGLU ------------------------------------------------------------------------
    for (int base = 0; base < n1p; base += S) {
#pragma unroll
        for (int st = 0; st < S; ++st) {
            const int i = base + st;
            issue((st + S - 1) % S, i + S - 1);
            if (i < n1) {
                const int u = i / s1.per, k = i - u * s1.per;
                const int rt = (c + u * G) * s1.r + s1.grp;
                const bool live = s1.active && rt < s1.tiles;
                if (k == 0) acc[0][0][0] = acc[0][0][1] = acc[1][0][0] = acc[1][0][1] = 0.0f;
                if (live) {
                    ARegs<1> a;
                    load_a_compact(a, codes, scales, la, s1.wv + s1.w * k);
                    int32_t dsum[1][2], msum[1][2];
                    compute_tile<1>(ring[st][0], a, acc[0], dsum, msum);
                    compute_tile<1>(ring[st][1], a, acc[1], dsum, msum);
                }
                if (k == s1.per - 1) {
                    reduce_unit(s1, u, live, 2);
                    if (live && s1.wv == 0) {
                        const int row = rt * 16 + slot;
#pragma unroll
                        for (int j = 0; j < 2; ++j)
                            if (2 * kq + j < n)
                                st_dev(p.h + (size_t)(2 * kq + j) * p.inter + row,
                                       silu_mul(acc[0][0][j], acc[1][0][j], p.silu_mode));
                    }
                }
            }
        }
    }

    // ---- barrier: h is complete device-wide -----------------------------------------------------------------
    // Only the wavefronts that stored wait for their stores; the others keep their tile requests in flight.
    if (s1.active && s1.wv == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (!grid_barrier<false>(p.sync, my_gen, ok, p.spin_ticks, [] {})) return;
    stage_rows<true>(codes, scales, p.h, p.inter, n, nb_i);
    __syncthreads();
    la = lane_a(lane, n, nb_i);

    // ---- phase 2: down ----------------------------------------------------------------------------------------
    for (int base = n1p; base < total; base += S) {
#pragma unroll
        for (int st = 0; st < S; ++st) {
            const int i = base + st;
            issue((st + S - 1) % S, i + S - 1);
            if (i < total) {
                const int i2 = i - n1p;
                const int u = i2 / sp2, q = i2 - u * sp2;
                const int rt = (c + u * G) * s2.r + s2.grp;
                const bool live = s2.active && rt < s2.tiles;
                if (q == 0) acc[0][0][0] = acc[0][0][1] = 0.0f;
                if (live) {
#pragma unroll
                    for (int half = 0; half < 2; ++half) {
                        const int k = 2 * q + half;
                        if (k < s2.per) {
                            ARegs<1> a;
                            load_a_compact(a, codes, scales, la, s2.wv + s2.w * k);
                            int32_t dsum[1][2], msum[1][2];
                            compute_tile<1>(ring[st][half], a, acc[0], dsum, msum);
                        }
                    }
                }
                if (q == sp2 - 1) {
                    reduce_unit(s2, u, live, 1);
                    if (live && s2.wv == 0) {
                        const int row = rt * 16 + slot;
#pragma unroll
                        for (int j = 0; j < 2; ++j)
                            if (2 * kq + j < n) p.y[(size_t)(2 * kq + j) * p.hidden + row] = acc[0][0][j];
                    }
                }
            }
        }
    }
}

constexpr int kRing = 4;

}  // namespace

size_t ffn_fused_lds_bytes(int n, int hidden, int inter) {
    const int nb = (hidden > inter ? hidden : inter) / kQK;
    return (size_t)n * nb * 256 + (size_t)n * nb * 4 + (size_t)2 * kWaves * 4 * 64 * 4 + 16;
}

hipError_t prepare_ffn_fused(size_t lds_bytes) {
    return hipFuncSetAttribute(reinterpret_cast<const void*>(ffn_fused_kernel<kRing>), hipFuncAttributeMaxDynamicSharedMemorySize,
                               (int)lds_bytes);
}

hipError_t launch_ffn_fused(const FfnFusedArgs& a, int n_workgroups, hipStream_t stream, hipEvent_t start, hipEvent_t stop) {
    const int nb_h = a.hidden / kQK, nb_i = a.inter / kQK;
    if (a.n < 1 || a.n > 8 || a.hidden <= 0 || (a.hidden % kQK) || a.inter <= 0 || (a.inter % kQK) || n_workgroups < 1 ||
        a.waves1 < 1 || a.waves1 > kWaves || (nb_h % a.waves1) || a.waves2 < 1 || a.waves2 > kWaves || (nb_i % a.waves2) ||
        !a.gate || !a.up || !a.down || !a.x || !a.h || !a.y || !a.sync)
        return hipErrorInvalidValue;
    const size_t lds = ffn_fused_lds_bytes(a.n, a.hidden, a.inter);
    if (start && stop) {
        hipExtLaunchKernelGGL((ffn_fused_kernel<kRing>), dim3((unsigned)n_workgroups), dim3(kThreads), lds, stream, start, stop, 0, a);
    } else {
        hipLaunchKernelGGL((ffn_fused_kernel<kRing>), dim3((unsigned)n_workgroups), dim3(kThreads), lds, stream, a);
    }
    return hipGetLastError();
}

}  // namespace mq
