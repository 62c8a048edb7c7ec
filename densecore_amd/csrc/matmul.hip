// Q4_K x Q8_K matmul for decode widths on gfx950 (dense and expert-grouped).
//
// Work decomposition
//   workgroup = one 16-row tile of the weight matrix (two matrices when gate and up are fused),
//               all of K; its W wavefronts take the super-blocks b = w, w+W, ... so that the
//               workgroup as a whole streams one contiguous run of tiles.
//   wavefront = per super-block: three coalesced 16-byte-per-lane loads bring one 2304-byte tile
//               (16 rows x 256 weights) straight into MFMA operand order; the next tile is
//               requested before the current one is consumed (two register stages, ping-pong; no request
//               is made past the wave's last super-block).
//   arithmetic, per tile and per group of 8 activation rows (independent of how many are live):
//       4 x v_mfma_i32_16x16x64_i8   one per 64-weight chunk.  Each activation row owns two M-side
//                                    slots with complementary zero halves (see common.h), so the
//                                    two 32-wide sub-blocks of the chunk come out as separate
//                                    int32 sums: sum q4*q8 per sub-block.
//       v_mad_i32_i24 with the 6-bit sub-block scales                       -> dot_scaled (int32)
//       4 x v_mfma_i32_16x16x64_i8   the 6-bit mins broadcast as the B operand: sum min*q8
//                                                                           -> min_dot   (int32)
//       fp32: acc += (d*yd)*dot_scaled - (dmin*yd)*min_dot  (core/src/llm/matmul/kquant_batched_kernels.h:299-301)
//   The two integers are exactly the reference's per-super-block sums; min_dot is formed from the
//   int8 codes instead of the 16 bsums, which is the same number because bsums[j] is by
//   construction the sum of codes 16j..16j+15 (core/src/kernels/hwy/hwy_moe_quant.cc:133-139).
//   epilogue: wave partials are added in wave order through LDS (deterministic), optional
//   silu(gate)*up, one store per (activation row, weight row).
//
// MFMA operand roles: A (M side) = 8 activation rows x 2 slots, B (N side) = 16 weight rows, so a
// lane's four accumulators belong to ONE weight row (lane%16) and to two activation rows
// (2*(lane/16) and 2*(lane/16)+1): it needs only that row's scales and writes two outputs.
#include <cstdlib>
#include <utility>

#include <hip/hip_ext.h>
#include <cmath>

#include "common.h"
#include "kernels.h"
#include "decode_tile.h"
#include "q8k_block.h"
#include "group_entry.h"

namespace mq {

namespace {

// f(std::integral_constant<int, 0>{}), ..., f(std::integral_constant<int, N - 1>{}) in order
template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// One workgroup: row tile blockIdx.x of group blockIdx.y (dense mode has a single group); its
// waves split the super-blocks of the row.  NMAT == 2: gate and up tiles of the same rows share
// the activations in registers and meet in silu(gate)*up.
// J == 1: a single activation row (dense, n == 1): the second of a lane's two activation rows is not formed at all.
// XQ (dense, n == 1): the activation row comes as fp32 (p.xf) and every wavefront quantizes the super-blocks it
// multiplies while their weight tiles travel -- the block quantizer of quantize_q8k_kernel, so the same codes,
// scales and result as the stand-alone quantizer followed by this kernel, one launch less.  (With two rows the
// repeated quantization costs what the saved launch gains, with four it loses a third.)
// REUSE_A (one-wave workgroups over several row tiles of rows that are two super-blocks long, the expert down
// projections): stage i multiplies super-block i % 2, which is also its register slot, so every slot keeps the
// activation operand it received with its first stage and later stages ask for weight tiles only -- a third of the
// load instructions instead of all of them (a stage is three tile loads and six operand loads).
// BM > 0 (one-wave workgroups over BM row tiles, an even number of super-blocks per row): the stages run block-major
// -- super-block b of all BM row tiles, then super-block b + 1 -- so that the activation operand of a super-block is
// requested once per workgroup instead of once per row tile (six of a stage's twelve load instructions are operand
// loads); each row tile keeps its own accumulators and all of them are stored at the end.
template <int NMAT, int TT, bool GROUPED, bool DEBUG, int WT, int J = 2, bool XQ = false, bool REUSE_A = false, int BM = 0>
__global__ void __launch_bounds__(512) matmul_kernel(const MatmulArgs p) {
    constexpr int kTileStride = tile_stride<WT>();
    extern __shared__ float red[];  // [W-1][NMAT][TT][2][64]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // uniform: keeps tile addresses scalar
    const int n_waves = blockDim.x >> 6;
    const int slot = lane & 15;  // A side: M slot (activation row slot/2, half slot%2); B side: weight row
    const int kq = lane >> 4;
    // A one-wave workgroup may own several consecutive row tiles (rt_per_wg): it streams them as one run of
    // tiles and finishes a row tile every nb stages.  Workgroups whose waves split K own exactly one.
    const int rt_per_wg = p.rt_per_wg > 1 ? p.rt_per_wg : 1;
    const int64_t rt = (int64_t)blockIdx.x * rt_per_wg;
    const int rt_count = (int)(((p.rows + 15) >> 4) - rt < rt_per_wg ? ((p.rows + 15) >> 4) - rt : rt_per_wg);
    const int64_t nb = p.nb;

    // ---- which activation rows does this workgroup see, and which weights ----
    const uint8_t* w[2] = {p.w0, p.w1};
    int count = (int)p.n;     // activation rows in this group
    int begin = 0;            // first entry (grouped mode)
    bool shared_group = false;
    int silu_mode = p.silu_mode;
    if (GROUPED) {
        // the three list reads are independent of each other (the lists are sized for every
        // possible group), so they cost one memory round trip, not three
        const int g = blockIdx.y;
        int ng, g_expert, g_begin, g_end;
        if (p.direct_ids) {  // few tokens: every (token, slot) pair is a group of its own, nothing was sorted
            ng = p.direct_top_k * (int)p.n;
            g_expert = p.direct_ids[g < ng ? g : 0];
            g_begin = g;
            g_end = g + 1;
            if (g < ng && (g_expert < 0 || g_expert >= p.n_experts)) return;  // dropped entry
        } else {
            ng = *p.n_groups;
            g_expert = p.group_expert[g];
            g_begin = p.group_begin[g];
            g_end = p.group_begin[g + 1];
        }
        if (g < ng) {
            const size_t eoff = (size_t)g_expert * p.expert_bytes;
            w[0] += eoff;
            if (NMAT == 2) w[1] += eoff;
            begin = g_begin;
            count = g_end - g_begin;
        } else if (g - ng < (p.sh_tokens + kTokTile * TT - 1) / (kTokTile * TT)) {
            // the shared expert sees every token: one group per pass of rows, so that its passes run
            // side by side instead of one after the other in a single workgroup
            shared_group = true;
            w[0] = p.sh_w0;
            w[1] = p.sh_w1;
            begin = (g - ng) * kTokTile * TT;
            count = p.sh_tokens - begin < kTokTile * TT ? p.sh_tokens - begin : kTokTile * TT;
            silu_mode = p.sh_silu_mode;
        } else {
            return;  // whole workgroup leaves together, before any barrier
        }
    }
    const uint8_t* tiles[NMAT];
#pragma unroll
    for (int m = 0; m < NMAT; ++m) tiles[m] = w[m] + tile_offset(rt, 0, nb, kTileStride);

    for (int chunk = 0; chunk < count; chunk += kTokTile * TT) {
        // activation row behind this lane's A slot, and activation / output rows of its two outputs
        size_t a_off[TT];
        int d_idx[TT][2], yrow[TT][2];
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
            // the three entries this lane needs, looked up together: its operand row and the two rows it
            // accumulates; a dead slot reads a live row and stores nothing
            const int pos[3] = {slot >> 1, 2 * kq, 2 * kq + 1};
            int ent[3], ars[3], yrs[3];
#pragma unroll
            for (int i = 0; i < 3; ++i) {
                const int e_raw = chunk + kTokTile * tt + pos[i];
                ent[i] = e_raw < count ? e_raw : count - 1;
            }
            entry_rows_n<GROUPED, 3>(p, shared_group, begin, ent, ars, yrs);
            a_off[tt] = aq_row_offset(ars[0], nb) + (size_t)kq * 256 + (size_t)(slot & 1) * 16;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                yrow[tt][j] = chunk + kTokTile * tt + pos[1 + j] < count ? yrs[1 + j] : -1;
                d_idx[tt][j] = (int)((size_t)(ars[1 + j] >> 3) * (size_t)nb * 8 + (size_t)(ars[1 + j] & 7));
            }
        }

        float acc[NMAT][TT][2];
#pragma unroll
        for (int m = 0; m < NMAT; ++m)
#pragma unroll
            for (int tt = 0; tt < TT; ++tt) acc[m][tt][0] = acc[m][tt][1] = 0.0f;

        // silu(gate)*up if fused, then one store per (activation row, weight row) of row tile `tile_rt`
        auto store_rows = [&](int64_t tile_rt) {
            const int64_t row = tile_rt * 16 + slot;
            if (row >= p.rows) return;
#pragma unroll
            for (int tt = 0; tt < TT; ++tt)
#pragma unroll
                for (int j = 0; j < J; ++j) {
                    if (yrow[tt][j] >= 0) {
                        float v = acc[0][tt][j];
                        if (NMAT == 2) v = silu_mul(v, acc[NMAT - 1][tt][j], silu_mode);
                        float* dst = p.y + (size_t)yrow[tt][j] * (size_t)p.ldy + (size_t)row;
                        if (p.out_aq) {  // another workgroup re-reads this value: store it device-coherently
                            __hip_atomic_store(dst, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        } else {
                            *dst = v;
                        }
                    }
                }
        };

        if constexpr (BM > 0) {
            // ---- block-major over BM row tiles: stage k of a pair of super-blocks (bb, bb + 1) is row tile k % BM of
            // super-block bb + k / BM; register slot k % 2 for the tiles, operand set (k / BM) % 2 for the activations.
            float accr[BM][NMAT][TT][2];
#pragma unroll
            for (int r = 0; r < BM; ++r)
#pragma unroll
                for (int m = 0; m < NMAT; ++m)
#pragma unroll
                    for (int tt = 0; tt < TT; ++tt) accr[r][m][tt][0] = accr[r][m][tt][1] = 0.0f;
            typename TileOf<WT>::Regs ring_t[2][NMAT];
            ARegs<TT> a_set[2];
            auto issue_k = [&](auto k_c, int bb) {
                constexpr int k = decltype(k_c)::value;
                constexpr int st = k & 1, par = (k / BM) & 1, r = k % BM;
                const int b = bb + k / BM;
#pragma unroll
                for (int m = 0; m < NMAT; ++m) load_tile_wt<WT>(ring_t[st][m], tiles[m] + ((size_t)r * nb + b) * kTileStride, lane);
                if constexpr (r == 0) load_a<TT>(a_set[par], p.aq + (size_t)b * 4096, p.ad + (size_t)b * 8, a_off, d_idx);
                asm volatile("" ::: "memory");  // requests stay in stage order
            };
            auto consume_k = [&](auto k_c) {
                constexpr int k = decltype(k_c)::value;
                constexpr int st = k & 1, par = (k / BM) & 1, r = k % BM;
#pragma unroll
                for (int m = 0; m < NMAT; ++m) {
                    int32_t dsum[TT][2], msum[TT][2];
                    if (GROUPED && TT == 1 && count == 1)  // most expert groups hold one row: its partner row is not formed
                        compute_tile_wt<TT, WT, 1>(ring_t[st][m], a_set[par], accr[r][m], dsum, msum, lane);
                    else
                        compute_tile_wt<TT, WT, J>(ring_t[st][m], a_set[par], accr[r][m], dsum, msum, lane);
                }
            };
            auto pair_of_blocks = [&](int bb, auto refill_c) {  // refill: the pair after this one exists
                constexpr bool refill = decltype(refill_c)::value;
                static_for<2 * BM>([&](auto k_c) {
                    constexpr int k = decltype(k_c)::value;
                    consume_k(k_c);
                    if constexpr (k + 2 < 2 * BM) issue_k(std::integral_constant<int, k + 2>{}, bb);
                    else if constexpr (refill) issue_k(std::integral_constant<int, k + 2 - 2 * BM>{}, bb + 2);
                });
            };
            issue_k(std::integral_constant<int, 0>{}, 0);
            issue_k(std::integral_constant<int, 1>{}, 0);
            int bb = 0;
            for (; bb + 2 < (int)nb; bb += 2) pair_of_blocks(bb, std::true_type{});
            pair_of_blocks(bb, std::false_type{});
#pragma unroll
            for (int r = 0; r < BM; ++r) {
#pragma unroll
                for (int m = 0; m < NMAT; ++m)
#pragma unroll
                    for (int tt = 0; tt < TT; ++tt) acc[m][tt][0] = accr[r][m][tt][0], acc[m][tt][1] = accr[r][m][tt][1];
                store_rows(rt + r);
            }
        } else
        // Stage i of this wave is super-block wave + i*W (several row tiles in a one-wave workgroup: tile i of the
        // contiguous run); two register stages, one in flight while the other is multiplied (ring2: no request is
        // ever made past the last stage).  All branches are wave-uniform and the loads themselves unconditional.
        if (wave < nb) {
            const int per_rt = (int)((nb - wave + n_waves - 1) / n_waves);  // super-blocks of this wave per row tile
            const int cnt = per_rt * rt_count;                              // stages of this wave
            typename TileOf<WT>::Regs ring_t[2][NMAT];
            ARegs<TT> ring_a[2];
            float4 ring_x[2];
            auto issue = [&](auto st_c, int i, auto first_c) {
                constexpr int st = decltype(st_c)::value;
                constexpr bool first = decltype(first_c)::value;
                // i == cnt (once, when cnt is odd): the same loads from fixed addresses in all lanes, a cache line each
                const bool valid = i < cnt;
                // several row tiles (one wave, per_rt == nb): stage i is tile i of the contiguous run,
                // super-block i % nb; one row tile: super-block wave + i*W
                const int t = valid ? (rt_per_wg > 1 ? i : wave + i * n_waves) : wave;
                const int b = rt_per_wg > 1 ? t % per_rt : t;
                const int ln = valid ? lane : 0;
#pragma unroll
                for (int m = 0; m < NMAT; ++m) load_tile_wt<WT>(ring_t[st][m], tiles[m] + (size_t)t * kTileStride, ln);
                if constexpr (XQ) {
                    ring_x[st] = *reinterpret_cast<const float4*>(p.xf + (size_t)b * kQK + ln * 4);
                } else if constexpr (REUSE_A && !first) {
                    // slot st still holds super-block st's operand
                } else {
                    size_t off[TT];
#pragma unroll
                    for (int tt = 0; tt < TT; ++tt) off[tt] = valid ? a_off[tt] : 0;
                    load_a<TT>(ring_a[st], p.aq + (size_t)b * 4096, p.ad + (size_t)b * 8, off, d_idx);
                }
            };
            auto consume = [&](auto st_c, int i) {
                constexpr int st = decltype(st_c)::value;
                ARegs<TT> quantized;
                if constexpr (XQ) {  // the row becomes row 0 of the operand
                    const float e[4] = {ring_x[st].x, ring_x[st].y, ring_x[st].z, ring_x[st].w};
                    a_from_lane_codes(quantized, quantize_block_q8k(e, lane), lane);
                }
                const ARegs<TT>& a_regs = XQ ? quantized : ring_a[st];
#pragma unroll
                for (int m = 0; m < NMAT; ++m) {
                    int32_t dsum[TT][2], msum[TT][2];
                    if (GROUPED && TT == 1 && count == 1)  // most expert groups hold one row: its partner row is not formed
                        compute_tile_wt<TT, WT, 1>(ring_t[st][m], a_regs, acc[m], dsum, msum, lane);
                    else
                        compute_tile_wt<TT, WT, J>(ring_t[st][m], a_regs, acc[m], dsum, msum, lane);
                    if (DEBUG && p.dbg_dot) {  // debug launches own one row tile per workgroup
                        const int b = wave + i * n_waves;
                        const int64_t row = rt * 16 + slot;
#pragma unroll
                        for (int tt = 0; tt < TT; ++tt)
#pragma unroll
                            for (int j = 0; j < 2; ++j) {
                                if (yrow[tt][j] >= 0 && row < p.rows) {
                                    const size_t idx = ((size_t)row * (size_t)p.n + (size_t)yrow[tt][j]) * nb + b;
                                    p.dbg_dot[idx] = dsum[tt][j];
                                    p.dbg_min[idx] = msum[tt][j];
                                }
                            }
                    }
                }
                if (rt_per_wg > 1 && (i + 1) % per_rt == 0) {  // a row tile is complete: store it, start the next
                    store_rows(rt + i / per_rt);
#pragma unroll
                    for (int m = 0; m < NMAT; ++m)
#pragma unroll
                        for (int tt = 0; tt < TT; ++tt) acc[m][tt][0] = acc[m][tt][1] = 0.0f;
                }
            };
            ring2(cnt, issue, consume);
        }

        // ---- cross-wave reduction in wave order, then the epilogue on wave 0 ----
        if (n_waves > 1) {
            if (wave > 0) {
#pragma unroll
                for (int m = 0; m < NMAT; ++m)
#pragma unroll
                    for (int tt = 0; tt < TT; ++tt)
#pragma unroll
                        for (int j = 0; j < J; ++j)
                            red[((((wave - 1) * NMAT + m) * TT + tt) * 2 + j) * 64 + lane] = acc[m][tt][j];
            }
            __syncthreads();
        }
        if (wave == 0 && rt_per_wg == 1) {
            if (n_waves > 1) {
#pragma unroll
                for (int m = 0; m < NMAT; ++m)
#pragma unroll
                    for (int tt = 0; tt < TT; ++tt)
#pragma unroll
                        for (int j = 0; j < J; ++j)
                            acc[m][tt][j] = add_wave_partials(acc[m][tt][j], n_waves, [&](int wv) {
                                return red[((((wv - 1) * NMAT + m) * TT + tt) * 2 + j) * 64 + lane];
                            });
            }
            store_rows(rt);
        }
        if (n_waves > 1 && chunk + kTokTile * TT < count) __syncthreads();  // red[] is reused by the next chunk
    }

    // ---- optional: the last workgroup to finish a 256-row block of y re-quantizes it to Q8_K ----
    if (p.out_aq) {
        __shared__ int is_last;
        const int out_nb = (int)(p.rows >> 8);
        const int hb = (int)(rt >> 4);
        // The y stores above are device-scope write-through stores.  A workgroup barrier does not
        // wait for global stores, so wait for their acknowledgement explicitly: after this they are
        // visible device-wide and the workgroup may be counted.  (A full release fence would write
        // back the whole L2 of this XCD on every workgroup.)
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (threadIdx.x == 0) {
            uint32_t* c = p.out_counters + (size_t)blockIdx.y * out_nb + hb;
            const uint32_t prev = atomicAdd(c, 1u);
            const uint32_t last = (uint32_t)(16 / rt_per_wg - 1);  // a 256-row block is 16 row tiles, rt_per_wg of them per workgroup
            is_last = prev == last;
            if (prev == last) atomicExch(c, 0u);  // leave the counters zero for the next launch
        }
        __syncthreads();
        if (is_last) {
            for (int e = wave; e < count; e += n_waves) {
                int ar, yr;
                entry_rows<GROUPED>(p, shared_group, begin, e, ar, yr);
                const float* src = p.y + (size_t)yr * (size_t)p.ldy + (size_t)hb * 256 + lane * 4;
                float v[4];
#pragma unroll
                for (int j = 0; j < 4; ++j)  // device-scope loads: other workgroups wrote these values
                    v[j] = __hip_atomic_load(src + j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                const Q8Lane r = quantize_block_q8k(v, lane);
                store_amajor(p.out_aq, p.out_ad, yr, hb, out_nb, lane, r);
            }
        }
    }
}

template <int NMAT, int TT, bool GROUPED, bool DEBUG, int WT, int J = 2, bool XQ = false, bool REUSE_A = false, int BM = 0>
hipError_t launch_one(const MatmulArgs& a, int waves, dim3 grid, hipStream_t stream, hipEvent_t start, hipEvent_t stop) {
    const size_t lds = waves > 1 ? (size_t)(waves - 1) * NMAT * TT * 2 * 64 * sizeof(float) : 0;
    if (start && stop) {
        // the events take the dispatch's own begin / end timestamps: no extra packets around the kernel
        hipExtLaunchKernelGGL((matmul_kernel<NMAT, TT, GROUPED, DEBUG, WT, J, XQ, REUSE_A, BM>), grid, dim3(64 * waves), lds, stream, start, stop,
                              0, a);
    } else {
        MQ_LAUNCH((matmul_kernel<NMAT, TT, GROUPED, DEBUG, WT, J, XQ, REUSE_A, BM>), grid, dim3(64 * waves), lds, stream, a);
    }
    return hipGetLastError();
}

}  // namespace

// Waves per workgroup: a compute unit holds 8 wavefronts of this kernel (2 per SIMD) and whole workgroups only;
// aim at having every workgroup of the launch resident at once -- a launch a few workgroups over that waits for
// a second round that starts when the first ones end -- with a count that divides the super-blocks of a row
// evenly and at most 8.
static int g_compute_units = 256;  // what an unpartitioned MI355X has; mq_init replaces it with the device's own count
void set_compute_units(int count) {
    if (count > 0) g_compute_units = count;
}
int compute_units() { return g_compute_units; }

int pick_waves(int64_t nb, int64_t workgroups) {
    const int64_t compute_units = g_compute_units;
    for (int64_t w = nb < 8 ? nb : 8; w > 1; --w)
        if (nb % w == 0 && workgroups <= compute_units * (8 / w)) return (int)w;
    return 1;
}

hipError_t launch_matmul(const MatmulArgs& a, hipStream_t stream, hipEvent_t start, hipEvent_t stop) {
    if (a.rows <= 0 || a.nb <= 0) return hipErrorInvalidValue;
    if (a.out_aq && (a.rows & 255)) return hipErrorInvalidValue;
    if (a.xf && (a.grouped || a.dbg_dot || a.out_aq || a.n != 1 || (reinterpret_cast<uintptr_t>(a.xf) & 15u))) return hipErrorInvalidValue;
    const int64_t rowtiles = (a.rows + 15) / 16;
    const int nmat = a.swiglu ? 2 : 1;
    const bool debug = a.dbg_dot != nullptr;
    if (a.wtype != kTypeQ4K && a.wtype != kTypeQ5K && a.wtype != kTypeQ6K) return hipErrorInvalidValue;
    // widest activation group this launch can see decides how many 8-row token tiles a pass holds
    const int64_t widest = a.grouped ? (a.n > a.sh_tokens ? a.n : a.sh_tokens) : a.n;
    // Expert groups rarely hold more than 8 rows at decode widths; the few that do (and the shared
    // expert) take a second pass over their 16 rows of weights, which then come from cache.
    const int tt = (a.grouped || widest <= 8) ? 1 : 2;
    const int groups = a.grouped ? a.max_groups + (a.sh_tokens + 8 * tt - 1) / (8 * tt) : 1;
    const int waves = pick_waves(a.nb, rowtiles * groups);
    // Short rows (few super-blocks) in one-wave workgroups: let a workgroup stream several row tiles, so that
    // its look-ups and activation addressing are paid once per ~16 tiles rather than once per row tile.
    // Expert-grouped gate/up in one-wave workgroups: a workgroup takes two row tiles and runs them block-major, so
    // that the activation operand of a super-block is requested once for both and the group look-ups are paid half as
    // often (measured, MoE block of 256 experts, top-8, row tiles per workgroup 1 / 2 / 4: 55.5 / 52.9 / 55.7 us at 12
    // tokens, 61.2 / 55.9 / 57.2 at 16, 80.0 / 74.6 / 79.8 at 32, 106.2 / 100.5 / 99.3 at 64, 148.1 / 137.8 / 149.2 at
    // 128; the down launch, whose workgroups already take eight row tiles, loses with any more).  With the fused output
    // quantization a workgroup must stay inside one 256-row block (16 row tiles).
    // Many groups (one-wave workgroups) of rows at least four super-blocks long: the kernel that gathers a group's rows
    // into LDS once per eight wavefronts, a row tile per wavefront (two while a wavefront would have fewer than eight
    // stages).  Measured on the MoE block of 256 experts, 2048 x 512, top-8: gate/up + SwiGLU 54.3 -> 52.1 us per
    // block at 16 tokens, 80.3 -> 73.4 at 32, 99.4 -> 93.6 at 64, 131.7 -> 123.8 at 128; mul_mat_id over the same
    // gate experts alone 24.8 -> 22.6 / 32.3 -> 28.9 / 46.0 -> 34.9 us at 16 / 32 / 64 tokens.  The down experts' rows
    // (two super-blocks) gain nothing there (the launch below keeps their operand in registers) and stay.
    if (a.grouped && waves == 1 && tt == 1 && a.nb >= 4 && grouped_lds_applies(a)) {
        int per_wave = 1;
        if (!a.out_aq) {
            while (per_wave < 8 && per_wave * a.nb * nmat < 8 && rowtiles >= 16 * per_wave) per_wave *= 2;
        }
        return launch_grouped_lds(a, per_wave, groups, stream, start, stop);
    }
    MatmulArgs b = a;
    b.rt_per_wg = 1;
    if (waves == 1 && !debug) {
        int64_t want = 16 / (a.nb * nmat);
        if (want < 1) want = 1;
        if (a.grouped && nmat == 2 && want == 1) want = 2;
        if (a.out_aq) {
            while (want > 1 && ((want & (want - 1)) || want > 16)) --want;  // a power of two up to 16 (rows % 256 == 0)
        } else {
            while (want > 1 && rowtiles % want) --want;  // an even split keeps the last workgroup full
        }
        b.rt_per_wg = (int)want;
    }
    const dim3 grid((unsigned)(rowtiles / b.rt_per_wg), (unsigned)groups);

#define MQ_LAUNCH_WT(NM, T, W)                                                                            \
    do {                                                                                                  \
        if (a.grouped && NM == 1 && T == 1 && waves == 1 && b.rt_per_wg > 1 && a.nb == 2)                  \
            return launch_one<1, 1, true, false, W, 2, false, true>(b, waves, grid, stream, start, stop);  \
        /* block-major order where its registers fit: Q4_K and Q5_K */                                        \
        if (a.grouped && NM == 2 && T == 1 && waves == 1 && b.rt_per_wg == 2 && a.nb % 2 == 0 && W != kWtQ6) \
            return launch_one<2, 1, true, false, W == kWtQ6 ? kWtQ4 : W, 2, false, false, 2>(b, waves, grid, stream, start, stop); \
        if (a.grouped) return launch_one<NM, T, true, false, W>(b, waves, grid, stream, start, stop);     \
        if (debug) return launch_one<NM, T, false, true, W>(b, waves, grid, stream, start, stop);         \
        if (T == 1 && a.xf) return launch_one<NM, 1, false, false, W, 1, true>(b, waves, grid, stream, start, stop); \
        if (T == 1 && a.n == 1) return launch_one<NM, 1, false, false, W, 1>(b, waves, grid, stream, start, stop); \
        return launch_one<NM, T, false, false, W>(b, waves, grid, stream, start, stop);                   \
    } while (0)
#define MQ_LAUNCH_NT(NM, T)                               \
    do {                                                 \
        if (a.wtype == kTypeQ6K) MQ_LAUNCH_WT(NM, T, kWtQ6); \
        if (a.wtype == kTypeQ5K) MQ_LAUNCH_WT(NM, T, kWtQ5); \
        MQ_LAUNCH_WT(NM, T, kWtQ4);                      \
    } while (0)

    if (nmat == 1) {
        if (tt == 1) MQ_LAUNCH_NT(1, 1);
        MQ_LAUNCH_NT(1, 2);
    } else {
        if (tt == 1) MQ_LAUNCH_NT(2, 1);
        MQ_LAUNCH_NT(2, 2);
    }
#undef MQ_LAUNCH_NT
#undef MQ_LAUNCH_WT
    return hipSuccess;
}

}  // namespace mq
