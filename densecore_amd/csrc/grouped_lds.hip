// Expert-grouped Q4_K / Q5_K / Q6_K x Q8_K product with a group's activations staged once per workgroup in LDS.
//
// matmul_kernel in its expert-grouped form gives every row tile (or pair of row tiles) of an expert group a one-wave
// workgroup of its own: each of them looks the group up, works out which activation rows sit behind its operand slots
// and then asks for that operand from global memory at every stage -- six loads per stage beside the weight tiles,
// all answered by the L2.  Here a workgroup of eight wavefronts takes 8 * R consecutive row tiles of one group
// (wavefront w the R tiles from 8 * R * blockIdx.x + R * w on), looks the group up once, gathers the group's (up to
// eight) activation rows into LDS once -- LDS-direct copies whose per-lane source address is the address the
// operand load of matmul_kernel would use, so the bytes land in operand order -- and every stage reads its operand
// from there.  A wavefront adds the super-blocks of a row tile in ascending order by itself, as the one-wave
// workgroups of matmul_kernel do: the same bits.  Used where launch_matmul would pick one-wave workgroups (many
// groups); the launches with few groups, whose wavefronts split K, stay on matmul_kernel.
//
// Operand conventions, group lists, the shared expert's extra groups and the fused Q8_K of
// the output (the last workgroup to finish a 256-row block quantizes it) are matmul_kernel's.
// RunQwen35NativeMoEGateUpRawQXKSwiGLU / the down callback group tokens by expert the same way
// (core/src/llm/moe/native.cpp:1664-1766, :3929-4345, :3051-3295).
#include <hip/hip_ext.h>

#include "common.h"
#include "kernels.h"
#include "decode_tile.h"
#include "q8k_block.h"
#include "group_entry.h"

namespace mq {

namespace {

typedef __attribute__((address_space(3))) void* lds_ptr_t;

template <int WT> constexpr int loads_per_tile() { return WT == kWtQ6 ? 5 : WT == kWtQ5 ? 4 : 3; }

bool g_enabled = true;

// LDS: [nb][4096] operand bytes in lane order (chunk (b, c) at (4 b + c) * 1024, lane l at + 16 l), then [nb][8]
// scales padded to whole 256-byte chunks.  R = p.rt_per_wg / 8 row tiles per wavefront.
template <int NMAT, int WT>
__global__ void __launch_bounds__(512, 4) grouped_lds_kernel(const MatmulArgs p) {
    constexpr int kTileStride = tile_stride<WT>();
    extern __shared__ __align__(16) uint8_t lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int slot = lane & 15, kq = lane >> 4;
    const int nb = (int)p.nb;
    const int R = p.rt_per_wg >> 3;
    const int64_t rowtiles = (p.rows + 15) >> 4;
    const int64_t rt_wg = (int64_t)blockIdx.x * p.rt_per_wg;
    int64_t rt0 = rt_wg + (int64_t)wave * R;                      // first row tile of this wavefront
    int rt_live = (int)(rowtiles - rt0 < R ? rowtiles - rt0 : R);  // row tiles of this wavefront that exist
    const bool dead = rt_live <= 0;
    if (dead) {  // past the last row tile: stream the last row tile again (it still takes part in the gather), store nothing
        rt0 = rowtiles - 1;
        rt_live = 1;
    }

    // ---- the group: its expert's weights and its entries ----
    const uint8_t* w[2] = {p.w0, p.w1};
    int count, begin;
    bool shared_group = false;
    int silu_mode = p.silu_mode;
    {
        const int g = blockIdx.y;
        int ng, g_expert, g_begin, g_end;
        if (p.direct_ids) {
            ng = p.direct_top_k * (int)p.n;
            g_expert = p.direct_ids[g < ng ? g : 0];
            g_begin = g;
            g_end = g + 1;
            if (g < ng && (g_expert < 0 || g_expert >= p.n_experts)) return;
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
        } else if (g - ng < (p.sh_tokens + kTokTile - 1) / kTokTile) {
            shared_group = true;
            w[0] = p.sh_w0;
            w[1] = p.sh_w1;
            begin = (g - ng) * kTokTile;
            count = p.sh_tokens - begin < kTokTile ? p.sh_tokens - begin : kTokTile;
            silu_mode = p.sh_silu_mode;
        } else {
            return;  // the whole workgroup leaves together, before any barrier
        }
    }
    const uint8_t* tiles[NMAT];
#pragma unroll
    for (int m = 0; m < NMAT; ++m) tiles[m] = w[m] + tile_offset(rt0, 0, nb, kTileStride);
    const int cnt = rt_live * nb;  // stages of this wavefront: tile i of its contiguous run, super-block i % nb

    uint8_t* a_lds = lds;
    const int d_floats = (nb * 8 + 63) & ~63;
    float* d_lds = reinterpret_cast<float*>(lds + (size_t)nb * 4096);
    const uint32_t a_base = (uint32_t)(uintptr_t)(lds_ptr_t)a_lds;
    const uint32_t d_base = (uint32_t)(uintptr_t)(lds_ptr_t)d_lds;

    for (int chunk = 0; chunk < count; chunk += kTokTile) {
        // ---- rows behind this lane: its operand slot (gather source), its two outputs ----
        // the four entries this lane needs, looked up together: its operand row, the two rows it accumulates, and the
        // row whose scale it gathers (row lane % 8 of super-block lane / 8, + 8 per round); a dead slot reads a live
        // row and stores nothing
        const int pos[4] = {slot >> 1, 2 * kq, 2 * kq + 1, lane & 7};
        int ent[4], ars[4], yrs[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) ent[i] = chunk + pos[i] < count ? chunk + pos[i] : count - 1;
        entry_rows_n<true, 4>(p, shared_group, begin, ent, ars, yrs);
        const size_t a_off = aq_row_offset(ars[0], nb) + (size_t)kq * 256 + (size_t)(slot & 1) * 16;
        const int yrow[2] = {chunk + pos[1] < count ? yrs[1] : -1, chunk + pos[2] < count ? yrs[2] : -1};
        const size_t d_row = (size_t)(ars[3] >> 3) * (size_t)nb * 8 + (size_t)(ars[3] & 7);

        if (chunk > 0) __syncthreads();  // everyone has finished reading the previous rows
        // ---- gather: operand chunk (b, c) = 1 KB in lane order; then the scales, eight super-blocks per copy ----
        for (int ch = wave; ch < nb * 4; ch += 8) {
            const uint8_t* g = p.aq + a_off + (size_t)(ch >> 2) * 4096 + (size_t)(ch & 3) * 1024;
            const uint32_t dst = a_base + (uint32_t)ch * 1024u;
            asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(g), "s"(dst) : "memory", "m0");
        }
        for (int c0 = wave; c0 < d_floats / 64; c0 += 8) {
            const int b = c0 * 8 + (lane >> 3);
            const float* g = p.ad + (size_t)(b < nb ? b : nb - 1) * 8 + d_row;  // the padding repeats the last super-block
            const uint32_t dst = d_base + (uint32_t)c0 * 256u;
            asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" : : "v"(g), "s"(dst) : "memory", "m0");
        }

        // A stage is ONE weight tile: with gate and up fused the stages alternate gate(b), up(b), gate(b + 1), ... so
        // that register slot 0 always holds a gate tile and slot 1 an up tile (two tiles of registers instead of four:
        // four wavefronts per SIMD fit); with one matrix the slots alternate over its tiles (cnt is even, host-checked).
        typename TileOf<WT>::Regs ring_t[2];
        auto issue = [&](auto st_c, int i) {  // tile i of the wavefront's run, matrix st (fused) or the only one
            constexpr int st = decltype(st_c)::value;
            load_tile_wt<WT>(ring_t[st], tiles[NMAT == 2 ? st : 0] + (size_t)i * kTileStride, lane);
        };
        float acc[NMAT][1][2];
#pragma unroll
        for (int m = 0; m < NMAT; ++m) acc[m][0][0] = acc[m][0][1] = 0.0f;

        auto store_rows = [&](int64_t tile_rt) {
            const int64_t row = tile_rt * 16 + slot;
            if (row >= p.rows) return;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                if (yrow[j] >= 0) {
                    float v = acc[0][0][j];
                    if (NMAT == 2) v = silu_mul(v, acc[NMAT - 1][0][j], silu_mode);
                    float* dst = p.y + (size_t)yrow[j] * (size_t)p.ldy + (size_t)row;
                    if (p.out_aq) {  // another workgroup re-reads this value: store it device-coherently
                        __hip_atomic_store(dst, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    } else {
                        *dst = v;
                    }
                }
            }
        };
        int b_next = 0, r_next = 0;  // super-block and row tile of the next tile to be multiplied
        ARegs<1> a;
        auto read_a = [&](int b) {
#pragma unroll
            for (int c = 0; c < 4; ++c) a.q[0][c] = *reinterpret_cast<const v4u*>(a_lds + (size_t)b * 4096 + c * 1024 + lane * 16);
#pragma unroll
            for (int j = 0; j < 2; ++j) a.yd[0][j] = d_lds[b * 8 + 2 * kq + j];
        };
        auto consume = [&](auto st_c) {
            constexpr int st = decltype(st_c)::value;
            constexpr int m = NMAT == 2 ? st : 0;
            const int b = b_next, r = r_next;
            if (NMAT == 1 || st == 0) read_a(b);  // gate and up of a super-block share the operand
            int32_t dsum[1][2], msum[1][2];
            compute_tile_wt<1, WT, 2>(ring_t[st], a, acc[m], dsum, msum, lane);
            if (NMAT == 1 || st == 1) {
                if (b == nb - 1) {  // a row tile is complete: store it (if it exists), start the next
                    if (!dead) store_rows(rt0 + r);
#pragma unroll
                    for (int mm = 0; mm < NMAT; ++mm) acc[mm][0][0] = acc[mm][0][1] = 0.0f;
                    b_next = 0;
                    r_next = r + 1;
                } else {
                    b_next = b + 1;
                }
            }
        };

        using S0 = std::integral_constant<int, 0>;
        using S1 = std::integral_constant<int, 1>;
        // tile index of stage s: s / 2 when fused (both slots work on the same tile index), s otherwise
        issue(S0{}, 0);
        asm volatile("" ::: "memory");
        issue(S1{}, NMAT == 2 ? 0 : 1);
        asm volatile("" ::: "memory");
        // the LDS-direct copies are older than the tile requests: they have landed once at most those are outstanding
        asm volatile("s_waitcnt vmcnt(%0)" : : "n"(2 * loads_per_tile<WT>()) : "memory");
        __builtin_amdgcn_s_barrier();  // no fence: a fence would wait for the outstanding weight tiles as well
        asm volatile("" ::: "memory");
        if constexpr (NMAT == 2) {
            int i = 0;
            for (; i + 1 < cnt; ++i) {
                consume(S0{});
                issue(S0{}, i + 1);
                asm volatile("" ::: "memory");
                consume(S1{});
                issue(S1{}, i + 1);
                asm volatile("" ::: "memory");
            }
            consume(S0{});
            consume(S1{});
        } else {
            int i = 0;
            for (; i + 2 < cnt; i += 2) {
                consume(S0{});
                issue(S0{}, i + 2);
                asm volatile("" ::: "memory");
                consume(S1{});
                issue(S1{}, i + 3);
                asm volatile("" ::: "memory");
            }
            consume(S0{});
            consume(S1{});
        }
    }

    // ---- optional: the last workgroup to finish a 256-row block of y re-quantizes it to Q8_K ----
    if (p.out_aq) {
        __shared__ int is_last;
        const int out_nb = (int)(p.rows >> 8);
        const int hb = (int)(rt_wg >> 4);
        // The y stores above are device-scope write-through stores; wait for their acknowledgement, then count the
        // workgroup (a release fence would write back the whole L2 of this XCD on every workgroup).
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (threadIdx.x == 0) {
            uint32_t* c = p.out_counters + (size_t)blockIdx.y * out_nb + hb;
            const uint32_t prev = atomicAdd(c, 1u);
            const uint32_t last = (uint32_t)(16 / p.rt_per_wg - 1);  // a 256-row block is 16 row tiles
            is_last = prev == last;
            if (prev == last) atomicExch(c, 0u);  // leave the counters zero for the next launch
        }
        __syncthreads();
        if (is_last) {
            for (int e = wave; e < count; e += 8) {
                int ar, yr;
                entry_rows<true>(p, shared_group, begin, e, ar, yr);
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

size_t lds_bytes(int64_t nb) { return (size_t)nb * 4096 + (size_t)((nb * 8 + 63) & ~63) * 4; }

template <int NMAT, int WT>
hipError_t launch_wt(const MatmulArgs& a, dim3 grid, hipStream_t stream, hipEvent_t start, hipEvent_t stop) {
    auto* kernel = &grouped_lds_kernel<NMAT, WT>;
    const size_t lds = lds_bytes(a.nb);
    static bool raised = false;  // per instantiation; the attribute belongs to the function, not to a launch
    if (!raised && lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
        raised = true;
    }
    if (start && stop) hipExtLaunchKernelGGL(kernel, grid, dim3(512), lds, stream, start, stop, 0, a);
    else MQ_LAUNCH(kernel, grid, dim3(512), lds, stream, a);
    return hipGetLastError();
}

}  // namespace

void set_grouped_lds(bool on) { g_enabled = on; }

// Whether the expert-grouped launch `a` (one-wave workgroups in matmul_kernel) runs here instead.
bool grouped_lds_applies(const MatmulArgs& a) {
    if (!g_enabled || !a.grouped || a.dbg_dot || a.xf) return false;
    if (a.out_aq && (a.rows & 255)) return false;
    if (a.nb & 1) return false;           // the stage loop runs in pairs
    if (!a.swiglu && (a.nb & 1)) return false;  // one matrix: the stage loop runs over pairs of super-blocks
    if (a.swiglu && a.wtype != kTypeQ4K) return false;  // fused Q5_K / Q6_K tiles do not fit four wavefronts per SIMD
    return lds_bytes(a.nb) <= 64 * 1024;       // two workgroups per compute unit keep their rows side by side
}

// rt_per_wave: row tiles a wavefront streams one after the other (1, 2, 4 or 8; with the fused output quantization a
// workgroup must stay inside a 256-row block: 1 or 2).
hipError_t launch_grouped_lds(const MatmulArgs& a, int rt_per_wave, int groups, hipStream_t stream, hipEvent_t start, hipEvent_t stop) {
    if (!grouped_lds_applies(a) || rt_per_wave < 1 || rt_per_wave > 8 || (rt_per_wave & (rt_per_wave - 1))) return hipErrorInvalidValue;
    if (a.out_aq && rt_per_wave > 2) return hipErrorInvalidValue;
    MatmulArgs b = a;
    b.rt_per_wg = 8 * rt_per_wave;
    const int64_t rowtiles = (a.rows + 15) / 16;
    const dim3 grid((unsigned)((rowtiles + b.rt_per_wg - 1) / b.rt_per_wg), (unsigned)groups);
    if (a.swiglu) return launch_wt<2, kWtQ4>(b, grid, stream, start, stop);
    if (a.wtype == kTypeQ6K) return launch_wt<1, kWtQ6>(b, grid, stream, start, stop);
    if (a.wtype == kTypeQ5K) return launch_wt<1, kWtQ5>(b, grid, stream, start, stop);
    if (a.wtype == kTypeQ4K) return launch_wt<1, kWtQ4>(b, grid, stream, start, stop);
    return hipErrorInvalidValue;
}

}  // namespace mq
