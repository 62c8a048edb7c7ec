// MoE gate/up + SwiGLU for decode widths with the router and the input quantizer inside, token-major.
//
// With few tokens nearly every (token, slot) pair has an expert of its own, so nothing is gained by grouping the
// pairs by expert -- and the two launches that only prepare the expert-grouped product (routing, Q8_K of the
// layer input) cost as much as the product.  Here a workgroup owns one (token, slot, 16-row tile) of the hidden
// rows and does everything it needs itself:
//   * its first wavefront routes the token (stable top-k over the logits in one wavefront, route_block.h;
//     ComputeQwenNativeMoEStableTopK, core/src/llm/moe/native.cpp:610-676) -- every workgroup of the token repeats
//     that, a few hundred instructions -- and one workgroup per token also forms the routing weights and writes
//     ids and weights out for the down projection (cb_moe_topk_weights_from_logits, :800-868);
//   * every wavefront quantizes the super-blocks of x it multiplies (the block quantizer of quantize_q8k_kernel)
//     while its weight tiles travel;
//   * hidden[t][k][r] = silu(gate_e[r] . q8k(x_t)) * (up_e[r] . q8k(x_t)), e = ids[t][k]
//     (RunQwen35NativeMoEGateUpRawQXKSwiGLU, core/src/llm/moe/native.cpp:3929-4345); the shared expert is slot
//     top_k of every token.
// Per-tile arithmetic, the wave split of K and the reduction order are those of matmul_kernel<2,1>: the same bits
// as routing + quantize + the expert-grouped launch.
#include "common.h"
#include "kernels.h"
#include "decode_tile.h"
#include "q8k_block.h"
#include "route_block.h"

namespace mq {

namespace {

constexpr int kStages = 3;  // register stages of a wavefront: a stage is one super-block of x and its two weight tiles

template <int WT>
__global__ void __launch_bounds__(512) moe_gateup_token_kernel(const MoeGateupTokenArgs p) {
    constexpr int kTileStride = tile_stride<WT>();
    extern __shared__ float red[];  // [W-1][2][64]
    __shared__ int ids_sh[8];
    __shared__ unsigned long long route_sh[kRouteScratch];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n_waves = blockDim.x >> 6;
    const int slot = lane & 15, kq = lane >> 4;
    const int64_t rt = blockIdx.x;
    const int slots = p.top_k + (p.sh_gate ? 1 : 0);
    const int tok = blockIdx.z, sl = blockIdx.y;
    const bool shared = sl >= p.top_k;
    const int nb = (int)p.nb;
    const int cnt = p.stages;  // super-blocks wave, wave + W, ... of this wavefront: W divides nb
    const float* xrow = p.x + (size_t)tok * (size_t)nb * kQK + lane * 4;

    // Ring of kStages register stages; the activations are requested first, they do not wait for the routing.
    typename TileOf<WT>::Regs ring_t[kStages][2];
    float4 ring_x[kStages];
    auto issue_x = [&](int st, int i) {
        const int b = i < cnt ? wave + i * n_waves : 0;  // a stage past the end re-reads block 0: the load count stays fixed
        ring_x[st] = *reinterpret_cast<const float4*>(xrow + (size_t)b * kQK);
    };
#pragma unroll
    for (int st = 0; st < kStages - 1; ++st) issue_x(st, st);

    // ---- routing (every workgroup of a routed slot; the shared expert needs none) ----
    int expert = 0;
    if (!shared) {
        if (wave == 0) {
            const float* row = p.logits + (size_t)tok * p.n_experts;
            auto load = [&](int e) { return row[e]; };
            int id;
            float logit;
            if (p.n_experts <= 256) route_token_wave_lds<4>(load, p.n_experts, p.top_k, lane, id, logit, route_sh);
            else route_token_wave_lds<8>(load, p.n_experts, p.top_k, lane, id, logit, route_sh);
            if (lane < p.top_k) ids_sh[lane] = id;
            if (rt == 0 && sl == 0) {  // one workgroup per token hands ids and weights to the down projection
                const float w = route_weight_lane(logit, lane, p.top_k, p.route_mode);
                if (lane < p.top_k) {
                    p.ids_out[(size_t)tok * p.top_k + lane] = id;
                    p.weights_out[(size_t)tok * p.top_k + lane] = w;
                }
            }
        }
        __syncthreads();
        expert = ids_sh[sl];
        if (expert < 0 || expert >= p.n_experts) return;  // dropped slot: the whole workgroup leaves, its row is never read
    }
    const uint8_t* tiles[2] = {(shared ? p.sh_gate : p.gate + (size_t)expert * p.expert_bytes) + tile_offset(rt, 0, nb, kTileStride),
                               (shared ? p.sh_up : p.up + (size_t)expert * p.expert_bytes) + tile_offset(rt, 0, nb, kTileStride)};
    auto issue_t = [&](int st, int i) {
        const int b = i < cnt ? wave + i * n_waves : 0;
#pragma unroll
        for (int m = 0; m < 2; ++m) load_tile_wt<WT>(ring_t[st][m], tiles[m] + (size_t)b * kTileStride, lane);
    };
#pragma unroll
    for (int st = 0; st < kStages - 1; ++st) issue_t(st, st);

    // while the first tiles travel their super-blocks of x are quantized (the token is row 0 of the operand)
    ACodes a_first[kStages - 1];
#pragma unroll
    for (int st = 0; st < kStages - 1; ++st) {
        const float e[4] = {ring_x[st].x, ring_x[st].y, ring_x[st].z, ring_x[st].w};
        a_codes_from_lane_codes(a_first[st], quantize_block_q8k(e, lane), lane);
    }
    float acc[2][1][2] = {{{0.0f, 0.0f}}, {{0.0f, 0.0f}}};
    for (int base = 0; base < cnt; base += kStages) {
#pragma unroll
        for (int st = 0; st < kStages; ++st) {
            const int i = base + st;
            issue_x((st + kStages - 1) % kStages, i + kStages - 1);
            issue_t((st + kStages - 1) % kStages, i + kStages - 1);
            if (i < cnt) {
                ARegs<1> a;
                if (st < kStages - 1 && base == 0) {
                    a_from_codes(a, a_first[st < kStages - 1 ? st : 0], lane);
                } else {
                    const float e[4] = {ring_x[st].x, ring_x[st].y, ring_x[st].z, ring_x[st].w};
                    a_from_lane_codes(a, quantize_block_q8k(e, lane), lane);
                }
#pragma unroll
                for (int m = 0; m < 2; ++m) {  // only row 0 of the operand is formed (J = 1)
                    int32_t dsum[1][2], msum[1][2];
                    compute_tile_wt<1, WT, 1>(ring_t[st][m], a, acc[m], dsum, msum, lane);
                }
            }
        }
    }

    // ---- partial sums meet in wave order (as in matmul_kernel), SwiGLU, one store per weight row ----
    if (n_waves > 1) {
        if (wave > 0) {
#pragma unroll
            for (int m = 0; m < 2; ++m) red[((wave - 1) * 2 + m) * 64 + lane] = acc[m][0][0];
        }
        __syncthreads();
    }
    if (wave == 0) {
        if (n_waves > 1) {
#pragma unroll
            for (int m = 0; m < 2; ++m)
                acc[m][0][0] = add_wave_partials(acc[m][0][0], n_waves, [&](int wv) { return red[((wv - 1) * 2 + m) * 64 + lane]; });
        }
        const int64_t row = rt * 16 + slot;
        if (kq == 0 && row < p.rows)
            p.hidden[((size_t)tok * slots + sl) * (size_t)p.rows + row] =
                silu_mul(acc[0][0][0], acc[1][0][0], shared ? p.sh_silu_mode : p.silu_mode);
    }
}

// The same product for more (token, row tile) pairs (a workgroup per (token, slot, row tile) routes its token and
// quantizes x by itself: 288 times per token).  Here a workgroup owns a (token, row tile) and a run of slots, W
// wavefronts per slot (the wave split of moe_gateup_token_waves: the same partial sums, added in the same order)
// -- all slots when there are enough (token, row tile) pairs for the chip, half or a third of them otherwise:
// wavefront 0 routes the token while the others quantize x into LDS -- once per workgroup instead of once per
// slot -- and after one barrier every wavefront streams its share of its expert's tiles against the shared codes.
template <int WT>
__global__ void __launch_bounds__(WT == kWtQ4 ? 1024 : 512) moe_gateup_slots_kernel(const MoeGateupTokenArgs p) {
    constexpr int kTileStride = tile_stride<WT>();
    extern __shared__ __attribute__((aligned(16))) uint8_t xq[];  // [nb][64] packed codes (lane l: elements 4l .. 4l+3), [nb] scales, then red [slots of the run][W-1][2][64]
    __shared__ int ids_sh[8];
    __shared__ unsigned long long route_sh[kRouteScratch];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int slots = p.top_k + (p.sh_gate ? 1 : 0);
    const int n_waves = blockDim.x >> 6, W = p.waves, per_wg = p.slots_per_wg;  // n_waves == per_wg * W
    const int slot = lane & 15, kq = lane >> 4;
    const int64_t rt = blockIdx.x;
    // wave = local slot * W + part (W is 1, 2, 4 or 8: nb % W == 0 and W <= 8 -- W == 3, 5, 6, 7 go the other way)
    const int wshift = W == 1 ? 0 : W == 2 ? 1 : W == 4 ? 2 : 3;
    const int local = wave >> wshift, part = wave & (W - 1);
    const int tok = blockIdx.z, sl = blockIdx.y * per_wg + local;
    const bool shared = sl >= p.top_k;
    const int nb = (int)p.nb, cnt = p.stages;  // super-blocks part, part + W, ... of this wavefront
    uint32_t* codes = reinterpret_cast<uint32_t*>(xq);
    float* scales = reinterpret_cast<float*>(xq + (size_t)nb * 256);
    float* red = scales + ((nb + 63) & ~63);

    if (wave == 0) {
        const float* row = p.logits + (size_t)tok * p.n_experts;
        auto load = [&](int e) { return row[e]; };
        int id;
        float logit;
        if (p.n_experts <= 256) route_token_wave_lds<4>(load, p.n_experts, p.top_k, lane, id, logit, route_sh);
        else route_token_wave_lds<8>(load, p.n_experts, p.top_k, lane, id, logit, route_sh);
        if (lane < p.top_k) ids_sh[lane] = id;
        if (rt == 0 && blockIdx.y == 0) {  // one workgroup per token hands ids and weights to the down projection
            const float w = route_weight_lane(logit, lane, p.top_k, p.route_mode);
            if (lane < p.top_k) {
                p.ids_out[(size_t)tok * p.top_k + lane] = id;
                p.weights_out[(size_t)tok * p.top_k + lane] = w;
            }
        }
    }
    if (wave > 0 || n_waves == 1) {  // the quantizing wavefronts share the super-blocks of x
        const int first = n_waves > 1 ? wave - 1 : 0, step = n_waves > 1 ? n_waves - 1 : 1;
        const float* xrow = p.x + (size_t)tok * (size_t)nb * kQK + lane * 4;
        for (int b = first; b < nb; b += step) {
            const float4 v = *reinterpret_cast<const float4*>(xrow + (size_t)b * kQK);
            const float e[4] = {v.x, v.y, v.z, v.w};
            const Q8Lane q = quantize_block_q8k(e, lane);
            codes[b * 64 + lane] = q.packed;
            if (lane == 0) scales[b] = q.d;
        }
    }
    __syncthreads();
    int expert = 0;
    bool live = sl < slots;  // the last run of slots may be shorter
    if (live && !shared) {
        expert = ids_sh[sl];
        live = expert >= 0 && expert < p.n_experts;  // dropped slot: its row is never read
    }
    if (!live && W == 1) return;  // no barrier follows
    float acc[2][1][2] = {{{0.0f, 0.0f}}, {{0.0f, 0.0f}}};
    if (live) {
        const uint8_t* tiles[2] = {(shared ? p.sh_gate : p.gate + (size_t)expert * p.expert_bytes) + tile_offset(rt, 0, nb, kTileStride),
                                   (shared ? p.sh_up : p.up + (size_t)expert * p.expert_bytes) + tile_offset(rt, 0, nb, kTileStride)};
        typename TileOf<WT>::Regs ring_t[kStages][2];
        auto issue_t = [&](int st, int i) {
            const int b = i < cnt ? part + i * W : 0;  // a stage past the end re-reads block 0: the load count stays fixed
#pragma unroll
            for (int m = 0; m < 2; ++m) load_tile_wt<WT>(ring_t[st][m], tiles[m] + (size_t)b * kTileStride, lane);
        };
#pragma unroll
        for (int st = 0; st < kStages - 1; ++st) issue_t(st, st);
        // this lane's words of a block's operand (a_codes_from_lane_codes): codes 64c + 32(slot & 1) + 8kq .. +7 of chunk c
        const int src = 8 * (slot & 1) + 2 * kq;
        const uint32_t even_slot = (slot & 1) ? 0u : 0xffffffffu, odd_slot = ~even_slot;
        for (int base = 0; base < cnt; base += kStages) {
#pragma unroll
            for (int st = 0; st < kStages; ++st) {
                const int i = base + st;
                issue_t((st + kStages - 1) % kStages, i + kStages - 1);
                if (i < cnt) {
                    const int b = part + i * W;
                    ARegs<1> a;
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const v2u v = *reinterpret_cast<const v2u*>(codes + b * 64 + 16 * c + src);
                        a.q[0][c] = v4u{v.x & even_slot, v.y & even_slot, v.x & odd_slot, v.y & odd_slot};  // as a_from_codes (q8k_block.h)
                    }
                    a.yd[0][0] = scales[b];
                    a.yd[0][1] = 0.0f;
#pragma unroll
                    for (int m = 0; m < 2; ++m) {  // only row 0 of the operand is formed (J = 1)
                        int32_t dsum[1][2], msum[1][2];
                        compute_tile_wt<1, WT, 1>(ring_t[st][m], a, acc[m], dsum, msum, lane);
                    }
                }
            }
        }
    }
    // partial sums of a slot meet in wave order (as in moe_gateup_token_kernel), SwiGLU, one store per weight row
    if (W > 1) {
        if (part > 0) {
#pragma unroll
            for (int m = 0; m < 2; ++m) red[((local * (W - 1) + part - 1) * 2 + m) * 64 + lane] = acc[m][0][0];
        }
        __syncthreads();
        if (!live || part > 0) return;
        for (int wv = 1; wv < W; ++wv) {
#pragma unroll
            for (int m = 0; m < 2; ++m) acc[m][0][0] = __fadd_rn(acc[m][0][0], red[((local * (W - 1) + wv - 1) * 2 + m) * 64 + lane]);
        }
    }
    const int64_t row = rt * 16 + slot;
    if (kq == 0 && row < p.rows)
        p.hidden[((size_t)tok * slots + sl) * (size_t)p.rows + row] =
            silu_mul(acc[0][0][0], acc[1][0][0], shared ? p.sh_silu_mode : p.silu_mode);
}

}  // namespace

// Wavefronts of this kernel that ONE compute unit holds at once: by the registers the compiled kernel takes (512 per
// SIMD lane, handed out in blocks of 8), four SIMDs per compute unit.
int moe_gateup_token_capacity(int wtype) {
    static int cached[3] = {0, 0, 0};
    const int k = wtype == kTypeQ6K ? 2 : wtype == kTypeQ5K ? 1 : 0;
    if (!cached[k]) {
        const void* fn = wtype == kTypeQ6K   ? reinterpret_cast<const void*>(moe_gateup_token_kernel<kWtQ6>)
                         : wtype == kTypeQ5K ? reinterpret_cast<const void*>(moe_gateup_token_kernel<kWtQ5>)
                                             : reinterpret_cast<const void*>(moe_gateup_token_kernel<kWtQ4>);
        hipFuncAttributes attr;
        int per_simd = 2;
        if (hipFuncGetAttributes(&attr, fn) == hipSuccess && attr.numRegs > 0) {
            per_simd = 512 / ((attr.numRegs + 7) / 8 * 8);
            per_simd = per_simd < 1 ? 1 : per_simd > 8 ? 8 : per_simd;
        }
        cached[k] = per_simd * 4;
    }
    return cached[k];
}

int moe_gateup_slots_capacity(int wtype) {
    static int cached[3] = {0, 0, 0};
    const int k = wtype == kTypeQ6K ? 2 : wtype == kTypeQ5K ? 1 : 0;
    if (!cached[k]) {
        const void* fn = wtype == kTypeQ6K   ? reinterpret_cast<const void*>(moe_gateup_slots_kernel<kWtQ6>)
                         : wtype == kTypeQ5K ? reinterpret_cast<const void*>(moe_gateup_slots_kernel<kWtQ5>)
                                             : reinterpret_cast<const void*>(moe_gateup_slots_kernel<kWtQ4>);
        hipFuncAttributes attr;
        int per_simd = 2;
        if (hipFuncGetAttributes(&attr, fn) == hipSuccess && attr.numRegs > 0) {
            per_simd = 512 / ((attr.numRegs + 7) / 8 * 8);
            per_simd = per_simd < 1 ? 1 : per_simd > 8 ? 8 : per_simd;
        }
        cached[k] = per_simd * 4;
    }
    return cached[k];
}

// Wavefronts per workgroup: as many as divide the super-blocks of a row evenly (at most 8) while all workgroups of
// the launch are resident at once -- a compute unit holds whole workgroups only.
int moe_gateup_token_waves(int64_t nb, int64_t rows, int64_t n, int slots, int wtype) {
    const int64_t workgroups = ((rows + 15) / 16) * n * slots;
    int device = 0, cus = 0;
    if (hipGetDevice(&device) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0)
        cus = 256;
    const int per_cu = moe_gateup_token_capacity(wtype);
    for (int64_t w = nb < 8 ? nb : 8; w > 1; --w)
        if (nb % w == 0 && workgroups <= (int64_t)cus * (per_cu / w)) return (int)w;
    return 1;
}

hipError_t launch_moe_gateup_token(const MoeGateupTokenArgs& a, hipStream_t stream) {
    if (a.n <= 0 || a.rows <= 0 || a.nb <= 0 || a.top_k <= 0 || a.top_k > 8 || a.n_experts < a.top_k || a.n_experts > 512 ||
        a.waves < 1 || a.waves > 8 || (a.nb % a.waves) || !a.gate || !a.up || !a.x || !a.logits || !a.hidden || !a.ids_out ||
        !a.weights_out || (a.sh_gate == nullptr) != (a.sh_up == nullptr))
        return hipErrorInvalidValue;
    const int slots = a.top_k + (a.sh_gate ? 1 : 0);
    // A workgroup per (token, row tile, run of slots) with W wavefronts per slot (moe_gateup_slots_kernel) where that
    // makes ONE round of one workgroup per compute unit with at least nine tenths of the units busy, and a slot takes
    // one or two wavefronts (four and eight tokens at 256 compute units and 32 row tiles).  MoE block of 256 + 1
    // experts, this form against the other at 1 .. 8 tokens with the nine-tenths rule off: 13.7 / 17.25 / 21.65 / 23.0 /
    // (18 wavefronts: not possible) / 30.25 / 31.9 / 33.35 us against 13.55 / 17.15 / 21.3 / 24.4 / 29.6 / 30.75 /
    // 31.5 / 35.0 -- with fewer units busy, or with four wavefronts per slot, nothing is gained.
    const int64_t pairs = ((a.rows + 15) / 16) * a.n;
    if ((a.waves == 1 || a.waves == 2) && a.n <= 65535 && (size_t)a.nb * 260 <= 32 * 1024) {
        const int cus = compute_units();
        const int cap = moe_gateup_slots_capacity(a.wtype);  // wavefronts of the kernel per compute unit
        int per_wg = 0, runs = 0;
        {
            int r = (int)(cus / (pairs > 0 ? pairs : 1));
            r = r < 1 ? 1 : r > slots ? slots : r;
            const int pw = (slots + r - 1) / r, waves = pw * a.waves;
            const int rr = (slots + pw - 1) / pw;
            // Q5_K / Q6_K tiles take more registers: workgroups of eight wavefronts at most
            if (waves <= (a.wtype == kTypeQ4K ? 16 : 8) && waves <= cap && pairs * rr <= cus && pairs * rr * 10 >= (int64_t)cus * 9)
                per_wg = pw, runs = rr;
        }
        if (per_wg > 0) {
            MoeGateupTokenArgs b = a;
            b.stages = (int)(a.nb / a.waves);
            b.slots_per_wg = per_wg;
            const dim3 grid((unsigned)((a.rows + 15) / 16), (unsigned)runs, (unsigned)a.n);
            const size_t lds = (size_t)a.nb * 256 + (size_t)((a.nb + 63) & ~(int64_t)63) * 4 + (size_t)per_wg * (a.waves - 1) * 2 * 64 * 4;
            const dim3 block(64 * per_wg * a.waves);
            if (a.wtype == kTypeQ6K) MQ_LAUNCH(moe_gateup_slots_kernel<kWtQ6>, grid, block, lds, stream, b);
            else if (a.wtype == kTypeQ5K) MQ_LAUNCH(moe_gateup_slots_kernel<kWtQ5>, grid, block, lds, stream, b);
            else if (a.wtype == kTypeQ4K) MQ_LAUNCH(moe_gateup_slots_kernel<kWtQ4>, grid, block, lds, stream, b);
            else return hipErrorInvalidValue;
            return hipGetLastError();
        }
    }
    const dim3 grid((unsigned)((a.rows + 15) / 16), (unsigned)slots, (unsigned)a.n);
    MoeGateupTokenArgs b = a;
    b.stages = (int)(a.nb / a.waves);
    const size_t lds = a.waves > 1 ? (size_t)(a.waves - 1) * 2 * 64 * sizeof(float) : 0;
    if (a.wtype == kTypeQ6K) MQ_LAUNCH(moe_gateup_token_kernel<kWtQ6>, grid, dim3(64 * a.waves), lds, stream, b);
    else if (a.wtype == kTypeQ5K) MQ_LAUNCH(moe_gateup_token_kernel<kWtQ5>, grid, dim3(64 * a.waves), lds, stream, b);
    else if (a.wtype == kTypeQ4K) MQ_LAUNCH(moe_gateup_token_kernel<kWtQ4>, grid, dim3(64 * a.waves), lds, stream, b);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

}  // namespace mq
