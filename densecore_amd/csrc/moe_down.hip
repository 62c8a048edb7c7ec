// MoE down projection with the weighted combine inside, token-major, for decode widths.
//
// The expert-grouped launch (matmul.hip) writes one partial row per (token, slot) and a second launch adds them
// up in routing order.  With few tokens almost every (token, slot) pair has an expert of its own, so grouping by
// expert shares nothing; here a workgroup owns one (token, 16-row tile) of the OUTPUT instead, streams the tiles
// of that token's top_k experts (and of the shared expert), and adds the results in routing order itself:
//   y[t][r] = sum_k w[t][k] * (down_e(t,k)[r] . q8k(hidden[t][k]))  (+ sigmoid(g . x[t]) * shared)
// (cb_qwen35_native_moe_down_q5k_weighted_logits, core/src/llm/moe/native.cpp:3051-3295; zero weights and ids out
// of range skipped as at :3237).  Per-tile arithmetic, the order of the super-block terms and of the slots, and
// the gate are those of the grouped launch + moe_combine_kernel: same bits, one launch less, no partial rows.
// kFromF32: the hidden rows come as fp32 and every wavefront quantizes the super-blocks it multiplies (the block
// quantizer of quantize_q8k_kernel: same codes and scale), which takes the re-quantization off the tail of the
// gate/up launch; the work is repeated by every workgroup of a token, a few hundred instructions each.
// Order of the requests: the token's experts (one vector load), the hidden rows and the gate operands go out first,
// the tile requests follow as soon as the experts are known, and the quantization, the gate and the routing weights
// are worked on while the tiles travel; requests are answered in order, so nothing that is needed early may be
// asked for after a tile.
#include "common.h"
#include "kernels.h"
#include "decode_tile.h"
#include "q8k_block.h"
#include "route_block.h"

namespace mq {

namespace {

constexpr int kWaves = 8;
constexpr int kItems = 3;  // (slot, super-block) items a wavefront keeps in flight

template <int WT, bool kFromF32>
__global__ void __launch_bounds__(kWaves * 64) moe_down_token_kernel(const MoeDownTokenArgs p) {
    constexpr int kTileStride = tile_stride<WT>();
    constexpr int J = kFromF32 ? 1 : 2;  // a row quantized here is row 0 of the operand: the second row is never formed
    extern __shared__ float term[];  // [slots * nb][16] terms, then [slots][16] weighted slot sums
    __shared__ float wave_sum[4];
    __shared__ float gate_sh;
    __shared__ int ids_sh[8];        // the token's experts and routing weights
    __shared__ float wts_sh[8];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int slot = lane & 15, kq = lane >> 4;
    const int64_t rt = blockIdx.x, t = blockIdx.y;
    const int nb = (int)p.nb, slots = p.top_k + (p.sh_w ? 1 : 0), n_items = slots * nb;
    float* prod = term + n_items * 16;
    auto item_slot = [&](int i) { return nb == 1 ? i : (int)__umulhi((uint32_t)i, p.inv_nb); };  // i / nb without a division

    // The token's experts and weights in lanes 0 .. top_k-1 of every wavefront: ONE request, made before anything
    // else, because the tile addresses wait for it (a scalar read per item would be a round trip per item).
    const int k_lane = lane < p.top_k ? lane : 0;
    const int id_lane = p.ids[t * p.top_k + k_lane];
    const float w_lane = p.weights[t * p.top_k + k_lane];

    for (int base = 0; base < n_items; base += kWaves * kItems) {
        typename TileOf<WT>::Regs tiles[kItems];
        ARegs<1> a[kItems];
        float4 hv[kItems];
        bool live[kItems];
        // the hidden rows first: they do not depend on the routing, and requests are answered in order
#pragma unroll
        for (int j = 0; j < kItems; ++j) {
            const int i = base + wave + kWaves * j;
            const int ii = i < n_items ? i : 0;
            const int sl = item_slot(ii), b = ii - sl * nb;
            const int64_t row = t * slots + sl;  // hidden row
            if (kFromF32) {
                hv[j] = *reinterpret_cast<const float4*>(p.hidden + (size_t)row * (size_t)(nb * kQK) + (size_t)b * kQK + lane * 4);
            } else {  // its 8-row tile comes along, only this row is kept
                const int64_t row0 = row & ~(int64_t)7;
                const size_t a_off[1] = {aq_row_offset(row0 + (slot >> 1), nb) + (size_t)kq * 256 + (size_t)(slot & 1) * 16};
                const int d_idx[1][2] = {{(int)ad_index(row0 + 2 * kq, 0, nb), (int)ad_index(row0 + 2 * kq + 1, 0, nb)}};
                load_a<1>(a[j], p.aq + (size_t)b * 4096, p.ad + (size_t)b * 8, a_off, d_idx);
            }
        }
        // the shared expert's gate, also ahead of the tile requests (moe_combine_kernel's order: thread j takes
        // columns j, j + 256, ... in turn; the operands are requested eight columns at a time)
        float gate_part = 0.0f;
        const bool with_gate = base == 0 && p.sh_w && p.sh_gate_inp;
        if (with_gate && tid < 256) {
            const float* gi = p.sh_gate_inp;
            const float* xr = p.x + t * p.rows;
            int64_t c = tid;
            for (; c + 7 * 256 < p.rows; c += 8 * 256) {
                float ga[8], xa[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) ga[u] = gi[c + u * 256], xa[u] = xr[c + u * 256];
#pragma unroll
                for (int u = 0; u < 8; ++u) gate_part = fmaf(ga[u], xa[u], gate_part);
            }
            for (; c < p.rows; c += 256) gate_part = fmaf(gi[c], xr[c], gate_part);
        }
        // the weight tiles: every load is issued; a missing or dropped item reads a harmless tile.  The experts
        // of all items are read out of the lanes first (branch-free), so that no tile request waits for a tile.
        const uint8_t* tile_ptr[kItems];
#pragma unroll
        for (int j = 0; j < kItems; ++j) {
            const int i = base + wave + kWaves * j;
            const int ii = i < n_items ? i : 0;
            const int sl = item_slot(ii), b = ii - sl * nb;
            const bool shared = sl >= p.top_k;
            const int e = __builtin_amdgcn_readlane(id_lane, sl & 7);
            live[j] = i < n_items && (shared || (e >= 0 && e < p.n_experts));
            const uint8_t* m = shared ? p.sh_w : p.w + (size_t)(live[j] ? e : 0) * p.expert_bytes;
            // (a harmless tile of this workgroup's own row tile: were it one fixed place for the whole launch, every
            // wavefront's spare requests would queue at the one memory channel that holds it)
            tile_ptr[j] = m + tile_offset(rt, live[j] ? b : 0, nb, kTileStride);
        }
#pragma unroll
        for (int j = 0; j < kItems; ++j) load_tile_wt<WT>(tiles[j], tile_ptr[j], lane);
        // while the tiles travel: the routing for the combine, the gate, the quantization of the hidden rows
        if (base == 0 && tid < p.top_k) ids_sh[tid] = id_lane, wts_sh[tid] = w_lane;
        if (with_gate && tid < 256) {
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) gate_part += __shfl_xor(gate_part, off, 64);
            if ((tid & 63) == 0) wave_sum[tid >> 6] = gate_part;
        }
        if (kFromF32) {
#pragma unroll
            for (int j = 0; j < kItems; ++j) {  // the row becomes row 0 of the operand
                const float e[4] = {hv[j].x, hv[j].y, hv[j].z, hv[j].w};
                a_from_lane_codes(a[j], quantize_block_q8k(e, lane), lane);
            }
        }
        if (base == 0 && p.sh_w) {
            float gate = 1.0f;
            if (p.sh_gate_inp) {
                __syncthreads();
                gate = stable_sigmoid((wave_sum[0] + wave_sum[1]) + (wave_sum[2] + wave_sum[3]));
            }
            if (tid == 0) gate_sh = gate;
        }
#pragma unroll
        for (int j = 0; j < kItems; ++j) {
            const int i = base + wave + kWaves * j;
            if (i < n_items) {  // wave-uniform
                float acc[1][2] = {{0.0f, 0.0f}};
                if (live[j]) {
                    int32_t dsum[1][2], msum[1][2];
                    compute_tile_wt<1, WT, J>(tiles[j], a[j], acc, dsum, msum, lane);
                }
                const int pos = kFromF32 ? 0 : (int)((t * slots + item_slot(i)) & 7);  // the row's place in its 8-row tile
                if (kq == (pos >> 1)) term[i * 16 + slot] = (pos & 1) ? acc[0][1] : acc[0][0];
            }
        }
    }
    __syncthreads();
    // The combine in the order of the two-launch form: a slot's super-block terms added in turn and the sum times
    // its weight -- every (slot, row) on a thread of its own -- then the slots in routing order, a row per thread.
    // A slot that the two-launch form skips (id out of range, zero weight) and the slots past the last one enter as
    // +0: the running sum starts at +0 and can never be -0, so adding +0 leaves its bits alone.
    if (tid < 9 * 16) {
        const int k = tid >> 4, r = tid & 15;
        float v = 0.0f;
        if (k < slots) {
            float part = __fadd_rn(0.0f, term[(k * nb) * 16 + r]);
            for (int b = 1; b < nb; ++b) part = __fadd_rn(part, term[(k * nb + b) * 16 + r]);
            const int e = ids_sh[k & 7];
            const float w = k < p.top_k ? wts_sh[k & 7] : gate_sh;
            const bool skip = k < p.top_k && (e < 0 || e >= p.n_experts || w == 0.0f);
            v = skip ? 0.0f : __fmul_rn(part, w);
        }
        prod[tid] = v;
    }
    __syncthreads();
    if (tid < 16) {
        const int64_t row = rt * 16 + tid;
        float v[9];
#pragma unroll
        for (int k = 0; k < 9; ++k) v[k] = prod[k * 16 + tid];
        float acc = 0.0f;
#pragma unroll
        for (int k = 0; k < 9; ++k) acc = __fadd_rn(acc, v[k]);
        if (row < p.rows) p.y[t * p.rows + row] = acc;
    }
}

// The same launch for more tokens (fp32 hidden rows): a workgroup owns `rt_per_wg` row tiles of one token and
// quantizes the token's hidden rows ONCE, into LDS -- with a workgroup per row tile every one of the 128 workgroups
// of a token repeats that, and from five tokens on the repetition is most of the launch's arithmetic.  The items
// (row tile, slot, super-block) go round the wavefronts with a ring of three tiles in flight; a row tile's terms are
// combined exactly as above (same bits).
template <int WT>
__global__ void __launch_bounds__(kWaves * 64) moe_down_rows_kernel(const MoeDownTokenArgs p) {
    constexpr int kTileStride = tile_stride<WT>();
    extern __shared__ float term[];  // [R * n_items][16] terms | [R][9][16] weighted slot sums | [n_items][64] codes | [n_items] scales
    __shared__ float wave_sum[4];
    __shared__ float gate_sh;
    __shared__ int ids_sh[8];
    __shared__ float wts_sh[8];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int slot = lane & 15, kq = lane >> 4;
    const int R = p.rt_per_wg;
    const int64_t rt0 = (int64_t)blockIdx.x * R, t = blockIdx.y;
    const int nb = (int)p.nb, slots = p.top_k + (p.sh_w ? 1 : 0), n_items = slots * nb, total = R * n_items;
    float* prod = term + total * 16;
    uint32_t* codes = reinterpret_cast<uint32_t*>(prod + R * 9 * 16);
    float* scales = reinterpret_cast<float*>(codes + n_items * 64);
    auto item_slot = [&](int i) { return nb == 1 ? i : (int)__umulhi((uint32_t)i, p.inv_nb); };       // i / nb
    auto item_tile_row = [&](int it) { return (int)__umulhi((uint32_t)it, p.inv_items); };            // it / n_items

    // the token's experts and weights in lanes 0 .. top_k-1 of every wavefront, ahead of everything that waits for them
    const int k_lane = lane < p.top_k ? lane : 0;
    const int id_lane = p.ids[t * p.top_k + k_lane];
    const float w_lane = p.weights[t * p.top_k + k_lane];
    // this wavefront's share of the hidden blocks (at most three per pass), requested before the tiles
    const float* hrow = p.hidden + (size_t)t * (size_t)slots * (size_t)(nb * kQK) + lane * 4;  // block i of the token at i * 256
    float gate_part = 0.0f;
    const bool with_gate = p.sh_w && p.sh_gate_inp;
    if (with_gate && tid < 256) {  // moe_combine_kernel's order: thread j takes columns j, j + 256, ... in turn
        const float* gi = p.sh_gate_inp;
        const float* xr = p.x + t * p.rows;
        int64_t c = tid;
        for (; c + 7 * 256 < p.rows; c += 8 * 256) {
            float ga[8], xa[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) ga[u] = gi[c + u * 256], xa[u] = xr[c + u * 256];
#pragma unroll
            for (int u = 0; u < 8; ++u) gate_part = fmaf(ga[u], xa[u], gate_part);
        }
        for (; c < p.rows; c += 256) gate_part = fmaf(gi[c], xr[c], gate_part);
    }
    for (int i0 = 0; i0 < n_items; i0 += kWaves * kItems) {
        float4 hv[kItems];
#pragma unroll
        for (int j = 0; j < kItems; ++j) {
            const int i = i0 + wave + kWaves * j;
            hv[j] = *reinterpret_cast<const float4*>(hrow + (size_t)(i < n_items ? i : 0) * kQK);
        }
#pragma unroll
        for (int j = 0; j < kItems; ++j) {
            const int i = i0 + wave + kWaves * j;
            if (i < n_items) {  // wave-uniform
                const float e[4] = {hv[j].x, hv[j].y, hv[j].z, hv[j].w};
                const Q8Lane q = quantize_block_q8k(e, lane);
                codes[i * 64 + lane] = q.packed;
                if (lane == 0) scales[i] = q.d;
            }
        }
    }
    if (tid < p.top_k) ids_sh[tid] = id_lane, wts_sh[tid] = w_lane;
    if (with_gate && tid < 256) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) gate_part += __shfl_xor(gate_part, off, 64);
        if ((tid & 63) == 0) wave_sum[tid >> 6] = gate_part;
    }
    __syncthreads();
    if (p.sh_w && tid == 0) gate_sh = with_gate ? stable_sigmoid((wave_sum[0] + wave_sum[1]) + (wave_sum[2] + wave_sum[3])) : 1.0f;

    // items wave, wave + 8, ... of the workgroup: item it = (row tile it / n_items, (slot, block) it % n_items)
    typename TileOf<WT>::Regs ring[kItems];
    bool live[kItems];
    const int cnt = wave < total ? (total - wave + kWaves - 1) >> 3 : 0;  // kWaves == 8
    auto issue = [&](int st, int q) {
        const int it = q < cnt ? wave + kWaves * q : 0;
        const int r = item_tile_row(it), i = it - r * n_items;
        const int sl = item_slot(i), b = i - sl * nb;
        const bool shared = sl >= p.top_k;
        const int e = __builtin_amdgcn_readlane(id_lane, sl & 7);
        live[st] = q < cnt && (shared || (e >= 0 && e < p.n_experts));
        const uint8_t* m = shared ? p.sh_w : p.w + (size_t)(live[st] ? e : 0) * p.expert_bytes;
        load_tile_wt<WT>(ring[st], m + tile_offset(rt0 + r, live[st] ? b : 0, nb, kTileStride), lane);  // dead: a tile of this workgroup's own rows, not one place for all
    };
#pragma unroll
    for (int st = 0; st < kItems - 1; ++st) issue(st, st);
    const int src = 8 * (slot & 1) + 2 * kq;  // this lane's words of a block's operand (a_codes_from_lane_codes)
    const uint32_t even_slot = (slot & 1) ? 0u : 0xffffffffu, odd_slot = ~even_slot;
    for (int q0 = 0; q0 < cnt; q0 += kItems) {
#pragma unroll
        for (int st = 0; st < kItems; ++st) {
            const int q = q0 + st;
            issue((st + kItems - 1) % kItems, q + kItems - 1);
            if (q < cnt) {
                const int it = wave + kWaves * q;
                const int r = item_tile_row(it), i = it - r * n_items;
                float acc[1][2] = {{0.0f, 0.0f}};
                if (live[st]) {
                    ARegs<1> a;
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const v2u v = *reinterpret_cast<const v2u*>(codes + i * 64 + 16 * c + src);
                        a.q[0][c] = v4u{v.x & even_slot, v.y & even_slot, v.x & odd_slot, v.y & odd_slot};  // as a_from_codes (q8k_block.h)
                    }
                    a.yd[0][0] = scales[i];
                    a.yd[0][1] = 0.0f;
                    int32_t dsum[1][2], msum[1][2];
                    compute_tile_wt<1, WT, 1>(ring[st], a, acc, dsum, msum, lane);
                }
                if (kq == 0) term[it * 16 + slot] = acc[0][0];
            }
        }
    }
    __syncthreads();
    // the combine of moe_down_token_kernel, per row tile
    for (int u = tid; u < R * 9 * 16; u += kWaves * 64) {
        const int r = u / 144, k = (u - r * 144) >> 4, row = u & 15;
        float v = 0.0f;
        if (k < slots) {
            const float* tr = term + (r * n_items + k * nb) * 16 + row;
            float part = __fadd_rn(0.0f, tr[0]);
            for (int b = 1; b < nb; ++b) part = __fadd_rn(part, tr[b * 16]);
            const int e = ids_sh[k & 7];
            const float w = k < p.top_k ? wts_sh[k & 7] : gate_sh;
            const bool skip = k < p.top_k && (e < 0 || e >= p.n_experts || w == 0.0f);
            v = skip ? 0.0f : __fmul_rn(part, w);
        }
        prod[u] = v;
    }
    __syncthreads();
    if (tid < R * 16) {
        const int r = tid >> 4, row = tid & 15;
        float v[9];
#pragma unroll
        for (int k = 0; k < 9; ++k) v[k] = prod[(r * 9 + k) * 16 + row];
        float acc = 0.0f;
#pragma unroll
        for (int k = 0; k < 9; ++k) acc = __fadd_rn(acc, v[k]);
        const int64_t orow = (rt0 + r) * 16 + row;
        if (orow < p.rows) p.y[t * p.rows + orow] = acc;
    }
}

}  // namespace

size_t moe_down_token_lds_bytes(int slots, int64_t nb) { return ((size_t)slots * (size_t)nb + 9) * 16 * sizeof(float); }

hipError_t launch_moe_down_token(const MoeDownTokenArgs& a, hipStream_t stream) {
    if (a.n <= 0 || a.rows <= 0 || (a.rows & 15) || a.nb <= 0 || a.top_k <= 0 || a.top_k > 8) return hipErrorInvalidValue;
    const int slots = a.top_k + (a.sh_w ? 1 : 0);
    const size_t lds = moe_down_token_lds_bytes(slots, a.nb);
    if (lds > kMoeDownTokenMaxLds) return hipErrorInvalidValue;
    const dim3 grid((unsigned)(a.rows / 16), (unsigned)a.n);
    if ((a.hidden == nullptr) == (a.aq == nullptr)) return hipErrorInvalidValue;  // one source of hidden rows
    MoeDownTokenArgs b = a;
    b.inv_nb = a.nb > 1 ? (uint32_t)(((uint64_t)1 << 32) / (uint64_t)a.nb) + 1u : 0u;  // nb < 2^16 by the LDS limit above
    // fp32 hidden rows and more workgroups than compute units: two or four row tiles of a token per workgroup, the
    // hidden rows quantized once per workgroup (moe_down_rows_kernel).  MoE block, 256 + 1 experts of 2048 x 512, with
    // at most two workgroups per compute unit instead of one: 24.2 / 26.9 us against 21.3 / 24.4 at three / four tokens.
    const int64_t rowtiles = a.rows / 16;
    int r_wg = 1;
    if (a.hidden) {
        while (r_wg < 4 && rowtiles * a.n > (int64_t)compute_units() * r_wg && rowtiles % (2 * r_wg) == 0) r_wg *= 2;
    }
    const int n_items = slots * (int)a.nb;
    if (r_wg > 1 && n_items > 1) {
        const size_t lds_rows = ((size_t)r_wg * n_items * 16 + (size_t)r_wg * 9 * 16 + (size_t)n_items * 65) * sizeof(float);
        if (lds_rows <= 48 * 1024 && (size_t)r_wg * n_items < 65536) {
            b.rt_per_wg = r_wg;
            b.inv_items = (uint32_t)(((uint64_t)1 << 32) / (uint64_t)n_items) + 1u;
            const dim3 grid_rows((unsigned)(rowtiles / r_wg), (unsigned)a.n);
            if (a.wtype == kTypeQ6K) MQ_LAUNCH(moe_down_rows_kernel<kWtQ6>, grid_rows, dim3(kWaves * 64), lds_rows, stream, b);
            else if (a.wtype == kTypeQ5K) MQ_LAUNCH(moe_down_rows_kernel<kWtQ5>, grid_rows, dim3(kWaves * 64), lds_rows, stream, b);
            else if (a.wtype == kTypeQ4K) MQ_LAUNCH(moe_down_rows_kernel<kWtQ4>, grid_rows, dim3(kWaves * 64), lds_rows, stream, b);
            else return hipErrorInvalidValue;
            return hipGetLastError();
        }
    }
#define MQ_DOWN_TOKEN(WT)                                                                                              \
    do {                                                                                                               \
        if (a.hidden) MQ_LAUNCH((moe_down_token_kernel<WT, true>), grid, dim3(kWaves * 64), lds, stream, b);  \
        else MQ_LAUNCH((moe_down_token_kernel<WT, false>), grid, dim3(kWaves * 64), lds, stream, b);          \
    } while (0)
    if (a.wtype == kTypeQ6K) MQ_DOWN_TOKEN(kWtQ6);
    else if (a.wtype == kTypeQ5K) MQ_DOWN_TOKEN(kWtQ5);
    else if (a.wtype == kTypeQ4K) MQ_DOWN_TOKEN(kWtQ4);
    else return hipErrorInvalidValue;
#undef MQ_DOWN_TOKEN
    return hipGetLastError();
}

}  // namespace mq
