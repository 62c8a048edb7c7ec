// A run of MoE decoder layers at decode width (n <= 8 tokens) as ONE persistent launch on gfx950.
//
// The reference executes a decoder graph node by node on a pool of CPU threads that meet at a spin
// barrier after every node (ggml_graph_compute as driven by core/src/llm/graph/decoder.cpp; the custom
// nodes of core/src/llm/moe/native.cpp:4831-4911).  At n <= 8 every node of such a layer moves a few
// megabytes, so on the GPU a launch per node is all latency: nine dependent launches per layer.  Here
// one workgroup per compute unit stays resident for the whole run of layers and the workgroups meet at a
// device-wide barrier between the phases of a layer, as the CPU threads do between nodes:
//
//   A  x += delta; rmsnorm; Q8_K                        (every workgroup, redundantly, into its own LDS)
//      qkv = W_qkv . q8k(h)                             row tiles spread over the workgroups        | barrier
//   B  o = W_o . q8k(qkv[:, :n_q])                      (input re-quantized by every workgroup)     | barrier
//   C  x += o; rmsnorm; Q8_K; logits = W_router . h2    one wavefront per (expert, token)           | barrier
//   D  top-k + softmax (one wavefront per token, keys in registers);
//      hidden = silu(gate_e . h2) * (up_e . h2)         per (token, slot) pair, shared expert extra | barrier
//   E  y = sum_k w_k * (down_e . q8k(hidden_k)) + sigmoid(g . h2) * shared                          | barrier
//
// The residual stream x lives in every workgroup's LDS (all replicas see the same numbers and apply the
// same arithmetic); what crosses workgroups (qkv, o, logits, hidden, y: a few KB each) is written with
// device-scope stores and read with device-scope loads, which is all the coherence the barrier needs --
// no cache write-back or invalidate.  Per-tile arithmetic, wave split of K, reduction order, rmsnorm,
// router dot, top-k, softmax and combine are those of the one-node kernels (matmul.hip, elementwise.hip,
// router.hip), so a fused run returns the bits of the node-by-node run.
//
// Barrier: two-level arrival counters (16 workgroups per first-level counter, every counter on its own
// 256-byte line) and a generation word that the waiters poll; counters return to zero by themselves.  A
// waiter gives up after a bounded time and raises a failure flag that every other waiter sees, so the
// launch always drains; the host reports the flag as an error.
#include "common.h"
#include "kernels.h"
#include "decode_tile.h"
#include "grid_sync.h"
#include "q8k_block.h"
#include "route_block.h"

namespace mq {

namespace {

constexpr int kWaves = 8;
constexpr int kThreads = kWaves * 64;
constexpr int kMaxSlots = 9;    // top_k <= 8 routed slots + the shared expert
constexpr int kMaxInterBlocks = 8;  // inter <= 2048
constexpr int kKeysPerLane = kDecoderMaxExperts / 64;

struct Shared {
    uint8_t* aq;    // A-major Q8_K codes of the current projection input, one 8-row tile: [nb][4096]
    float* ad;      // [nb][8]
    float* xres;    // residual stream [n][hidden]
    float* red;     // cross-wave partial sums [7][2][2][64]
    float* term;    // down-projection terms per (slot, super-block) [kMaxSlots][kMaxInterBlocks][16]
    float* scale;   // [8] rmsnorm scale per token
    float* gate;    // [8] shared-expert gate per token
    float* vsum;    // [32] partial sums per (token, wavefront of a 256-thread workgroup)
    float* wts;     // [8][8] routing weights
    int32_t* ids;   // [8][8] routed experts
    int* ok;        // barrier verdict of this workgroup
};

// Per-token sums over the columns in the order of a 256-thread workgroup of the one-node kernels: thread j
// takes columns j, j + 256, ... with fused multiply-adds, a butterfly inside each of the four wavefronts,
// then (w0 + w1) + (w2 + w3).  Here the (token, wavefront) pairs are spread over the eight wavefronts;
// term(t, c, acc) returns the running sum with column c of token t added, finish(t, total) consumes a total.
// kBlocks: the order of add_rmsnorm_blocks_kernel instead -- wavefront v takes the super-blocks v, v + 4, ... and
// lane l their elements 4l .. 4l+3 in turn.
template <bool kBlocks, typename Term, typename Finish>
__device__ __forceinline__ void token_sums(const Shared& s, int n, int hidden, Term term, Finish finish) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int i = wave; i < 4 * n; i += kWaves) {
        const int t = i >> 2, v = i & 3;
        float acc = 0.0f;
        if (kBlocks) {
            for (int c0 = v * kQK + lane * 4; c0 < hidden; c0 += 4 * kQK) {
#pragma unroll
                for (int q = 0; q < 4; ++q) acc = term(t, c0 + q, acc);
            }
        } else {
#pragma unroll 4
            for (int c = v * 64 + lane; c < hidden; c += 256) acc = term(t, c, acc);
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
        if (lane == 0) s.vsum[i] = acc;
    }
    __syncthreads();
    if (tid < n) finish(tid, (s.vsum[4 * tid] + s.vsum[4 * tid + 1]) + (s.vsum[4 * tid + 2] + s.vsum[4 * tid + 3]));
    __syncthreads();
}

// xres[t][c] += delta[t][c] (delta: device-scope reads; may be null), then scale[t] = 1/sqrt(mean(x^2) + eps)
// with the summation order of add_rmsnorm_kernel.
__device__ __forceinline__ void residual_norm(const Shared& s, const float* delta, int n, int hidden, float eps) {
    const int tid = threadIdx.x;
    if (delta) {
        for (int i = tid; i < n * hidden; i += kThreads) s.xres[i] = __fadd_rn(s.xres[i], ld_dev(delta + i));
        __syncthreads();
    }
    token_sums<true>(
        s, n, hidden,
        [&](int t, int c, float acc) {
            const float v = s.xres[t * hidden + c];
            return __fmaf_rn(v, v, acc);
        },
        [&](int t, float total) { s.scale[t] = __fdiv_rn(1.0f, __fsqrt_rn(__fadd_rn(__fdiv_rn(total, (float)hidden), eps))); });
}

// normalised value of column c of token t, as add_rmsnorm_kernel forms it
__device__ __forceinline__ float normed_at(const Shared& s, const float* __restrict__ weight, int t, int hidden, int c) {
    const float sw = weight ? __fmul_rn(s.scale[t], weight[c]) : s.scale[t];
    return __fmul_rn(s.xres[t * hidden + c], sw);
}

// Q8_K of n rows into the LDS A tile, one wavefront per (row, super-block).  get(t, c) returns element c of row t.
template <typename Get>
__device__ __forceinline__ void quantize_rows(const Shared& s, int n, int nb, Get get) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int u = wave; u < n * nb; u += kWaves) {
        const int t = u / nb, b = u - t * nb;
        const int c0 = b * kQK + lane * 4;
        const float e[4] = {get(t, c0), get(t, c0 + 1), get(t, c0 + 2), get(t, c0 + 3)};
        store_amajor(s.aq, s.ad, t, b, nb, lane, quantize_block_q8k(e, lane));
    }
}

// This lane's A operand of super-block b from the LDS tile (rows past the live ones read the last live row;
// their results are never stored).
__device__ __forceinline__ void load_a_lds(ARegs<1>& a, const Shared& s, int b, int n, int lane) {
    const int slot = lane & 15, kq = lane >> 4;
    const int row = (slot >> 1) < n ? (slot >> 1) : n - 1;
    const uint8_t* base = s.aq + (size_t)b * 4096 + row * 32 + kq * 256 + (slot & 1) * 16;
#pragma unroll
    for (int c = 0; c < 4; ++c) a.q[0][c] = *reinterpret_cast<const v4u*>(base + c * 1024);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int r = 2 * kq + j < n ? 2 * kq + j : n - 1;
        a.yd[0][j] = s.ad[b * 8 + r];
    }
}

// Pulls `bytes` bytes at p (16-byte aligned, a multiple of 16) towards this compute unit's caches: the whole
// workgroup reads them once and folds them into `sink`, which only exists so that the reads survive.
__device__ __forceinline__ void warm(const void* p, size_t bytes, uint32_t& sink) {
    const v4u* q = reinterpret_cast<const v4u*>(p);
    for (size_t i = threadIdx.x; i < bytes / 16; i += kThreads) {
        const v4u v = q[i];
        sink ^= v.x ^ v.y ^ v.z ^ v.w;
    }
}

// The weight tiles of super-block `wave` of row tile rt, requested ahead of their use.
template <int NMAT>
__device__ __forceinline__ void fetch_tiles(TileRegs (&t)[NMAT], const uint8_t* const (&w)[NMAT], int64_t rt, int nb) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // a wavefront past the last super-block fetches block 0 and never uses it: the load count stays uniform
    const int b = wave < nb ? wave : 0;
#pragma unroll
    for (int m = 0; m < NMAT; ++m) load_tile(t[m], w[m] + tile_offset(rt, b, nb), lane);
}

// One 16-row tile of NMAT matrices against the LDS activations: the waves split the super-blocks
// (b = wave, wave + 8, ...), partial sums meet in wave order, wave 0 ends up with the totals.  `first` holds
// the tiles of super-block `wave` (fetch_tiles).
// `order`: the wavefronts per row tile of the one-node launch whose summation order is to be kept when every
// wavefront here holds one super-block (nb <= 8): that launch adds the super-blocks w, w + order, ... in each of
// its `order` wavefronts and then the wavefronts' sums in turn.  order == 8 is this kernel's own order.
template <int NMAT>
__device__ __forceinline__ void tile_rows(const Shared& s, const TileRegs (&first)[NMAT], const uint8_t* const (&w)[NMAT],
                                          int64_t rt, int nb, int n, float (&acc)[NMAT][1][2], int order = kWaves) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
#pragma unroll
    for (int m = 0; m < NMAT; ++m) acc[m][0][0] = acc[m][0][1] = 0.0f;
    if (wave < nb) {
        ARegs<1> a;
        load_a_lds(a, s, wave, n, lane);
#pragma unroll
        for (int m = 0; m < NMAT; ++m) {
            int32_t dsum[1][2], msum[1][2];
            compute_tile<1>(first[m], a, acc[m], dsum, msum);
        }
    }
    for (int b = wave + kWaves; b < nb; b += kWaves) {
        TileRegs t[NMAT];
#pragma unroll
        for (int m = 0; m < NMAT; ++m) load_tile(t[m], w[m] + tile_offset(rt, b, nb), lane);
        ARegs<1> a;
        load_a_lds(a, s, b, n, lane);
#pragma unroll
        for (int m = 0; m < NMAT; ++m) {
            int32_t dsum[1][2], msum[1][2];
            compute_tile<1>(t[m], a, acc[m], dsum, msum);
        }
    }
    if (wave > 0) {
#pragma unroll
        for (int m = 0; m < NMAT; ++m)
#pragma unroll
            for (int j = 0; j < 2; ++j) s.red[(((wave - 1) * NMAT + m) * 2 + j) * 64 + lane] = acc[m][0][j];
    }
    __syncthreads();
    if (wave == 0) {
        if (order >= kWaves || nb > kWaves) {
            for (int wv = 1; wv < kWaves; ++wv) {
#pragma unroll
                for (int m = 0; m < NMAT; ++m)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        acc[m][0][j] = __fadd_rn(acc[m][0][j], s.red[(((wv - 1) * NMAT + m) * 2 + j) * 64 + lane]);
            }
        } else {
            // wavefront wv of this kernel holds the term of super-block wv alone (zero past the last one)
            float total[NMAT][2];
            for (int ow = 0; ow < order; ++ow) {
                float part[NMAT][2];
#pragma unroll
                for (int m = 0; m < NMAT; ++m)
#pragma unroll
                    for (int j = 0; j < 2; ++j) part[m][j] = ow == 0 ? acc[m][0][j] : s.red[(((ow - 1) * NMAT + m) * 2 + j) * 64 + lane];
                for (int b = ow + order; b < nb; b += order) {
#pragma unroll
                    for (int m = 0; m < NMAT; ++m)
#pragma unroll
                        for (int j = 0; j < 2; ++j) part[m][j] = __fadd_rn(part[m][j], s.red[(((b - 1) * NMAT + m) * 2 + j) * 64 + lane]);
                }
#pragma unroll
                for (int m = 0; m < NMAT; ++m)
#pragma unroll
                    for (int j = 0; j < 2; ++j) total[m][j] = ow == 0 ? part[m][j] : __fadd_rn(total[m][j], part[m][j]);
            }
#pragma unroll
            for (int m = 0; m < NMAT; ++m)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[m][0][j] = total[m][j];
        }
    }
}

// Dense projection of the LDS activations: y[t][row] for every live token, row tiles spread over the grid.
// `first` holds the tiles of this workgroup's first row tile (requested during the barrier that precedes the
// phase); the next row tile's are requested before the current one is multiplied.
__device__ __forceinline__ void dense_phase(const Shared& s, const uint8_t* w, int64_t rows, int nb, int n, float* y,
                                            int64_t ldy, TileRegs (&first)[1]) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int slot = lane & 15, kq = lane >> 4;
    const int64_t rowtiles = (rows + 15) >> 4;
    const uint8_t* const ws[1] = {w};
    for (int64_t rt = blockIdx.x; rt < rowtiles; rt += gridDim.x) {
        TileRegs next[1];
        const bool more = rt + gridDim.x < rowtiles;
        if (more) fetch_tiles<1>(next, ws, rt + gridDim.x, nb);
        float acc[1][1][2];
        tile_rows<1>(s, first, ws, rt, nb, n, acc);
        const int64_t row = rt * 16 + slot;
        if (wave == 0 && row < rows) {
#pragma unroll
            for (int j = 0; j < 2; ++j)
                if (2 * kq + j < n) st_dev(y + (size_t)(2 * kq + j) * ldy + row, acc[0][0][j]);
        }
        __syncthreads();  // red[] is reused by the next row tile
        if (more) first[0] = next[0];
    }
}

constexpr int kItems = 3;  // (slot, super-block) items of the down projection a wavefront keeps in flight

__global__ void __launch_bounds__(kThreads) decoder_layers_kernel(const DecoderArgs p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int slot = lane & 15, kq = lane >> 4;
    const int n = p.n, hidden = p.hidden, inter = p.inter, top_k = p.top_k, n_experts = p.n_experts;
    const int nb_h = hidden / kQK, nb_q = p.n_q / kQK, nb_i = inter / kQK;
    const int nb_max = nb_h > nb_q ? nb_h : nb_q;
    const int slots = top_k + (p.has_shared ? 1 : 0);

    Shared s;
    {
        uint8_t* at = lds_raw;
        s.aq = at;
        at += (size_t)nb_max * 4096;
        s.ad = reinterpret_cast<float*>(at);
        at += (size_t)nb_max * 8 * sizeof(float);
        s.xres = reinterpret_cast<float*>(at);
        at += (size_t)n * hidden * sizeof(float);
        s.red = reinterpret_cast<float*>(at);
        at += (size_t)(kWaves - 1) * 2 * 2 * 64 * sizeof(float);
        s.term = reinterpret_cast<float*>(at);
        at += (size_t)kMaxSlots * kMaxInterBlocks * 16 * sizeof(float);
        s.scale = reinterpret_cast<float*>(at);
        s.gate = s.scale + 8;
        s.vsum = s.gate + 8;
        s.wts = s.vsum + 32;
        s.ids = reinterpret_cast<int32_t*>(s.wts + 64);
        s.ok = reinterpret_cast<int*>(s.ids + 64);
    }
    if (ld_dev(p.sync + 2 * kSyncLine) != 0u) return;  // an earlier launch abandoned a barrier: the state is unusable
    uint32_t my_gen = ld_dev(p.sync + kSyncLine);      // cannot move before this workgroup's own first arrival
    uint32_t sink = 0u;  // see warm()

    // Weights of this workgroup's first row tile of a dense projection, requested a phase ahead.  Workgroups
    // without a row tile fetch tile 0 and never use it, so that the registers are defined on every path.
    auto request_dense = [&](TileRegs (&dst)[1], const uint8_t* w, int64_t rows, int nb) {
        const uint8_t* const ws[1] = {w};
        fetch_tiles<1>(dst, ws, (int64_t)blockIdx.x < ((rows + 15) >> 4) ? blockIdx.x : 0, nb);
    };
    TileRegs ahead_qkv[1];
    request_dense(ahead_qkv, p.layers[0].wqkv, p.layers[0].qkv_rows, nb_h);

    for (int i = tid; i < n * hidden; i += kThreads) s.xres[i] = p.x_in[i];
    __syncthreads();

    // sigmoid(sh_gate_inp . h2[t]) with the summation order of moe_combine_kernel; h2 = the MoE block's input
    auto shared_gates = [&](const DecoderLayerDev& L) {
        if (!p.has_shared) return;
        if (!L.sh_gate_inp) {
            if (tid < n) s.gate[tid] = 1.0f;
            __syncthreads();
            return;
        }
        const float* gi = L.sh_gate_inp;
        const float* wn = L.ffn_norm;
        token_sums<false>(
            s, n, hidden,
            [&](int t, int c, float acc) { return fmaf(gi[c], normed_at(s, wn, t, hidden, c), acc); },
            [&](int t, float total) { s.gate[t] = stable_sigmoid(total); });
    };

    const float* delta = nullptr;
    for (int li = 0; li < p.n_layers; ++li) {
        const DecoderLayerDev& L = p.layers[li];

        // ---- A: residual add, rmsnorm, Q8_K, qkv projection -------------------------------------------
        residual_norm(s, delta, n, hidden, p.eps);
        {
            const float* wn = L.attn_norm;
            quantize_rows(s, n, nb_h, [&](int t, int c) { return normed_at(s, wn, t, hidden, c); });
        }
        __syncthreads();
        dense_phase(s, L.wqkv, L.qkv_rows, nb_h, n, p.qkv, L.qkv_rows, ahead_qkv);
        TileRegs ahead_wo[1];
        if (!grid_barrier(p.sync, my_gen, s.ok, p.spin_ticks, [&] { request_dense(ahead_wo, L.wo, hidden, nb_q); })) return;

        // ---- B: output projection of the first n_q columns ---------------------------------------------
        {
            const float* src = p.qkv;
            const int64_t ld = L.qkv_rows;
            quantize_rows(s, n, nb_q, [&](int t, int c) { return ld_dev(src + (size_t)t * ld + c); });
        }
        __syncthreads();
        dense_phase(s, L.wo, hidden, nb_q, n, p.o, hidden, ahead_wo);
        if (!grid_barrier(p.sync, my_gen, s.ok, p.spin_ticks, [&] {
                // what phase C reads that does not depend on o: this workgroup's first router row, the gate vector
                if ((int)blockIdx.x < n_experts) warm(L.router + (size_t)blockIdx.x * hidden, (size_t)hidden * 4, sink);
                if (p.has_shared && L.sh_gate_inp) warm(L.sh_gate_inp, (size_t)hidden * 4, sink);
            }))
            return;

        // ---- C: residual add, rmsnorm, Q8_K, router projection -----------------------------------------
        residual_norm(s, p.o, n, hidden, p.eps);
        {
            const float* wn = L.ffn_norm;
            quantize_rows(s, n, nb_h, [&](int t, int c) { return normed_at(s, wn, t, hidden, c); });
        }
        __syncthreads();
        // one wavefront per (token, expert), the dot of router_logits_kernel; the last wavefront takes the
        // first unit so that the gates below, which start with the first wavefronts, run beside it
        for (int u = (kWaves - 1 - wave) * gridDim.x + blockIdx.x; u < n * n_experts; u += kWaves * gridDim.x) {
            const int t = u / n_experts, e = u - t * n_experts;
            const float* wr = L.router + (size_t)e * hidden;
            float acc = 0.0f;
            for (int c = lane * 4; c + 3 < hidden; c += 256) {
                const float4 a = *reinterpret_cast<const float4*>(wr + c);
                acc = __fmaf_rn(a.x, normed_at(s, L.ffn_norm, t, hidden, c), acc);
                acc = __fmaf_rn(a.y, normed_at(s, L.ffn_norm, t, hidden, c + 1), acc);
                acc = __fmaf_rn(a.z, normed_at(s, L.ffn_norm, t, hidden, c + 2), acc);
                acc = __fmaf_rn(a.w, normed_at(s, L.ffn_norm, t, hidden, c + 3), acc);
            }
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
            if (lane == 0) st_dev(p.logits + (size_t)t * n_experts + e, acc);
        }
        shared_gates(L);
        if (!grid_barrier(p.sync, my_gen, s.ok, p.spin_ticks, [&] {
                // the shared expert's gate/up tiles of this workgroup's first unit do not wait for the routing
                if (p.has_shared && (int)blockIdx.x < inter / 16) {
                    warm(L.sh_gate + tile_offset(blockIdx.x, 0, nb_h), (size_t)nb_h * kTileBytes, sink);
                    warm(L.sh_up + tile_offset(blockIdx.x, 0, nb_h), (size_t)nb_h * kTileBytes, sink);
                }
            }))
            return;

        // ---- D: routing, then gate/up + SwiGLU per (token, slot) and for the shared expert -------------------
        float routed_logit = 0.0f;  // lane k of wavefront t: logit of token t's k-th expert
        if (wave < n) {
            const bool fixed = L.fixed_logits != nullptr;
            const float* row = (fixed ? L.fixed_logits : p.logits) + (size_t)wave * n_experts;
            auto load = [&](int e) { return fixed ? row[e] : ld_dev(row + e); };
            int id;
            if (n_experts <= 256) route_token_wave<4>(load, n_experts, top_k, lane, id, routed_logit);
            else route_token_wave<kKeysPerLane>(load, n_experts, top_k, lane, id, routed_logit);
            if (lane < top_k) s.ids[wave * 8 + lane] = id;
        }
        __syncthreads();
        {
            const int rt_i = inter / 16;
            const int pairs = n * top_k;
            const int sh_units = p.has_shared ? rt_i : 0;
            const int units = sh_units + pairs * rt_i;
            // unit u -> (shared pass or (token, slot) pair, row tile); a dropped pair (id out of range) has no
            // weights.  The shared expert's units come first: their weights do not wait for the routing and
            // were pulled into cache during the barrier.
            auto unit_weights = [&](int u, const uint8_t* (&ws)[2], int& t, int& k, int& rt, bool& shared) -> bool {
                shared = u < sh_units;
                const int g = shared ? 0 : (u - sh_units) / rt_i;
                rt = shared ? u : (u - sh_units) - g * rt_i;
                t = shared ? 0 : g / top_k;
                k = shared ? top_k : g - t * top_k;
                const int e = shared ? 0 : s.ids[t * 8 + k];
                if (!shared && (e < 0 || e >= n_experts)) return false;
                ws[0] = shared ? L.sh_gate : L.gate_exps + (size_t)e * L.gu_expert_bytes;
                ws[1] = shared ? L.sh_up : L.up_exps + (size_t)e * L.gu_expert_bytes;
                return true;
            };
            TileRegs cur[2], nxt[2];
            const uint8_t* ws[2];
            const uint8_t* wn[2];
            int t = 0, k = 0, rt = 0, tn = 0, kn = 0, rtn = 0;
            bool shared = false, sharedn = false;
            // Every fetch is issued whether or not the unit exists: the number of loads in flight is then the same
            // on every path and the waits can count them.
            // (a missing unit re-reads `again`, tiles that were fetched a moment ago and still sit in cache)
            auto fetch_unit = [&](int u, TileRegs (&dst)[2], const uint8_t* (&w)[2], int& tt, int& kk, int& rr, bool& sh,
                                  const uint8_t* const (&again)[2], int again_rt) -> bool {
                bool live = false;
                if (u < units) live = unit_weights(u, w, tt, kk, rr, sh);
                if (!live) {
                    w[0] = again[0], w[1] = again[1];
                    rr = again_rt;
                }
                const uint8_t* const wc[2] = {w[0], w[1]};
                fetch_tiles<2>(dst, wc, rr, nb_h);
                return live;
            };
            const uint8_t* const cold[2] = {L.gate_exps, L.up_exps};
            bool live = fetch_unit(blockIdx.x, cur, ws, t, k, rt, shared, cold, 0);
            for (int u = blockIdx.x; u < units; u += gridDim.x) {
                const uint8_t* const here[2] = {ws[0], ws[1]};
                const bool live_n = fetch_unit(u + gridDim.x, nxt, wn, tn, kn, rtn, sharedn, here, rt);
                if (live) {  // the whole workgroup takes the same branch
                    const uint8_t* const wc[2] = {ws[0], ws[1]};
                    float acc[2][1][2];
                    tile_rows<2>(s, cur, wc, rt, nb_h, n, acc, p.gateup_order);
                    if (wave == 0) {
                        const int mode = shared ? 2 : p.silu_mode;
#pragma unroll
                        for (int j = 0; j < 2; ++j) {
                            const int r = 2 * kq + j;  // activation row of this accumulator
                            if (r < n && (shared || r == t))
                                st_dev(p.mid + ((size_t)r * slots + k) * inter + rt * 16 + slot,
                                       silu_mul(acc[0][0][j], acc[1][0][j], mode));
                        }
                    }
                    __syncthreads();
                }
                live = live_n;
                cur[0] = nxt[0], cur[1] = nxt[1];
                ws[0] = wn[0], ws[1] = wn[1];
                t = tn, k = kn, rt = rtn, shared = sharedn;
            }
        }

        // ---- E: down projection per slot, weighted combine in routing order -----------------------------------
        // A unit is one (token, 16-row tile); its slots x super-blocks are spread over the wavefronts.
        const int rt_h = hidden / 16;
        const int n_items = slots * nb_i;
        TileRegs etile[kItems];
        auto item_tile = [&](int t, int rt, int i) -> const uint8_t* {  // null for a dropped slot
            const int sl = i / nb_i, b = i - sl * nb_i;
            const bool shared = sl >= top_k;
            const int e = shared ? 0 : s.ids[t * 8 + sl];
            if (!shared && (e < 0 || e >= n_experts)) return nullptr;
            return (shared ? L.sh_down : L.down_exps + (size_t)e * L.down_expert_bytes) + tile_offset(rt, b, nb_i);
        };
        auto fetch_items = [&](int t, int rt, int base) {
#pragma unroll
            for (int j = 0; j < kItems; ++j) {
                const int i = base + wave + kWaves * j;
                const uint8_t* w = i < n_items ? item_tile(t, rt, i) : nullptr;
                load_tile(etile[j], w ? w : L.down_exps, lane);  // a dropped item reads a harmless tile
            }
        };
        const bool e_unit = (int)blockIdx.x < n * rt_h;
        if (!grid_barrier(p.sync, my_gen, s.ok, p.spin_ticks, [&] {
                if (e_unit) fetch_items(blockIdx.x / rt_h, blockIdx.x % rt_h, 0);
            }))
            return;

        // quantize this wavefront's hidden blocks, multiply them by the tiles in etile[], park the terms in LDS
        auto load_hidden = [&](float (&ev)[kItems][4], int t, int base) {
#pragma unroll
            for (int j = 0; j < kItems; ++j) {
                const int i = base + wave + kWaves * j;
                const int ii = i < n_items ? i : 0;
                const int sl = ii / nb_i, b = ii - sl * nb_i;
                const float* hrow = p.mid + ((size_t)t * slots + sl) * inter + b * kQK + lane * 4;
#pragma unroll
                for (int q = 0; q < 4; ++q) ev[j][q] = ld_dev(hrow + q);
            }
        };
        auto multiply_items = [&](const float (&ev)[kItems][4], int t, int rt, int base) {
#pragma unroll
            for (int j = 0; j < kItems; ++j) {
                const int i = base + wave + kWaves * j;
                if (i < n_items) {  // wave-uniform
                    float acc[1][2] = {{0.0f, 0.0f}};
                    if (item_tile(t, rt, i)) {
                        ARegs<1> a;
                        a_from_lane_codes(a, quantize_block_q8k(ev[j], lane), lane);
                        int32_t dsum[1][2], msum[1][2];
                        compute_tile<1>(etile[j], a, acc, dsum, msum);
                    }
                    if (kq == 0) s.term[i * 16 + slot] = acc[0][0];
                }
            }
        };
        float ev[kItems][4];
        if (e_unit) load_hidden(ev, blockIdx.x / rt_h, 0);
        // the routing weights are first needed by the combine below: formed while the hidden rows travel
        if (wave < n) {
            const float w = route_weight_lane(routed_logit, lane, top_k, p.route_mode);
            if (lane < top_k) {
                s.wts[wave * 8 + lane] = w;
                if (blockIdx.x == 0) {
                    if (p.ids_out) p.ids_out[((size_t)li * n + wave) * top_k + lane] = s.ids[wave * 8 + lane];
                    if (p.wts_out) p.wts_out[((size_t)li * n + wave) * top_k + lane] = w;
                }
            }
        }
        for (int u = blockIdx.x; u < n * rt_h; u += gridDim.x) {
            const int t = u / rt_h, rt = u - t * rt_h;
            if (u != (int)blockIdx.x) {  // the first unit's tiles and hidden rows are already on their way
                fetch_items(t, rt, 0);
                load_hidden(ev, t, 0);
            }
            multiply_items(ev, t, rt, 0);
            for (int base = kWaves * kItems; base < n_items; base += kWaves * kItems) {
                fetch_items(t, rt, base);
                load_hidden(ev, t, base);
                multiply_items(ev, t, rt, base);
            }
            __syncthreads();
            if (tid < 16) {
                // per slot the super-block terms in order, then the slots in routing order (moe_combine_kernel)
                float acc = 0.0f;
                for (int k = 0; k < slots; ++k) {
                    float part = s.term[(k * nb_i) * 16 + tid];
                    for (int b = 1; b < nb_i; ++b) part = __fadd_rn(part, s.term[(k * nb_i + b) * 16 + tid]);
                    if (k < top_k) {
                        const int e = s.ids[t * 8 + k];
                        const float w = s.wts[t * 8 + k];
                        if (e < 0 || e >= n_experts || w == 0.0f) continue;
                        acc = __fadd_rn(acc, __fmul_rn(part, w));
                    } else {
                        acc = __fadd_rn(acc, __fmul_rn(part, s.gate[t]));
                    }
                }
                st_dev(p.y + (size_t)t * hidden + rt * 16 + tid, acc);
            }
            __syncthreads();
        }
        {
            // the next layer's first projection (the last layer re-requests its own: unused, but defined)
            const DecoderLayerDev& N = p.layers[li + 1 < p.n_layers ? li + 1 : li];
            if (!grid_barrier(p.sync, my_gen, s.ok, p.spin_ticks, [&] {
                    request_dense(ahead_qkv, N.wqkv, N.qkv_rows, nb_h);
                }))
                return;
        }
        delta = p.y;
    }

    // ---- the last residual add ---------------------------------------------------------------------------------
    for (int i = blockIdx.x * kThreads + tid; i < n * hidden; i += gridDim.x * kThreads)
        p.out[i] = __fadd_rn(s.xres[i], ld_dev(p.y + i));
    if (sink == 0x9e3779b9u && p.n < 0) p.out[0] = 0.0f;  // never true: keeps the warm-up reads alive
}

}  // namespace

size_t decoder_layers_lds_bytes(const DecoderArgs& a) {
    const int nb_h = a.hidden / kQK, nb_q = a.n_q / kQK;
    const int nb_max = nb_h > nb_q ? nb_h : nb_q;
    return (size_t)nb_max * 4096 + (size_t)nb_max * 8 * 4 + (size_t)a.n * a.hidden * 4 + (size_t)(kWaves - 1) * 2 * 2 * 64 * 4 +
           (size_t)kMaxSlots * kMaxInterBlocks * 16 * 4 + (8 + 8 + 32 + 64 + 64 + 4) * 4;
}

size_t decoder_sync_bytes(int n_workgroups) {
    return (size_t)(4 + (n_workgroups + kSyncGroup - 1) / kSyncGroup) * kSyncLine * sizeof(uint32_t);
}

hipError_t prepare_decoder_layers(size_t lds_bytes) {
    return hipFuncSetAttribute(reinterpret_cast<const void*>(decoder_layers_kernel),
                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
}

hipError_t launch_decoder_layers(const DecoderArgs& a, int n_workgroups, hipStream_t stream) {
    if (!a.layers || a.n_layers < 1 || a.n < 1 || a.n > 8 || a.top_k < 1 || a.top_k > 8 || a.n_experts < a.top_k || a.n_experts > kDecoderMaxExperts ||
        a.hidden <= 0 || (a.hidden % kQK) || a.inter <= 0 || (a.inter % kQK) || a.inter > kMaxInterBlocks * kQK ||
        n_workgroups < 1 || a.n_q <= 0 || (a.n_q % kQK))
        return hipErrorInvalidValue;
    MQ_LAUNCH(decoder_layers_kernel, dim3((unsigned)n_workgroups), dim3(kThreads), decoder_layers_lds_bytes(a),
                       stream, a);
    return hipGetLastError();
}

}  // namespace mq
