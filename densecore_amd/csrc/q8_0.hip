// Q8_0 weights x Q8_0 activations at decode widths: y[m][r] = sum_blocks fp16(dx) * fp16(dy) * sum_32 qx * qy.
//
// The reference sends Q8_0 weight matrices (token embeddings used as output head, some attention tensors of
// mixed-precision files) through the same GEMV / small-batch callbacks as the K-quants, with the activations
// quantized to Q8_0 too (core/src/llm/matmul/batched_exec.cpp:630; four-column kernel Q8SmallBatchDot4,
// core/src/llm/matmul/q8_small_batch.h:29-77: per 32-weight block an integer dot and one fused multiply-add with
// fp16(dx) * fp16(dy)).  Here:
//   * quantize_q80_kernel: one wavefront per (row, 256 values): the maximum magnitude of each 32-value block over
//     its eight lanes, d = amax / 127 stored as fp16, codes = round-half-even(x * (127 / amax)) -- ggml's x86
//     quantizer, which lives in a submodule the reference tree does not carry (its parity is unpinned) -- written
//     as the split-slot A operand of common.h (the element order of Q8_K's codes) plus eight fp16 scales per row
//     and 256 values;
//   * q80_matmul_kernel: workgroup = 16 weight rows, its wavefronts split the 256-weight groups of the row and keep
//     a ring of tiles in flight as matmul_kernel does; one K=64 MFMA yields the integer sums of two 32-weight
//     blocks for eight activation rows; acc = fma(dx * dy, float(sum), acc) block by block; partial sums of the
//     wavefronts meet in wave order.  More than eight rows: passes of eight over the same 16 weight rows.
// Integer block sums are exact (mq_debug_block_sums writes them out); fp32 differs from the reference's eight-lane
// order by rounding only.
#include "common.h"
#include "kernels.h"
#include "decode_tile.h"

namespace mq {

namespace {

constexpr int kStages = 3;

__global__ void __launch_bounds__(256) quantize_q80_kernel(const float* __restrict__ x, int64_t n, int64_t ldx, int64_t nb,
                                                           uint8_t* __restrict__ aq, uint16_t* __restrict__ ah) {
    const int lane = threadIdx.x & 63;
    const int64_t unit = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (unit >= n * nb) return;
    int64_t m, b;
    split_unit(unit, nb, m, b);
    const float4 v = *reinterpret_cast<const float4*>(x + m * ldx + b * kQK + lane * 4);
    const float e[4] = {v.x, v.y, v.z, v.w};
    float local = fmaxf(fmaxf(fabsf(e[0]), fabsf(e[1])), fmaxf(fabsf(e[2]), fabsf(e[3])));
    // largest magnitude of the block = of the eight lanes 8g .. 8g+7 (non-negative floats order like their bits)
    uint32_t a = __float_as_uint(local), t;
    t = dpp_u32<kDppXor1>(a);
    a = t > a ? t : a;
    t = dpp_u32<kDppXor2>(a);
    a = t > a ? t : a;
    t = dpp_u32<kDppHalfMirror>(a);
    a = t > a ? t : a;
    const float amax = __uint_as_float(a);
    const float d = __fdiv_rn(amax, 127.0f);
    const float id = amax != 0.0f ? __fdiv_rn(127.0f, amax) : 0.0f;
    uint32_t packed = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) packed |= ((uint32_t)(int)rintf(__fmul_rn(e[j], id)) & 0xffu) << (8 * j);
    // element 4*lane+j: block g = lane/8, index 4*(lane%8)+j; the codes go to the half of the row's slot that
    // belongs to the block's parity, zeros to the other half (the A-major layout of common.h)
    const int g = lane >> 3, h = g & 1, kq = (lane & 7) >> 1;
    const size_t off = aq_offset(m, b, g >> 1, kq, h, nb) + (size_t)(lane & 1) * 4;
    *reinterpret_cast<uint32_t*>(aq + off + h * 8) = packed;
    *reinterpret_cast<uint32_t*>(aq + off + (1 - h) * 8) = 0u;
    if ((lane & 7) == 0) ah[ad_index(m, b, nb) * 8 + g] = __half_as_ushort(__float2half_rn(d));
}

struct Tile80 {
    v4u q[4];  // B operands of the four 64-weight chunks
    v4u sc;    // the eight fp16 d of weight row lane % 16
};
struct A80 {
    v4u q[4];    // split-slot A operand
    v4u s0, s1;  // the eight fp16 d of activation rows 2 kq and 2 kq + 1
};

__device__ __forceinline__ void unpack_halves(const v4u w, float (&out)[8]) {
    const uint32_t words[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        out[2 * i] = half_bits_to_float(words[i] & 0xffffu);
        out[2 * i + 1] = half_bits_to_float(words[i] >> 16);
    }
}

__global__ void __launch_bounds__(512) q80_matmul_kernel(const Q80MatmulArgs p) {
    extern __shared__ float red[];  // [W-1][2][64]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n_waves = blockDim.x >> 6;
    const int slot = lane & 15, kq = lane >> 4;
    int64_t rt = blockIdx.x;
    const int nb = (int)p.nb;
    const uint8_t* w = p.w;
    int first = 0, last = (int)p.n;  // activation rows this workgroup multiplies (dense, pairs), or entries of its group
    int g_begin = 0;                 // expert-grouped: first entry of the group (or first token of a shared-expert pass)
    bool g_shared = false;
    const bool grouped = p.group_begin != nullptr;
    if (p.pair_ids) {
        // expert-routed: the grid is flat, workgroup = column g * rowtiles + row tile (a grid's second dimension ends
        // at 65535, a prefill-width block has more pairs); column g is hidden row g = token * slots + slot alone,
        // against the expert that the token's slot names (slots past top_k: the shared expert); rows of dropped
        // pairs are left as they are
        const uint32_t rowtiles = (uint32_t)((p.rows + 15) >> 4);
        const int g = (int)(blockIdx.x / rowtiles), tok = g / p.slots, k = g - tok * p.slots;
        rt = (int64_t)(blockIdx.x - (uint32_t)g * rowtiles);
        if (k < p.top_k) {
            const int e = p.pair_ids[tok * p.top_k + k];
            if (e < 0 || e >= p.n_experts) return;  // the whole workgroup, before any barrier
            w += (size_t)e * p.expert_bytes;
        } else {
            w = p.sh_w;
        }
        first = g;
        last = g + 1;
    } else if (grouped) {
        const int g = blockIdx.y, ng = *p.n_groups;
        const int gi = g < p.max_groups ? g : 0;  // columns of the shared expert read group 0's entries and drop them
        const int g_expert = p.group_expert[gi], b0 = p.group_begin[gi], b1 = p.group_begin[gi + 1];
        if (g < ng) {
            w += (size_t)g_expert * p.expert_bytes;
            g_begin = b0;
            last = b1 - b0;
        } else if (g - ng < (p.sh_tokens + kTokTile - 1) / kTokTile) {
            g_shared = true;
            w = p.sh_w;
            g_begin = (g - ng) * kTokTile;
            last = p.sh_tokens - g_begin < kTokTile ? p.sh_tokens - g_begin : kTokTile;
        } else {
            return;  // the whole workgroup, before any barrier
        }
    }
    // hidden / output row of entry e of the group
    auto group_row = [&](int e) {
        if (g_shared) return (g_begin + e) * p.slots + p.top_k;
        return p.entry_token[g_begin + e] * p.slots + p.entry_k[g_begin + e];
    };
    const uint8_t* tiles = w + tile_offset(rt, 0, nb, kTile80Bytes);
    const int cnt = wave < nb ? (nb - wave + n_waves - 1) / n_waves : 0;  // 256-weight groups wave, wave + W, ...

    for (int chunk = first; chunk < last; chunk += kTokTile) {
        const int count = last - chunk < kTokTile ? last - chunk : kTokTile;
        // a dead slot reads a live row of the pass and stores nothing
        const int a_ent = chunk + ((slot >> 1) < count ? (slot >> 1) : count - 1);
        const int arow = grouped ? group_row(a_ent) : a_ent;
        const size_t a_off = aq_row_offset(arow, nb) + (size_t)kq * 256 + (size_t)(slot & 1) * 16;
        int yrow[2];
        size_t s_off[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const bool live = 2 * kq + j < count;
            const int ent = chunk + (live ? 2 * kq + j : count - 1);
            const int r = grouped ? group_row(ent) : ent;
            yrow[j] = live ? r : -1;
            s_off[j] = ad_index(r, 0, nb) * 8;  // + b * 64 halves per group
        }
        float acc[2] = {0.0f, 0.0f};
        if (cnt > 0) {
            Tile80 ring_t[kStages];
            A80 ring_a[kStages];
            auto issue = [&](int st, int i) {
                const int b = i < cnt ? wave + i * n_waves : wave;  // past the end: the first group again, the load count stays fixed
                const uint8_t* tile = tiles + (size_t)b * kTile80Bytes;
#pragma unroll
                for (int c = 0; c < 4; ++c) ring_t[st].q[c] = load_stream16(tile + c * 1024 + lane * 16);
                ring_t[st].sc = load_stream16(tile + kTile80SOff + slot * 16);
#pragma unroll
                for (int c = 0; c < 4; ++c) ring_a[st].q[c] = load16(p.aq + (size_t)b * 4096 + a_off + c * 1024);
                ring_a[st].s0 = load16(p.ah + s_off[0] + (size_t)b * 64);
                ring_a[st].s1 = load16(p.ah + s_off[1] + (size_t)b * 64);
            };
#pragma unroll
            for (int st = 0; st < kStages - 1; ++st) issue(st, st);
            for (int base = 0; base < cnt; base += kStages) {
#pragma unroll
                for (int st = 0; st < kStages; ++st) {
                    const int i = base + st;
                    issue((st + kStages - 1) % kStages, i + kStages - 1);
                    if (i < cnt) {
                        float dx[8], dy[2][8];
                        unpack_halves(ring_t[st].sc, dx);
                        unpack_halves(ring_a[st].s0, dy[0]);
                        unpack_halves(ring_a[st].s1, dy[1]);
#pragma unroll
                        for (int c = 0; c < 4; ++c) {
                            const v4u av = ring_a[st].q[c], bv = ring_t[st].q[c];
                            const v4i a16 = {(int)av.x, (int)av.y, (int)av.z, (int)av.w};
                            const v4i b16 = {(int)bv.x, (int)bv.y, (int)bv.z, (int)bv.w};
                            const v4i zero = {0, 0, 0, 0};
                            // s[0], s[2]: block 2c of activation rows 2kq and 2kq+1;  s[1], s[3]: block 2c+1
                            const v4i s = __builtin_amdgcn_mfma_i32_16x16x64_i8(a16, b16, zero, 0, 0, 0);
#pragma unroll
                            for (int j = 0; j < 2; ++j)
#pragma unroll
                                for (int h = 0; h < 2; ++h) {
                                    const int k = 2 * c + h;
                                    acc[j] = __fmaf_rn(__fmul_rn(dx[k], dy[j][k]), (float)s[2 * j + h], acc[j]);
                                    if (p.dbg_sum && yrow[j] >= 0 && rt * 16 + slot < p.rows)
                                        p.dbg_sum[(((size_t)(rt * 16 + slot) * (size_t)p.n + (size_t)yrow[j]) * (size_t)nb +
                                                   (size_t)(wave + i * n_waves)) * 8 + k] = s[2 * j + h];
                                }
                        }
                    }
                }
            }
        }
        if (n_waves > 1) {
            if (wave > 0) {
                red[((wave - 1) * 2 + 0) * 64 + lane] = acc[0];
                red[((wave - 1) * 2 + 1) * 64 + lane] = acc[1];
            }
            __syncthreads();
        }
        if (wave == 0) {
            for (int wv = 1; wv < n_waves; ++wv) {
                acc[0] = __fadd_rn(acc[0], red[((wv - 1) * 2 + 0) * 64 + lane]);
                acc[1] = __fadd_rn(acc[1], red[((wv - 1) * 2 + 1) * 64 + lane]);
            }
            const int64_t row = rt * 16 + slot;
            if (row < p.rows) {
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    if (yrow[j] >= 0) p.y[(size_t)yrow[j] * (size_t)p.ldy + (size_t)row] = acc[j];
            }
        }
        if (n_waves > 1 && chunk + kTokTile < last) __syncthreads();  // red[] is reused by the next pass
    }
}

}  // namespace

size_t q80_scale_bytes(int64_t n, int64_t nb) { return ad_count(n, nb) * 8 * sizeof(uint16_t); }

hipError_t launch_quantize_q80(const float* x, int64_t n, int64_t ldx, int64_t cols, uint8_t* aq, uint16_t* ah, hipStream_t stream) {
    const int64_t nb = cols / kQK, units = n * nb;
    if (units == 0) return hipSuccess;
    if (units >= (int64_t)1 << 31) return hipErrorInvalidValue;  // split_unit divides in 32 bits
    if ((cols % kQK) || ldx < cols || (ldx & 3) || (reinterpret_cast<uintptr_t>(x) & 15u)) return hipErrorInvalidValue;
    MQ_LAUNCH(quantize_q80_kernel, dim3((unsigned)((units + 3) / 4)), dim3(256), 0, stream, x, n, ldx, nb, aq, ah);
    return hipGetLastError();
}

hipError_t launch_q80_matmul(const Q80MatmulArgs& a, hipStream_t stream) {
    if (a.rows <= 0 || a.nb <= 0 || a.n <= 0 || !a.w || !a.aq || !a.ah || !a.y || a.ldy < a.rows) return hipErrorInvalidValue;
    const bool grouped = a.group_begin != nullptr;
    if ((a.pair_ids || grouped) && (a.top_k <= 0 || a.slots < a.top_k || a.n % a.slots || a.dbg_sum || (a.slots > a.top_k && !a.sh_w)))
        return hipErrorInvalidValue;
    if (grouped && (a.pair_ids || !a.group_expert || !a.n_groups || !a.entry_token || !a.entry_k || a.max_groups <= 0)) return hipErrorInvalidValue;
    const int64_t rowtiles = (a.rows + 15) / 16;
    if (grouped) {
        const int64_t columns = (int64_t)a.max_groups + (a.sh_tokens + kTokTile - 1) / kTokTile;
        if (columns > 65535) return hipErrorInvalidValue;
        const int waves = pick_waves(a.nb, rowtiles * columns);
        MQ_LAUNCH(q80_matmul_kernel, dim3((unsigned)rowtiles, (unsigned)columns), dim3(64 * waves),
                           waves > 1 ? (size_t)(waves - 1) * 2 * 64 * sizeof(float) : 0, stream, a);
        return hipGetLastError();
    }
    const int64_t columns = a.pair_ids ? a.n : 1;
    if (rowtiles * columns >= (int64_t)1 << 31) return hipErrorInvalidValue;
    const int waves = pick_waves(a.nb, rowtiles * columns);
    MQ_LAUNCH(q80_matmul_kernel, dim3((unsigned)(rowtiles * columns)), dim3(64 * waves),
                       waves > 1 ? (size_t)(waves - 1) * 2 * 64 * sizeof(float) : 0, stream, a);
    return hipGetLastError();
}

}  // namespace mq
