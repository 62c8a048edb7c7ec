// MoE routing on the device: stable top-k + softmax over the selected logits, the expert-grouped
// work list ("gather tokens by expert"), and the routing-order weighted combine.  Nothing here
// returns to the host; the matmul kernels read the lists these kernels write.
#include <type_traits>

#include "common.h"
#include "kernels.h"
#include "q8k_block.h"
#include "route_block.h"

namespace mq {

namespace {

constexpr int kMaxExperts = 2048;

// Routing of one token by one workgroup of 256 threads.  Up to 512 experts: one wavefront, keys in registers.
// More: all threads turn the logits into sort keys in
// LDS; wavefront 0 then extracts the top_k largest keys one after the other (lane l owns the experts
// e = l mod 64: a local maximum over its keys, a 6-step butterfly across the lanes, and the owner of
// the winner clears it).  The keys are unique and totally ordered exactly like
// ComputeQwenNativeMoEStableTopK (core/src/llm/moe/native.cpp:610-645), so the k-th extraction is the
// k-th expert of the routing order.  keys: max(n_experts, kRouteScratch) 64-bit words of LDS; sel: 8 floats + 8 ints of LDS.
__device__ __forceinline__ void route_token_block(const float* __restrict__ row, int n_experts, int top_k, int mode,
                                                  unsigned long long* keys, float* sel_logit, int32_t* sel_id,
                                                  int32_t* __restrict__ ids_out, float* __restrict__ w_out,
                                                  bool coherent_ids) {
    const int tid = threadIdx.x;
    if (n_experts <= 512) {
        // few enough experts for one wavefront's registers: eight 32-bit keys per lane, winners by ballot,
        // softmax lane-parallel (route_block.h); the other wavefronts only pass the barriers
        if (tid < 64) {
            int id;
            float logit;
            auto load = [&](int e) { return row[e]; };
            if (n_experts <= 256) route_token_wave_lds<4>(load, n_experts, top_k, tid, id, logit, keys);
            else route_token_wave_lds<8>(load, n_experts, top_k, tid, id, logit, keys);
            const float w = route_weight_lane(logit, tid, top_k, mode);
            if (tid < top_k) {
                sel_id[tid] = id;
                w_out[tid] = w;
            }
        }
        __syncthreads();
        if (tid < top_k) {
            if (coherent_ids) {
                __hip_atomic_store(ids_out + tid, sel_id[tid], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            } else {
                ids_out[tid] = sel_id[tid];
            }
        }
        return;
    }
    for (int e = tid; e < n_experts; e += 256) keys[e] = route_key(row[e], e);
    __syncthreads();
    if (tid < 64) {
        for (int r = 0; r < top_k; ++r) {
            unsigned long long best = 0ull;  // below every key
            for (int e = tid; e < n_experts; e += 64) {
                const unsigned long long k = keys[e];
                best = k > best ? k : best;
            }
            best = wave_max_key(best);
            const int id = (int)~(uint32_t)best;
            if (tid == (id & 63)) keys[id] = 0ull;  // the owning lane is the only one that reads this key again
            if (tid == 0) {
                sel_id[r] = id;
                sel_logit[r] = route_key_logit(best);
            }
        }
        if (tid == 0) {
            float l[8];
            for (int k = 0; k < top_k; ++k) l[k] = sel_logit[k];
            route_weights(l, top_k, mode, w_out);
        }
    }
    __syncthreads();
    if (tid < top_k) {
        if (coherent_ids) {
            __hip_atomic_store(ids_out + tid, sel_id[tid], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else {
            ids_out[tid] = sel_id[tid];
        }
    }
}

__global__ void __launch_bounds__(256) route_topk_kernel(const float* __restrict__ logits, int n_experts, int top_k,
                                                         int mode, int32_t* __restrict__ ids,
                                                         float* __restrict__ weights) {
    extern __shared__ unsigned long long route_sh[];  // [n_experts] keys, then 8 floats, 8 ints
    float* sel_logit = reinterpret_cast<float*>(route_sh + (n_experts > kRouteScratch ? n_experts : kRouteScratch));
    int32_t* sel_id = reinterpret_cast<int32_t*>(sel_logit + 8);
    const int64_t tok = blockIdx.x;
    route_token_block(logits + tok * n_experts, n_experts, top_k, mode, route_sh, sel_logit, sel_id, ids + tok * top_k,
                      weights + tok * top_k, false);
}

// Weights of already-selected experts from the raw logits (core/src/llm/moe/native.cpp:2305-2357):
// invalid ids weigh 0 and take no part in the max; one thread per token.
__global__ void __launch_bounds__(64) weights_from_ids_kernel(const float* __restrict__ logits, int n_experts, int n,
                                                              const int32_t* __restrict__ ids, int top_k,
                                                              float* __restrict__ weights) {
    const int tok = blockIdx.x * 64 + threadIdx.x;
    if (tok >= n) return;
    const float* row = logits + (size_t)tok * n_experts;
    float l[8];
    bool ok[8];
    float mx = -INFINITY;
    for (int k = 0; k < top_k; ++k) {
        const int e = ids[(size_t)tok * top_k + k];
        ok[k] = e >= 0 && e < n_experts;
        l[k] = ok[k] ? row[e] : 0.0f;
        if (ok[k] && l[k] > mx) mx = l[k];
    }
    if (!isfinite(mx)) mx = 0.0f;
    float den = 0.0f;
    for (int k = 0; k < top_k; ++k) {
        l[k] = ok[k] ? expf(__fsub_rn(l[k], mx)) : 0.0f;
        if (ok[k]) den = __fadd_rn(den, l[k]);
    }
    den = den < 6.103515625e-5f ? 6.103515625e-5f : den;  // std::max(den, floor): a NaN den is replaced too
    for (int k = 0; k < top_k; ++k) weights[(size_t)tok * top_k + k] = __fdiv_rn(l[k], den);
}

// Counting sort of the (token, k) pairs by expert, by one workgroup.  Pairs keep their natural
// (token, k) order inside an expert, which is the (expert, token, k) order of
// core/src/llm/moe/native.cpp:1726-1730.  Experts nobody selected produce no group.
// ids may live in LDS or in global memory; count[] is n_experts ints of LDS.
// token_mask (LDS, n_experts * (mask_words | 1) + 1 words, or null): one bit per (expert, token).  A pair's place inside
// its group is the number of earlier pairs of the same expert; when no token names an expert twice (always so for
// routed ids) that is the number of earlier tokens whose bit is set -- a population count instead of a scan over
// all earlier pairs.  A repeated (expert, token) raises the word after the masks and the scan is used.
__device__ __forceinline__ void group_entries(const int32_t* ids, int n_entries, int top_k, int n_experts,
                                              int32_t* count, int32_t* __restrict__ group_expert,
                                              int32_t* __restrict__ group_begin, int32_t* __restrict__ n_groups,
                                              int32_t* __restrict__ entry_token, int32_t* __restrict__ entry_k,
                                              uint32_t* token_mask = nullptr, int mask_words = 0, int part = 0, int parts = 1,
                                              uint16_t* mask_prefix = nullptr) {
    const int tid = threadIdx.x, nt = blockDim.x;
    // an expert's mask words are an odd number of words apart: the lanes of a wavefront (consecutive pairs, different
    // experts) walk their experts' words side by side, and an even stride puts them all on one LDS bank (225 us
    // against 20 for the grouping of 2048 tokens)
    const int mask_stride = mask_words | 1;
    for (int e = tid; e < n_experts; e += nt) count[e] = 0;
    if (token_mask)
        for (int w = tid; w <= n_experts * mask_stride; w += nt) token_mask[w] = 0u;
    __syncthreads();
    for (int i = tid; i < n_entries; i += nt) {
        const int e = ids[i];
        if (e >= 0 && e < n_experts) {
            atomicAdd(&count[e], 1);
            if (token_mask) {
                const int t = i / top_k;
                const uint32_t bit = 1u << (t & 31);
                if (atomicOr(&token_mask[e * mask_stride + (t >> 5)], bit) & bit) token_mask[n_experts * mask_stride] = 1u;
            }
        }
    }
    __syncthreads();
    if (tid < 64) {  // wave 0: exclusive scan over the experts, lane l covers a run of consecutive experts
        const int per = (n_experts + 63) / 64;
        const int e0 = tid * per;
        int sum = 0, active = 0;
        for (int j = 0; j < per; ++j) {
            const int e = e0 + j;
            if (e < n_experts) {
                sum += count[e];
                active += count[e] > 0;
            }
        }
        int off = sum, g = active;  // inclusive scans across lanes
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int o = __shfl_up(off, d, 64);
            const int og = __shfl_up(g, d, 64);
            if (tid >= d) {
                off += o;
                g += og;
            }
        }
        const int total = __shfl(off, 63, 64), groups = __shfl(g, 63, 64);
        off -= sum;
        g -= active;
        for (int j = 0; j < per; ++j) {
            const int e = e0 + j;
            if (e < n_experts) {
                const int c = count[e];
                count[e] = off;
                if (c > 0) {
                    if (part == 0) {
                        group_expert[g] = e;
                        group_begin[g] = off;
                    }
                    ++g;
                }
                off += c;
            }
        }
        if (tid == 0 && part == 0) {
            group_begin[groups] = total;
            *n_groups = groups;
        }
    }
    __syncthreads();
    const bool by_mask = token_mask && token_mask[n_experts * mask_stride] == 0u;
    // mask_prefix (LDS, n_experts * mask_stride 16-bit words, or null; at most 65535 tokens): the number of set bits in an
    // expert's mask words before word w, so that a pair's place costs one look-up and one population count instead of a
    // walk over all the expert's earlier words (half of them on average: at 2048 tokens 32 LDS reads per pair)
    if (by_mask && mask_prefix) {
        for (int e = tid; e < n_experts; e += nt) {
            const uint32_t* m = token_mask + e * mask_stride;
            uint16_t* pre = mask_prefix + e * mask_stride;
            int run = 0;
            for (int w = 0; w < mask_words; ++w) {
                pre[w] = (uint16_t)run;
                run += __popc(m[w]);
            }
        }
        __syncthreads();
    }
    // several workgroups (parts > 1) all build the counts and masks, each places its share of the pairs
    for (int i = part * nt + tid; i < n_entries; i += parts * nt) {
        const int e = ids[i];
        if (e < 0 || e >= n_experts) continue;
        int rank = 0;  // earlier pairs routed to the same expert
        int j = 0;
        if (by_mask) {
            const int t = i / top_k;
            const uint32_t* m = token_mask + e * mask_stride;
            if (mask_prefix) rank = mask_prefix[e * mask_stride + (t >> 5)];
            else
                for (int w = 0; w < (t >> 5); ++w) rank += __popc(m[w]);
            rank += __popc(m[t >> 5] & ((1u << (t & 31)) - 1u));
            j = i;  // nothing left to scan
        }
        for (; j + 16 <= i; j += 16) {
            int v16[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) v16[u] = ids[j + u];
#pragma unroll
            for (int u = 0; u < 16; ++u) rank += v16[u] == e;
        }
        for (; j < i; ++j) rank += ids[j] == e;
        const int pos = count[e] + rank;
        entry_token[pos] = i / top_k;
        entry_k[pos] = i - (i / top_k) * top_k;
    }
}

__global__ void __launch_bounds__(1024) build_groups_kernel(const int32_t* __restrict__ ids, int n_entries,
                                                            int top_k, int n_experts, int use_lds, int mask_words, int with_prefix,
                                                            int32_t* __restrict__ group_expert,
                                                            int32_t* __restrict__ group_begin,
                                                            int32_t* __restrict__ n_groups,
                                                            int32_t* __restrict__ entry_token,
                                                            int32_t* __restrict__ entry_k) {
    extern __shared__ int32_t sh[];  // [n_experts] counts -> offsets, [n_entries] ids when they fit, then the token masks
    int32_t* count = sh;
    const int32_t* src = ids;
    if (use_lds) {
        int32_t* ids_s = sh + n_experts;
        for (int i = threadIdx.x; i < n_entries; i += blockDim.x) ids_s[i] = ids[i];
        src = ids_s;  // the barrier inside group_entries orders these stores
    }
    uint32_t* masks = mask_words ? reinterpret_cast<uint32_t*>(sh + n_experts + (use_lds ? n_entries : 0)) : nullptr;
    uint16_t* prefix = with_prefix ? reinterpret_cast<uint16_t*>(masks + n_experts * (mask_words | 1) + 1) : nullptr;
    group_entries(src, n_entries, top_k, n_experts, count, group_expert, group_begin, n_groups, entry_token, entry_k, masks, mask_words,
                  (int)blockIdx.x, (int)gridDim.x, prefix);
}

// Router and grouping in one launch (decode widths): a workgroup per token routes it; the last
// workgroup to finish gathers all ids and builds the expert groups.  `arrivals` is one zeroed
// uint32 in device memory that the kernel leaves zero again.  Workgroups past `route_blocks` do an
// unrelated job that needs nothing from the router and would otherwise cost a launch of its own: they
// quantize the layer input to Q8_K (four (row, super-block) units each, as quantize_q8k_kernel does).
__global__ void __launch_bounds__(1024) route_and_group_kernel(const float* __restrict__ logits, int n_experts, int n,
                                                              int top_k, int mode, int32_t* __restrict__ ids,
                                                              float* __restrict__ weights, uint32_t* arrivals,
                                                              int32_t* __restrict__ group_expert,
                                                              int32_t* __restrict__ group_begin,
                                                              int32_t* __restrict__ n_groups,
                                                              int32_t* __restrict__ entry_token,
                                                              int32_t* __restrict__ entry_k, int build_groups,
                                                              int route_blocks, int mask_words, int wave_parallel,
                                                              const float* __restrict__ qx, int64_t q_ldx, int64_t q_nb,
                                                              uint8_t* __restrict__ q_aq, float* __restrict__ q_ad) {
    if ((int)blockIdx.x >= route_blocks) {
        const int lane = threadIdx.x & 63;
        const int64_t unit = (int64_t)(blockIdx.x - route_blocks) * (blockDim.x >> 6) + (threadIdx.x >> 6);
        if (unit >= (int64_t)n * q_nb) return;
        int64_t m, b;
        split_unit(unit, q_nb, m, b);
        const float4 v = *reinterpret_cast<const float4*>(qx + m * q_ldx + b * kQK + lane * 4);
        const float e[4] = {v.x, v.y, v.z, v.w};
        store_amajor(q_aq, q_ad, m, b, q_nb, lane, quantize_block_q8k(e, lane));
        return;
    }
    extern __shared__ unsigned long long route_sh[];  // keys | sel | then reused: counts, ids
    __shared__ int is_last;
    float* sel_logit = reinterpret_cast<float*>(route_sh + (n_experts > kRouteScratch ? n_experts : kRouteScratch));
    int32_t* sel_id = reinterpret_cast<int32_t*>(sel_logit + 8);
    if (wave_parallel) {
        // One workgroup for all tokens, a token per wavefront (and round): the ids go to LDS as they are found and the
        // grouping follows behind one barrier -- no device-coherent stores, arrival count and re-read between them.
        const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, n_waves = blockDim.x >> 6;
        unsigned long long* scratch = route_sh + wave * kRouteScratch;
        int32_t* count = reinterpret_cast<int32_t*>(route_sh + n_waves * kRouteScratch);
        int32_t* ids_s = count + n_experts;
        // the logits of all tokens of this wavefront (at most two: 32 tokens, 16 wavefronts) are requested first;
        // ids and weights leave for global memory after the grouping (a store ahead of a barrier makes it wait)
        int id_keep[2];
        float w_keep[2];
        auto route_all = [&](auto kpl_c) {
            constexpr int KPL = decltype(kpl_c)::value;
            float lg[2][KPL];
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                const int tok = wave + r * n_waves < n ? wave + r * n_waves : n - 1;
                const float* row = logits + (size_t)tok * n_experts;
                route_load_logits<KPL>([&](int e) { return row[e]; }, n_experts, lane, lg[r]);
            }
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                const int tok = wave + r * n_waves;
                id_keep[r] = -1, w_keep[r] = 0.0f;
                if (tok < n) {  // wave-uniform
                    float logit;
                    route_logits_wave_lds<KPL>(lg[r], n_experts, top_k, lane, id_keep[r], logit, scratch);
                    w_keep[r] = route_weight_lane(logit, lane, top_k, mode);
                    if (lane < top_k) ids_s[tok * top_k + lane] = id_keep[r];
                }
            }
        };
        if (n_experts <= 256) route_all(std::integral_constant<int, 4>{});
        else route_all(std::integral_constant<int, 8>{});
        // group_entries zeroes its counters and passes a barrier before it reads the ids
        if (build_groups)
            group_entries(ids_s, n * top_k, top_k, n_experts, count, group_expert, group_begin, n_groups, entry_token, entry_k,
                          mask_words ? reinterpret_cast<uint32_t*>(ids_s + n * top_k) : nullptr, mask_words);
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const int tok = wave + r * n_waves;
            if (tok < n && lane < top_k) {
                ids[(size_t)tok * top_k + lane] = id_keep[r];
                weights[(size_t)tok * top_k + lane] = w_keep[r];
            }
        }
        return;
    }
    const bool solo = route_blocks == 1;  // one or two tokens: one workgroup does everything, no handshake
    const int per_block = solo ? n : 1;
    for (int t = 0; t < per_block; ++t) {
        const int tok = blockIdx.x * per_block + t;
        route_token_block(logits + (size_t)tok * n_experts, n_experts, top_k, mode, route_sh, sel_logit, sel_id,
                          ids + (size_t)tok * top_k, weights + (size_t)tok * top_k, !solo);
        __syncthreads();  // keys / sel are reused by the next token and by the grouping below
    }
    if (!build_groups) return;  // the consumer takes the ids as they are (few tokens)
    if (!solo) {
        // the ids were stored device-coherently; wait for their acknowledgement before being counted
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (threadIdx.x == 0) {
            const uint32_t prev = atomicAdd(arrivals, 1u);
            is_last = prev == (uint32_t)(n - 1);
            if (is_last) atomicExch(arrivals, 0u);
        }
        __syncthreads();
        if (!is_last) return;
    }
    int32_t* count = reinterpret_cast<int32_t*>(route_sh);
    int32_t* ids_s = count + n_experts;
    const int n_entries = n * top_k;
    for (int i = threadIdx.x; i < n_entries; i += blockDim.x)
        ids_s[i] = solo ? ids[i] : __hip_atomic_load(ids + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    group_entries(ids_s, n_entries, top_k, n_experts, count, group_expert, group_begin, n_groups, entry_token, entry_k,
                  mask_words ? reinterpret_cast<uint32_t*>(ids_s + n_entries) : nullptr, mask_words);
}

// grid = (ceil(rows/256), n).  Routed experts are added in routing order k = 0..top_k-1
// (core/src/llm/moe/native.cpp:3233-3285), zero weights skipped (:3237); then the shared expert
// scaled by sigmoid(sh_gate_inp . x) (core/src/llm/graph/decoder.cpp:2545-2600).
__global__ void __launch_bounds__(256) moe_combine_kernel(const float* __restrict__ part, int top_k, int slots,
                                                          int64_t rows, const float* __restrict__ weights,
                                                          const int32_t* __restrict__ ids, int n_experts,
                                                          int has_shared, const float* __restrict__ sh_gate_inp,
                                                          const float* __restrict__ x, float* __restrict__ y) {
    __shared__ float wave_sum[4];
    const int64_t tok = blockIdx.y;
    const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
    // Every partial row, id and weight is requested before anything else and unconditionally (a slot past top_k or
    // a row past the end re-reads slot 0 / row 0; a dropped slot's row may hold anything: it is read and thrown
    // away), so that all of them and the gate operands below travel together.
    const int64_t rr = r < rows ? r : 0;
    float pv[9], wk[8];
    int ek[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const int kk = k < top_k ? k : 0;
        ek[k] = ids[tok * top_k + kk];
        wk[k] = weights[tok * top_k + kk];
        pv[k] = part[(tok * slots + kk) * rows + rr];
    }
    pv[8] = part[(tok * slots + (has_shared ? top_k : 0)) * rows + rr];
    float gate = 1.0f;
    if (has_shared && sh_gate_inp) {
        // thread j takes columns j, j + 256, ... in turn; the operands are requested eight columns at a time so that
        // their latencies overlap instead of adding up
        const float* xr = x + tok * rows;
        float acc = 0.0f;
        int64_t c = threadIdx.x;
        for (; c + 7 * 256 < rows; c += 8 * 256) {
            float ga[8], xa[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) ga[u] = sh_gate_inp[c + u * 256], xa[u] = xr[c + u * 256];
#pragma unroll
            for (int u = 0; u < 8; ++u) acc = fmaf(ga[u], xa[u], acc);
        }
        for (; c < rows; c += 256) acc = fmaf(sh_gate_inp[c], xr[c], acc);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
        if ((threadIdx.x & 63) == 0) wave_sum[threadIdx.x >> 6] = acc;
        __syncthreads();
        gate = stable_sigmoid((wave_sum[0] + wave_sum[1]) + (wave_sum[2] + wave_sum[3]));
    }
    if (r >= rows) return;
    // the sum runs in routing order
    float acc = 0.0f;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const bool live = k < top_k && ek[k] >= 0 && ek[k] < n_experts && wk[k] != 0.0f;
        if (live) acc = __fadd_rn(acc, __fmul_rn(pv[k], wk[k]));
    }
    if (has_shared) acc = __fadd_rn(acc, __fmul_rn(pv[8], gate));
    y[tok * rows + r] = acc;
}

// The work list as (expert, token, k) triples in list order, for comparison with the reference's sorted assignments
// (core/src/llm/moe/native.cpp:1664-1733); one workgroup.
__global__ void __launch_bounds__(256) flatten_groups_kernel(const int32_t* __restrict__ group_expert,
                                                             const int32_t* __restrict__ group_begin,
                                                             const int32_t* __restrict__ n_groups,
                                                             const int32_t* __restrict__ entry_token,
                                                             const int32_t* __restrict__ entry_k, int max_entries,
                                                             int32_t* __restrict__ triples, int32_t* __restrict__ count) {
    const int groups = *n_groups;
    for (int g = 0; g < groups; ++g) {
        const int b = group_begin[g], e = group_begin[g + 1];
        for (int i = b + (int)threadIdx.x; i < e && i < max_entries; i += 256) {
            triples[3 * i] = group_expert[g];
            triples[3 * i + 1] = entry_token[i];
            triples[3 * i + 2] = entry_k[i];
        }
    }
    if (threadIdx.x == 0) *count = group_begin[groups];
}

__global__ void __launch_bounds__(256) fill_zero_kernel(float* __restrict__ p, size_t count) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * 256;
    for (; i < count; i += stride) p[i] = 0.0f;
}

__global__ void __launch_bounds__(1024) skeleton_kernel() {}

}  // namespace

int g_skeleton = 0;

hipError_t launch_skeleton(dim3 grid, dim3 block, size_t lds, hipStream_t stream) {
    static bool raised = false;
    if (!raised) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(skeleton_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
        raised = true;
    }
    hipLaunchKernelGGL(skeleton_kernel, grid, block, lds, stream);
    return hipGetLastError();
}

hipError_t launch_route_topk(const float* logits, int64_t n_experts, int64_t n, int top_k, int mode, int32_t* ids,
                             float* weights, hipStream_t stream) {
    if (n_experts > kMaxExperts || top_k > 8) return hipErrorInvalidValue;
    const size_t lds = (size_t)(n_experts > kRouteScratch ? n_experts : kRouteScratch) * 8 + 64;
    MQ_LAUNCH(route_topk_kernel, dim3((unsigned)n), dim3(256), lds, stream, logits, (int)n_experts, top_k, mode,
                       ids, weights);
    return hipGetLastError();
}

hipError_t launch_weights_from_ids(const float* logits, int64_t n_experts, int64_t n, const int32_t* ids, int top_k,
                                   float* weights, hipStream_t stream) {
    if (top_k > 8 || top_k <= 0) return hipErrorInvalidValue;
    MQ_LAUNCH(weights_from_ids_kernel, dim3((unsigned)((n + 63) / 64)), dim3(64), 0, stream, logits,
                       (int)n_experts, (int)n, ids, top_k, weights);
    return hipGetLastError();
}

hipError_t launch_build_groups(const int32_t* ids, int64_t n, int top_k, int64_t n_experts, int32_t* group_expert,
                               int32_t* group_begin, int32_t* n_groups, int32_t* entry_token, int32_t* entry_k,
                               hipStream_t stream) {
    const int64_t entries = n * top_k;
    if (entries > (int64_t)1 << 30 || n_experts > 8192) return hipErrorInvalidValue;
    const int threads = entries >= 1024 ? 1024 : (entries > 256 ? 512 : 256);
    // one bit per (expert, token) when that fits the 160 KB of a compute unit (256 experts: up to 4096 tokens); without
    // it a pair's place in its group is found by scanning all earlier pairs -- 394 us at 512 tokens against 17 at 256.
    // The ids join them in LDS while there is room (16384 pairs at 2048 tokens and 256 experts).
    size_t lds = (size_t)n_experts * 4;
    int mask_words = n <= 4096 ? (int)((n + 31) / 32) : 0;
    if (lds + ((size_t)n_experts * (mask_words | 1) + 1) * 4 > 150 * 1024) mask_words = 0;
    if (mask_words) lds += ((size_t)n_experts * (mask_words | 1) + 1) * 4;
    // from 512 tokens the prefix counts of the masks join them (where they fit), ahead of the ids
    const size_t prefix_bytes = ((size_t)n_experts * (mask_words | 1) * 2 + 3) & ~(size_t)3;
    const int with_prefix = mask_words >= 16 && lds + prefix_bytes <= 150 * 1024;
    if (with_prefix) lds += prefix_bytes;
    const int use_lds = lds + (size_t)entries * 4 <= 150 * 1024;
    if (use_lds) lds += (size_t)entries * 4;
    if (lds > 64 * 1024) {
        static bool raised = false;
        if (!raised) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&build_groups_kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess) return e;
            raised = true;
        }
    }
    // placing a pair is a population count over its expert's mask words and two scattered stores: beyond a few thousand
    // pairs several workgroups share that part (each repeats the cheap counting): 43 -> 16 us at 16384 pairs
    const unsigned parts = entries >= 3072 ? 8u : 1u;
    MQ_LAUNCH(build_groups_kernel, dim3(parts), dim3(threads), lds, stream, ids, (int)entries, top_k,
                       (int)n_experts, use_lds, mask_words, with_prefix, group_expert, group_begin, n_groups, entry_token, entry_k);
    return hipGetLastError();
}

hipError_t launch_route_and_group(const float* logits, int64_t n_experts, int64_t n, int top_k, int mode, int32_t* ids,
                                  float* weights, uint32_t* arrivals, int32_t* group_expert, int32_t* group_begin,
                                  int32_t* n_groups, int32_t* entry_token, int32_t* entry_k, bool build_groups,
                                  const float* qx, int64_t q_ldx, int64_t q_cols, uint8_t* q_aq, float* q_ad, hipStream_t stream) {
    if (n_experts > kMaxExperts || top_k > 8) return hipErrorInvalidValue;
    const size_t lds_route = (size_t)(n_experts > kRouteScratch ? n_experts : kRouteScratch) * 8 + 64;
    // one bit per (expert, token) for the grouping (see launch_build_groups)
    const int mask_words = n <= 4096 ? (int)((n + 31) / 32) : 0;
    const size_t lds_group = (size_t)n_experts * 4 + (size_t)n * top_k * 4 + (mask_words ? ((size_t)n_experts * (mask_words | 1) + 1) * 4 : 0);
    if (lds_group > 60 * 1024 || n * top_k >= 3072) {  // prefill widths: route, then group over several workgroups, quantize on its own
        hipError_t e = launch_route_topk(logits, n_experts, n, top_k, mode, ids, weights, stream);
        if (e != hipSuccess) return e;
        e = launch_build_groups(ids, n, top_k, n_experts, group_expert, group_begin, n_groups, entry_token, entry_k,
                                stream);
        if (e != hipSuccess || !qx) return e;
        return launch_quantize_q8k(qx, n, q_ldx, q_cols, nullptr, 0, q_aq, q_ad, stream);
    }
    // Up to 32 tokens and 512 experts: one workgroup routes a token or two per wavefront and groups right away.  Against
    // one workgroup per token + the last one to arrive grouping (device-coherent id stores, an arrival count, a re-read):
    // 6.0 against 8 us at 16 tokens, but 13.5 against 9 at 64 -- sixteen wavefronts on one compute unit route a token
    // in 1.5-1.9 us each (they share its four SIMDs), and the handshake costs about 3 us.
    const int threads = n <= 4 ? 256 : n <= 8 ? 512 : 1024;
    const size_t lds_wave = (size_t)(threads / 64) * kRouteScratch * 8 + lds_group;
    const bool wave_parallel = n <= 32 && n_experts <= 512 && lds_wave <= 60 * 1024;
    const int route_blocks = wave_parallel || n <= 2 ? 1 : (int)n;
    const int block = wave_parallel ? threads : 256;
    const int64_t q_nb = q_cols / kQK;
    const int64_t per_block = block / 64;
    const int64_t quant_blocks = qx ? (n * q_nb + per_block - 1) / per_block : 0;
    const size_t lds = wave_parallel ? lds_wave : (lds_route > lds_group ? lds_route : lds_group);
    MQ_LAUNCH(route_and_group_kernel, dim3((unsigned)(route_blocks + quant_blocks)), dim3(block), lds, stream, logits,
                       (int)n_experts, (int)n, top_k, mode, ids, weights, arrivals, group_expert, group_begin, n_groups,
                       entry_token, entry_k, build_groups ? 1 : 0, route_blocks, mask_words, wave_parallel ? 1 : 0, qx, q_ldx,
                       q_nb, q_aq, q_ad);
    return hipGetLastError();
}

hipError_t launch_moe_combine(const float* part, int64_t n, int top_k, int slots, int64_t rows, const float* weights,
                              const int32_t* ids, int64_t n_experts, int has_shared, const float* sh_gate_inp,
                              const float* x, float* y, hipStream_t stream) {
    if (top_k < 0 || top_k > 8) return hipErrorInvalidValue;
    MQ_LAUNCH(moe_combine_kernel, dim3((unsigned)((rows + 255) / 256), (unsigned)n), dim3(256), 0, stream, part,
                       top_k, slots, rows, weights, ids, (int)n_experts, has_shared, sh_gate_inp, x, y);
    return hipGetLastError();
}

hipError_t launch_flatten_groups(const int32_t* group_expert, const int32_t* group_begin, const int32_t* n_groups,
                                 const int32_t* entry_token, const int32_t* entry_k, int max_entries, int32_t* triples,
                                 int32_t* count, hipStream_t stream) {
    MQ_LAUNCH(flatten_groups_kernel, dim3(1), dim3(256), 0, stream, group_expert, group_begin, n_groups, entry_token,
                       entry_k, max_entries, triples, count);
    return hipGetLastError();
}

hipError_t launch_fill_zero(float* p, size_t count, hipStream_t stream) {
    if (count == 0) return hipSuccess;
    size_t blocks = (count + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    MQ_LAUNCH(fill_zero_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, p, count);
    return hipGetLastError();
}

}  // namespace mq
