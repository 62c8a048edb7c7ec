// MoE routing on the device: stable top-k + softmax over the selected logits, the expert-grouped
// work list ("gather tokens by expert"), and the routing-order weighted combine.  Nothing here
// returns to the host; the matmul kernels read the lists these kernels write.
#include "common.h"
#include "kernels.h"

namespace mq {

namespace {

// core/src/llm/moe/native.cpp:610-619: non-NaN before NaN, larger logit first, lower id on ties.
__device__ __forceinline__ bool precedes(float a, int ia, float b, int ib) {
    const bool an = isnan(a), bn = isnan(b);
    if (an != bn) return !an;
    if (a > b) return true;
    if (a < b) return false;
    return ia < ib;
}

constexpr int kMaxPerLane = 16;  // up to 1024 experts per token

// One wavefront per token.  Lane l owns experts l, l+64, ...; each of the top_k rounds takes the
// best remaining candidate of the wave.
__global__ void __launch_bounds__(256) route_topk_kernel(const float* __restrict__ logits, int n_experts, int64_t n,
                                                         int top_k, int mode, int32_t* __restrict__ ids,
                                                         float* __restrict__ weights) {
    const int lane = threadIdx.x & 63;
    const int64_t tok = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (tok >= n) return;
    const float* row = logits + tok * n_experts;
    float v[kMaxPerLane];
    uint32_t live = 0;
#pragma unroll
    for (int j = 0; j < kMaxPerLane; ++j) {
        const int e = lane + 64 * j;
        v[j] = 0.0f;
        if (e < n_experts) {
            v[j] = row[e];
            live |= 1u << j;
        }
    }
    float sel_logit = 0.0f;  // lane k keeps the k-th selected logit
    int sel_id = -1;
    for (int k = 0; k < top_k; ++k) {
        float best = 0.0f;
        int best_id = 0x7fffffff;  // "none": loses to every real candidate below
        bool have = false;
#pragma unroll
        for (int j = 0; j < kMaxPerLane; ++j) {
            if (live & (1u << j)) {
                const int e = lane + 64 * j;
                if (!have || precedes(v[j], e, best, best_id)) {
                    best = v[j];
                    best_id = e;
                    have = true;
                }
            }
        }
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const float ob = __shfl_xor(best, off, 64);
            const int oid = __shfl_xor(best_id, off, 64);
            const bool ohave = oid != 0x7fffffff;
            if (ohave && (!have || precedes(ob, oid, best, best_id))) {
                best = ob;
                best_id = oid;
                have = true;
            }
        }
        if ((best_id & 63) == lane) live &= ~(1u << (best_id >> 6));
        if (lane == k) {
            sel_logit = best;
            sel_id = best_id;
        }
    }
    if (lane < top_k) ids[tok * top_k + lane] = sel_id;

    // softmax over the selected logits, summed in routing order on one lane
    float l[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) l[k] = __shfl(sel_logit, k < top_k ? k : 0, 64);
    if (lane != 0) return;
    float w[8];
    float* out = weights + tok * top_k;
    if (mode == 0) {  // core/src/llm/moe/native.cpp:650-675
        float mx = -INFINITY;
        bool all_finite = true;
        for (int k = 0; k < top_k; ++k) {
            all_finite = all_finite && isfinite(l[k]);
            if (isfinite(l[k])) mx = fmaxf(mx, l[k]);
        }
        float den = 0.0f;
        if (all_finite && isfinite(mx)) {
            for (int k = 0; k < top_k; ++k) {
                w[k] = expf(__fsub_rn(l[k], mx));
                den = __fadd_rn(den, w[k]);
            }
        }
        if (!(den > 0.0f) || !isfinite(den)) {
            for (int k = 0; k < top_k; ++k) out[k] = __fdiv_rn(1.0f, (float)top_k);
            return;
        }
        for (int k = 0; k < top_k; ++k) out[k] = __fdiv_rn(w[k], den);
    } else if (mode == 1) {  // core/src/llm/moe/native.cpp:2321-2355
        float mx = -INFINITY;
        for (int k = 0; k < top_k; ++k) mx = fmaxf(mx, l[k]);
        if (!isfinite(mx)) mx = 0.0f;
        float den = 0.0f;
        for (int k = 0; k < top_k; ++k) {
            w[k] = expf(__fsub_rn(l[k], mx));
            den = __fadd_rn(den, w[k]);
        }
        den = fmaxf(den, 6.103515625e-5f);
        for (int k = 0; k < top_k; ++k) out[k] = __fdiv_rn(w[k], den);
    } else {  // core/src/llm/moe/native.cpp:822-866
        float mx = -INFINITY;
        for (int k = 0; k < top_k; ++k)
            if (isfinite(l[k])) mx = fmaxf(mx, l[k]);
        float den = 0.0f;
        for (int k = 0; k < top_k; ++k)
            if (isfinite(l[k]) && isfinite(mx)) den = __fadd_rn(den, expf(__fsub_rn(l[k], mx)));
        const bool uniform = !(den > 0.0f) || !isfinite(den);
        den = uniform ? 1.0f : fmaxf(den, 6.103515625e-5f);
        const float uni = __fdiv_rn(1.0f, (float)top_k);
        for (int k = 0; k < top_k; ++k)
            out[k] = (uniform || !isfinite(l[k]) || !isfinite(mx)) ? uni : __fdiv_rn(expf(__fsub_rn(l[k], mx)), den);
    }
}

// Single workgroup.  Counting sort of the (token, k) pairs by expert; pairs keep their natural
// (token, k) order inside an expert, which is the (expert, token, k) order of
// core/src/llm/moe/native.cpp:1726-1730.  Experts nobody selected produce no group.
__global__ void __launch_bounds__(1024) build_groups_kernel(const int32_t* __restrict__ ids, int n_entries,
                                                            int top_k, int n_experts, int32_t* __restrict__ group_expert,
                                                            int32_t* __restrict__ group_begin,
                                                            int32_t* __restrict__ n_groups,
                                                            int32_t* __restrict__ entry_token,
                                                            int32_t* __restrict__ entry_k) {
    extern __shared__ int32_t sh[];  // [n_experts] counts -> offsets, [n_experts] group index
    int32_t* count = sh;
    int32_t* gidx = sh + n_experts;
    const int tid = threadIdx.x, nt = blockDim.x;
    for (int e = tid; e < n_experts; e += nt) count[e] = 0;
    __syncthreads();
    for (int i = tid; i < n_entries; i += nt) {
        const int e = ids[i];
        if (e >= 0 && e < n_experts) atomicAdd(&count[e], 1);
    }
    __syncthreads();
    if (tid == 0) {  // n_experts is a few hundred: a serial scan costs less than a barrier tree here
        int off = 0, g = 0;
        for (int e = 0; e < n_experts; ++e) {
            const int c = count[e];
            count[e] = off;
            if (c > 0) {
                group_expert[g] = e;
                group_begin[g] = off;
                gidx[e] = g;
                ++g;
            }
            off += c;
        }
        group_begin[g] = off;
        *n_groups = g;
    }
    __syncthreads();
    for (int i = tid; i < n_entries; i += nt) {
        const int e = ids[i];
        if (e < 0 || e >= n_experts) continue;
        int rank = 0;  // earlier pairs routed to the same expert
        for (int j = 0; j < i; ++j) rank += ids[j] == e;
        const int pos = count[e] + rank;
        entry_token[pos] = i / top_k;
        entry_k[pos] = i - (i / top_k) * top_k;
    }
}

__device__ __forceinline__ float stable_sigmoid(float x) {  // core/src/llm/graph/fused_ops.cpp:451-458
    if (x >= 0.0f) {
        const float z = expf(-x);
        return __fdiv_rn(1.0f, __fadd_rn(1.0f, z));
    }
    const float z = expf(x);
    return __fdiv_rn(z, __fadd_rn(1.0f, z));
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
    float gate = 1.0f;
    if (has_shared && sh_gate_inp) {
        float acc = 0.0f;
        for (int64_t c = threadIdx.x; c < rows; c += 256) acc = fmaf(sh_gate_inp[c], x[tok * rows + c], acc);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
        if ((threadIdx.x & 63) == 0) wave_sum[threadIdx.x >> 6] = acc;
        __syncthreads();
        gate = stable_sigmoid((wave_sum[0] + wave_sum[1]) + (wave_sum[2] + wave_sum[3]));
    }
    if (r >= rows) return;
    float acc = 0.0f;
    for (int k = 0; k < top_k; ++k) {
        const int e = ids[tok * top_k + k];
        const float w = weights[tok * top_k + k];
        if (e < 0 || e >= n_experts || w == 0.0f) continue;
        acc = __fadd_rn(acc, __fmul_rn(part[(tok * slots + k) * rows + r], w));
    }
    if (has_shared) acc = __fadd_rn(acc, __fmul_rn(part[(tok * slots + top_k) * rows + r], gate));
    y[tok * rows + r] = acc;
}

__global__ void __launch_bounds__(256) fill_zero_kernel(float* __restrict__ p, size_t count) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * 256;
    for (; i < count; i += stride) p[i] = 0.0f;
}

}  // namespace

hipError_t launch_route_topk(const float* logits, int64_t n_experts, int64_t n, int top_k, int mode, int32_t* ids,
                             float* weights, hipStream_t stream) {
    if (n_experts > 64 * kMaxPerLane || top_k > 8) return hipErrorInvalidValue;
    hipLaunchKernelGGL(route_topk_kernel, dim3((unsigned)((n + 3) / 4)), dim3(256), 0, stream, logits, (int)n_experts, n,
                       top_k, mode, ids, weights);
    return hipGetLastError();
}

hipError_t launch_build_groups(const int32_t* ids, int64_t n, int top_k, int64_t n_experts, int32_t* group_expert,
                               int32_t* group_begin, int32_t* n_groups, int32_t* entry_token, int32_t* entry_k,
                               hipStream_t stream) {
    const int64_t entries = n * top_k;
    if (entries > (int64_t)1 << 30 || n_experts > 8192) return hipErrorInvalidValue;
    const int threads = entries >= 1024 ? 1024 : (entries > 256 ? 512 : 256);
    hipLaunchKernelGGL(build_groups_kernel, dim3(1), dim3(threads), (size_t)n_experts * 8, stream, ids, (int)entries,
                       top_k, (int)n_experts, group_expert, group_begin, n_groups, entry_token, entry_k);
    return hipGetLastError();
}

hipError_t launch_moe_combine(const float* part, int64_t n, int top_k, int slots, int64_t rows, const float* weights,
                              const int32_t* ids, int64_t n_experts, int has_shared, const float* sh_gate_inp,
                              const float* x, float* y, hipStream_t stream) {
    hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)((rows + 255) / 256), (unsigned)n), dim3(256), 0, stream, part,
                       top_k, slots, rows, weights, ids, (int)n_experts, has_shared, sh_gate_inp, x, y);
    return hipGetLastError();
}

hipError_t launch_fill_zero(float* p, size_t count, hipStream_t stream) {
    if (count == 0) return hipSuccess;
    size_t blocks = (count + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, p, count);
    return hipGetLastError();
}

}  // namespace mq
