// The two small fp32 operators that sit between the quantized matmuls of a decoder layer: the
// fused residual add + RMSNorm that feeds every projection, and the F32 router projection that
// produces the MoE logits.  Both are bandwidth-trivial; they exist so that a decode step stays on
// the device between the Q4_K kernels.
#include "common.h"
#include "kernels.h"
#include "q8k_block.h"

namespace mq {

namespace {

// sum[t] = x[t] + delta[t] (delta may be null); normed[t] = sum[t] * (rsqrt(mean(sum^2) + eps) * weight)
// AddRMSNorm (core/src/kernels/hwy/hwy_normalization.cc:102-153; plain form in
// core/tests/kernels/test_normalization.cpp:57-68).  One workgroup per token; the squares are
// summed per thread in column order, then across lanes and waves in a fixed order.  This general form takes
// rows of any length and alignment; rows of whole super-blocks take add_rmsnorm_blocks_kernel below.
// When q_aq is given (cols % 256 == 0) the normalised row also leaves as Q8_K in the layout the matmul
// kernels read, quantized from the very floats that normed_out receives.
__global__ void __launch_bounds__(256) add_rmsnorm_kernel(const float* x, const float* __restrict__ delta,
                                                          const float* __restrict__ weight, int64_t cols, float eps,
                                                          float* sum_out, float* __restrict__ normed_out,
                                                          uint8_t* __restrict__ q_aq, float* __restrict__ q_ad) {
    __shared__ float wave_sum[4];
    const int64_t base = (int64_t)blockIdx.x * cols;
    float ssq = 0.0f;
    for (int64_t c = threadIdx.x; c < cols; c += 256) {
        const float v = delta ? __fadd_rn(x[base + c], delta[base + c]) : x[base + c];
        if (sum_out) sum_out[base + c] = v;
        ssq = __fmaf_rn(v, v, ssq);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) ssq += __shfl_xor(ssq, off, 64);
    if ((threadIdx.x & 63) == 0) wave_sum[threadIdx.x >> 6] = ssq;
    __syncthreads();
    const float total = (wave_sum[0] + wave_sum[1]) + (wave_sum[2] + wave_sum[3]);
    const float scale = __fdiv_rn(1.0f, __fsqrt_rn(__fadd_rn(__fdiv_rn(total, (float)cols), eps)));
    auto normed = [&](int64_t c) {
        // sum_out may alias x: a thread re-reads what it stored itself rather than adding delta twice
        const float v = sum_out ? sum_out[base + c] : (delta ? __fadd_rn(x[base + c], delta[base + c]) : x[base + c]);
        const float sw = weight ? __fmul_rn(scale, weight[c]) : scale;
        return __fmul_rn(v, sw);
    };
    if (!q_aq) {
        for (int64_t c = threadIdx.x; c < cols; c += 256) normed_out[base + c] = normed(c);
        return;
    }
    // one wavefront per super-block, lane l holds its elements 4l .. 4l+3
    __syncthreads();  // pass 1 stored sum_out with another thread-to-column mapping
    const int lane = threadIdx.x & 63;
    const int64_t nb = cols / kQK;
    for (int64_t b = threadIdx.x >> 6; b < nb; b += 4) {
        const int64_t c0 = b * kQK + lane * 4;
        const float e[4] = {normed(c0), normed(c0 + 1), normed(c0 + 2), normed(c0 + 3)};
        if (normed_out) *reinterpret_cast<float4*>(normed_out + base + c0) = make_float4(e[0], e[1], e[2], e[3]);
        store_amajor(q_aq, q_ad, blockIdx.x, b, nb, lane, quantize_block_q8k(e, lane));
    }
}

// The same operator for rows of whole super-blocks (cols % 256 == 0: every projection input), one pass: wavefront v of
// the workgroup owns the super-blocks v, v + 4, ... of the row and lane l their elements 4l .. 4l+3 -- the mapping
// the quantizer wants -- from the first load on, and keeps up to kKeep super-blocks in registers, so nothing is read
// twice and nothing waits for a store.  The squares are summed per thread in that order (super-block by
// super-block, element by element), then across the lanes of a wavefront by butterfly, then (w0 + w1) + (w2 + w3).
// kKeep == 0: longer rows; the thread re-reads what it stored (or adds again).
template <int kKeep>
__global__ void __launch_bounds__(256) add_rmsnorm_blocks_kernel(const float* x, const float* __restrict__ delta,
                                                                 const float* __restrict__ weight, int64_t cols, float eps,
                                                                 float* sum_out, float* __restrict__ normed_out,
                                                                 uint8_t* __restrict__ q_aq, float* __restrict__ q_ad) {
    __shared__ float wave_sum[4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t base = (int64_t)blockIdx.x * cols;
    const int64_t nb = cols / kQK;
    auto fetch = [&](int64_t c0) {
        float4 a = *reinterpret_cast<const float4*>(x + base + c0);
        if (delta) {
            const float4 d = *reinterpret_cast<const float4*>(delta + base + c0);
            a.x = __fadd_rn(a.x, d.x), a.y = __fadd_rn(a.y, d.y), a.z = __fadd_rn(a.z, d.z), a.w = __fadd_rn(a.w, d.w);
        }
        return a;
    };
    float4 kept[kKeep > 0 ? kKeep : 1];
    float ssq = 0.0f;
    auto first_pass = [&](int64_t b, float4& slot) {
        const int64_t c0 = b * kQK + lane * 4;
        const float4 a = fetch(c0);
        if (sum_out) *reinterpret_cast<float4*>(sum_out + base + c0) = a;
        ssq = __fmaf_rn(a.x, a.x, ssq);
        ssq = __fmaf_rn(a.y, a.y, ssq);
        ssq = __fmaf_rn(a.z, a.z, ssq);
        ssq = __fmaf_rn(a.w, a.w, ssq);
        slot = a;
    };
    // kKeep > 0: every operand of the row -- x, residual, norm weights -- is requested first and unconditionally (a
    // block past the end re-reads block 0, a missing residual or weight re-reads x), and nothing is stored before
    // the barrier: conditional loads go out one round trip after the other, and a barrier waits for earlier stores.
    float4 wn[kKeep > 0 ? kKeep : 1];
    if (kKeep > 0) {
        const float* dp = delta ? delta : x;
        const float* wp = weight ? weight : x;
        float4 dl[kKeep > 0 ? kKeep : 1];
#pragma unroll
        for (int i = 0; i < kKeep; ++i) {
            const int64_t c0 = (wave + 4 * i < nb ? wave + 4 * i : 0) * kQK + lane * 4;
            kept[i] = *reinterpret_cast<const float4*>(x + base + c0);
            dl[i] = *reinterpret_cast<const float4*>(dp + base + c0);
            wn[i] = *reinterpret_cast<const float4*>(wp + c0);
        }
#pragma unroll
        for (int i = 0; i < kKeep; ++i) {
            if (wave + 4 * i < nb) {
                float4 a = kept[i];
                if (delta) {
                    const float4 d = dl[i];
                    a.x = __fadd_rn(a.x, d.x), a.y = __fadd_rn(a.y, d.y), a.z = __fadd_rn(a.z, d.z), a.w = __fadd_rn(a.w, d.w);
                }
                ssq = __fmaf_rn(a.x, a.x, ssq);
                ssq = __fmaf_rn(a.y, a.y, ssq);
                ssq = __fmaf_rn(a.z, a.z, ssq);
                ssq = __fmaf_rn(a.w, a.w, ssq);
                kept[i] = a;
            }
        }
    } else {
        for (int64_t b = wave; b < nb; b += 4) first_pass(b, kept[0]);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) ssq += __shfl_xor(ssq, off, 64);
    if (lane == 0) wave_sum[wave] = ssq;
    __syncthreads();
    const float total = (wave_sum[0] + wave_sum[1]) + (wave_sum[2] + wave_sum[3]);
    const float scale = __fdiv_rn(1.0f, __fsqrt_rn(__fadd_rn(__fdiv_rn(total, (float)cols), eps)));
    auto second_pass = [&](int64_t b, const float4& a) {
        const int64_t c0 = b * kQK + lane * 4;
        float4 w = make_float4(1.0f, 1.0f, 1.0f, 1.0f);
        if (weight) w = *reinterpret_cast<const float4*>(weight + c0);
        const float e[4] = {__fmul_rn(a.x, weight ? __fmul_rn(scale, w.x) : scale), __fmul_rn(a.y, weight ? __fmul_rn(scale, w.y) : scale),
                            __fmul_rn(a.z, weight ? __fmul_rn(scale, w.z) : scale), __fmul_rn(a.w, weight ? __fmul_rn(scale, w.w) : scale)};
        if (normed_out) *reinterpret_cast<float4*>(normed_out + base + c0) = make_float4(e[0], e[1], e[2], e[3]);
        if (q_aq) store_amajor(q_aq, q_ad, blockIdx.x, b, nb, lane, quantize_block_q8k(e, lane));
    };
    if (kKeep > 0) {
#pragma unroll
        for (int i = 0; i < kKeep; ++i) {
            if (wave + 4 * i < nb) {
                const int64_t b = wave + 4 * i, c0 = b * kQK + lane * 4;
                const float4 a = kept[i], w = wn[i];
                // sum_out may alias x: every thread has read its own elements long before it stores them
                if (sum_out) *reinterpret_cast<float4*>(sum_out + base + c0) = a;
                const float e[4] = {__fmul_rn(a.x, weight ? __fmul_rn(scale, w.x) : scale), __fmul_rn(a.y, weight ? __fmul_rn(scale, w.y) : scale),
                                    __fmul_rn(a.z, weight ? __fmul_rn(scale, w.z) : scale), __fmul_rn(a.w, weight ? __fmul_rn(scale, w.w) : scale)};
                if (normed_out) *reinterpret_cast<float4*>(normed_out + base + c0) = make_float4(e[0], e[1], e[2], e[3]);
                if (q_aq) store_amajor(q_aq, q_ad, blockIdx.x, b, nb, lane, quantize_block_q8k(e, lane));
            }
        }
    } else {
        for (int64_t b = wave; b < nb; b += 4) {
            const int64_t c0 = b * kQK + lane * 4;
            // sum_out may alias x: the thread re-reads what it stored itself rather than adding delta twice
            second_pass(b, sum_out ? *reinterpret_cast<const float4*>(sum_out + base + c0) : fetch(c0));
        }
    }
}

// logits[t][e] = w[e] . x[t], fp32 (the ffn_gate_inp projection, core/src/llm/graph/decoder.cpp:2265).
// One wavefront per (expert, token): lanes stride the columns, fixed-order butterfly at the end.
__global__ void __launch_bounds__(256) router_logits_kernel(const float* __restrict__ w, int64_t n_experts,
                                                            int64_t cols, const float* __restrict__ x, int64_t ldx,
                                                            float* __restrict__ logits) {
    const int lane = threadIdx.x & 63;
    const int64_t e = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t t = blockIdx.y;
    if (e >= n_experts) return;
    const float* wr = w + e * cols;
    const float* xr = x + t * ldx;
    float acc = 0.0f;
    auto add4 = [&](const float4& a, const float4& b) {
        acc = __fmaf_rn(a.x, b.x, acc);
        acc = __fmaf_rn(a.y, b.y, acc);
        acc = __fmaf_rn(a.z, b.z, acc);
        acc = __fmaf_rn(a.w, b.w, acc);
    };
    // same order of additions as one column group after the other; the operands of eight groups are requested
    // together so that their latencies overlap (a row of 2048 columns is one such batch)
    int64_t c = (int64_t)lane * 4;
    for (; c + 7 * 256 + 3 < cols; c += 8 * 256) {
        float4 a[8], b[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            a[u] = *reinterpret_cast<const float4*>(wr + c + u * 256);
            b[u] = *reinterpret_cast<const float4*>(xr + c + u * 256);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) add4(a[u], b[u]);
    }
    for (; c + 3 < cols; c += 256) add4(*reinterpret_cast<const float4*>(wr + c), *reinterpret_cast<const float4*>(xr + c));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
    if (lane == 0) logits[t * n_experts + e] = acc;
}

// Residual add + RMSNorm + router projection in one launch: workgroup (g, t) normalises row t itself (the
// arithmetic and the summation order of add_rmsnorm_blocks_kernel, repeated by every workgroup of the row: 8 KB
// of loads), parks the normalised row in LDS and its four wavefronts form the logits of the experts 4g .. 4g+3
// (router_logits_kernel's order); workgroup g = 0 also writes the sum and the normalised row out.  Same bits as
// the two launches.  sum_out must not be x or delta: other workgroups still read them.
__global__ void __launch_bounds__(256) add_rmsnorm_router_kernel(const float* __restrict__ x, const float* __restrict__ delta,
                                                                 const float* __restrict__ weight, int64_t cols, float eps,
                                                                 float* __restrict__ sum_out, float* __restrict__ normed_out,
                                                                 const float* __restrict__ w_router, int64_t n_experts,
                                                                 float* __restrict__ logits) {
    extern __shared__ __attribute__((aligned(16))) float row_sh[];  // [cols]
    __shared__ float wave_sum[4];
    constexpr int kKeep = 4;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t t = blockIdx.y, base = t * cols, nb = cols / kQK;
    const bool writer = blockIdx.x == 0;
    // this wavefront's router row does not depend on the norm: its first eight chunks are requested before anything
    // else, so that their trip from HBM overlaps the norm instead of following it
    const int64_t ex = (int64_t)blockIdx.x * 4 + wave;
    const float* wr = w_router + (ex < n_experts ? ex : 0) * cols;
    const bool ahead = cols >= 8 * 256;  // wave-uniform
    float4 first[8];
    if (ahead) {
#pragma unroll
        for (int u = 0; u < 8; ++u) first[u] = *reinterpret_cast<const float4*>(wr + lane * 4 + u * 256);
    }
    // The operands of the norm are requested together and unconditionally (a block past the end re-reads block 0,
    // a missing residual or weight re-reads x): conditional loads would go out one round trip after the other.
    const float* dp = delta ? delta : x;
    const float* wp = weight ? weight : x;
    float4 kept[kKeep], dl[kKeep], wn[kKeep];
#pragma unroll
    for (int i = 0; i < kKeep; ++i) {
        const int64_t b = wave + 4 * i;
        const int64_t c0 = (b < nb ? b : 0) * kQK + lane * 4;
        kept[i] = *reinterpret_cast<const float4*>(x + base + c0);
        dl[i] = *reinterpret_cast<const float4*>(dp + base + c0);
        wn[i] = *reinterpret_cast<const float4*>(wp + c0);
    }
    float ssq = 0.0f;
#pragma unroll
    for (int i = 0; i < kKeep; ++i) {
        if (wave + 4 * i < nb) {
            float4 a = kept[i];
            if (delta) {
                const float4 d = dl[i];
                a.x = __fadd_rn(a.x, d.x), a.y = __fadd_rn(a.y, d.y), a.z = __fadd_rn(a.z, d.z), a.w = __fadd_rn(a.w, d.w);
            }
            ssq = __fmaf_rn(a.x, a.x, ssq);
            ssq = __fmaf_rn(a.y, a.y, ssq);
            ssq = __fmaf_rn(a.z, a.z, ssq);
            ssq = __fmaf_rn(a.w, a.w, ssq);
            kept[i] = a;
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) ssq += __shfl_xor(ssq, off, 64);
    if (lane == 0) wave_sum[wave] = ssq;
    __syncthreads();
    const float total = (wave_sum[0] + wave_sum[1]) + (wave_sum[2] + wave_sum[3]);
    const float scale = __fdiv_rn(1.0f, __fsqrt_rn(__fadd_rn(__fdiv_rn(total, (float)cols), eps)));
#pragma unroll
    for (int i = 0; i < kKeep; ++i) {
        if (wave + 4 * i < nb) {
            const int64_t c0 = (int64_t)(wave + 4 * i) * kQK + lane * 4;
            const float4 a = kept[i], w = wn[i];
            const float4 e = make_float4(__fmul_rn(a.x, weight ? __fmul_rn(scale, w.x) : scale), __fmul_rn(a.y, weight ? __fmul_rn(scale, w.y) : scale),
                                         __fmul_rn(a.z, weight ? __fmul_rn(scale, w.z) : scale), __fmul_rn(a.w, weight ? __fmul_rn(scale, w.w) : scale));
            *reinterpret_cast<float4*>(row_sh + c0) = e;
        }
    }
    __syncthreads();
    // a wavefront without an expert of its own forms expert 0's logit again and drops it (it may still have stores to make)
    float acc = 0.0f;
    auto add4 = [&](const float4& a, const float4& b) {
        acc = __fmaf_rn(a.x, b.x, acc);
        acc = __fmaf_rn(a.y, b.y, acc);
        acc = __fmaf_rn(a.z, b.z, acc);
        acc = __fmaf_rn(a.w, b.w, acc);
    };
    int64_t c = (int64_t)lane * 4;
    if (ahead) {
#pragma unroll
        for (int u = 0; u < 8; ++u) add4(first[u], *reinterpret_cast<const float4*>(row_sh + c + u * 256));
        c += 8 * 256;
    }
    for (; c + 7 * 256 + 3 < cols; c += 8 * 256) {
        float4 a[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) a[u] = *reinterpret_cast<const float4*>(wr + c + u * 256);
#pragma unroll
        for (int u = 0; u < 8; ++u) add4(a[u], *reinterpret_cast<const float4*>(row_sh + c + u * 256));
    }
    for (; c + 3 < cols; c += 256) add4(*reinterpret_cast<const float4*>(wr + c), *reinterpret_cast<const float4*>(row_sh + c));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
    if (lane == 0 && ex < n_experts) logits[t * n_experts + ex] = acc;
    if (writer) {  // last: a store ahead of a barrier would make the barrier wait for it
#pragma unroll
        for (int i = 0; i < kKeep; ++i) {
            if (wave + 4 * i < nb) {
                const int64_t c0 = (int64_t)(wave + 4 * i) * kQK + lane * 4;
                if (sum_out) *reinterpret_cast<float4*>(sum_out + base + c0) = kept[i];
                if (normed_out) *reinterpret_cast<float4*>(normed_out + base + c0) = *reinterpret_cast<const float4*>(row_sh + c0);
            }
        }
    }
}

// out = silu(gate) * up, element by element over [n][cols] with their own row strides: the node between the gate / up
// products and the down product of a dense FFN (cb_silu_mul_fused, core/src/llm/graph/fused_ops.cpp:317-366).
__global__ void __launch_bounds__(256) silu_mul_kernel(const float* __restrict__ gate, const float* __restrict__ up, int64_t n,
                                                       int64_t cols, int64_t ld_gate, int64_t ld_up, float* __restrict__ out,
                                                       int64_t ld_out, int mode) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n * cols) return;
    const uint32_t row = (uint32_t)i / (uint32_t)cols, c = (uint32_t)i - row * (uint32_t)cols;  // n * cols < 2^31 (launcher)
    out[(size_t)row * ld_out + c] = silu_mul(gate[(size_t)row * ld_gate + c], up[(size_t)row * ld_up + c], mode);
}

// out[t] = sigmoid(logit[t]) * src[t] with the two-sided sigmoid of core/src/llm/graph/fused_ops.cpp:451-458
// (cb_apply_shared_scalar_gate, :437-475): the scalar gate of the shared expert.
__global__ void __launch_bounds__(256) scale_rows_sigmoid_kernel(const float* __restrict__ src, int64_t n, int64_t cols, int64_t ld_src,
                                                                 const float* __restrict__ logit, int64_t ld_logit,
                                                                 float* __restrict__ out, int64_t ld_out) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n * cols) return;
    const uint32_t row = (uint32_t)i / (uint32_t)cols, c = (uint32_t)i - row * (uint32_t)cols;
    const float x = logit[(size_t)row * ld_logit];
    float g;
    if (x >= 0.0f) {
        g = __fdiv_rn(1.0f, __fadd_rn(1.0f, expf(-x)));
    } else {
        const float z = expf(x);
        g = __fdiv_rn(z, __fadd_rn(1.0f, z));
    }
    out[(size_t)row * ld_out + c] = __fmul_rn(src[(size_t)row * ld_src + c], g);
}

}  // namespace

hipError_t launch_add_rmsnorm_router(const float* x, const float* delta, const float* weight, int64_t n, int64_t cols, float eps,
                                     float* sum_out, float* normed_out, const float* w_router, int64_t n_experts, float* logits,
                                     hipStream_t stream) {
    if (n == 0) return hipSuccess;
    if ((cols % kQK) || cols > 4 * 4 * kQK || n > 65535 || n_experts <= 0) return hipErrorInvalidValue;
    MQ_LAUNCH(add_rmsnorm_router_kernel, dim3((unsigned)((n_experts + 3) / 4), (unsigned)n), dim3(256),
                       (size_t)cols * sizeof(float), stream, x, delta, weight, cols, eps, sum_out, normed_out, w_router, n_experts,
                       logits);
    return hipGetLastError();
}

hipError_t launch_add_rmsnorm(const float* x, const float* delta, const float* weight, int64_t n, int64_t cols,
                              float eps, float* sum_out, float* normed_out, uint8_t* q_aq, float* q_ad,
                              hipStream_t stream) {
    if (n == 0) return hipSuccess;
    if (q_aq && (cols % kQK)) return hipErrorInvalidValue;
    const bool vec = (cols % kQK) == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(delta) |
                                            reinterpret_cast<uintptr_t>(weight) | reinterpret_cast<uintptr_t>(sum_out) |
                                            reinterpret_cast<uintptr_t>(normed_out)) & 15u) == 0;
    if (vec && cols <= 4 * 4 * kQK) {
        MQ_LAUNCH(add_rmsnorm_blocks_kernel<4>, dim3((unsigned)n), dim3(256), 0, stream, x, delta, weight, cols, eps,
                           sum_out, normed_out, q_aq, q_ad);
    } else if (vec) {
        MQ_LAUNCH(add_rmsnorm_blocks_kernel<0>, dim3((unsigned)n), dim3(256), 0, stream, x, delta, weight, cols, eps,
                           sum_out, normed_out, q_aq, q_ad);
    } else {
        MQ_LAUNCH(add_rmsnorm_kernel, dim3((unsigned)n), dim3(256), 0, stream, x, delta, weight, cols, eps, sum_out,
                           normed_out, q_aq, q_ad);
    }
    return hipGetLastError();
}

hipError_t launch_router_logits(const float* w, int64_t n_experts, int64_t cols, const float* x, int64_t n, int64_t ldx,
                                float* logits, hipStream_t stream) {
    if (n == 0) return hipSuccess;
    if (n > 65535) return hipErrorInvalidValue;
    MQ_LAUNCH(router_logits_kernel, dim3((unsigned)((n_experts + 3) / 4), (unsigned)n), dim3(256), 0, stream, w,
                       n_experts, cols, x, ldx, logits);
    return hipGetLastError();
}

hipError_t launch_silu_mul(const float* gate, const float* up, int64_t n, int64_t cols, int64_t ld_gate, int64_t ld_up, float* out,
                           int64_t ld_out, int mode, hipStream_t stream) {
    if (n * cols == 0) return hipSuccess;
    if (n * cols >= (int64_t)1 << 31) return hipErrorInvalidValue;
    MQ_LAUNCH(silu_mul_kernel, dim3((unsigned)((n * cols + 255) / 256)), dim3(256), 0, stream, gate, up, n, cols, ld_gate, ld_up,
                       out, ld_out, mode);
    return hipGetLastError();
}

hipError_t launch_scale_rows_sigmoid(const float* src, int64_t n, int64_t cols, int64_t ld_src, const float* logit, int64_t ld_logit,
                                     float* out, int64_t ld_out, hipStream_t stream) {
    if (n * cols == 0) return hipSuccess;
    if (n * cols >= (int64_t)1 << 31) return hipErrorInvalidValue;
    MQ_LAUNCH(scale_rows_sigmoid_kernel, dim3((unsigned)((n * cols + 255) / 256)), dim3(256), 0, stream, src, n, cols, ld_src,
                       logit, ld_logit, out, ld_out);
    return hipGetLastError();
}

}  // namespace mq
