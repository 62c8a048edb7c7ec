// Q8_K activation quantizer for gfx950: one wavefront per 256-value super-block.
//
// Bit-exact with the reference quantizer (core/src/kernels/hwy/hwy_moe_quant.cc:103-143):
//   * the extreme element is the FIRST one of largest magnitude and keeps its sign, so the
//     cross-lane arg-max breaks ties towards the lower index;
//   * iscale = -127/max and d = 1/iscale are correctly rounded divisions;
//   * iscale*x is rounded before the +1.5*2^23 add (no FMA contraction), which then yields
//     round-half-even in the low mantissa bits.
#include "common.h"
#include "kernels.h"

namespace mq {

namespace {

__device__ __forceinline__ int nearest_int_rne(float v) {
    const float biased = __fadd_rn(v, 12582912.0f);
    return (__float_as_int(biased) & 0x007fffff) - 0x00400000;
}

__global__ void __launch_bounds__(256) quantize_q8k_kernel(const float* __restrict__ x, int64_t n, int64_t ldx,
                                                           int64_t nb, uint8_t* __restrict__ q8_std,
                                                           size_t q8_row_bytes, uint8_t* __restrict__ aq,
                                                           float* __restrict__ ad) {
    const int lane = threadIdx.x & 63;
    const int64_t unit = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);  // (row, block) pair
    if (unit >= n * nb) return;
    const int64_t m = unit / nb;
    const int64_t b = unit - m * nb;

    const float4 v = *reinterpret_cast<const float4*>(x + m * ldx + b * kQK + lane * 4);
    const float e[4] = {v.x, v.y, v.z, v.w};

    // first-of-largest-magnitude within the lane, then across the wave (lower index wins ties)
    float best_abs = 0.0f, best = 0.0f;
    int best_idx = lane * 4;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float a = fabsf(e[j]);
        if (a > best_abs) {
            best_abs = a;
            best = e[j];
            best_idx = lane * 4 + j;
        }
    }
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const float o_abs = __shfl_xor(best_abs, off, 64);
        const float o_val = __shfl_xor(best, off, 64);
        const int o_idx = __shfl_xor(best_idx, off, 64);
        if (o_abs > best_abs || (o_abs == best_abs && o_idx < best_idx)) {
            best_abs = o_abs;
            best = o_val;
            best_idx = o_idx;
        }
    }

    int q[4] = {0, 0, 0, 0};
    float d = 0.0f;
    if (best_abs != 0.0f) {
        const float iscale = __fdiv_rn(-127.0f, best);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int r = nearest_int_rne(__fmul_rn(iscale, e[j]));
            q[j] = r > 127 ? 127 : r;
        }
        d = __fdiv_rn(1.0f, iscale);
    }
    const uint32_t packed = (uint32_t)(q[0] & 0xff) | ((uint32_t)(q[1] & 0xff) << 8) | ((uint32_t)(q[2] & 0xff) << 16) |
                            ((uint32_t)(q[3] & 0xff) << 24);
    int s = q[0] + q[1] + q[2] + q[3];
    s += __shfl_xor(s, 1, 64);
    s += __shfl_xor(s, 2, 64);  // lanes 4j..4j+3 now hold the sum of elements 16j..16j+15

    if (q8_std) {
        uint8_t* blk = q8_std + (size_t)m * q8_row_bytes + (size_t)b * kQ8Block;
        *reinterpret_cast<uint32_t*>(blk + 4 + lane * 4) = packed;
        if ((lane & 3) == 0) *reinterpret_cast<int16_t*>(blk + 260 + (lane >> 2) * 2) = (int16_t)s;
        if (lane == 0) *reinterpret_cast<float*>(blk) = d;
    }
    if (aq) {
        // element 4*lane+j: sub-block g = lane/8, index in sub-block 4*(lane%8)+j
        const int g = lane >> 3;
        const int kq = (lane & 7) >> 1;
        const size_t off = aq_offset(m, b, g >> 1, kq, nb) + (size_t)(g & 1) * 8 + (size_t)(lane & 1) * 4;
        *reinterpret_cast<uint32_t*>(aq + off) = packed;
        if (lane == 0) ad[ad_index(m, b, nb)] = d;
    }
}

__global__ void __launch_bounds__(256) q8k_to_amajor_kernel(const uint8_t* __restrict__ q8_std, int64_t n,
                                                            size_t q8_row_bytes, int64_t nb, uint8_t* __restrict__ aq,
                                                            float* __restrict__ ad) {
    const int lane = threadIdx.x & 63;
    const int64_t unit = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (unit >= n * nb) return;
    const int64_t m = unit / nb;
    const int64_t b = unit - m * nb;
    const uint8_t* blk = q8_std + (size_t)m * q8_row_bytes + (size_t)b * kQ8Block;
    const uint32_t packed = *reinterpret_cast<const uint32_t*>(blk + 4 + lane * 4);
    const int g = lane >> 3;
    const int kq = (lane & 7) >> 1;
    const size_t off = aq_offset(m, b, g >> 1, kq, nb) + (size_t)(g & 1) * 8 + (size_t)(lane & 1) * 4;
    *reinterpret_cast<uint32_t*>(aq + off) = packed;
    if (lane == 0) ad[ad_index(m, b, nb)] = *reinterpret_cast<const float*>(blk);
}

}  // namespace

hipError_t launch_quantize_q8k(const float* x, int64_t n, int64_t ldx, int64_t k, void* q8_std, size_t q8_row_bytes,
                               uint8_t* aq, float* ad, hipStream_t stream) {
    const int64_t nb = k / kQK;
    const int64_t units = n * nb;
    if (units == 0) return hipSuccess;
    const unsigned grid = (unsigned)((units + 3) / 4);
    hipLaunchKernelGGL(quantize_q8k_kernel, dim3(grid), dim3(256), 0, stream, x, n, ldx, nb, (uint8_t*)q8_std,
                       q8_row_bytes, aq, ad);
    return hipGetLastError();
}

hipError_t launch_q8k_to_amajor(const void* q8_std, int64_t n, size_t q8_row_bytes, int64_t k, uint8_t* aq, float* ad,
                                hipStream_t stream) {
    const int64_t nb = k / kQK;
    const int64_t units = n * nb;
    if (units == 0) return hipSuccess;
    const unsigned grid = (unsigned)((units + 3) / 4);
    hipLaunchKernelGGL(q8k_to_amajor_kernel, dim3(grid), dim3(256), 0, stream, (const uint8_t*)q8_std, n, q8_row_bytes,
                       nb, aq, ad);
    return hipGetLastError();
}

}  // namespace mq
