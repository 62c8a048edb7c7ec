// Q8_K activation quantizer for gfx950: one wavefront per 256-value super-block (q8k_block.h holds
// the arithmetic and its bit-exactness notes).
#include "common.h"
#include "kernels.h"
#include "q8k_block.h"

namespace mq {

namespace {

__global__ void __launch_bounds__(256) quantize_q8k_kernel(const float* __restrict__ x, int64_t n, int64_t ldx,
                                                           int64_t nb, uint8_t* __restrict__ q8_std,
                                                           size_t q8_row_bytes, uint8_t* __restrict__ aq,
                                                           float* __restrict__ ad) {
    const int lane = threadIdx.x & 63;
    const int64_t unit = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);  // (row, block) pair
    if (unit >= n * nb) return;
    int64_t m, b;
    split_unit(unit, nb, m, b);

    const float4 v = *reinterpret_cast<const float4*>(x + m * ldx + b * kQK + lane * 4);
    const float e[4] = {v.x, v.y, v.z, v.w};
    const Q8Lane r = quantize_block_q8k(e, lane);

    if (q8_std) {
        uint8_t* blk = q8_std + (size_t)m * q8_row_bytes + (size_t)b * kQ8Block;
        *reinterpret_cast<uint32_t*>(blk + 4 + lane * 4) = r.packed;
        if ((lane & 3) == 0) *reinterpret_cast<int16_t*>(blk + 260 + (lane >> 2) * 2) = (int16_t)r.bsum;
        if (lane == 0) *reinterpret_cast<float*>(blk) = r.d;
    }
    if (aq) store_amajor(aq, ad, m, b, nb, lane, r);
}

__global__ void __launch_bounds__(256) q8k_to_amajor_kernel(const uint8_t* __restrict__ q8_std, int64_t n,
                                                            size_t q8_row_bytes, int64_t nb, uint8_t* __restrict__ aq,
                                                            float* __restrict__ ad) {
    const int lane = threadIdx.x & 63;
    const int64_t unit = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (unit >= n * nb) return;
    int64_t m, b;
    split_unit(unit, nb, m, b);
    const uint8_t* blk = q8_std + (size_t)m * q8_row_bytes + (size_t)b * kQ8Block;
    Q8Lane r;
    r.packed = *reinterpret_cast<const uint32_t*>(blk + 4 + lane * 4);
    r.d = *reinterpret_cast<const float*>(blk);
    r.bsum = 0;
    store_amajor(aq, ad, m, b, nb, lane, r);
}

}  // namespace

hipError_t launch_quantize_q8k(const float* x, int64_t n, int64_t ldx, int64_t k, void* q8_std, size_t q8_row_bytes,
                               uint8_t* aq, float* ad, hipStream_t stream) {
    const int64_t nb = k / kQK;
    const int64_t units = n * nb;
    if (units == 0) return hipSuccess;
    if (units >= (int64_t)1 << 31) return hipErrorInvalidValue;  // split_unit divides in 32 bits
    const unsigned grid = (unsigned)((units + 3) / 4);
    MQ_LAUNCH(quantize_q8k_kernel, dim3(grid), dim3(256), 0, stream, x, n, ldx, nb, (uint8_t*)q8_std,
                       q8_row_bytes, aq, ad);
    return hipGetLastError();
}

hipError_t launch_q8k_to_amajor(const void* q8_std, int64_t n, size_t q8_row_bytes, int64_t k, uint8_t* aq, float* ad,
                                hipStream_t stream) {
    const int64_t nb = k / kQK;
    const int64_t units = n * nb;
    if (units == 0) return hipSuccess;
    if (units >= (int64_t)1 << 31) return hipErrorInvalidValue;  // split_unit divides in 32 bits
    const unsigned grid = (unsigned)((units + 3) / 4);
    MQ_LAUNCH(q8k_to_amajor_kernel, dim3(grid), dim3(256), 0, stream, (const uint8_t*)q8_std, n, q8_row_bytes,
                       nb, aq, ad);
    return hipGetLastError();
}

}  // namespace mq
