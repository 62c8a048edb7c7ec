// Single-row GEMV with the Q8_K quantizer inside (n == 1, short rows): y[r] = W[r] . q8k(x).
//
// At n = 1 the stand-alone quantizer launch costs about as much as the product itself.  Here every
// wavefront quantizes the super-blocks it multiplies: lane l loads x[256 b + 4l .. +3], the wave runs the
// same block quantizer as quantize_q8k_kernel (q8k_block.h: bit-identical codes and scale), and eight
// cross-lane reads put the codes into the split-slot A operand (row 0 owns M slots 0 and 1, common.h).
// The work is repeated by every workgroup, which is why the kernel is used only when a wave sees at most
// two super-blocks; workgroup shape, accumulation order and epilogue are those of matmul_kernel<1,1>, so
// the result is bit-identical to quantize + matmul.
// cb_gemv_custom quantizes on thread 0 and multiplies on all threads (core/src/llm/matmul/gemv_exec.cpp:298-341).
#include "common.h"
#include "kernels.h"
#include "decode_tile.h"
#include "q8k_block.h"

namespace mq {

namespace {

constexpr int kMaxStages = 2;

__global__ void __launch_bounds__(512) gemv1_fused_kernel(const uint8_t* __restrict__ w, int64_t rows, int64_t nb,
                                                          const float* __restrict__ x, float* __restrict__ y) {
    extern __shared__ float red[];  // [W-1][64]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n_waves = blockDim.x >> 6;
    const int slot = lane & 15, kq = lane >> 4;
    const int64_t rt = blockIdx.x;
    const uint8_t* tiles = w + tile_offset(rt, 0, nb);
    const int cnt = wave < nb ? (int)((nb - wave + n_waves - 1) / n_waves) : 0;  // <= kMaxStages (host-checked)

    TileRegs t[kMaxStages];
    float4 xv[kMaxStages];
#pragma unroll
    for (int i = 0; i < kMaxStages; ++i) {
        const int b = i < cnt ? wave + i * n_waves : 0;
        load_tile(t[i], tiles + (size_t)b * kTileBytes, lane);
        xv[i] = *reinterpret_cast<const float4*>(x + (size_t)b * kQK + lane * 4);
    }
    float acc[1][2] = {{0.0f, 0.0f}};
#pragma unroll
    for (int i = 0; i < kMaxStages; ++i) {
        if (i < cnt) {
            const float e[4] = {xv[i].x, xv[i].y, xv[i].z, xv[i].w};
            const Q8Lane q = quantize_block_q8k(e, lane);
            // code 4L + j sits in byte j of lane L.  Slot s (0: even sub-block, 1: odd) of k-group kq needs the
            // eight codes 64c + 32s + 8kq + (0..7) of chunk c: lanes 16c + 8s + 2kq and the next one.
            ARegs<1> a;
            const int src = 8 * (slot & 1) + 2 * kq;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const uint32_t lo = (uint32_t)__shfl((int)q.packed, 16 * c + src, 64);
                const uint32_t hi = (uint32_t)__shfl((int)q.packed, 16 * c + src + 1, 64);
                a.q[0][c] = slot == 0 ? v4u{lo, hi, 0u, 0u} : (slot == 1 ? v4u{0u, 0u, lo, hi} : v4u{0u, 0u, 0u, 0u});
            }
            a.yd[0][0] = q.d;   // row 0 (meaningful in k-group 0 only, the others are never stored)
            a.yd[0][1] = 0.0f;
            int32_t dsum[1][2], msum[1][2];
            compute_tile<1>(t[i], a, acc, dsum, msum);
        }
    }
    // cross-wave reduction in wave order, epilogue on wave 0 (as matmul_kernel)
    if (n_waves > 1) {
        if (wave > 0) red[(wave - 1) * 64 + lane] = acc[0][0];
        __syncthreads();
    }
    if (wave == 0) {
        float v = acc[0][0];
        for (int wv = 1; wv < n_waves; ++wv) v = __fadd_rn(v, red[(wv - 1) * 64 + lane]);
        const int64_t row = rt * 16 + slot;
        if (kq == 0 && row < rows) y[row] = v;
    }
}

}  // namespace

bool gemv1_fused_applies(int64_t nb, int waves) { return waves >= 1 && (nb + waves - 1) / waves <= kMaxStages; }

hipError_t launch_gemv1_fused(const uint8_t* w, int64_t rows, int64_t nb, const float* x, float* y, int waves,
                              hipStream_t stream) {
    if (!gemv1_fused_applies(nb, waves) || rows <= 0) return hipErrorInvalidValue;
    const int64_t rowtiles = (rows + 15) / 16;
    hipLaunchKernelGGL(gemv1_fused_kernel, dim3((unsigned)rowtiles), dim3(64 * waves),
                       waves > 1 ? (size_t)(waves - 1) * 64 * sizeof(float) : 0, stream, w, rows, nb, x, y);
    return hipGetLastError();
}

}  // namespace mq
