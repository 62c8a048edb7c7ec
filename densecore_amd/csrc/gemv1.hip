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

__device__ __forceinline__ void gemv1_fused_body(const uint8_t* __restrict__ w, int64_t rows, int64_t nb, const float* __restrict__ x,
                                                 float* __restrict__ y, int64_t rt, float* red) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n_waves = blockDim.x >> 6;
    const int slot = lane & 15, kq = lane >> 4;
    const uint8_t* tiles = w + tile_offset(rt, 0, nb);
    const int cnt = (wave < nb ? 1 : 0) + (wave + n_waves < nb ? 1 : 0);  // super-blocks wave, wave + W (at most kMaxStages, host-checked; no division)

    // The activations are requested before the tiles (requests are answered in order) and quantized while the
    // tiles travel; only row 0 of the operand is formed (J = 1).
    TileRegs t[kMaxStages];
    float4 xv[kMaxStages];
#pragma unroll
    for (int i = 0; i < kMaxStages; ++i) xv[i] = *reinterpret_cast<const float4*>(x + (size_t)(i < cnt ? wave + i * n_waves : 0) * kQK + lane * 4);
#pragma unroll
    for (int i = 0; i < kMaxStages; ++i) load_tile(t[i], tiles + (size_t)(i < cnt ? wave + i * n_waves : 0) * kTileBytes, lane);
    // code 4L + j sits in byte j of lane L.  Slot s (0: even sub-block, 1: odd) of k-group kq needs the eight codes
    // 64c + 32s + 8kq + (0..7) of chunk c: lanes 16c + 8s + 2kq and the next one (a_codes_from_lane_codes).
    ACodes codes[kMaxStages];
#pragma unroll
    for (int i = 0; i < kMaxStages; ++i) {
        const float e[4] = {xv[i].x, xv[i].y, xv[i].z, xv[i].w};
        a_codes_from_lane_codes(codes[i], quantize_block_q8k(e, lane), lane);
    }
    float acc[1][2] = {{0.0f, 0.0f}};
#pragma unroll
    for (int i = 0; i < kMaxStages; ++i) {
        if (i < cnt) {
            ARegs<1> a;  // row 0 (meaningful in k-group 0 only, the others are never stored)
            a_from_codes(a, codes[i], lane);
            int32_t dsum[1][2], msum[1][2];
            compute_tile<1, false, 1>(t[i], a, acc, dsum, msum);
        }
    }
    // cross-wave reduction in wave order, epilogue on wave 0 (as matmul_kernel)
    if (n_waves > 1) {
        if (wave > 0) red[(wave - 1) * 64 + lane] = acc[0][0];
        __syncthreads();
    }
    if (wave == 0) {
        float v = acc[0][0];
        if (n_waves > 1) v = add_wave_partials(v, n_waves, [&](int wv) { return red[(wv - 1) * 64 + lane]; });
        const int64_t row = rt * 16 + slot;
        if (kq == 0 && row < rows) y[row] = v;
    }
}

__global__ void __launch_bounds__(512) gemv1_fused_kernel(const uint8_t* __restrict__ w, int64_t rows, int64_t nb,
                                                          const float* __restrict__ x, float* __restrict__ y) {
    extern __shared__ float red[];  // [W-1][64]
    gemv1_fused_body(w, rows, nb, x, y, blockIdx.x, red);
}

// Several matrices against ONE activation row in one launch (the q, k and v projections of a layer, the gate and up
// projections of an FFN: core/src/llm/graph/decoder.cpp:1092-1099, :2662-2663 emit them as separate nodes on the same
// input).  The grid is the matrices' row tiles one after the other, RT consecutive row tiles of one matrix to a
// workgroup; per row tile the arithmetic, the wave split and the reduction order are the single-matrix kernel's, so the
// bits are those of one launch per matrix -- whose dispatch and first trip to memory are paid once here, and whose
// quantization of x (every workgroup repeats it) once per RT row tiles: with a thousand workgroups that repetition,
// not memory, is what a launch costs.
template <int RT>
__global__ void __launch_bounds__(512) gemv1_multi_kernel(const Gemv1MultiArgs p) {
    extern __shared__ float red[];  // [RT][W-1][64]
    const int g = blockIdx.x;
    int m = 0;
#pragma unroll
    for (int i = 1; i < kGemvMultiMax; ++i) m += (i < p.count && g >= p.rt_begin[i]) ? 1 : 0;  // begins ascend: a count, no search
    const uint8_t* w = p.w[m];
    const int64_t rows = p.rows[m], nb = p.nb;
    const int64_t rowtiles = (rows + 15) >> 4;
    const int64_t rt0 = (int64_t)(g - p.rt_begin[m]) * RT;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n_waves = blockDim.x >> 6;
    const int slot = lane & 15, kq = lane >> 4;
    const int cnt = (wave < nb ? 1 : 0) + (wave + n_waves < nb ? 1 : 0);
    TileRegs t[RT][kMaxStages];
    float4 xv[kMaxStages];
#pragma unroll
    for (int i = 0; i < kMaxStages; ++i) xv[i] = *reinterpret_cast<const float4*>(p.x + (size_t)(i < cnt ? wave + i * n_waves : 0) * kQK + lane * 4);
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        // a row tile past the matrix's last streams the last one again and stores nothing
        const uint8_t* tiles = w + tile_offset(rt0 + r < rowtiles ? rt0 + r : rowtiles - 1, 0, nb);
#pragma unroll
        for (int i = 0; i < kMaxStages; ++i) load_tile(t[r][i], tiles + (size_t)(i < cnt ? wave + i * n_waves : 0) * kTileBytes, lane);
    }
    ACodes codes[kMaxStages];
#pragma unroll
    for (int i = 0; i < kMaxStages; ++i) {
        const float e[4] = {xv[i].x, xv[i].y, xv[i].z, xv[i].w};
        a_codes_from_lane_codes(codes[i], quantize_block_q8k(e, lane), lane);
    }
    float acc[RT][1][2];
#pragma unroll
    for (int r = 0; r < RT; ++r) acc[r][0][0] = acc[r][0][1] = 0.0f;
#pragma unroll
    for (int i = 0; i < kMaxStages; ++i) {
        if (i < cnt) {
            ARegs<1> a;
            a_from_codes(a, codes[i], lane);
#pragma unroll
            for (int r = 0; r < RT; ++r) {
                int32_t dsum[1][2], msum[1][2];
                compute_tile<1, false, 1>(t[r][i], a, acc[r], dsum, msum);
            }
        }
    }
    if (n_waves > 1) {
        if (wave > 0) {
#pragma unroll
            for (int r = 0; r < RT; ++r) red[(r * (n_waves - 1) + wave - 1) * 64 + lane] = acc[r][0][0];
        }
        __syncthreads();
    }
    if (wave == 0) {
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            float v = acc[r][0][0];
            if (n_waves > 1) v = add_wave_partials(v, n_waves, [&](int wv) { return red[(r * (n_waves - 1) + wv - 1) * 64 + lane]; });
            const int64_t row = (rt0 + r) * 16 + slot;
            if (kq == 0 && rt0 + r < rowtiles && row < rows) p.y[m][row] = v;
        }
    }
}

// The same GEMV with the residual add and the RMSNorm of its input inside as well (one row):
//     s = x + delta;  h = s * (weight / sqrt(mean(s^2) + eps));  y[r] = W[r] . q8k(h)
// The first four wavefronts of every workgroup sum the squares of the row exactly as add_rmsnorm_blocks_kernel does
// (wavefront v takes the super-blocks v, v + 4, ..., lane l their elements 4l .. 4l+3; butterfly; (w0 + w1) +
// (w2 + w3)) while the weight tiles travel -- 8 KB of loads repeated per workgroup -- then every wavefront
// normalises and quantizes the super-blocks it multiplies.  Workgroup 0 also writes s out (sum_out must not be x or
// delta: the other workgroups still read them).  Same bits as mq_add_rmsnorm_q8k followed by the product.
__global__ void __launch_bounds__(512) gemv1_norm_fused_kernel(const uint8_t* __restrict__ w, int64_t rows, int64_t nb,
                                                               const float* __restrict__ x, const float* __restrict__ delta,
                                                               const float* __restrict__ weight, float eps,
                                                               float* __restrict__ sum_out, float* __restrict__ y) {
    extern __shared__ float red[];  // [W-1][64]
    __shared__ float wave_sum[4];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n_waves = blockDim.x >> 6;
    const int slot = lane & 15, kq = lane >> 4;
    const int64_t rt = blockIdx.x;
    const uint8_t* tiles = w + tile_offset(rt, 0, nb);
    const int cnt = (wave < nb ? 1 : 0) + (wave + n_waves < nb ? 1 : 0);  // super-blocks wave, wave + W (at most kMaxStages, host-checked; no division)
    // Every request is unconditional (without a residual or without norm weights x is simply read again) and made
    // before the tile requests: requests are answered in order, and the norm must not wait for the tiles.
    const float* dp = delta ? delta : x;
    const float* wp = weight ? weight : x;
    auto add = [&](float4 a, const float4& d) {
        if (delta) a.x = __fadd_rn(a.x, d.x), a.y = __fadd_rn(a.y, d.y), a.z = __fadd_rn(a.z, d.z), a.w = __fadd_rn(a.w, d.w);
        return a;
    };
    // sum of squares in the order of the 256-thread norm kernel: virtual wavefront v = 0..3 takes the super-blocks
    // v, v + 4, ... (at most four of them here); with four or more wavefronts wavefront v is virtual wavefront v
    const bool four = n_waves >= 4;
    const int v4 = wave & 3;
    float4 sx[4], sd[4];
    if (four) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int64_t c0 = (int64_t)(v4 + 4 * k < nb ? v4 + 4 * k : 0) * kQK + lane * 4;
            sx[k] = *reinterpret_cast<const float4*>(x + c0);
            sd[k] = *reinterpret_cast<const float4*>(dp + c0);
        }
    }
    TileRegs t[kMaxStages];
    float4 xv[kMaxStages], dv[kMaxStages], wn[kMaxStages];
#pragma unroll
    for (int i = 0; i < kMaxStages; ++i) {
        const int64_t c0 = (int64_t)(i < cnt ? wave + i * n_waves : 0) * kQK + lane * 4;
        xv[i] = *reinterpret_cast<const float4*>(x + c0);
        dv[i] = *reinterpret_cast<const float4*>(dp + c0);
        wn[i] = *reinterpret_cast<const float4*>(wp + c0);
    }
#pragma unroll
    for (int i = 0; i < kMaxStages; ++i) load_tile(t[i], tiles + (size_t)(i < cnt ? wave + i * n_waves : 0) * kTileBytes, lane);
    if (four) {
        if (wave < 4) {
            float ssq = 0.0f;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                if (v4 + 4 * k < nb) {
                    const float4 a = add(sx[k], sd[k]);
                    ssq = __fmaf_rn(a.x, a.x, ssq);
                    ssq = __fmaf_rn(a.y, a.y, ssq);
                    ssq = __fmaf_rn(a.z, a.z, ssq);
                    ssq = __fmaf_rn(a.w, a.w, ssq);
                }
            }
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) ssq += __shfl_xor(ssq, off, 64);
            if (lane == 0) wave_sum[wave] = ssq;
        }
    } else {
        for (int v = wave; v < 4; v += n_waves) {
            float ssq = 0.0f;
            for (int64_t b = v; b < nb; b += 4) {
                const int64_t c0 = b * kQK + lane * 4;
                const float4 a = add(*reinterpret_cast<const float4*>(x + c0), *reinterpret_cast<const float4*>(dp + c0));
                ssq = __fmaf_rn(a.x, a.x, ssq);
                ssq = __fmaf_rn(a.y, a.y, ssq);
                ssq = __fmaf_rn(a.z, a.z, ssq);
                ssq = __fmaf_rn(a.w, a.w, ssq);
            }
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) ssq += __shfl_xor(ssq, off, 64);
            if (lane == 0) wave_sum[v] = ssq;
        }
    }
    __syncthreads();
    const float total = (wave_sum[0] + wave_sum[1]) + (wave_sum[2] + wave_sum[3]);
    const float scale = __fdiv_rn(1.0f, __fsqrt_rn(__fadd_rn(__fdiv_rn(total, (float)(nb * kQK)), eps)));

    // normalise and quantize while the tiles travel, then multiply (only row 0 of the operand is formed)
    ACodes codes[kMaxStages];
#pragma unroll
    for (int i = 0; i < kMaxStages; ++i) {
        xv[i] = add(xv[i], dv[i]);
        const float4 a = xv[i], w = wn[i];
        const float e[4] = {__fmul_rn(a.x, weight ? __fmul_rn(scale, w.x) : scale), __fmul_rn(a.y, weight ? __fmul_rn(scale, w.y) : scale),
                            __fmul_rn(a.z, weight ? __fmul_rn(scale, w.z) : scale), __fmul_rn(a.w, weight ? __fmul_rn(scale, w.w) : scale)};
        a_codes_from_lane_codes(codes[i], quantize_block_q8k(e, lane), lane);
    }
    float acc[1][2] = {{0.0f, 0.0f}};
#pragma unroll
    for (int i = 0; i < kMaxStages; ++i) {
        if (i < cnt) {
            ARegs<1> ar;
            a_from_codes(ar, codes[i], lane);
            int32_t dsum[1][2], msum[1][2];
            compute_tile<1, false, 1>(t[i], ar, acc, dsum, msum);
        }
    }
    if (n_waves > 1) {
        if (wave > 0) red[(wave - 1) * 64 + lane] = acc[0][0];
        __syncthreads();
    }
    if (wave == 0) {
        float v = acc[0][0];
        if (n_waves > 1) v = add_wave_partials(v, n_waves, [&](int wv) { return red[(wv - 1) * 64 + lane]; });
        const int64_t row = rt * 16 + slot;
        if (kq == 0 && row < rows) y[row] = v;
    }
    if (rt == 0 && sum_out) {  // last: a store ahead of a barrier would make the barrier wait for it
#pragma unroll
        for (int i = 0; i < kMaxStages; ++i)
            if (i < cnt) *reinterpret_cast<float4*>(sum_out + (int64_t)(wave + i * n_waves) * kQK + lane * 4) = xv[i];
    }
}

// Up to eight rows, the same two ideas: every wavefront quantizes the super-blocks it multiplies -- one block per
// row, parked as compact codes in a corner of LDS that only this wavefront uses (block of row t at t * 256, its
// 64-byte chunks permuted by t & 3 so that the rows an MFMA reads side by side fall on different banks) and read
// back as the split-slot A operand (common.h) -- and with kNorm the residual add and the RMSNorm of the rows run
// inside as in gemv1_norm_fused_kernel.  Wave split of K, accumulation order and epilogue are matmul_kernel<1,1>'s:
// the bits of quantize (or mq_add_rmsnorm_q8k) + matmul.
// RMAX (2, 4 or 8 >= n) bounds the registers of the stage operands, which are requested before the tiles.
template <bool kNorm, int RMAX>
__global__ void __launch_bounds__(512) gemvn_fused_kernel(const uint8_t* __restrict__ w, int64_t rows, int64_t nb,
                                                          const float* __restrict__ x, int64_t ldx, const float* __restrict__ delta,
                                                          const float* __restrict__ weight, float eps, float* __restrict__ sum_out,
                                                          float* __restrict__ y, int64_t ldy, int n) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];  // [W][8 * 256 + 32] codes and scales, then red [W-1][2][64]
    __shared__ float wave_sum[8][4];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n_waves = blockDim.x >> 6;
    const int slot = lane & 15, kq = lane >> 4;
    const int64_t rt = blockIdx.x;
    const uint8_t* tiles = w + tile_offset(rt, 0, nb);
    const int cnt = (wave < nb ? 1 : 0) + (wave + n_waves < nb ? 1 : 0);  // super-blocks wave, wave + W (at most kMaxStages, host-checked; no division)
    uint8_t* codes = lds_raw + (size_t)wave * (8 * 256 + 32);
    float* scales = reinterpret_cast<float*>(codes + 8 * 256);
    float* red = reinterpret_cast<float*>(lds_raw + (size_t)n_waves * (8 * 256 + 32));
    const int64_t cols = nb * kQK;
    // Requests are unconditional (a row past n re-reads the last row, a stage past the end block 0, a missing
    // residual or weight x) and those of the stages go out before the tiles: requests are answered in order.
    const float* dp = kNorm && delta ? delta : x;
    const int64_t ldd = kNorm && delta ? cols : ldx;
    const float* wp = kNorm && weight ? weight : x;
    auto add = [&](float4 a, const float4& d) {
        if (kNorm && delta) a.x = __fadd_rn(a.x, d.x), a.y = __fadd_rn(a.y, d.y), a.z = __fadd_rn(a.z, d.z), a.w = __fadd_rn(a.w, d.w);
        return a;
    };
    float4 xv[kMaxStages][RMAX], dv[kMaxStages][kNorm ? RMAX : 1], wn[kMaxStages];
#pragma unroll
    for (int i = 0; i < kMaxStages; ++i) {
        const int64_t c0 = (int64_t)(i < cnt ? wave + i * n_waves : 0) * kQK + lane * 4;
#pragma unroll
        for (int r = 0; r < RMAX; ++r) {
            const int rr = r < n ? r : n - 1;
            xv[i][r] = *reinterpret_cast<const float4*>(x + (size_t)rr * ldx + c0);
            if (kNorm) dv[i][r] = *reinterpret_cast<const float4*>(dp + (size_t)rr * ldd + c0);
        }
        if (kNorm) wn[i] = *reinterpret_cast<const float4*>(wp + c0);
    }
    TileRegs t[kMaxStages];
#pragma unroll
    for (int i = 0; i < kMaxStages; ++i) load_tile(t[i], tiles + (size_t)(i < cnt ? wave + i * n_waves : 0) * kTileBytes, lane);

    float scale[RMAX];
#pragma unroll
    for (int r = 0; r < RMAX; ++r) scale[r] = 1.0f;
    if (kNorm) {
        // sums of squares in the order of the 256-thread norm kernel: virtual wavefront v = 0..3, row by row
        for (int v = wave; v < 4; v += n_waves) {
            for (int r = 0; r < n; ++r) {
                float ssq = 0.0f;
                for (int64_t b = v; b < nb; b += 4) {
                    const int64_t c0 = b * kQK + lane * 4;
                    const float4 a = add(*reinterpret_cast<const float4*>(x + (size_t)r * ldx + c0), *reinterpret_cast<const float4*>(dp + (size_t)r * ldd + c0));
                    ssq = __fmaf_rn(a.x, a.x, ssq);
                    ssq = __fmaf_rn(a.y, a.y, ssq);
                    ssq = __fmaf_rn(a.z, a.z, ssq);
                    ssq = __fmaf_rn(a.w, a.w, ssq);
                }
#pragma unroll
                for (int off = 32; off > 0; off >>= 1) ssq += __shfl_xor(ssq, off, 64);
                if (lane == 0) wave_sum[r][v] = ssq;
            }
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < RMAX; ++r) {
            if (r < n) {
                const float total = (wave_sum[r][0] + wave_sum[r][1]) + (wave_sum[r][2] + wave_sum[r][3]);
                scale[r] = __fdiv_rn(1.0f, __fsqrt_rn(__fadd_rn(__fdiv_rn(total, (float)cols), eps)));
            }
        }
    }

    // this lane's part of the A operand: row (slot / 2, the last live one for a dead slot), half slot % 2
    const int arow = (slot >> 1) < n ? (slot >> 1) : n - 1;
    const int a_off = arow * 256 + 32 * (slot & 1) + 8 * kq, a_swz = arow & 3;
    const uint32_t keep_lo = (slot & 1) ? 0u : 0xffffffffu, keep_hi = ~keep_lo;
    const int d0 = 2 * kq < n ? 2 * kq : n - 1, d1 = 2 * kq + 1 < n ? 2 * kq + 1 : n - 1;

    float acc[1][2] = {{0.0f, 0.0f}};
#pragma unroll
    for (int i = 0; i < kMaxStages; ++i) {
        if (i < cnt) {
            const float4 wv = wn[i];
#pragma unroll
            for (int r = 0; r < RMAX; ++r) {
                if (r < n) {  // wave-uniform
                    const float4 a = kNorm ? add(xv[i][r], dv[i][r]) : xv[i][r];
                    xv[i][r] = a;
                    float e[4] = {a.x, a.y, a.z, a.w};
                    if (kNorm) {
                        e[0] = __fmul_rn(a.x, weight ? __fmul_rn(scale[r], wv.x) : scale[r]);
                        e[1] = __fmul_rn(a.y, weight ? __fmul_rn(scale[r], wv.y) : scale[r]);
                        e[2] = __fmul_rn(a.z, weight ? __fmul_rn(scale[r], wv.z) : scale[r]);
                        e[3] = __fmul_rn(a.w, weight ? __fmul_rn(scale[r], wv.w) : scale[r]);
                    }
                    const Q8Lane q = quantize_block_q8k(e, lane);
                    *reinterpret_cast<uint32_t*>(codes + r * 256 + ((((lane >> 4) ^ (r & 3)) << 6) | ((lane & 15) << 2))) = q.packed;
                    if (lane == 0) scales[r] = q.d;
                }
            }
            __builtin_amdgcn_wave_barrier();  // the codes above are read by other lanes of this wavefront below
            ARegs<1> ar;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const v2u v = *reinterpret_cast<const v2u*>(codes + a_off + ((c ^ a_swz) << 6));
                ar.q[0][c] = v4u{v.x & keep_lo, v.y & keep_lo, v.x & keep_hi, v.y & keep_hi};
            }
            ar.yd[0][0] = scales[d0];
            ar.yd[0][1] = scales[d1];
            __builtin_amdgcn_wave_barrier();  // the next stage overwrites the codes
            int32_t dsum[1][2], msum[1][2];
            compute_tile<1>(t[i], ar, acc, dsum, msum);
        }
    }
    if (n_waves > 1) {
        if (wave > 0) {
            red[((wave - 1) * 2 + 0) * 64 + lane] = acc[0][0];
            red[((wave - 1) * 2 + 1) * 64 + lane] = acc[0][1];
        }
        __syncthreads();
    }
    if (wave == 0) {
        if (n_waves > 1) {
#pragma unroll
            for (int j = 0; j < 2; ++j)
                acc[0][j] = add_wave_partials(acc[0][j], n_waves, [&](int wv) { return red[((wv - 1) * 2 + j) * 64 + lane]; });
        }
        const int64_t row = rt * 16 + slot;
        if (row < rows) {
#pragma unroll
            for (int j = 0; j < 2; ++j)
                if (2 * kq + j < n) y[(size_t)(2 * kq + j) * ldy + row] = acc[0][j];
        }
    }
    if (kNorm && rt == 0 && sum_out) {  // last: a store ahead of a barrier would make the barrier wait for it
#pragma unroll
        for (int i = 0; i < kMaxStages; ++i) {
            if (i < cnt) {
                const int64_t c0 = (int64_t)(wave + i * n_waves) * kQK + lane * 4;
#pragma unroll
                for (int r = 0; r < RMAX; ++r)
                    if (r < n) *reinterpret_cast<float4*>(sum_out + (size_t)r * cols + c0) = xv[i][r];
            }
        }
    }
}

}  // namespace

hipError_t launch_gemvn_fused(const uint8_t* w, int64_t rows, int64_t nb, const float* x, int64_t ldx, const float* delta,
                              const float* weight, float eps, float* sum_out, float* y, int64_t ldy, int n, bool norm, int waves,
                              hipStream_t stream) {
    if (!gemv1_fused_applies(nb, waves) || rows <= 0 || n < 1 || n > 8) return hipErrorInvalidValue;
    const int64_t rowtiles = (rows + 15) / 16;
    const size_t lds = (size_t)waves * (8 * 256 + 32) + (waves > 1 ? (size_t)(waves - 1) * 2 * 64 * sizeof(float) : 0);
#define MQ_GEMVN(NORM, RMAX)                                                                                                 \
    MQ_LAUNCH((gemvn_fused_kernel<NORM, RMAX>), dim3((unsigned)rowtiles), dim3(64 * waves), lds, stream, w, rows, nb, x, ldx, \
                       delta, weight, eps, sum_out, y, ldy, n)
    if (norm) {
        if (n <= 2) MQ_GEMVN(true, 2);
        else if (n <= 4) MQ_GEMVN(true, 4);
        else MQ_GEMVN(true, 8);
    } else {
        if (n <= 2) MQ_GEMVN(false, 2);
        else if (n <= 4) MQ_GEMVN(false, 4);
        else MQ_GEMVN(false, 8);
    }
#undef MQ_GEMVN
    return hipGetLastError();
}

hipError_t launch_gemv1_norm_fused(const uint8_t* w, int64_t rows, int64_t nb, const float* x, const float* delta,
                                   const float* weight, float eps, float* sum_out, float* y, int waves, hipStream_t stream) {
    if (!gemv1_fused_applies(nb, waves) || rows <= 0) return hipErrorInvalidValue;
    const int64_t rowtiles = (rows + 15) / 16;
    MQ_LAUNCH(gemv1_norm_fused_kernel, dim3((unsigned)rowtiles), dim3(64 * waves),
                       waves > 1 ? (size_t)(waves - 1) * 64 * sizeof(float) : 0, stream, w, rows, nb, x, delta, weight, eps, sum_out,
                       y);
    return hipGetLastError();
}

bool gemv1_fused_applies(int64_t nb, int waves) { return waves >= 1 && (nb + waves - 1) / waves <= kMaxStages; }

hipError_t launch_gemv1_fused(const uint8_t* w, int64_t rows, int64_t nb, const float* x, float* y, int waves,
                              hipStream_t stream) {
    if (!gemv1_fused_applies(nb, waves) || rows <= 0) return hipErrorInvalidValue;
    const int64_t rowtiles = (rows + 15) / 16;
    MQ_LAUNCH(gemv1_fused_kernel, dim3((unsigned)rowtiles), dim3(64 * waves),
                       waves > 1 ? (size_t)(waves - 1) * 64 * sizeof(float) : 0, stream, w, rows, nb, x, y);
    return hipGetLastError();
}

hipError_t launch_gemv1_multi(const Gemv1MultiArgs& a, int waves, hipStream_t stream) {
    if (a.count < 1 || a.count > kGemvMultiMax || !gemv1_fused_applies(a.nb, waves) || !a.x) return hipErrorInvalidValue;
    int64_t all_tiles = 0;
    for (int i = 0; i < a.count; ++i) {
        if (!a.w[i] || !a.y[i] || a.rows[i] <= 0) return hipErrorInvalidValue;
        all_tiles += (a.rows[i] + 15) / 16;
    }
    // row tiles per workgroup: as many as leave every compute unit a workgroup (at most four)
    const int64_t per_cu = all_tiles / compute_units();
    const int rt = per_cu >= 4 ? 4 : per_cu >= 2 ? 2 : 1;
    Gemv1MultiArgs b = a;
    int total = 0;
    for (int i = 0; i < a.count; ++i) {
        b.rt_begin[i] = total;
        total += (int)(((a.rows[i] + 15) / 16 + rt - 1) / rt);
    }
    for (int i = a.count; i <= kGemvMultiMax; ++i) b.rt_begin[i] = total;
    const size_t lds = waves > 1 ? (size_t)rt * (waves - 1) * 64 * sizeof(float) : 0;
    if (rt == 4) MQ_LAUNCH(gemv1_multi_kernel<4>, dim3((unsigned)total), dim3(64 * waves), lds, stream, b);
    else if (rt == 2) MQ_LAUNCH(gemv1_multi_kernel<2>, dim3((unsigned)total), dim3(64 * waves), lds, stream, b);
    else MQ_LAUNCH(gemv1_multi_kernel<1>, dim3((unsigned)total), dim3(64 * waves), lds, stream, b);
    return hipGetLastError();
}

}  // namespace mq
