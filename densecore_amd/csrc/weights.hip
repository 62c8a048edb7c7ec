// Weight re-tiling (ggml block_q4_K / block_q5_K / block_q6_K / Q8_0 rows <-> the 16-row tile layouts of common.h)
// and the on-device synthetic fill.  One thread moves one 8-byte word of a block; each such word lands in one
// contiguous 8-byte slot of a tile (tile_word_offset, tile_word_offset_q5, tile_word_offset_q6,
// tile_word_offset_q80).  The last "word" of a block_q6_K is its two-byte d, and so are the last eight "words" of
// a row's eight Q8_0 blocks.
#include "common.h"
#include "kernels.h"

namespace mq {

namespace {

// 8-byte words per block: 18 (Q4_K), 22 (Q5_K), 26 + the two-byte d (Q6_K), 32 + eight two-byte d (eight Q8_0 blocks)
__host__ __device__ inline int words_per_block(int type) {
    return type == kTypeQ80 ? 40 : type == kTypeQ6K ? 27 : block_bytes_of(type) / 8;
}
// a word that is a lone fp16 scale (two bytes)
__host__ __device__ inline bool scale_word(int type, int word) {
    return (type == kTypeQ6K && word == 26) || (type == kTypeQ80 && word >= 32);
}
// where a word starts inside its block in a ggml row
__host__ __device__ inline int row_word_offset(int type, int word) { return type == kTypeQ80 ? row_word_offset_q80(word) : word * 8; }
// Q6_K: the qh words are stored with bit 5 of every code flipped (common.h)
__host__ __device__ inline uint64_t stored_form(uint64_t v, int type, int word) {
    return (type == kTypeQ6K && word >= 16 && word < 24) ? v ^ 0xAAAAAAAAAAAAAAAAull : v;
}

__device__ __forceinline__ bool decode_word(int64_t idx, int64_t rows, int64_t nb, int type, int64_t& row, int64_t& b,
                                            int& word) {
    const int wpb = words_per_block(type);
    const int64_t per_row = nb * wpb;
    row = idx / per_row;
    if (row >= rows) return false;
    const int64_t rem = idx - row * per_row;
    b = rem / wpb;
    word = (int)(rem - b * wpb);
    return true;
}

// where word `word` of row r's block lives inside its tile
__device__ __forceinline__ size_t word_in_tiles(int64_t row, int64_t b, int64_t nb, int word, int type) {
    const int r = (int)(row & 15);
    return tile_offset(row >> 4, b, nb, tile_bytes_of(type)) +
           (size_t)(type == kTypeQ80   ? tile_word_offset_q80(r, word)
                    : type == kTypeQ6K ? tile_word_offset_q6(r, word)
                    : type == kTypeQ5K ? tile_word_offset_q5(r, word)
                                       : tile_word_offset(r, word));
}

__global__ void __launch_bounds__(256) tile_weights_kernel(const uint8_t* __restrict__ raw, int64_t rows, int64_t nb,
                                                           int type, size_t row_bytes, size_t expert_bytes,
                                                           uint8_t* __restrict__ tiled, size_t tiled_expert_bytes) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    int64_t row, b;
    int word;
    if (!decode_word(idx, rows, nb, type, row, b, word)) return;
    const int64_t e = blockIdx.y;
    const uint8_t* src = raw + (size_t)e * expert_bytes + (size_t)row * row_bytes + (size_t)b * block_bytes_of(type) + row_word_offset(type, word);
    uint8_t* dst = tiled + (size_t)e * tiled_expert_bytes + word_in_tiles(row, b, nb, word, type);
    // the blocks are only 2-byte aligned in general: go through 2-byte loads to stay correct for odd host strides
    const uint16_t* s16 = reinterpret_cast<const uint16_t*>(src);
    if (scale_word(type, word)) {  // fp16 d (Q6_K: padded to four bytes)
        if (type == kTypeQ6K) *reinterpret_cast<uint32_t*>(dst) = (uint32_t)s16[0];
        else *reinterpret_cast<uint16_t*>(dst) = s16[0];
        return;
    }
    const uint64_t v = (uint64_t)s16[0] | ((uint64_t)s16[1] << 16) | ((uint64_t)s16[2] << 32) | ((uint64_t)s16[3] << 48);
    *reinterpret_cast<uint64_t*>(dst) = stored_form(v, type, word);
}

__global__ void __launch_bounds__(256) untile_weights_kernel(const uint8_t* __restrict__ tiled, int64_t rows,
                                                             int64_t nb, int type, size_t row_bytes,
                                                             size_t expert_bytes, uint8_t* __restrict__ raw,
                                                             size_t tiled_expert_bytes) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    int64_t row, b;
    int word;
    if (!decode_word(idx, rows, nb, type, row, b, word)) return;
    const int64_t e = blockIdx.y;
    const uint8_t* src = tiled + (size_t)e * tiled_expert_bytes + word_in_tiles(row, b, nb, word, type);
    uint8_t* dst = raw + (size_t)e * expert_bytes + (size_t)row * row_bytes + (size_t)b * block_bytes_of(type) + row_word_offset(type, word);
    uint16_t* d16 = reinterpret_cast<uint16_t*>(dst);
    if (scale_word(type, word)) {
        d16[0] = *reinterpret_cast<const uint16_t*>(src);
        return;
    }
    const uint64_t v = stored_form(*reinterpret_cast<const uint64_t*>(src), type, word);
    d16[0] = (uint16_t)v;
    d16[1] = (uint16_t)(v >> 16);
    d16[2] = (uint16_t)(v >> 32);
    d16[3] = (uint16_t)(v >> 48);
}

// fp16(0.001 + 0.009*u), u = top 24 bits of the word / 2^24, each step rounded in fp32.
__device__ __forceinline__ uint32_t unit_scale_f16(uint64_t w) {
    const float u = __fmul_rn((float)(uint32_t)(w >> 40), 5.9604644775390625e-08f);
    const float v = __fadd_rn(0.001f, __fmul_rn(0.009f, u));
    return (uint32_t)__half_as_ushort(__float2half_rn(v));
}

__global__ void __launch_bounds__(256) synth_weights_kernel(uint64_t seed, int64_t rows, int64_t nb, int type,
                                                            uint8_t* __restrict__ tiled, size_t tiled_expert_bytes) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    int64_t row, b;
    int word;
    if (!decode_word(idx, rows, nb, type, row, b, word)) return;
    const int64_t e = blockIdx.y;
    // stream position of this word in the flat [expert][row][block][words per block] order
    const uint64_t flat_block = ((uint64_t)e * (uint64_t)rows + (uint64_t)row) * (uint64_t)nb + (uint64_t)b;
    const uint64_t pos = flat_block * (uint64_t)words_per_block(type) + (uint64_t)word;
    uint64_t v = mix64(seed + (pos + 1) * kGamma);
    uint8_t* dst = tiled + (size_t)e * tiled_expert_bytes + word_in_tiles(row, b, nb, word, type);
    if (type == kTypeQ80) {  // codes in [-127, 127] (ggml never writes -128), one d per 32 weights
        if (word >= 32) {
            *reinterpret_cast<uint16_t*>(dst) =
                (uint16_t)unit_scale_f16(mix64((seed ^ kScaleStream) + (flat_block * 8 + (uint64_t)(word - 32) + 1) * kGamma));
            return;
        }
        uint64_t fixed = 0;
        for (int i = 0; i < 8; ++i) {
            const uint64_t byte = (v >> (8 * i)) & 0xffu;
            fixed |= (byte == 0x80u ? 0x81ull : byte) << (8 * i);
        }
        v = fixed;
    } else if (type == kTypeQ6K) {  // d is the block's last field
        if (word == 26) {
            *reinterpret_cast<uint32_t*>(dst) = unit_scale_f16(mix64((seed ^ kScaleStream) + (flat_block * 2 + 1) * kGamma));
            return;
        }
    } else if (word == 0) {
        const uint64_t s0 = mix64((seed ^ kScaleStream) + (flat_block * 2 + 1) * kGamma);
        const uint64_t s1 = mix64((seed ^ kScaleStream) + (flat_block * 2 + 2) * kGamma);
        v = (v & 0xffffffff00000000ull) | (uint64_t)unit_scale_f16(s0) | ((uint64_t)unit_scale_f16(s1) << 16);
    }
    *reinterpret_cast<uint64_t*>(dst) = stored_form(v, type, word);
}

inline dim3 word_grid(int64_t rows, int64_t nb, int64_t n_experts, int type) {
    const int64_t words = rows * nb * words_per_block(type);
    return dim3((unsigned)((words + 255) / 256), (unsigned)n_experts);
}

}  // namespace

hipError_t launch_tile_weights(const uint8_t* raw, int64_t rows, int64_t nb, int type, size_t row_bytes,
                               size_t expert_bytes, int64_t n_experts, uint8_t* tiled, size_t tiled_expert_bytes,
                               hipStream_t stream) {
    hipLaunchKernelGGL(tile_weights_kernel, word_grid(rows, nb, n_experts, type), dim3(256), 0, stream, raw, rows, nb,
                       type, row_bytes, expert_bytes, tiled, tiled_expert_bytes);
    return hipGetLastError();
}

hipError_t launch_untile_weights(const uint8_t* tiled, int64_t rows, int64_t nb, int type, size_t row_bytes,
                                 size_t expert_bytes, int64_t n_experts, uint8_t* raw, size_t tiled_expert_bytes,
                                 hipStream_t stream) {
    hipLaunchKernelGGL(untile_weights_kernel, word_grid(rows, nb, n_experts, type), dim3(256), 0, stream, tiled, rows, nb,
                       type, row_bytes, expert_bytes, raw, tiled_expert_bytes);
    return hipGetLastError();
}

hipError_t launch_synth_weights(uint64_t seed, int64_t rows, int64_t nb, int type, int64_t n_experts, uint8_t* tiled,
                                size_t tiled_expert_bytes, hipStream_t stream) {
    hipLaunchKernelGGL(synth_weights_kernel, word_grid(rows, nb, n_experts, type), dim3(256), 0, stream, seed, rows, nb,
                       type, tiled, tiled_expert_bytes);
    return hipGetLastError();
}

}  // namespace mq
