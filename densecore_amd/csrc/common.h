// Shared constants, layouts and small device helpers for the gfx950 Q4_K x Q8_K kernels.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mq {

constexpr int kQK = 256;             // weights per super-block
constexpr int kQ4Block = 144;        // bytes of block_q4_K
constexpr int kQ8Block = 292;        // bytes of block_q8_K
constexpr int kTileRows = 16;        // weight rows per tile (the N side of a 16x16 MFMA)
constexpr int kTileBytes = kTileRows * kQ4Block;  // 2304
constexpr int kTileQBytes = kTileRows * 128;      // 2048: nibble part

// ---------------------------------------------------------------------------------------------
// Weight layout in HBM ("row-tile major"): a matrix of `rows` x `cols` is cut into tiles of 16
// rows x one super-block.  Tile (rt, b) sits at ((rt * nb + b) * 2304) bytes; a wave reads it
// with three fully coalesced 16-byte-per-lane loads and gets its MFMA B operand without any
// shuffle:
//   bytes [i*1024 + lane*16, +16), i = 0,1   lane = kq*16 + r  (r = row in tile, kq = 0..3)
//        [0..7]  = qs[r][32*(2i)   + 8*kq .. +7]   -> low nibbles: sub-block 4i,   elements 8kq..8kq+7
//                                                     high nibbles: sub-block 4i+1
//        [8..15] = qs[r][32*(2i+1) + 8*kq .. +7]   -> sub-blocks 4i+2 (low) and 4i+3 (high)
//   bytes [2048 + r*16, +16)                 = {fp16 d, fp16 dmin, scales[12]} of row r
// Same 144 bytes per 256 weights as ggml's block_q4_K; only the order differs.
// ---------------------------------------------------------------------------------------------
__host__ __device__ inline size_t tile_offset(int64_t rt, int64_t b, int64_t nb, int tile_bytes = kTileBytes) {
    return (size_t)(rt * nb + b) * (size_t)tile_bytes;
}

// Offset inside a tile of the 8-byte word `word` (0..17) of row r's block_q4_K.
__host__ __device__ inline int tile_word_offset(int r, int word) {
    if (word < 2) return kTileQBytes + r * 16 + word * 8;
    const int j = word - 2;        // qs[8j .. 8j+7]
    const int chunk = j >> 2;      // 32-byte chunk of qs
    const int kq = j & 3;
    return (chunk >> 1) * 1024 + (kq * 16 + r) * 16 + (chunk & 1) * 8;
}

// ---------------------------------------------------------------------------------------------
// Q5_K (block_q5_K, 176 bytes: Q4_K plus qh[32], one high bit per weight -- bit s of qh[l] belongs to
// element l of sub-block s; core/src/kernels/hwy/hwy_moe_quant.cc:36-45,177-200).  Same tile as Q4_K with
// the high bits appended: 2816 bytes per 16 rows x one super-block,
//   bytes [0, 2304)                          as above (nibbles, then headers)
//   bytes [2304 + (kq*16 + r)*8, +8)         = qh[r][8*kq .. 8*kq+7]: all eight sub-block bits of the eight
//                                              elements whose nibbles lane (kq, r) holds
// Word w of a block_q5_K (8 bytes each, 22 of them): 0..1 header, 2..5 qh, 6..21 qs.
// ---------------------------------------------------------------------------------------------
constexpr int kQ5Block = 176;
constexpr int kTile5Bytes = kTileRows * kQ5Block;  // 2816
constexpr int kTileHBytes = kTileBytes;            // offset of the qh part
constexpr int kTypeQ4K = 12, kTypeQ5K = 13, kTypeQ6K = 14;  // ggml_type values

// ---------------------------------------------------------------------------------------------
// Q6_K (block_q6_K, 210 bytes: ql[128] low nibbles, qh[64] top two bits, scales[16] signed bytes -- one per
// 16 weights --, fp16 d; core/src/llm/matmul/q6_small_batch.h:13-24,56-76).  Element 128 j + 32 z + l has
// nibble ql[64 j + 32 (z & 1) + l] (low for z < 2, high otherwise) and top bits (qh[32 j + l] >> 2 z) & 3; the
// weight is d * scale * (code - 32).  Tile of 16 rows x one super-block, 3392 bytes:
//   bytes [j*1024 + (kq*16 + r)*16, +16), j = 0,1 = ql[64 j + 8 kq .. +7], ql[64 j + 32 + 8 kq .. +7] of row r:
//        low nibbles are the 64-weight chunk 2 j of the MFMA loop, high nibbles chunk 2 j + 1
//   bytes [2048 + (kq*16 + r)*16, +16)            = qh[8 kq .. +7], qh[32 + 8 kq .. +7], every byte XOR 0xAA:
//        with bit 5 of each code flipped the six bits are the two's complement of (code - 32), so that
//        (bits << 2) read as a signed byte is 4 * (code - 32) -- the B operand needs no subtraction
//   bytes [3072 + r*16, +16)                      = scales[16] of row r
//   bytes [3328 + r*4, +4)                        = fp16 d of row r, two zero bytes
// Words of a block_q6_K as the re-tiling kernels move them: 0..15 ql, 16..23 qh, 24..25 scales (8 bytes each),
// 26 = d (2 bytes).
// ---------------------------------------------------------------------------------------------
constexpr int kQ6Block = 210;
constexpr int kTile6HOff = 2048, kTile6SOff = 3072, kTile6DOff = 3328;
constexpr int kTile6Bytes = 3392;
__host__ __device__ inline int tile_word_offset_q6(int r, int word) {
    if (word < 16) {
        const int x = word * 8, j = x >> 6, within = x & 63;
        return j * 1024 + (((within & 31) >> 3) * 16 + r) * 16 + (within >> 5) * 8;
    }
    if (word < 24) {
        const int x = (word - 16) * 8, j = x >> 5;
        return kTile6HOff + (((x & 31) >> 3) * 16 + r) * 16 + j * 8;
    }
    if (word < 26) return kTile6SOff + r * 16 + (word - 24) * 8;
    return kTile6DOff + r * 4;
}
// ---------------------------------------------------------------------------------------------
// Q8_0 (fp16 d, int8 qs[32]; 34 bytes per 32 weights, core/src/llm/matmul/q8_small_batch.h:9-14).  Eight
// consecutive blocks of a row -- 256 weights, 272 bytes -- take the place of a super-block.  Tile of 16 rows x 256
// weights, 4352 bytes:
//   bytes [c*1024 + (kq*16 + r)*16, +16), c = 0..3 = qs[8 kq .. +7] of block 2c, then of block 2c + 1, of row r:
//        the B operand of the MFMA over the 64-weight chunk c, the same element order as the Q4_K tile
//   bytes [4096 + r*16, +16)                       = the eight fp16 d of row r
// Words as the re-tiling kernels move them: 0..31 = eight code bytes each (word 4k + j = qs[8j .. 8j+7] of block
// k), 32..39 = the two-byte d of block k = word - 32.
// ---------------------------------------------------------------------------------------------
constexpr int kTypeQ80 = 8;  // ggml_type value
constexpr int kQ80Block = 34, kQ80Super = 8 * kQ80Block;
constexpr int kTile80SOff = 4096, kTile80Bytes = 4352;
__host__ __device__ inline int tile_word_offset_q80(int r, int word) {
    if (word >= 32) return kTile80SOff + r * 16 + (word - 32) * 2;
    const int k = word >> 2, j = word & 3;
    return (k >> 1) * 1024 + (j * 16 + r) * 16 + (k & 1) * 8;
}
// byte offset of a word inside the 272 bytes of its eight blocks in a ggml row
__host__ __device__ inline int row_word_offset_q80(int word) {
    return word >= 32 ? (word - 32) * kQ80Block : (word >> 2) * kQ80Block + 2 + (word & 3) * 8;
}
__host__ __device__ inline int tile_bytes_of(int type) {
    return type == kTypeQ80 ? kTile80Bytes : type == kTypeQ6K ? kTile6Bytes : type == kTypeQ5K ? kTile5Bytes : kTileBytes;
}
// bytes of one row's 256 weights in ggml's layout
__host__ __device__ inline int block_bytes_of(int type) {
    return type == kTypeQ80 ? kQ80Super : type == kTypeQ6K ? kQ6Block : type == kTypeQ5K ? kQ5Block : kQ4Block;
}
__host__ __device__ inline int tile_word_offset_q5(int r, int word) {
    if (word < 2) return kTileQBytes + r * 16 + word * 8;
    if (word < 6) return kTileHBytes + ((word - 2) * 16 + r) * 8;
    return tile_word_offset(r, word - 4);  // qs words 6..21 map like Q4_K's 2..17
}

// ---------------------------------------------------------------------------------------------
// Activation layout consumed by the matmul kernels ("A-major Q8_K"): the same int8 codes and fp32
// scales as block_q8_K, ordered so that a wave reads the A operand of v_mfma_i32_16x16x64_i8 with
// coalesced 16-byte loads.  One MFMA covers a 64-weight chunk, i.e. two 32-wide sub-blocks with
// different scales; to keep their partial sums apart every activation row owns TWO of the 16
// M-side slots: slot 2t holds the codes of the even sub-block in bytes 0..7 and zeros in bytes
// 8..15, slot 2t+1 the reverse.  The products against the zero halves vanish, so output slot 2t is
// the dot over sub-block 2c alone and slot 2t+1 the dot over sub-block 2c+1.  A tile is therefore
// 8 activation rows.  Row m lives in tile m/8, position t = m%8:
//   codes : [m/8][b][c 0..3][kq 0..3][slot 0..15][16 B]      (4096 B per tile and super-block)
//           slot 2t   = {qs[64c + 8kq .. +7], 0 x 8}
//           slot 2t+1 = {0 x 8, qs[64c + 32 + 8kq .. +7]}
//   scale : [m/8][b][t] fp32
// ---------------------------------------------------------------------------------------------
constexpr int kTokTile = 8;  // activation rows per MFMA (two M-side slots each)
__host__ __device__ inline size_t aq_row_offset(int64_t m, int64_t nb) {  // row part of the address
    return (size_t)(m >> 3) * (size_t)nb * 4096 + (size_t)(m & 7) * 32;
}
__host__ __device__ inline size_t aq_offset(int64_t m, int64_t b, int c, int kq, int h, int64_t nb) {
    return aq_row_offset(m, nb) + (size_t)b * 4096 + (size_t)(c * 4 + kq) * 256 + (size_t)h * 16;
}
__host__ __device__ inline size_t ad_index(int64_t m, int64_t b, int64_t nb) {
    return ((size_t)(m >> 3) * nb + b) * 8 + (size_t)(m & 7);
}
__host__ __device__ inline size_t aq_bytes(int64_t n_rows, int64_t nb) {
    return (size_t)((n_rows + 7) >> 3) * nb * 4096;
}
__host__ __device__ inline size_t ad_count(int64_t n_rows, int64_t nb) {
    return (size_t)((n_rows + 7) >> 3) * nb * 8;
}

// SplitMix64 finaliser: the synthetic-weight recipe shared with densecore_amd/synth.py.
__host__ __device__ inline uint64_t mix64(uint64_t z) {
    z ^= z >> 30;
    z *= 0xBF58476D1CE4E5B9ull;
    z ^= z >> 27;
    z *= 0x94D049BB133111EBull;
    z ^= z >> 31;
    return z;
}
constexpr uint64_t kGamma = 0x9E3779B97F4A7C15ull;
constexpr uint64_t kScaleStream = 0x5CA1E5CA1E5CA1E5ull;

#if defined(__HIPCC__)
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float half_bits_to_float(uint32_t h16) {
    return __half2float(__ushort_as_half((unsigned short)h16));
}

// Streaming 16-byte load for weights that are read exactly once.
__device__ __forceinline__ v4u load_stream16(const void* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const v4u*>(p));
}
__device__ __forceinline__ v4u load16(const void* p) { return *reinterpret_cast<const v4u*>(p); }

// Value of lane (i ^ 1), (i ^ 2), the mirrored lane of each 8, of each 16: data-parallel-primitive moves,
// an order of magnitude cheaper than a cross-lane read through LDS.
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t x) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, CTRL, 0xf, 0xf, true);
}
constexpr int kDppXor1 = 0xB1, kDppXor2 = 0x4E, kDppHalfMirror = 0x141, kDppMirror = 0x140;

// Maximum of an unsigned value over the 64 lanes, returned in every lane (wave-uniform).
// acc + the partial sums of the wavefronts 1 .. n_waves-1 (n_waves <= 8) in wave order, part(wv) reading wavefront wv's
// value from LDS: all seven reads are requested first (a wavefront past the end re-reads wavefront 1: its value is
// read and dropped) -- inside a loop over a run-time wave count every read is a round trip to LDS of its own.
template <class Part>
__device__ __forceinline__ float add_wave_partials(float acc, int n_waves, Part part) {
    float v[7];
#pragma unroll
    for (int wv = 1; wv < 8; ++wv) v[wv - 1] = part(wv < n_waves ? wv : 1);
#pragma unroll
    for (int wv = 1; wv < 8; ++wv)
        if (wv < n_waves) acc = __fadd_rn(acc, v[wv - 1]);
    return acc;
}

// unit = row * nb + block, split again.  The launchers keep the unit count below 2^31, so the division is a
// 32-bit one: a 64-bit division is some 150 dependent scalar instructions at the head of a kernel that otherwise
// runs for a few microseconds.
__device__ __forceinline__ void split_unit(int64_t unit, int64_t nb, int64_t& row, int64_t& block) {
    const uint32_t q = (uint32_t)unit / (uint32_t)nb;
    row = (int64_t)q;
    block = (int64_t)((uint32_t)unit - q * (uint32_t)nb);
}

__device__ __forceinline__ uint32_t wave_max_u32(uint32_t x) {
    uint32_t t;
    t = dpp_u32<kDppXor1>(x);
    x = t > x ? t : x;
    t = dpp_u32<kDppXor2>(x);
    x = t > x ? t : x;
    t = dpp_u32<kDppHalfMirror>(x);
    x = t > x ? t : x;
    t = dpp_u32<kDppMirror>(x);
    x = t > x ? t : x;
    const uint32_t a = __builtin_amdgcn_readlane(x, 0), b = __builtin_amdgcn_readlane(x, 16);
    const uint32_t c = __builtin_amdgcn_readlane(x, 32), d = __builtin_amdgcn_readlane(x, 48);
    const uint32_t ab = a > b ? a : b, cd = c > d ? c : d;
    return ab > cd ? ab : cd;
}

// The reference's fast exp (core/src/backend/cpu_backend_internal.h:99-114): unfused Horner.
__device__ __forceinline__ float fast_exp_plain(float x) {
    x = x < -50.0f ? -50.0f : x;
    x = x > 50.0f ? 50.0f : x;
    const float y = __fmul_rn(x, 1.4426950408889634f);
    const float fl = floorf(y);
    const float f = __fsub_rn(y, fl);
    const float inner = __fadd_rn(0.224494337302845f, __fmul_rn(f, 0.07944023841053369f));
    const float mid = __fadd_rn(0.6960656421638072f, __fmul_rn(f, inner));
    const float p = __fadd_rn(1.0f, __fmul_rn(f, mid));
    const int ebits = ((int)fl + 127) << 23;
    return __fmul_rn(__int_as_float(ebits), p);
}
// core/src/kernels/hwy/hwy_fastexp.h:13-47: the same cubic with fused multiply-adds.
__device__ __forceinline__ float fast_exp_fma(float x) {
    x = fmaxf(fminf(x, 50.0f), -50.0f);
    const float y = __fmul_rn(x, 1.4426950408889634f);
    const float fl = floorf(y);
    const float f = __fsub_rn(y, fl);
    float p = __fmaf_rn(f, 0.07944023841053369f, 0.224494337302845f);
    p = __fmaf_rn(f, p, 0.6960656421638072f);
    p = __fmaf_rn(f, p, 1.0f);
    const int ebits = ((int)fl + 127) << 23;
    return __fmul_rn(__int_as_float(ebits), p);
}
// silu(gate) * up in the three orders the reference uses (see include/mi355_q4k.h MQ_SILU_*).
__device__ __forceinline__ float silu_mul(float g, float u, int mode) {
    if (mode == 1) return __fmul_rn(__fdiv_rn(g, __fadd_rn(1.0f, fast_exp_plain(-g))), u);
    if (mode == 2) {
        const float sig = __fdiv_rn(1.0f, __fadd_rn(1.0f, fast_exp_fma(__fmul_rn(g, -1.0f))));
        return __fmul_rn(__fmul_rn(g, sig), u);
    }
    return __fmul_rn(__fdiv_rn(g, __fadd_rn(1.0f, expf(-g))), u);
}
#endif

}  // namespace mq
