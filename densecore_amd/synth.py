"""Seeded synthetic tensors for the Q4_K x Q8_K path.

Counter-based (SplitMix64 finaliser over ``seed + (i+1)*gamma``) so any slice
can be produced independently, in any order, on the host (numpy, here) or on
the device (the library's fill kernel uses the same integer recipe for the
multi-gigabyte weight sets of the decode-step workload).

Recipes
-------
* Q4_K super-block (144 B, layout of ``block_q4_K``): all 144 bytes uniform
  random -- i.e. every 6-bit scale/min and every 4-bit quant is uniform -- then
  ``d`` and ``dmin`` overwritten with ``fp16(U(0.001, 0.01))``.  This is the
  raw-block filling the reference's own micro-benchmark uses
  (core/tests/benchmarks/q4_down_rowpair.cpp:38-46) with the positive scale
  range of the benchmark configuration.
* activations / router logits: fp32 N(0, 1) by Box-Muller on the same stream.
"""
from __future__ import annotations

import numpy as np

QK_K = 256
Q4K_BLOCK_BYTES = 144
Q5K_BLOCK_BYTES = 176
Q6K_BLOCK_BYTES = 210
Q8K_BLOCK_BYTES = 292
GGML_TYPE_Q4_K = 12
GGML_TYPE_Q5_K = 13
GGML_TYPE_Q6_K = 14
GGML_TYPE_Q8_0 = 8
Q80_BLOCK_BYTES = 34       # fp16 d + 32 int8 codes
Q80_GROUP_BYTES = 8 * 34   # the eight blocks that cover 256 weights of a row
# bytes of 256 weights of a row, per weight type
BLOCK_BYTES = {GGML_TYPE_Q4_K: Q4K_BLOCK_BYTES, GGML_TYPE_Q5_K: Q5K_BLOCK_BYTES, GGML_TYPE_Q6_K: Q6K_BLOCK_BYTES,
               GGML_TYPE_Q8_0: Q80_GROUP_BYTES}

_GAMMA = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def mix64(z: np.ndarray) -> np.ndarray:
    """SplitMix64 output function on a uint64 array."""
    z = z.astype(np.uint64, copy=True)
    with np.errstate(over="ignore"):
        z ^= z >> np.uint64(30)
        z *= _M1
        z ^= z >> np.uint64(27)
        z *= _M2
        z ^= z >> np.uint64(31)
    return z


def stream_u64(seed: int, start: int, count: int) -> np.ndarray:
    """Words ``start .. start+count-1`` of the stream named by ``seed``."""
    with np.errstate(over="ignore"):
        idx = np.arange(start + 1, start + count + 1, dtype=np.uint64)
        return mix64(np.uint64(seed & 0xFFFFFFFFFFFFFFFF) + idx * _GAMMA)


def tensor_seed(*parts) -> int:
    """Stable 64-bit seed from a tuple such as ("cfg3", "gate", layer, expert)."""
    h = 0xCBF29CE484222325
    for p in parts:
        for b in str(p).encode() + b"\x1f":
            h = ((h ^ b) * 0x100000001B3) & 0xFFFFFFFFFFFFFFFF
    return h


def unit_scale_f16(words: np.ndarray) -> np.ndarray:
    """fp16(0.001 + 0.009*u), u = top 24 bits / 2^24, every step in fp32."""
    u = (words >> np.uint64(40)).astype(np.float32) * np.float32(2.0 ** -24)
    v = np.float32(0.001) + np.float32(0.009) * u
    return v.astype(np.float16)


def q4k_blocks(seed: int, n_blocks: int, first_block: int = 0) -> np.ndarray:
    """``[n_blocks, 144]`` uint8 array of seeded Q4_K super-blocks."""
    words = stream_u64(seed, first_block * 18, n_blocks * 18).reshape(n_blocks, 18)
    raw = words.view(np.uint8).reshape(n_blocks, Q4K_BLOCK_BYTES).copy()
    sw = stream_u64(seed ^ 0x5CA1E5CA1E5CA1E5, first_block * 2, n_blocks * 2).reshape(n_blocks, 2)
    raw[:, 0:2] = unit_scale_f16(sw[:, 0]).view(np.uint8).reshape(n_blocks, 2)
    raw[:, 2:4] = unit_scale_f16(sw[:, 1]).view(np.uint8).reshape(n_blocks, 2)
    return raw


def q5k_blocks(seed: int, n_blocks: int, first_block: int = 0) -> np.ndarray:
    """``[n_blocks, 176]`` uint8 array of seeded Q5_K super-blocks: the Q4_K recipe over 22 words a block
    (d, dmin, scales[12], qh[32], qs[128]; core/src/kernels/hwy/hwy_moe_quant.cc:36-45)."""
    words = stream_u64(seed, first_block * 22, n_blocks * 22).reshape(n_blocks, 22)
    raw = words.view(np.uint8).reshape(n_blocks, Q5K_BLOCK_BYTES).copy()
    sw = stream_u64(seed ^ 0x5CA1E5CA1E5CA1E5, first_block * 2, n_blocks * 2).reshape(n_blocks, 2)
    raw[:, 0:2] = unit_scale_f16(sw[:, 0]).view(np.uint8).reshape(n_blocks, 2)
    raw[:, 2:4] = unit_scale_f16(sw[:, 1]).view(np.uint8).reshape(n_blocks, 2)
    return raw


def q5k_matrix(seed: int, rows: int, cols: int) -> np.ndarray:
    """Row-major Q5_K matrix ``[rows, cols/256 * 176]`` uint8 (ggml row layout)."""
    if cols % QK_K:
        raise ValueError("cols must be a multiple of 256")
    nb = cols // QK_K
    return q5k_blocks(seed, rows * nb).reshape(rows, nb * Q5K_BLOCK_BYTES)


def q6k_blocks(seed: int, n_blocks: int, first_block: int = 0) -> np.ndarray:
    """``[n_blocks, 210]`` uint8 array of seeded Q6_K super-blocks (ql[128], qh[64], scales[16] signed, fp16 d;
    core/src/llm/matmul/q6_small_batch.h:13-24): 27 stream words a block, the first 210 bytes of them taken,
    then ``d`` overwritten with ``fp16(U(0.001, 0.01))``."""
    words = stream_u64(seed, first_block * 27, n_blocks * 27).reshape(n_blocks, 27)
    raw = words.view(np.uint8).reshape(n_blocks, 216)[:, :Q6K_BLOCK_BYTES].copy()
    sw = stream_u64(seed ^ 0x5CA1E5CA1E5CA1E5, first_block * 2, n_blocks * 2).reshape(n_blocks, 2)
    raw[:, 208:210] = unit_scale_f16(sw[:, 0]).view(np.uint8).reshape(n_blocks, 2)
    return raw


def q6k_matrix(seed: int, rows: int, cols: int) -> np.ndarray:
    """Row-major Q6_K matrix ``[rows, cols/256 * 210]`` uint8 (ggml row layout)."""
    if cols % QK_K:
        raise ValueError("cols must be a multiple of 256")
    nb = cols // QK_K
    return q6k_blocks(seed, rows * nb).reshape(rows, nb * Q6K_BLOCK_BYTES)


def q80_matrix(seed: int, rows: int, cols: int) -> np.ndarray:
    """Row-major Q8_0 matrix ``[rows, cols/32 * 34]`` uint8 (ggml row layout).  Per 256 weights of a row: 40 stream
    words, the first 32 of them the codes of the eight blocks in order (a byte 0x80 becomes 0x81: ggml's quantizer
    never writes -128), and ``d = fp16(U(0.001, 0.01))`` per block from the scale stream."""
    if cols % QK_K:
        raise ValueError("cols must be a multiple of 256")
    groups = rows * cols // QK_K
    words = stream_u64(seed, 0, groups * 40).reshape(groups, 40)
    codes = np.ascontiguousarray(words[:, :32]).view(np.uint8).reshape(groups, 8, 32).copy()
    codes[codes == 0x80] = 0x81
    raw = np.zeros((groups, 8, Q80_BLOCK_BYTES), np.uint8)
    raw[:, :, 2:] = codes
    sw = stream_u64(seed ^ 0x5CA1E5CA1E5CA1E5, 0, groups * 8).reshape(groups, 8)
    raw[:, :, 0:2] = unit_scale_f16(sw).view(np.uint8).reshape(groups, 8, 2)
    return raw.reshape(rows, cols // 32 * Q80_BLOCK_BYTES)


def q4k_matrix(seed: int, rows: int, cols: int) -> np.ndarray:
    """Row-major Q4_K matrix ``[rows, cols/256 * 144]`` uint8 (ggml row layout)."""
    if cols % QK_K:
        raise ValueError("cols must be a multiple of 256")
    nb = cols // QK_K
    return q4k_blocks(seed, rows * nb).reshape(rows, nb * Q4K_BLOCK_BYTES)


def normal_f32(seed: int, shape) -> np.ndarray:
    """fp32 N(0,1), Box-Muller in float64 on the counter stream."""
    count = int(np.prod(shape))
    w = stream_u64(seed, 0, 2 * count).reshape(count, 2)
    u1 = ((w[:, 0] >> np.uint64(11)).astype(np.float64) + 1.0) * (2.0 ** -53)  # (0, 1]
    u2 = (w[:, 1] >> np.uint64(11)).astype(np.float64) * (2.0 ** -53)
    z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
    return z.astype(np.float32).reshape(shape)


def q4k_row_bytes(cols: int) -> int:
    return cols // QK_K * Q4K_BLOCK_BYTES


def q8k_row_bytes(cols: int) -> int:
    return cols // QK_K * Q8K_BLOCK_BYTES
