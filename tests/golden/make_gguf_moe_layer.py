"""One MoE layer as a GGUF v3 file, written from the published container layout without anything of this repository
(only `struct`): the independent statement of the format and of the tensor names that mq_gguf_load_moe_layer is tested
against.

    python tests/golden/make_gguf_moe_layer.py [out.gguf]      # prints the SHA-256; writes the file when a path is given

Tensors, named as a Q4_K_M-style model file of the qwen35moe architecture names them: blk.0.ffn_gate_exps.weight /
ffn_up_exps.weight (Q4_K, [256, 256, 3]), ffn_down_exps.weight (Q5_K, [256, 256, 3]), the shared expert
ffn_{gate,up,down}_shexp.weight, its scalar gate ffn_gate_inp_shexp.weight (F32 [256]) and the router ffn_gate_inp.weight
(F16 [256, 3]); metadata "general.architecture" and "<arch>.expert_used_count".  331 KB of blocks: too long to keep as
hex, so tests call moe_layer_file() and pin the result by its SHA-256.  Block bytes come from a 32-bit linear
congruential generator; the high byte of d and dmin is overwritten so that both are fp16 values in [2^-7, 2^-6)."""
import hashlib
import struct
import sys


def _lcg_bytes(seed: int, count: int) -> bytearray:
    out, state = bytearray(count), seed & 0xFFFFFFFF
    for i in range(count):
        state = (state * 1664525 + 1013904223) & 0xFFFFFFFF
        out[i] = state >> 24
    return out


def _kquant_rows(seed: int, rows: int, block_bytes: int) -> bytes:
    """rows x one super-block; fp16 d (and dmin) forced into [2^-7, 2^-6)."""
    raw = _lcg_bytes(seed, rows * block_bytes)
    for r in range(rows):
        base = r * block_bytes
        for off in (0, 2):                     # Q4_K / Q5_K: d at 0, dmin at 2
            raw[base + off + 1] = 0x20         # sign 0, exponent 8 (2^-7), top mantissa bits 0
    return bytes(raw)


def moe_layer_file() -> bytes:
    hidden = inter = 256
    n_exp, used = 3, 2
    tensors = []                               # (name, dims, type, bytes)
    tensors.append(("blk.0.ffn_gate_exps.weight", [hidden, inter, n_exp], 12, _kquant_rows(11, inter * n_exp, 144)))
    tensors.append(("blk.0.ffn_up_exps.weight", [hidden, inter, n_exp], 12, _kquant_rows(12, inter * n_exp, 144)))
    tensors.append(("blk.0.ffn_down_exps.weight", [inter, hidden, n_exp], 13, _kquant_rows(13, hidden * n_exp, 176)))
    tensors.append(("blk.0.ffn_gate_shexp.weight", [hidden, inter], 12, _kquant_rows(14, inter, 144)))
    tensors.append(("blk.0.ffn_up_shexp.weight", [hidden, inter], 12, _kquant_rows(15, inter, 144)))
    tensors.append(("blk.0.ffn_down_shexp.weight", [inter, hidden], 13, _kquant_rows(16, hidden, 176)))
    gate_inp = struct.pack(f"<{hidden}f", *[((i * 37) % 64 - 32) / 512.0 for i in range(hidden)])
    tensors.append(("blk.0.ffn_gate_inp_shexp.weight", [hidden], 0, gate_inp))
    # router as F16: exactly representable values k / 256, k in -128..127
    router = b"".join(struct.pack("<e", (((e * hidden + i) * 29) % 256 - 128) / 256.0) for e in range(n_exp) for i in range(hidden))
    tensors.append(("blk.0.ffn_gate_inp.weight", [hidden, n_exp], 1, router))
    align = 32
    out = bytearray(b"GGUF" + struct.pack("<IQQ", 3, len(tensors), 2))

    def s(text: str) -> bytes:
        return struct.pack("<Q", len(text)) + text.encode()

    out += s("general.architecture") + struct.pack("<I", 8) + s("qwen35moe")
    out += s("qwen35moe.expert_used_count") + struct.pack("<II", 4, used)
    offset = 0
    for name, dims, ttype, blob in tensors:
        out += s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims) + struct.pack("<IQ", ttype, offset)
        offset += -(-len(blob) // align) * align
    out += b"\0" * (-len(out) % align)
    for _, _, _, blob in tensors:
        out += blob + b"\0" * (-len(blob) % align)
    return bytes(out)


if __name__ == "__main__":
    blob = moe_layer_file()
    print(len(blob), "bytes, sha256", hashlib.sha256(blob).hexdigest())
    if len(sys.argv) > 1:
        open(sys.argv[1], "wb").write(blob)
