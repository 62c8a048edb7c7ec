"""Writes tests/golden/gguf_v3_by_hand.hex: a small GGUF v3 file spelled out field by field from the published
container layout (magic, version, counts; one key of every metadata value type; two tensor infos; padding to
general.alignment; tensor data), as annotated hex.  Nothing of this repository is imported: the file is a second,
independent statement of the layout that the C++ reader (densecore_amd/host/gguf_ingest.cpp) is tested against,
besides the files the package's own writer produces.

    python tests/golden/make_gguf_fixture.py
"""
import os
import struct

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "gguf_v3_by_hand.hex")
lines = []
size = 0


def emit(blob: bytes, note: str):
    global size
    lines.append(f"{blob.hex():<48s} # @{size}: {note}")
    size += len(blob)


def string(s: str, note: str):
    emit(struct.pack("<Q", len(s)), f"{note}: string length {len(s)}")
    if s:
        emit(s.encode(), f"  \"{s}\"")


def key(name: str, type_id: int, type_name: str):
    string(name, "key")
    emit(struct.pack("<I", type_id), f"  value type {type_id} ({type_name})")


emit(b"GGUF", "magic")
emit(struct.pack("<I", 3), "version 3")
emit(struct.pack("<Q", 2), "tensor count")
emit(struct.pack("<Q", 15), "metadata key count")
key("t.u8", 0, "UINT8"); emit(struct.pack("<B", 200), "  200")
key("t.i8", 1, "INT8"); emit(struct.pack("<b", -100), "  -100")
key("t.u16", 2, "UINT16"); emit(struct.pack("<H", 60000), "  60000")
key("t.i16", 3, "INT16"); emit(struct.pack("<h", -30000), "  -30000")
key("t.u32", 4, "UINT32"); emit(struct.pack("<I", 4000000000), "  4000000000")
key("t.i32", 5, "INT32"); emit(struct.pack("<i", -2000000000), "  -2000000000")
key("t.f32", 6, "FLOAT32"); emit(struct.pack("<f", 1.5), "  1.5")
key("t.bool", 7, "BOOL"); emit(struct.pack("<B", 1), "  true")
key("t.str", 8, "STRING"); string("hello gguf", "  value")
key("t.arr_i32", 9, "ARRAY"); emit(struct.pack("<I", 5), "  element type 5 (INT32)"); emit(struct.pack("<Q", 3), "  3 elements")
emit(struct.pack("<iii", 7, -8, 9), "  7, -8, 9")
key("t.arr_str", 9, "ARRAY"); emit(struct.pack("<I", 8), "  element type 8 (STRING)"); emit(struct.pack("<Q", 2), "  2 elements")
string("ab", "  element 0"); string("", "  element 1")
key("t.u64", 10, "UINT64"); emit(struct.pack("<Q", 1 << 40), "  2^40")
key("t.i64", 11, "INT64"); emit(struct.pack("<q", -(1 << 41)), "  -2^41")
key("t.f64", 12, "FLOAT64"); emit(struct.pack("<d", -0.25), "  -0.25")
key("general.alignment", 4, "UINT32"); emit(struct.pack("<I", 64), "  64")
# tensor infos: name, n_dims, ne[n_dims], ggml type, offset from the start of the data section
string("a.weight", "tensor 0 name")
emit(struct.pack("<I", 2), "  2 dimensions")
emit(struct.pack("<QQ", 256, 2), "  ne = [256, 2]")
emit(struct.pack("<I", 12), "  type 12 (Q4_K): 2 rows x 1 block x 144 bytes = 288 bytes")
emit(struct.pack("<Q", 0), "  offset 0")
string("b.bias", "tensor 1 name")
emit(struct.pack("<I", 1), "  1 dimension")
emit(struct.pack("<Q", 5), "  ne = [5]")
emit(struct.pack("<I", 0), "  type 0 (F32): 20 bytes")
emit(struct.pack("<Q", 320), "  offset 320 (288 rounded up to the alignment)")
pad = -size % 64
emit(b"\0" * pad, f"padding to the alignment: the data section starts at {size + pad}")
DATA_START = size
a = bytes((i * 7 + 3) & 0xFF for i in range(288))
for i in range(0, 288, 24):
    emit(a[i:i + 24], f"a.weight bytes {i}..{i + 23}: (7 i + 3) mod 256")
emit(b"\0" * 32, "padding to offset 320")
emit(struct.pack("<5f", 1.0, -2.5, 0.0, 3.25, 0.001), "b.bias = 1.0, -2.5, 0.0, 3.25, 0.001")
with open(OUT, "w") as f:
    f.write("# GGUF v3, little endian, written out by hand (see make_gguf_fixture.py beside this file).\n")
    f.write(f"# {size} bytes; data section at {DATA_START}.  Hex bytes, then '#', the file offset and what the bytes are.\n")
    f.write("\n".join(lines) + "\n")
print(OUT, size, "bytes")
