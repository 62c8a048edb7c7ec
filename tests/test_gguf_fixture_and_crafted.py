"""The C++ GGUF reader against (1) a file spelled out by hand from the published v3 layout
(tests/golden/gguf_v3_by_hand.hex: one key of every metadata type, two tensor infos, alignment padding) -- a statement
of the format that does not come from this package's own writer -- and (2) crafted headers whose 64-bit fields are
chosen to wrap the reader's size arithmetic: each must be refused at open, none may yield a tensor whose bytes lie
outside the mapping.  Runs without a GPU.  (Agreement with ggml's own gguf_init_from_file stays unpinned: ggml is not
part of this build and the reference ships no .gguf file.)"""
import ctypes
import os
import struct

import pytest

from densecore_amd import gguf

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "gguf_v3_by_hand.hex")


def fixture_bytes() -> bytes:
    out = bytearray()
    for line in open(GOLDEN):
        out += bytes.fromhex(line.split("#", 1)[0].strip())
    return bytes(out)


def test_hand_written_file(tmp_path):
    blob = fixture_bytes()
    assert len(blob) == 852 and blob[:4] == b"GGUF"
    path = str(tmp_path / "by_hand.gguf")
    open(path, "wb").write(blob)
    with gguf.GgufFile(path) as g:
        ints = {"t.u8": 200, "t.i8": -100, "t.u16": 60000, "t.i16": -30000, "t.u32": 4000000000, "t.i32": -2000000000,
                "t.bool": 1, "t.u64": 1 << 40, "t.i64": -(1 << 41), "general.alignment": 64}
        for key, want in ints.items():
            assert g.get_int(key) == want, key
        assert g.get_string("t.str") == "hello gguf"
        for key in ("t.f32", "t.f64", "t.arr_i32", "t.arr_str", "t.str"):
            with pytest.raises(KeyError):
                g.get_int(key)
        ts = g.tensors()
        assert [(t["name"], t["type"], t["ne"], t["offset"], t["nbytes"]) for t in ts] == [
            ("a.weight", 12, [256, 2], 0, 288), ("b.bias", 0, [5], 320, 20)]
        assert ctypes.string_at(ts[0]["data"], 288) == bytes((i * 7 + 3) & 0xFF for i in range(288))
        assert struct.unpack("<5f", ctypes.string_at(ts[1]["data"], 20)) == struct.unpack(
            "<5f", struct.pack("<5f", 1.0, -2.5, 0.0, 3.25, 0.001))
        assert g.find("b.bias") == 1 and g.find("a") == -1
    # the same bytes cut anywhere inside the header or the data are refused
    for cut in (7, 23, 39, 100, 300, 511, 700, 851):
        p = str(tmp_path / f"cut_{cut}.gguf")
        open(p, "wb").write(blob[:cut])
        with pytest.raises(ValueError):
            gguf.GgufFile(p)


def _file(tensors, data=b"\0" * 4096) -> bytes:
    """A GGUF v3 file with no metadata and the given raw tensor infos (name, dims, type, offset)."""
    out = bytearray(b"GGUF" + struct.pack("<IQQ", 3, len(tensors), 0))
    for name, dims, ttype, offset in tensors:
        out += struct.pack("<Q", len(name)) + name.encode() + struct.pack("<I", len(dims))
        for d in dims:
            out += struct.pack("<Q", d & 0xFFFFFFFFFFFFFFFF)
        out += struct.pack("<IQ", ttype, offset & 0xFFFFFFFFFFFFFFFF)
    out += b"\0" * (-len(out) % 32)
    return bytes(out) + data


CRAFTED = {
    # (ne0 / 256) * 144 * ne1 wraps to a small number: 2^61 rows of one block
    "size_product_wraps": [("w", [256, 1 << 61], 12, 0)],
    # three large dimensions whose product wraps to exactly 0
    "size_product_wraps_to_zero": [("w", [256, 1 << 32, 1 << 32], 12, 0)],
    # a negative dimension read as a huge unsigned one
    "negative_rows": [("w", [256, -1], 12, 0)],
    "negative_experts": [("w", [256, 16, -4], 12, 0)],
    "zero_rows": [("w", [256, 0], 12, 0)],
    # base + offset wraps round to a small address
    "offset_wraps": [("w", [256, 1], 12, (1 << 64) - 32)],
    "offset_past_end": [("w", [256, 1], 12, 1 << 40)],
    "size_past_end": [("w", [256, 64], 12, 0)],
    "row_not_whole_blocks": [("w", [200, 4], 12, 0)],
    "misaligned_offset": [("w", [256, 1], 12, 8)],
    "f32_size_wraps": [("b", [1 << 62, 4], 0, 0)],
}


@pytest.mark.parametrize("name", sorted(CRAFTED))
def test_crafted_tensor_tables_are_refused(tmp_path, name):
    path = str(tmp_path / f"{name}.gguf")
    open(path, "wb").write(_file(CRAFTED[name]))
    with pytest.raises(ValueError):
        gguf.GgufFile(path)


def test_the_same_table_with_honest_numbers_opens(tmp_path):
    path = str(tmp_path / "honest.gguf")
    open(path, "wb").write(_file([("w", [256, 16], 12, 0), ("b", [8], 0, 2304)]))
    with gguf.GgufFile(path) as g:
        assert [t["nbytes"] for t in g.tensors()] == [2304, 32]


def test_upload_refuses_shapes_whose_size_wraps():
    """The device-side entry points take shapes from such headers: they must refuse what does not fit, with or
    without a GPU, before any size is multiplied out unchecked."""
    from densecore_amd import _lib
    L = _lib.load()
    h = ctypes.c_void_p()
    buf = (ctypes.c_uint8 * 4096)()
    for rows, cols, experts, row_bytes, expert_bytes in [((1 << 61), 256, 1, 144, 0), (16, 256, (1 << 60), 144, 2304),
                                                         (1 << 31, 256, 1 << 31, 144, 1 << 40), (-5, 256, 1, 144, 0)]:
        rc = L.mq_weight_upload_typed(12, buf, ctypes.c_int64(rows), ctypes.c_int64(cols), ctypes.c_int64(experts),
                                      ctypes.c_size_t(row_bytes), ctypes.c_size_t(expert_bytes), ctypes.byref(h))
        assert rc != 0 and not h.value
