"""The content key of the adapters' weight cache (mq_ggml_weight_fingerprint), held to what the reference's own test
of its fingerprint asserts (core/tests/runtime/test_q4k_fingerprint.cpp): empty input is 0, every sampled byte and the
length take part, unaligned input is fine, equal bytes give equal keys, swapped bytes differ.  Runs without a GPU."""
import ctypes as C

import numpy as np

from densecore_amd import ggml_adapter as ga


def fp(buf: np.ndarray, size=None) -> int:
    return ga.lib().mq_ggml_weight_fingerprint(C.c_void_p(buf.ctypes.data), buf.size if size is None else size)


def sampled(size: int) -> np.ndarray:
    """Offsets the key reads: all of a short input; the first and last 4 KiB plus 64 x 16 bytes spread over the rest."""
    if size <= 8192:
        return np.ones(size, bool)
    m = np.zeros(size, bool)
    m[:4096] = m[-4096:] = True
    inner = size - 8192
    if inner >= 1024:
        step = inner // 64
        for i in range(64):
            m[4096 + i * step:4096 + i * step + 16] = True
    else:
        m[4096:-4096] = True
    return m


def test_empty_input_is_zero():
    one = np.ones(1, np.uint8)
    assert ga.lib().mq_ggml_weight_fingerprint(None, 100) == 0
    assert fp(one, 0) == 0 and fp(one) != 0


def test_every_sampled_byte_takes_part_and_unaligned_input_is_fine():
    for size in (1, 3, 4, 7, 8, 31, 4095, 4096, 4097, 8191, 8192, 8193, 9000, 16385, 40000):
        storage = np.zeros(size + 1, np.uint8)
        data = storage[1:]  # odd address
        data[:] = (np.arange(size) * 37 + 11).astype(np.uint8)
        original = fp(data)
        assert original == fp(data.copy())
        mask = sampled(size)
        step = 1 if size <= 8193 else 7  # every byte of the short ones, a dense sweep of the long ones
        for i in range(0, size, step):
            data[i] ^= 0x80
            changed = fp(data) != original
            data[i] ^= 0x80
            assert changed == bool(mask[i]), (size, i)
        assert fp(data) == original


def test_length_takes_part():
    data = np.zeros(16385, np.uint8)
    assert fp(data, 16384) != fp(data, 16385)


def test_swapped_bytes_differ():
    for first in range(8):
        data = np.zeros(64, np.uint8)
        data[first] = 1
        original = fp(data)
        for second in range(first + 1, 8):
            data[first], data[second] = data[second], data[first]
            assert fp(data) != original
            data[first], data[second] = data[second], data[first]
