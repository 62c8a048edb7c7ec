"""CPU-side checks of the C ABI: the library loads without a GPU, exports every symbol the public
header declares, and refuses work loudly when no device is present."""
import os
import re

import pytest

from densecore_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols(header="mi355_q4k.h"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mq_[a-z0-9_]+)\s*\(", text)))


def test_header_and_loader_agree():
    assert declared_symbols() == sorted(_lib.EXPORTS)
    assert declared_symbols("mi355_q4k_debug.h") == sorted(_lib.DEBUG_EXPORTS)
    assert not [s for s in declared_symbols() if s.startswith(("mq_debug", "mq_census"))], "instruments belong in the debug header"


def test_library_exports_every_declared_symbol():
    L = _lib.load()
    for name in declared_symbols() + declared_symbols("mi355_q4k_debug.h"):
        assert hasattr(L, name), name


def test_ggml_adapter_library_exports_every_declared_symbol():
    import ctypes

    from densecore_amd import ggml_adapter
    _lib.load()
    L = ctypes.CDLL(ggml_adapter.LIB_PATH, mode=ctypes.RTLD_GLOBAL)
    declared = declared_symbols("mi355_q4k_ggml.h")
    assert declared == sorted(ggml_adapter.EXPORTS)
    for name in declared:
        assert hasattr(L, name), name
    # the ctypes mirror must have ggml's layout: data at 248, name at 256, 336 bytes in all
    assert ggml_adapter.GgmlTensor.data.offset == 248 and ctypes.sizeof(ggml_adapter.GgmlTensor) == 336


@pytest.mark.skipif(os.path.exists("/dev/kfd"), reason="a GPU is present")
def test_no_gpu_is_a_loud_error_not_a_fallback():
    L = _lib.load()
    assert L.mq_init(0) != 0
    assert b"no HIP device" in L.mq_last_error()
    with pytest.raises(_lib.MqError):
        _lib.lib()
