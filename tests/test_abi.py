"""CPU-side checks of the C ABI: libkq.so loads, exports every symbol include/kq.h declares, and
the registry / host-only entry points behave (no GPU compute is called)."""
import ctypes as C
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "mlx-kquant_amd", "lib", "libkq.so")


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(LIB):
        subprocess.check_call([sys.executable, os.path.join(ROOT, "mlx-kquant_amd", "build.py")])
    return C.CDLL(LIB)


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "kq.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(kq_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_exported(lib):
    names = _declared_symbols()
    assert len(names) >= 14
    for n in names:
        assert hasattr(lib, n), n


def test_registry_matches_python_geometry(lib):
    sys.path.insert(0, os.path.join(ROOT, "mlx-kquant_amd"))
    import kq

    assert kq.codecs() == list(kq.CODEC_GEOMETRY) or sorted(kq.codecs()) == sorted(kq.CODEC_GEOMETRY)
    import oracle_lib as O

    assert kq.codecs() == O.ALL_CODECS
    for name in kq.codecs():
        _, _, bpb, wpb = kq.codec_geometry.geometry(name)
        assert (wpb, bpb) == O.geometry(name)
        assert kq.codec_has_matmul(name) and kq.codec_has_moe_glu(name)
    assert not kq.codec_has_matmul("nope") and not kq.codec_has_moe_glu("nope")
    assert kq.bytes_per_row("q4_k", 4096) == 2304 and kq.bytes_per_row("q6_k", 14336) == 11760
    assert kq.weights_per_row("mxfp4", 1530) == 2880
    with pytest.raises(ValueError):
        kq.bytes_per_row("q4_k", 100)


def test_error_codes_without_gpu(lib):
    lib.kq_last_error.restype = C.c_char_p
    lib.kq_dequantize.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_int, C.c_int, C.c_void_p]
    assert lib.kq_dequantize(None, None, 256, 99, 0, None) == -1
    assert b"codec" in lib.kq_last_error()
    assert lib.kq_dequantize(None, None, 100, 2, 0, None) == -1  # not a whole number of blocks
    assert lib.kq_dequantize(None, None, 0, 2, 0, None) == 0  # empty tensor is a no-op
    assert lib.kq_codec_id(b"q4_k") == 2 and lib.kq_codec_id(b"zzz") == -1


def test_python_front_end_refuses_cpu_tensors():
    sys.path.insert(0, os.path.join(ROOT, "mlx-kquant_amd"))
    import torch

    import kq

    w = torch.zeros((4, 144), dtype=torch.uint8)
    with pytest.raises(RuntimeError):
        kq.dequantize(w, None, "q4_k")
    with pytest.raises(RuntimeError):
        kq.quantized_matmul(torch.zeros((1, 256), dtype=torch.float16), w, None, "q4_k")
    with pytest.raises(ValueError):
        kq.quantized_matmul(torch.zeros((1, 128), dtype=torch.float16), w, None, "q4_k")
