"""The C-ABI library loads and exports exactly what include/chadq.h declares.  No GPU, no compute calls."""
import ctypes
import os
import re

import pytest

from chadslab_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "chadq.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(chadq_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_something():
    syms = declared_symbols()
    assert "chadq_gemv_i4g32" in syms and "chadq_version" in syms and len(syms) >= 10


def test_library_is_built_in_tree():
    assert _lib.LIB_PATH.exists(), "run `python -m chadslab_amd.build` (or __graft_entry__.build())"
    assert str(_lib.LIB_PATH).startswith(ROOT)


def test_every_declared_symbol_is_exported():
    lib = ctypes.CDLL(str(_lib.LIB_PATH))
    for name in declared_symbols():
        assert hasattr(lib, name), "libchadq.so does not export %s" % name


def test_python_binding_covers_the_header():
    assert sorted(_lib.SIGNATURES) == declared_symbols()


def test_version_and_arch_without_a_gpu():
    lib = _lib.load()
    assert lib.chadq_version() >= 100
    assert lib.chadq_arch() == b"gfx950"
    assert lib.chadq_last_error() is not None


def test_ops_refuse_cpu_tensors():
    import torch

    from chadslab_amd import QWeightInt4G32, ops

    qw = QWeightInt4G32(torch.zeros(4, 16, dtype=torch.uint8), torch.ones(4, 1, dtype=torch.float16))
    with pytest.raises(ValueError, match="GPU tensor"):
        ops.qgemv(torch.zeros(1, 32, dtype=torch.bfloat16), qw)
    with pytest.raises(ValueError, match="GPU tensor"):
        ops.unpack_int4(torch.zeros(4, 16, dtype=torch.uint8))


def test_host_side_quantizer_matches_oracle():
    import numpy as np
    import torch

    import chadslab_amd as C
    from oracle import chadq_oracle as O

    w = (np.random.Generator(np.random.PCG64(7)).standard_normal((24, 96)) * 0.1).astype(np.float32)
    qw = C.quantize_int4_g32(torch.from_numpy(w))
    p, s = O.quantize_int4_g32(w)
    assert np.array_equal(qw.packed.numpy(), p) and np.array_equal(qw.scale.numpy(), s)
    q8 = C.quantize_int8_row(torch.from_numpy(w))
    w8, s8 = O.quantize_int8_row(w)
    assert np.array_equal(q8.w.numpy(), w8) and np.array_equal(q8.scale.numpy(), s8)
    with pytest.raises(ValueError):
        C.QWeightInt4G32(torch.zeros(4, 16, dtype=torch.uint8), torch.ones(4, 2, dtype=torch.float16))
