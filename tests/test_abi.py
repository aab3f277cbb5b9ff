"""The C-ABI library loads on a machine without a GPU and exports every symbol include/miq.h declares."""
import ctypes
import os
import re

from conftest import ROOT


def _declared():
    text = open(os.path.join(ROOT, "include", "miq.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(miq_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from aimet_amd import _lib
    lib = ctypes.CDLL(_lib.LIB_PATH)
    names = _declared()
    assert len(names) >= 30
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/miq.h but not exported"
    # and the Python binding knows each one
    assert set(names) == set(_lib.EXPORTED_SYMBOLS)


def test_host_entry_points_need_no_gpu():
    from aimet_amd import ops
    e = ops.fill_encoding_info(3, -5, 10)
    assert abs(e.min - (-4.2857142857142857)) < 1e-12 and abs(e.max - 10.714285714285714) < 1e-12
    e = ops.get_computed_encodings(6, -18, 10, False, False, False)
    assert e.offset == -41 and abs(e.delta - 0.4444) < 1e-3


def test_errors_are_reported_not_thrown():
    from aimet_amd import _lib
    e = _lib.Encoding()
    rc = _lib.lib.miq_fill_encoding_info(99, 0.0, 1.0, ctypes.byref(e))
    assert rc == -1 and b"bitwidth" in _lib.lib.miq_last_error()
    try:
        _lib.check(rc)
    except RuntimeError as exc:
        assert "bitwidth" in str(exc)
    else:
        raise AssertionError("check() must raise")


def test_cpu_tensors_are_rejected():
    import pytest
    import torch
    from aimet_amd import ops
    with pytest.raises(RuntimeError):
        ops.qdq_per_tensor(torch.zeros(8), -1.0, 1.0, 8)


def test_host_encoding_math_matches_oracle(oracle):
    import numpy as np
    from aimet_amd import ops
    rng = np.random.default_rng(0)
    for _ in range(300):
        lo, hi = sorted(rng.normal(0, 4, 2))
        for bw in (4, 8, 16):
            a = ops.fill_encoding_info(bw, lo, hi)
            b = oracle.fill_encoding_info(bw, lo, hi)
            assert (a.min, a.max, a.delta, a.offset, a.bw) == b.astuple()
            for sym, strict, uns in ((0, 0, 0), (1, 0, 0), (1, 1, 0), (1, 0, 1)):
                a = ops.get_computed_encodings(bw, lo, hi, sym, strict, uns)
                b = oracle.get_computed_encodings(bw, lo, hi, sym, strict, uns)
                assert (a.min, a.max, a.delta, a.offset, a.bw) == b.astuple()
