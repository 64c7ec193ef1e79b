"""CPU-side checks of the boundary: the shared library loads and exports every
symbol include/tpuhip.h declares, and the ctypes prototypes cover them all."""
import os
import re

import pytest

from tpu_compiler_amd import _lib, capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "tpuhip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tpuhip_[a-z0-9_]+)\s*\(", text)))


def test_library_is_built():
    assert os.path.exists(_lib.LIB_PATH), "run python -m tpu_compiler_amd.build"


def test_every_declared_symbol_is_exported_and_bound():
    lib = _lib.load()
    names = declared_symbols()
    assert len(names) > 30
    for name in names:
        assert hasattr(lib, name), "libtpuhip.so does not export " + name
        assert name in capi.PROTOTYPES, "no ctypes prototype for " + name
    for name in capi.PROTOTYPES:
        assert name in names, name + " is bound but not declared in tpuhip.h"
    capi.bind(lib)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libtpuhip.so"))
    with pytest.raises(_lib.TpuHipUnavailable):
        _lib.load()


def test_host_side_tables_need_no_gpu():
    # the 256-entry table builders are host code: check them against the oracle here
    import numpy as np
    import oracle_lib as O
    lib = capi.bind()
    x = np.arange(-128, 128, dtype=np.int16).astype(np.int8)
    for rp, mp, rn, mn in ((0, 1, 7, 13), (5, 33, 10, 102), (0, 0, 6, 6), (3, 9, 0, 1)):
        t = np.empty(256, np.int8)
        assert lib.tpuhip_leaky_relu_table(rp, mp, rn, mn, t.ctypes.data) == 0
        assert np.array_equal(t[x.view(np.uint8)], O.leaky_relu_i8(x, rp, mp, rn, mn))
    for lo, hi, r, m in ((0, 93, 0, 1), (-20, 50, 2, 3), (0, 127, 0, 1)):
        t = np.empty(256, np.int8)
        assert lib.tpuhip_clip_table(lo, hi, r, m, t.ctypes.data) == 0
        assert np.array_equal(t[x.view(np.uint8)], O.clip_i8(x, lo, hi, r, m))
    t = np.empty(256, np.int8)
    assert lib.tpuhip_leaky_relu_table(31, 1, 0, 1, t.ctypes.data) == capi.C.c_int(1).value
    assert b"rshift" in lib.tpuhip_last_error()
