"""The shared library loads on a CPU-only machine and exports every symbol
the header declares (no compute calls here)."""
import ctypes as C
import os
import re

import pytest

from wayruntime_amd import hipattn

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(wr_hip_(?:attn|proj|rows)_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared("wr_hip_attn.h")
    assert len(names) >= 20
    lib = C.CDLL(hipattn.HIP_SO)
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_binding_covers_every_declared_symbol():
    lib = hipattn.load()
    for n in _declared("wr_hip_attn.h"):
        if n == "wr_hip_attn_set_log":
            continue
        assert getattr(lib, n).argtypes is not None, n


def test_entry_points_refuse_to_run_before_init():
    # No device is touched: every entry point must report WR_HIP_ERR_STATE
    # rather than fall back to anything.
    if hipattn._inited:
        pytest.skip("library already initialised in this process")
    lib = hipattn.load()
    h = C.c_void_p()
    hd = (C.c_uint32 * 1)(128)
    assert lib.wr_hip_attn_kv_create(1, hd, 8, 128, C.byref(h)) == hipattn.ERR_STATE
    assert lib.wr_hip_attn_sync() == hipattn.ERR_STATE
    assert lib.wr_hip_attn_dev_alloc(1024) is None
