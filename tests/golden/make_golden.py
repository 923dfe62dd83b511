#!/usr/bin/env python3
"""Writes the fixtures in this directory from the COMPILED REFERENCE
(``oracle/_ref/libwayref.so``, built by ``make -C oracle ref`` from the
reference's own sources).  Run from the repository root where the reference
tree is available:

    python tests/golden/make_golden.py

Inputs come from tests/golden/cases.py (integer-hash fills, regenerated
bit-for-bit by the tests), so the files hold expected outputs only:

    attn_golden.npz   one float32 array per attention case
    rope_golden.npz   one float32 array per RoPE case
    mathx_golden.npz  exp/log/sqrt/sin/cos on fixed grids
    f16_golden.npz    truncating encode of fixed float32 bit patterns,
                      decode of all 65536 binary16 patterns (as uint32 bits)
    ops_golden.npz    RMS normalisation and GGML-layout matmul outputs (the
                      matmul through whichever SIMD variant this host selects;
                      its variant number is stored beside the outputs)
"""
from __future__ import annotations

import ctypes as C
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import oracle  # noqa: E402
from tests.golden import cases  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def main() -> None:
    oracle.build(ref=True)
    if not oracle.have_ref():
        raise SystemExit("reference build not available; cannot write fixtures")
    ref = oracle.ref()

    attn = {}
    for case in cases.ATTN_CASES:
        name, _sq, _nq, _nkv, _hd, _rows, seq_k, sc, win, _dt = case
        q, k, v = cases.attn_inputs(case)
        rc, out = oracle.ref_attention(q, k, v, seq_k=seq_k, scale_override=sc, window=win)
        assert rc == 0, (name, rc)
        attn[name] = out
    np.savez(os.path.join(HERE, "attn_golden.npz"), **attn)

    rope = {}
    for case in cases.ROPE_CASES:
        name, _seq, _heads, _hd, pos, theta, nrot = case
        x = cases.rope_input(case)
        y = np.empty_like(x)
        tx, ty = oracle.wrap(x), oracle.wrap(y)
        rc = ref.wri_op_rope(C.byref(tx), C.byref(ty), pos, theta, nrot)
        assert rc == 0, (name, rc)
        rope[name] = y
    np.savez(os.path.join(HERE, "rope_golden.npz"), **rope)

    mathx = {}
    for fn in ("exp", "log", "sqrt", "sin", "cos"):
        f = getattr(ref, "wri_" + fn)
        mathx[fn] = np.array([f(float(x)) for x in cases.math_grid(fn)], dtype=np.float32)
    np.savez_compressed(os.path.join(HERE, "mathx_golden.npz"), **mathx)

    bits = cases.f16_encode_bits()
    # exact bit patterns (NaN payloads included) go in as raw 4-byte buffers
    enc = np.array([ref.wri_f32_to_f16(C.c_float.from_buffer_copy(int(b).to_bytes(4, "little")))
                    for b in bits], dtype=np.uint16)
    dec = np.array([ref.wri_f16_to_f32(h) for h in range(65536)], dtype=np.float32).view(np.uint32)
    np.savez_compressed(os.path.join(HERE, "f16_golden.npz"), encode=enc, decode_bits=dec)

    ops = {}
    ref.wri_op_rmsnorm.argtypes = [C.POINTER(oracle.Tensor)] * 3 + [C.c_float]
    ref.wri_op_matmul.argtypes = [C.POINTER(oracle.Tensor)] * 3
    ref.wri_simd_matmul_variant.restype = C.c_int
    for case in cases.NORM_CASES:
        name, _rows, _dim, wn, eps = case
        x, w = cases.norm_inputs(case)
        y = np.empty_like(x)
        tx, ty = oracle.wrap(x), oracle.wrap(y)
        tw = oracle.wrap(w) if wn else None
        rc = ref.wri_op_rmsnorm(C.byref(tx), C.byref(tw) if wn else None, C.byref(ty), eps)
        assert rc == 0, (name, rc)
        ops["norm_" + name] = y
    GGML_WEIGHT = 1 << 3                               # src/core/internal.h:113-118
    for case in cases.MATMUL_CASES:
        name, rows, n_in, n_out, _std = case
        x, w16 = cases.matmul_inputs(case)
        # the loader widens F16 weights to F32 before any multiply (loader.c:164-190)
        w32 = np.array([ref.wri_f16_to_f32(int(h)) for h in w16.reshape(-1)],
                       dtype=np.float32).reshape(n_out, n_in)
        y = np.empty((rows, n_out), dtype=np.float32)
        ta, tc = oracle.wrap(x), oracle.wrap(y)
        tb = oracle.wrap(w32, shape=(n_in, n_out), flags=GGML_WEIGHT)
        rc = ref.wri_op_matmul(C.byref(ta), C.byref(tb), C.byref(tc))
        assert rc == 0, (name, rc)
        ops["matmul_" + name] = y
    ref.wri_op_fused_silu_mul.argtypes = [C.POINTER(oracle.Tensor)] * 3
    g, u = cases.silu_inputs()
    y = np.empty_like(g)
    tg, tu, ty = oracle.wrap(g), oracle.wrap(u), oracle.wrap(y)
    assert ref.wri_op_fused_silu_mul(C.byref(tg), C.byref(tu), C.byref(ty)) == 0
    ops["silu_mul"] = y
    ops["matmul_variant"] = np.array([ref.wri_simd_matmul_variant()], dtype=np.int32)
    np.savez(os.path.join(HERE, "ops_golden.npz"), **ops)

    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    main()
