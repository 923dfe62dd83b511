"""Shared helpers for the parity tests."""
from __future__ import annotations

import numpy as np

import oracle
from wayruntime_amd import synth

MAX_ABS = 2e-3        # tolerance stated for the attention outputs
REL_L2 = 1e-3


def errors(got: np.ndarray, want: np.ndarray):
    g = got.astype(np.float64).ravel()
    w = want.astype(np.float64).ravel()
    max_abs = float(np.max(np.abs(g - w)))
    rel_l2 = float(np.linalg.norm(g - w) / max(np.linalg.norm(w), 1e-30))
    return max_abs, rel_l2


def assert_close(got, want, what=""):
    assert not np.isnan(got).any(), f"{what}: NaN in device output"
    max_abs, rel_l2 = errors(got, want)
    assert max_abs <= MAX_ABS and rel_l2 <= REL_L2, \
        f"{what}: max_abs={max_abs:.3e} (<= {MAX_ABS}), rel_l2={rel_l2:.3e} (<= {REL_L2})"
    return max_abs, rel_l2


def make_kv(seed: int, rows: int, nkv: int, hd: int, gen=synth.normal):
    """(k32, v32 float32, k16, v16 truncated bit patterns) [rows, nkv, hd]."""
    k32 = gen(seed, (rows, nkv, hd))
    v32 = gen(seed + 1, (rows, nkv, hd))
    return k32, v32, synth.f32_to_f16_trunc(k32), synth.f32_to_f16_trunc(v32)


def oracle_decode(q, k16, v16, seq_k, scale_override=0.0, window=0):
    """q [nq, hd] -> [nq, hd] through the CPU oracle."""
    oracle.set_attn_max_seq(1 << 20)
    return oracle.attention(q[None], k16, v16, seq_k=seq_k, scale_override=scale_override,
                            window=window)[0]
