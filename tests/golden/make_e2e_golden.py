#!/usr/bin/env python3
"""Writes tests/golden/e2e_qwen3_golden.npz from the COMPILED REFERENCE
(oracle/_ref/libwayref.so): the end-to-end workload on the random-init
Qwen3-0.6B-architecture model (28 layers, hidden 1024, 16/8 heads, head_dim 128,
F16 weights N(0, 0.02) from seed 0x5EED0100).

    python tests/golden/make_e2e_golden.py [--small | --small16 | --gemma]

Workload: 128 prompt token ids uniform in [0, vocab) from splitmix64, prefill of
the first 127, then 129 greedy steps (the last prompt token plus 128 generated
tokens).  Stored per step: the greedy token, the top-2 logit gap and eight
probe logits, plus a CRC of the model file so a test can tell "inputs differ"
from "results differ".  --small writes the same for a 2-layer toy model
(e2e_tiny_golden.npz) that the CPU-only tests can run in a second; --small16
for a 3-layer toy model whose every dimension is a multiple of 32 (vocab 320),
the smallest shape that can run with its weights on the device
(e2e_small16_golden.npz); --gemma for a 6-layer toy model of the reference's
Gemma family (local layers with a 16-key window and head_dim 32, global layers
with head_dim 64 and partial rotary, the last two layers reading earlier
layers' caches, logit soft cap): e2e_gemma_golden.npz.
"""
from __future__ import annotations

import ctypes as C
import os
import sys
import tempfile
import zlib

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import oracle  # noqa: E402
from wayruntime_amd import gguf_writer as gw, synth  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))

TINY = gw.ModelShape(n_layers=2, hidden=64, ffn=128, n_q=4, n_kv=2, head_dim=32, vocab=300,
                     context=512)
SMALL16 = gw.ModelShape(n_layers=3, hidden=128, ffn=256, n_q=4, n_kv=2, head_dim=64, vocab=320,
                        context=512)
GEMMA_TOY = gw.ModelShape(arch="gemma4", n_layers=6, hidden=96, ffn=160, n_q=4, n_kv=2, head_dim=64,
                          vocab=288, context=512, rope_base=1e6, head_dim_swa=32, sliding_window=16,
                          shared_kv_layers=2, swa_pattern=(True, True, False, True, True, False),
                          softcap=30.0, rope_base_swa=1e4)
GEMMA_SEED, GEMMA_STD = 0x5EED0102, 0.08     # a seed whose greedy stream has top-2 gaps >= 0.02
PROBES = 8


def workload(shape: gw.ModelShape, n_prompt: int):
    r = synth.splitmix64(synth.config_seed(1, 0), n_prompt)
    return (r % np.uint64(shape.vocab)).astype(np.uint32)


def file_crc(path: str) -> int:
    crc = 0
    with open(path, "rb") as f:
        while True:
            b = f.read(1 << 24)
            if not b:
                break
            crc = zlib.crc32(b, crc)
    return crc


def run_reference(path: str, prompt: np.ndarray, n_steps: int, max_ctx: int):
    ref = oracle.ref()
    ref.wr_engine_create.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
    ref.wr_model_load.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p, C.POINTER(C.c_void_p)]
    ref.wr_session_create.argtypes = [C.c_void_p, C.c_void_p, C.POINTER(C.c_void_p)]
    ref.wr_prefill.argtypes = [C.c_void_p, C.POINTER(C.c_uint32), C.c_uint32]
    ref.wr_step.argtypes = [C.c_void_p, C.c_uint32]
    ref.wr_step.restype = C.POINTER(C.c_float)
    for fn in ("wr_session_destroy", "wr_model_free", "wr_engine_destroy"):
        getattr(ref, fn).argtypes = [C.c_void_p]
        getattr(ref, fn).restype = None

    class SessionParams(C.Structure):
        _fields_ = [("max_context", C.c_uint32)]

    eng, mdl, ses = C.c_void_p(), C.c_void_p(), C.c_void_p()
    assert ref.wr_engine_create(None, C.byref(eng)) == 0
    assert ref.wr_model_load(eng, path.encode(), None, C.byref(mdl)) == 0
    sp = SessionParams(max_ctx)
    assert ref.wr_session_create(mdl, C.byref(sp), C.byref(ses)) == 0
    ids = (C.c_uint32 * (len(prompt) - 1))(*[int(t) for t in prompt[:-1]])
    assert ref.wr_prefill(ses, ids, len(prompt) - 1) == len(prompt) - 1

    tokens, gaps, probes = [], [], []
    tok = int(prompt[-1])
    for step in range(n_steps):
        lp = ref.wr_step(ses, tok)
        assert lp, f"wr_step failed at step {step}"
        logits = np.ctypeslib.as_array(lp, shape=(run_reference.vocab,)).copy()
        order = np.argsort(-logits, kind="stable")[:2]
        best = int(np.argmax(logits))                      # first maximum: ties keep the lower id
        tokens.append(best)
        gaps.append(float(logits[order[0]] - logits[order[1]]))
        probes.append(logits[np.linspace(0, run_reference.vocab - 1, PROBES).astype(int)])
        tok = best
        if step % 16 == 0:
            print(f"  step {step}: token {best} gap {gaps[-1]:.4f}", flush=True)
    ref.wr_session_destroy(ses)
    ref.wr_model_free(mdl)
    ref.wr_engine_destroy(eng)
    return (np.array(tokens, dtype=np.uint32), np.array(gaps, dtype=np.float32),
            np.array(probes, dtype=np.float32))


def main() -> None:
    small = "--small" in sys.argv
    small16 = "--small16" in sys.argv
    gemma = "--gemma" in sys.argv
    oracle.build(ref=True)
    shape = TINY if small else (SMALL16 if small16 else (GEMMA_TOY if gemma else gw.QWEN3_0_6B))
    n_prompt, n_steps = (12, 20) if small else ((40, 40) if (small16 or gemma) else (128, 129))
    out = os.path.join(HERE, "e2e_tiny_golden.npz" if small else
                       ("e2e_small16_golden.npz" if small16 else
                        ("e2e_gemma_golden.npz" if gemma else "e2e_qwen3_golden.npz")))
    with tempfile.TemporaryDirectory(dir="/tmp") as d:
        path = os.path.join(d, "model.gguf")
        if gemma:
            gw.write_model(path, shape, seed=GEMMA_SEED, std=GEMMA_STD)
        else:
            gw.write_model(path, shape)
        crc = file_crc(path)
        prompt = workload(shape, n_prompt)
        run_reference.vocab = shape.vocab
        tokens, gaps, probes = run_reference(path, prompt, n_steps, n_prompt + n_steps - 1)
    np.savez(out, prompt=prompt, tokens=tokens, gaps=gaps, probes=probes,
             model_crc=np.array([crc], dtype=np.uint64))
    print(out, "min gap", float(gaps.min()), "tokens", tokens[:8], "...")


if __name__ == "__main__":
    main()
