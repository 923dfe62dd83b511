"""Writes random-init GGUF v3 model files of the Llama / Qwen3 architectures and
of the reference's Gemma family ("gemma4": sandwich norms, per-layer head_dim,
sliding-window layers, KV-shared layers; no per-layer-input tables).

No checkpoints can be fetched here, so the end-to-end workload runs on weights
drawn from a fixed seed: matmul weights F16 ~ N(0, std), norm vectors F32 = 1
(Gemma files: 1 + 0.1 N(0, 1), so that every norm weight matters).
The file follows the GGUF container layout (magic, version 3, tensor and
key/value counts, typed key/values, tensor infos, aligned data section) and the
tensor names / orientations the reference loader expects
(reference: src/core/loader.c:283-401 names, :217-231 orientation;
src/core/gguf.c:897-938 architecture keys).
"""
from __future__ import annotations

import struct
from dataclasses import dataclass

import numpy as np


GGML_F32, GGML_F16 = 0, 1
T_U32, T_F32, T_BOOL, T_STR, T_ARR = 4, 6, 7, 8, 9
ALIGN = 32


@dataclass
class ModelShape:
    arch: str = "qwen3"
    n_layers: int = 28
    hidden: int = 1024
    ffn: int = 3072
    n_q: int = 16
    n_kv: int = 8
    head_dim: int = 128
    vocab: int = 151936
    context: int = 40960
    rope_base: float = 1e6
    rms_eps: float = 1e-6
    tied_head: bool = True
    # Gemma family only (src/core/loader.c:576-628, src/core/gguf.c:920-938)
    head_dim_swa: int = 0            # head_dim of sliding-window layers (0 = same)
    sliding_window: int = 0
    shared_kv_layers: int = 0        # trailing layers that read an earlier layer's cache
    swa_pattern: tuple = ()          # per layer: True = sliding-window (local) layer
    softcap: float = 0.0             # final-logit soft cap
    rope_base_swa: float = 0.0

    def layer_head_dim(self, l: int) -> int:
        if self.arch == "gemma4" and self.swa_pattern and self.swa_pattern[l] and self.head_dim_swa:
            return self.head_dim_swa
        return self.head_dim


QWEN3_0_6B = ModelShape()


def _s(b: str) -> bytes:
    raw = b.encode()
    return struct.pack("<Q", len(raw)) + raw


def _kv_u32(key, v):
    return _s(key) + struct.pack("<II", T_U32, v)


def _kv_f32(key, v):
    return _s(key) + struct.pack("<If", T_F32, v)


def _kv_str(key, v):
    return _s(key) + struct.pack("<I", T_STR) + _s(v)


def _kv_bools(key, vals):
    return (_s(key) + struct.pack("<IIQ", T_ARR, T_BOOL, len(vals)) +
            bytes(1 if v else 0 for v in vals))


def tensor_plan(m: ModelShape):
    """[(name, dims innermost-first, ggml type)] in file order."""
    plan = [("token_embd.weight", (m.hidden, m.vocab), GGML_F16),
            ("output_norm.weight", (m.hidden,), GGML_F32)]
    if not m.tied_head:
        plan.append(("output.weight", (m.hidden, m.vocab), GGML_F16))
    gemma = m.arch == "gemma4"
    for l in range(m.n_layers):
        p = f"blk.{l}."
        hd = m.layer_head_dim(l)
        plan += [(p + "attn_norm.weight", (m.hidden,), GGML_F32),
                 (p + "attn_q.weight", (m.hidden, m.n_q * hd), GGML_F16),
                 (p + "attn_k.weight", (m.hidden, m.n_kv * hd), GGML_F16),
                 (p + "attn_v.weight", (m.hidden, m.n_kv * hd), GGML_F16)]
        if m.arch == "qwen3" or gemma:
            plan += [(p + "attn_q_norm.weight", (hd,), GGML_F32),
                     (p + "attn_k_norm.weight", (hd,), GGML_F32)]
        plan += [(p + "attn_output.weight", (m.n_q * hd, m.hidden), GGML_F16)]
        if gemma:
            plan += [(p + "post_attention_norm.weight", (m.hidden,), GGML_F32)]
        plan += [(p + "ffn_norm.weight", (m.hidden,), GGML_F32),
                 (p + "ffn_gate.weight", (m.hidden, m.ffn), GGML_F16),
                 (p + "ffn_up.weight", (m.hidden, m.ffn), GGML_F16),
                 (p + "ffn_down.weight", (m.ffn, m.hidden), GGML_F16)]
        if gemma:
            plan += [(p + "post_ffw_norm.weight", (m.hidden,), GGML_F32)]
    return plan


def write_model(path: str, m: ModelShape, seed: int = 0x5EED0100, std: float = 0.02) -> None:
    a = m.arch
    kvs = [
        _kv_str("general.architecture", a),
        _kv_str("general.name", f"random-init {a} (seed {seed:#x})"),
        _kv_u32("general.alignment", ALIGN),
        _kv_u32(f"{a}.block_count", m.n_layers),
        _kv_u32(f"{a}.context_length", m.context),
        _kv_u32(f"{a}.embedding_length", m.hidden),
        _kv_u32(f"{a}.feed_forward_length", m.ffn),
        _kv_u32(f"{a}.attention.head_count", m.n_q),
        _kv_u32(f"{a}.attention.head_count_kv", m.n_kv),
        _kv_u32(f"{a}.attention.key_length", m.head_dim),
        _kv_u32(f"{a}.attention.value_length", m.head_dim),
        _kv_f32(f"{a}.attention.layer_norm_rms_epsilon", m.rms_eps),
        _kv_f32(f"{a}.rope.freq_base", m.rope_base),
    ]
    if a == "gemma4":
        assert len(m.swa_pattern) == m.n_layers
        kvs += [
            _kv_u32(f"{a}.attention.key_length_swa", m.head_dim_swa),
            _kv_u32(f"{a}.attention.sliding_window", m.sliding_window),
            _kv_u32(f"{a}.attention.shared_kv_layers", m.shared_kv_layers),
            _kv_f32(f"{a}.final_logit_softcapping", m.softcap),
            _kv_f32(f"{a}.rope.freq_base_swa", m.rope_base_swa),
            _kv_bools(f"{a}.attention.sliding_window_pattern", m.swa_pattern),
        ]
    plan = tensor_plan(m)
    infos, offset, sizes = [], 0, []
    for name, dims, typ in plan:
        n = int(np.prod(dims))
        nbytes = n * (4 if typ == GGML_F32 else 2)
        infos.append(_s(name) + struct.pack("<I", len(dims)) +
                     b"".join(struct.pack("<Q", d) for d in dims) +
                     struct.pack("<IQ", typ, offset))
        sizes.append((n, nbytes, offset))
        offset += (nbytes + ALIGN - 1) // ALIGN * ALIGN

    head = b"GGUF" + struct.pack("<IQQ", 3, len(plan), len(kvs)) + b"".join(kvs) + b"".join(infos)
    pad = (-len(head)) % ALIGN
    with open(path, "wb") as f:
        f.write(head + b"\0" * pad)
        base = f.tell()
        for i, ((name, dims, typ), (n, nbytes, off)) in enumerate(zip(plan, sizes)):
            assert f.tell() == base + off
            if typ == GGML_F32 and a == "gemma4":
                rng = np.random.Generator(np.random.PCG64([seed, 1000 + i]))
                data = (np.float32(1.0) + np.float32(0.1) *
                        rng.standard_normal(n, dtype=np.float32)).tobytes()
            elif typ == GGML_F32:
                data = np.ones(n, dtype=np.float32).tobytes()           # norm scales
            else:
                data = _weights(seed, i, n, std).tobytes()
            f.write(data)
            f.write(b"\0" * ((-nbytes) % ALIGN))


def _weights(seed: int, idx: int, n: int, std: float) -> np.ndarray:
    """N(0, std) float16 values for tensor number idx (PCG64 stream per tensor)."""
    rng = np.random.Generator(np.random.PCG64([seed, idx]))
    return (rng.standard_normal(n, dtype=np.float32) * np.float32(std)).astype(np.float16)
