"""ctypes access to the CPU oracle (``libwr_oracle.so``) and, when it has been
built, to the compiled reference (``_ref/libwayref.so``).

TEST INFRASTRUCTURE.  Only the test-suite, the smoke check and the CPU-baseline
leg of the benchmark import this package; the shipped library never does.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(_HERE, "libwr_oracle.so")
REF_SO = os.path.join(_HERE, "_ref", "libwayref.so")

WRO_OK, WRO_ERR_INVAL, WRO_ERR_NOMEM = 0, -4, -5
WRO_ERR_CTX_FULL, WRO_ERR_LIMIT, WRO_ERR_INTERNAL = -6, -8, -10
DTYPE_F32, DTYPE_F16 = 0, 1
GROWABLE = 1 << 1


HOSTCPU_SO = os.path.join(_HERE, "libwayruntime_cpuattn.so")


def build(ref: bool = True) -> None:
    """Compile the oracle, the host engine on the CPU test double, and the
    reference when its tree is present."""
    subprocess.check_call(["make", "-s", "-C", _HERE, "oracle", "hostcpu"] + (["ref"] if ref else []))


class Tensor(C.Structure):
    """Mirror of the tensor descriptor subset (wr_oracle.h: wro_tensor); the
    reference's wr_tensor has the same field order and types
    (src/core/internal.h:121-132), so the same class describes both."""
    _fields_ = [
        ("data", C.c_void_p),
        ("size_bytes", C.c_uint64),
        ("shape", C.c_uint32 * 8),
        ("ndim", C.c_uint8),
        ("dtype", C.c_uint8),
        ("flags", C.c_uint16),
        ("valid_rows", C.c_uint32),
    ]


def wrap(arr: np.ndarray, shape=None, flags: int = 0, valid_rows: int = 0) -> Tensor:
    """Describe a contiguous float32 / uint16(F16 bits) array as a tensor."""
    assert arr.flags["C_CONTIGUOUS"]
    if arr.dtype == np.float32:
        dt = DTYPE_F32
    elif arr.dtype == np.uint16:
        dt = DTYPE_F16
    else:
        raise TypeError(arr.dtype)
    shape = tuple(arr.shape if shape is None else shape)
    t = Tensor()
    t.data = arr.ctypes.data
    t.size_bytes = arr.nbytes
    for i, s in enumerate(shape):
        t.shape[i] = s
    t.ndim = len(shape)
    t.dtype = dt
    t.flags = flags
    t.valid_rows = valid_rows
    t._keep = arr
    return t


_f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
_u16p = np.ctypeslib.ndpointer(dtype=np.uint16, flags="C_CONTIGUOUS")
_u32p = np.ctypeslib.ndpointer(dtype=np.uint32, flags="C_CONTIGUOUS")


def _load_oracle() -> C.CDLL:
    if not os.path.exists(ORACLE_SO):
        build(ref=False)
    lib = C.CDLL(ORACLE_SO)
    for name in ("wro_exp", "wro_log", "wro_sqrt", "wro_sin", "wro_cos"):
        getattr(lib, name).restype = C.c_float
        getattr(lib, name).argtypes = [C.c_float]
    lib.wro_f16_to_f32.restype = C.c_float
    lib.wro_f16_to_f32.argtypes = [C.c_uint16]
    lib.wro_f32_to_f16.restype = C.c_uint16
    lib.wro_f32_to_f16.argtypes = [C.c_float]
    lib.wro_set_attn_max_seq.argtypes = [C.c_uint32]
    lib.wro_get_attn_max_seq.restype = C.c_uint32
    lib.wro_tensor_set_valid_rows.argtypes = [C.POINTER(Tensor), C.c_uint32]
    lib.wro_op_gqa_attention.argtypes = [C.POINTER(Tensor)] * 4 + [
        C.c_float, C.c_uint32, C.POINTER(C.c_uint64)]
    lib.wro_attention_f16kv.restype = None
    lib.wro_attention_f16kv.argtypes = [_f32p, _u16p, _u16p, _f32p] + [C.c_uint32] * 5 + [
        C.c_float, C.c_uint32]
    lib.wro_kv_append_row.argtypes = [C.POINTER(Tensor), _f32p, C.c_uint32, C.c_uint32]
    lib.wro_causal_prefill_rows.restype = None
    lib.wro_causal_prefill_rows.argtypes = [_f32p, _u16p, _u16p, _f32p] + [C.c_uint32] * 6 + [
        C.c_float, C.c_uint32]
    lib.wro_rope.argtypes = [_f32p] + [C.c_uint32] * 4 + [C.c_float, C.c_uint32]
    lib.wro_rope_table.argtypes = [_f32p] + [C.c_uint32] * 3 + [C.c_float, C.c_uint32]
    lib.wro_rope_table.restype = C.c_int
    lib.wro_matmul_w16.argtypes = [_f32p, _u16p, _f32p] + [C.c_uint32] * 3
    lib.wro_silu_mul.argtypes = [_f32p, _f32p, _f32p, C.c_uint64]
    lib.wro_rmsnorm.argtypes = [_f32p, C.c_void_p, C.c_uint32, _f32p, C.c_uint32, C.c_uint32,
                                C.c_float]
    return lib


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        _lib = _load_oracle()
    return _lib


# ----------------------------------------------------------------- helpers --

def exp(x: float) -> float:
    return lib().wro_exp(x)


def f32_to_f16(x: float) -> int:
    return lib().wro_f32_to_f16(x)


def f16_to_f32(h: int) -> float:
    return lib().wro_f16_to_f32(h)


def set_attn_max_seq(cap: int) -> None:
    lib().wro_set_attn_max_seq(cap)


def attention(q: np.ndarray, k16: np.ndarray, v16: np.ndarray, seq_k: int | None = None,
              scale_override: float = 0.0, window: int = 0) -> np.ndarray:
    """q [seq_q, nq, hd] float32; k16/v16 [rows, nkv, hd] uint16 F16 bits.
    Returns [seq_q, nq, hd] float32 (non-causal, as the reference op)."""
    seq_q, nq, hd = q.shape
    rows, nkv, hd2 = k16.shape
    assert hd2 == hd and v16.shape == k16.shape and nq % nkv == 0
    seq_k = rows if seq_k is None else seq_k
    assert 0 < seq_k <= rows
    out = np.empty_like(q)
    lib().wro_attention_f16kv(np.ascontiguousarray(q), np.ascontiguousarray(k16),
                              np.ascontiguousarray(v16), out, seq_q, nq, nkv, hd, seq_k,
                              scale_override, window)
    return out


def causal_prefill(q: np.ndarray, k16: np.ndarray, v16: np.ndarray, p0: int = 0,
                   scale_override: float = 0.0, window: int = 0, rows=None,
                   threads: int = 1) -> np.ndarray:
    """Row i of q [T, nq, hd] attends keys 0..p0+i of the cache.  ``rows``
    (iterable of row indices) limits the computation to a sample; other rows of
    the result are NaN.  ``threads`` > 1 spreads rows over a thread pool (the
    oracle is re-entrant and ctypes releases the GIL)."""
    T, nq, hd = q.shape
    nkv = k16.shape[1]
    assert k16.shape[0] >= p0 + T
    q = np.ascontiguousarray(q)
    k16 = np.ascontiguousarray(k16)
    v16 = np.ascontiguousarray(v16)
    out = np.full_like(q, np.nan)
    fn = lib().wro_causal_prefill_rows

    def run(lo, hi):
        fn(q, k16, v16, out, p0, lo, hi, nq, nkv, hd, scale_override, window)

    if rows is None:
        spans = [(0, T)]
        if threads > 1:
            # balance the triangular cost: split by equal area
            edges = [0]
            total = float((p0 + T) ** 2 - p0 ** 2)
            for j in range(1, threads * 4):
                want = p0 ** 2 + total * j / (threads * 4)
                edges.append(min(T, max(edges[-1], int(np.sqrt(want)) - p0)))
            edges.append(T)
            spans = [(a, b) for a, b in zip(edges[:-1], edges[1:]) if b > a]
    else:
        spans = [(int(r), int(r) + 1) for r in rows]
    if threads > 1 and len(spans) > 1:
        from concurrent.futures import ThreadPoolExecutor
        with ThreadPoolExecutor(threads) as ex:
            list(ex.map(lambda s: run(*s), spans))
    else:
        for s in spans:
            run(*s)
    return out


def rope(x: np.ndarray, pos: int, theta: float, n_rot_pairs: int = 0) -> np.ndarray:
    """x [seq, heads, hd] float32 -> rotated copy."""
    y = np.ascontiguousarray(x, dtype=np.float32).copy()
    rc = lib().wro_rope(y, y.shape[0], y.shape[1], y.shape[2], pos, theta, n_rot_pairs)
    if rc != 0:
        raise ValueError(rc)
    return y


def rope_table(seq: int, hd: int, pos: int, theta: float, n_rot_pairs: int = 0) -> np.ndarray:
    """(cos, sin) of the angles wro_rope uses: float32 [seq, n_rot, 2]."""
    buf = np.zeros((seq, hd // 2, 2), dtype=np.float32)
    n_rot = lib().wro_rope_table(buf, seq, hd, pos, theta, n_rot_pairs)
    if n_rot < 0:
        raise ValueError(n_rot)
    return np.ascontiguousarray(buf.reshape(-1)[: seq * n_rot * 2].reshape(seq, n_rot, 2))


def matmul_w16(x: np.ndarray, w16: np.ndarray) -> np.ndarray:
    """x [M, K] float32, w16 [N, K] F16 bit patterns -> x . W^T, float32 [M, N]."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    w16 = np.ascontiguousarray(w16, dtype=np.uint16)
    y = np.empty((x.shape[0], w16.shape[0]), dtype=np.float32)
    rc = lib().wro_matmul_w16(x, w16, y, x.shape[0], x.shape[1], w16.shape[0])
    if rc != 0:
        raise ValueError(rc)
    return y


def silu_mul(g: np.ndarray, u: np.ndarray) -> np.ndarray:
    g = np.ascontiguousarray(g, dtype=np.float32)
    u = np.ascontiguousarray(u, dtype=np.float32)
    out = np.empty_like(g)
    rc = lib().wro_silu_mul(g.reshape(-1), u.reshape(-1), out.reshape(-1), g.size)
    if rc != 0:
        raise ValueError(rc)
    return out


def rmsnorm(x: np.ndarray, w, eps: float) -> np.ndarray:
    """Rows of x (last axis = dim) normalised; w float32 [wn] or None."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    dim = x.shape[-1]
    rows = x.size // dim
    out = np.empty_like(x)
    if w is None:
        wp, wn = None, 0
    else:
        w = np.ascontiguousarray(w, dtype=np.float32)
        wp, wn = w.ctypes.data, w.size
    rc = lib().wro_rmsnorm(x.reshape(-1), wp, wn, out.reshape(-1), rows, dim, eps)
    if rc != 0:
        raise ValueError(rc)
    return out


# --------------------------------------------------------------- reference --

def have_ref() -> bool:
    return os.path.exists(REF_SO)


_ref = None


def ref() -> C.CDLL:
    """The compiled reference (only where ``oracle/_ref`` has been built)."""
    global _ref
    if _ref is None:
        r = C.CDLL(REF_SO)
        for name in ("wri_exp", "wri_log", "wri_sqrt", "wri_sin", "wri_cos"):
            getattr(r, name).restype = C.c_float
            getattr(r, name).argtypes = [C.c_float]
        r.wri_f16_to_f32.restype = C.c_float
        r.wri_f16_to_f32.argtypes = [C.c_uint16]
        r.wri_f32_to_f16.restype = C.c_uint16
        r.wri_f32_to_f16.argtypes = [C.c_float]
        r.wri_op_gqa_attention.argtypes = [C.POINTER(Tensor)] * 4 + [C.c_float, C.c_uint32]
        r.wri_op_rope.argtypes = [C.POINTER(Tensor), C.POINTER(Tensor), C.c_uint32,
                                  C.c_float, C.c_uint32]
        _ref = r
    return _ref


def ref_attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, seq_k: int | None = None,
                  scale_override: float = 0.0, window: int = 0):
    """Run the compiled reference op.  k/v may be uint16 (F16) or float32."""
    out = np.empty_like(q)
    flags = GROWABLE if seq_k is not None else 0
    tq, tk, tv, tc = wrap(q), wrap(k, flags=flags, valid_rows=seq_k or 0), \
        wrap(v, flags=flags, valid_rows=seq_k or 0), wrap(out)
    rc = ref().wri_op_gqa_attention(C.byref(tq), C.byref(tk), C.byref(tv), C.byref(tc),
                                    scale_override, window)
    return rc, out
