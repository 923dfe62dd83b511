"""ctypes binding of the C ABI in ``include/wr_hip_attn.h`` — used by the tests
and the benchmark.  The product is the shared library; this module only passes
numpy buffers through.  There is no fallback: if the library is missing or
no gfx950 device is present, loading / ``init`` raises.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

PKG = os.path.dirname(os.path.abspath(__file__))
HIP_SO = os.environ.get("WR_HIP_ATTN_LIB") or os.path.join(PKG, "libwr_hip_attn.so")

OK = 0
ERR_UNSUPPORTED, ERR_INVAL, ERR_NOMEM, ERR_CTX_FULL = -3, -4, -5, -6
ERR_STATE, ERR_LIMIT, ERR_INTERNAL = -7, -8, -10
QKV_V_NORM, QKV_Q_ONLY = 1, 2          # flags of wr_hip_rows_qkv_append_dev
ATTN_MAX_SEQ = 131072
BATCH_MAX = 16

_vp = C.c_void_p
_u32 = C.c_uint32
_f32p = C.POINTER(C.c_float)


class HipAttnError(RuntimeError):
    def __init__(self, rc: int, what: str):
        super().__init__(f"{what} failed with wr_status {rc}")
        self.rc = rc


def load() -> C.CDLL:
    if not os.path.exists(HIP_SO):
        raise FileNotFoundError(
            f"{HIP_SO} is not built (run `python -m wayruntime_amd.build`); there is no CPU path")
    lib = C.CDLL(HIP_SO)
    sig = {
        "wr_hip_attn_init": (C.c_int, [C.c_int]),
        "wr_hip_attn_shutdown": (None, []),
        "wr_hip_attn_calls": (C.c_uint64, []),
        "wr_hip_attn_device_name": (C.c_char_p, []),
        "wr_hip_attn_caps": (_u32, []),
        "wr_hip_attn_kv_create": (C.c_int, [_u32, C.POINTER(_u32), _u32, _u32, C.POINTER(_vp)]),
        "wr_hip_attn_kv_destroy": (None, [_vp]),
        "wr_hip_attn_kv_bytes": (C.c_uint64, [_vp]),
        "wr_hip_attn_append": (C.c_int, [_vp, _u32, _u32, _u32, _vp, _vp]),
        "wr_hip_attn_kv_read": (C.c_int, [_vp, _u32, _u32, _u32, _vp, _vp]),
        "wr_hip_attn_kv_write": (C.c_int, [_vp, _u32, _u32, _u32, _vp, _vp]),
        "wr_hip_attn_decode": (C.c_int, [_vp, _u32, _u32, _vp, _vp, _u32, C.c_float, _u32]),
        "wr_hip_attn_decode_batched": (C.c_int, [_u32, C.POINTER(_vp), _u32, C.POINTER(_u32),
                                                 C.POINTER(_vp), C.POINTER(_vp), _u32, C.c_float,
                                                 _u32]),
        "wr_hip_attn_prefill": (C.c_int, [_vp, _u32, _u32, _u32, _vp, _vp, _u32, C.c_float, _u32]),
        "wr_hip_attn_append_decode": (C.c_int, [_vp, _u32, _u32, _vp, _vp, _vp, _vp, _u32, C.c_float,
                                                _u32]),
        "wr_hip_attn_append_decode_batched": (C.c_int, [_u32, C.POINTER(_vp), _u32, C.POINTER(_u32),
                                                        C.POINTER(_vp), C.POINTER(_vp),
                                                        C.POINTER(_vp), C.POINTER(_vp), _u32,
                                                        C.c_float, _u32]),
        "wr_hip_attn_dev_alloc": (_vp, [C.c_size_t]),
        "wr_hip_attn_dev_free": (None, [_vp]),
        "wr_hip_attn_h2d": (C.c_int, [_vp, _vp, C.c_size_t]),
        "wr_hip_attn_d2h": (C.c_int, [_vp, _vp, C.c_size_t]),
        "wr_hip_attn_sync": (C.c_int, []),
        "wr_hip_attn_stream": (_vp, []),
        "wr_hip_attn_append_dev": (C.c_int, [_vp, _u32, _u32, _u32, _vp, _vp]),
        "wr_hip_attn_append_batched_dev": (C.c_int, [_u32, C.POINTER(_vp), _u32, C.POINTER(_u32),
                                                     _vp, _vp]),
        "wr_hip_attn_append_rope": (C.c_int, [_vp, _u32, _u32, _u32, _vp, _vp, _vp, _u32]),
        "wr_hip_attn_rope_dev": (C.c_int, [_vp, _vp, _u32, _u32, _u32, _u32]),
        "wr_hip_attn_rope_table_dev": (C.c_int, [_vp, _u32, _u32, C.POINTER(_u32), _u32, C.c_float,
                                                 _u32]),
        "wr_hip_attn_decode_batched_dev": (C.c_int, [_u32, C.POINTER(_vp), _u32, C.POINTER(_u32),
                                                     _vp, _vp, _u32, C.c_float, _u32]),
        "wr_hip_attn_decode_batched_dev_noalloc": (C.c_int, [_u32, C.POINTER(_vp), _u32,
                                                             C.POINTER(_u32), _vp, _vp, _u32,
                                                             C.c_float, _u32]),
        "wr_hip_attn_append_decode_batched_dev": (C.c_int, [_u32, C.POINTER(_vp), _u32, C.POINTER(_u32),
                                                            _vp, _u32, _u32, _vp, _vp, C.c_float, _vp,
                                                            _u32, _vp, C.c_float, _u32]),
        "wr_hip_attn_prefill_dev": (C.c_int, [_vp, _u32, _u32, _u32, _vp, _vp, _u32, C.c_float,
                                              _u32]),
        "wr_hip_proj_weight_create": (C.c_int, [_u32, C.POINTER(_vp), C.POINTER(_u32), _u32,
                                                C.POINTER(_vp)]),
        "wr_hip_proj_weight_destroy": (None, [_vp]),
        "wr_hip_proj_weight_rows": (_u32, [_vp]),
        "wr_hip_proj_weight_cols": (_u32, [_vp]),
        "wr_hip_proj_rows": (C.c_int, [_vp, _u32, _vp, _vp]),
        "wr_hip_proj_rows_dev": (C.c_int, [_vp, _u32, _vp, _u32, _vp, _vp, _u32]),
        "wr_hip_proj_rows_norm_dev": (C.c_int, [_vp, _u32, _vp, _u32, _vp, C.c_float, _vp, _vp, _u32]),
        "wr_hip_proj_rows_swiglu_dev": (C.c_int, [_vp, _u32, _vp, _u32, _vp, _vp, _u32]),
        "wr_hip_rows_rmsnorm_dev": (C.c_int, [_vp, _u32, _vp, _u32, _vp, _u32, _u32, _u32, C.c_float]),
        "wr_hip_rows_qkv_prep_dev": (C.c_int, [_vp, _u32, _u32, _u32, _u32, _u32, _vp, _vp, C.c_float,
                                               _vp, _u32, _vp, _vp, _vp]),
        "wr_hip_rows_qkv_append_dev": (C.c_int, [_vp, _u32, _u32, _u32, _vp, _vp, C.c_float, _vp, _u32, _u32,
                                                 C.POINTER(_vp), _u32, C.POINTER(_u32), _vp, _u32]),
        "wr_hip_rows_qkv_append_q16_dev": (C.c_int, [_vp, _u32, _u32, _u32, _vp, _vp, C.c_float, _vp, _u32, _u32,
                                                     C.POINTER(_vp), _u32, C.POINTER(_u32), _vp, C.c_float, _u32]),
        "wr_hip_attn_prefill_q16_dev": (C.c_int, [_vp, _u32, _u32, _u32, _vp, _vp, _u32, C.c_float, _u32]),
        "wr_hip_rows_rmsnorm_add_dev": (C.c_int, [_vp, _u32, _vp, _u32, _vp, _u32, _u32, _u32, C.c_float]),
        "wr_hip_proj_rows_geglu_dev": (C.c_int, [_vp, _u32, _vp, _u32, _vp, _vp, _u32]),
        "wr_hip_rows_swiglu_dev": (C.c_int, [_vp, _u32, _vp, _u32, _u32, _u32]),
        "wr_hip_attn_host_alloc": (_vp, [C.c_size_t]),
        "wr_hip_attn_host_free": (None, [_vp]),
        "wr_hip_attn_set_tuning": (None, [_u32, C.c_int]),
        "wr_hip_attn_set_prefill_one_wave": (None, [C.c_int]),
        "wr_hip_attn_profile_begin": (C.c_int, [_u32]),
        "wr_hip_attn_profile_end": (C.c_int, [C.POINTER(C.c_double), C.POINTER(_u32)]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


_lib = None
_inited = False


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        _lib = load()
    return _lib


def init(device: int = 0) -> None:
    """Initialise once per process (idempotent for this module)."""
    global _inited
    if _inited:
        return
    rc = lib().wr_hip_attn_init(device)
    if rc != OK:
        raise HipAttnError(rc, "wr_hip_attn_init")
    _inited = True


def shutdown() -> None:
    global _inited
    if _inited:
        lib().wr_hip_attn_shutdown()
        _inited = False


def _check(rc: int, what: str) -> None:
    if rc != OK:
        raise HipAttnError(rc, what)


def _ptr(a: np.ndarray) -> int:
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data


class KVCache:
    """One session's device cache (wr_hip_kv)."""

    def __init__(self, n_layers: int, hd, nkv: int, max_ctx: int):
        init()
        hds = [hd] * n_layers if isinstance(hd, int) else list(hd)
        assert len(hds) == n_layers
        self.n_layers, self.hd, self.nkv, self.max_ctx = n_layers, hds, nkv, max_ctx
        arr = (_u32 * n_layers)(*hds)
        h = _vp()
        _check(lib().wr_hip_attn_kv_create(n_layers, arr, nkv, max_ctx, C.byref(h)), "kv_create")
        self.h = h

    def close(self) -> None:
        if getattr(self, "h", None):
            lib().wr_hip_attn_kv_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def bytes(self) -> int:
        return lib().wr_hip_attn_kv_bytes(self.h)

    # ---- host-pointer entry points -------------------------------------
    def append(self, layer: int, pos: int, k: np.ndarray, v: np.ndarray) -> int:
        """k, v float32 [n_rows, nkv, hd]; returns the wr_status."""
        k = np.ascontiguousarray(k, dtype=np.float32)
        v = np.ascontiguousarray(v, dtype=np.float32)
        assert k.shape == v.shape
        return lib().wr_hip_attn_append(self.h, layer, pos, k.shape[0], _ptr(k), _ptr(v))

    def append_rope(self, layer: int, pos: int, k: np.ndarray, v: np.ndarray,
                    cos_sin: np.ndarray) -> int:
        """k (before rotation), v float32 [n_rows, nkv, hd]; cos_sin float32
        [n_rows, n_rot, 2]; returns the wr_status."""
        k = np.ascontiguousarray(k, dtype=np.float32)
        v = np.ascontiguousarray(v, dtype=np.float32)
        cs = np.ascontiguousarray(cos_sin, dtype=np.float32)
        assert k.shape == v.shape and cs.shape[0] == k.shape[0] and cs.shape[2] == 2
        return lib().wr_hip_attn_append_rope(self.h, layer, pos, k.shape[0], _ptr(k), _ptr(v),
                                             _ptr(cs), cs.shape[1])

    def write_f16(self, layer: int, pos: int, k16: np.ndarray, v16: np.ndarray,
                  chunk_rows: int = 8192) -> None:
        k16 = np.ascontiguousarray(k16, dtype=np.uint16)
        v16 = np.ascontiguousarray(v16, dtype=np.uint16)
        for lo in range(0, k16.shape[0], chunk_rows):
            hi = min(k16.shape[0], lo + chunk_rows)
            _check(lib().wr_hip_attn_kv_write(self.h, layer, pos + lo, hi - lo,
                                              _ptr(k16[lo:hi]), _ptr(v16[lo:hi])), "kv_write")

    def read_f16(self, layer: int, pos: int, n_rows: int):
        shape = (n_rows, self.nkv, self.hd[layer])
        k = np.empty(shape, dtype=np.uint16)
        v = np.empty(shape, dtype=np.uint16)
        _check(lib().wr_hip_attn_kv_read(self.h, layer, pos, n_rows, _ptr(k), _ptr(v)), "kv_read")
        return k, v

    def decode(self, layer: int, seq_k: int, q: np.ndarray, scale_override: float = 0.0,
               window: int = 0) -> np.ndarray:
        """q float32 [nq, hd] -> float32 [nq, hd]."""
        q = np.ascontiguousarray(q, dtype=np.float32)
        out = np.empty_like(q)
        _check(lib().wr_hip_attn_decode(self.h, layer, seq_k, _ptr(q), _ptr(out), q.shape[0],
                                        scale_override, window), "decode")
        return out

    def append_decode(self, layer: int, pos: int, k: np.ndarray, v: np.ndarray, q: np.ndarray,
                      scale_override: float = 0.0, window: int = 0) -> np.ndarray:
        """Row k, v float32 [nkv, hd] stored at pos, then q float32 [nq, hd] attends keys
        0 .. pos: append + decode in one call."""
        k = np.ascontiguousarray(k, dtype=np.float32)
        v = np.ascontiguousarray(v, dtype=np.float32)
        q = np.ascontiguousarray(q, dtype=np.float32)
        out = np.empty_like(q)
        _check(lib().wr_hip_attn_append_decode(self.h, layer, pos, _ptr(k), _ptr(v), _ptr(q),
                                               _ptr(out), q.shape[0], scale_override, window),
               "append_decode")
        return out

    def prefill(self, layer: int, p0: int, q: np.ndarray, scale_override: float = 0.0,
                window: int = 0) -> np.ndarray:
        """q float32 [T, nq, hd] -> float32 [T, nq, hd]."""
        q = np.ascontiguousarray(q, dtype=np.float32)
        out = np.empty_like(q)
        _check(lib().wr_hip_attn_prefill(self.h, layer, p0, q.shape[0], _ptr(q), _ptr(out),
                                         q.shape[1], scale_override, window), "prefill")
        return out


def decode_batched(caches, layer: int, seq_k, qs, scale_override: float = 0.0, window: int = 0):
    """qs: list of float32 [nq, hd]; returns list of outputs."""
    n = len(caches)
    qs = [np.ascontiguousarray(q, dtype=np.float32) for q in qs]
    outs = [np.empty_like(q) for q in qs]
    kvp = (_vp * n)(*[c.h for c in caches])
    sk = (_u32 * n)(*[int(s) for s in seq_k])
    qp = (_vp * n)(*[_ptr(q) for q in qs])
    op = (_vp * n)(*[_ptr(o) for o in outs])
    _check(lib().wr_hip_attn_decode_batched(n, kvp, layer, sk, qp, op, qs[0].shape[0],
                                            scale_override, window), "decode_batched")
    return outs


def append_decode_batched(caches, layer: int, pos, ks, vs, qs, scale_override: float = 0.0,
                          window: int = 0):
    """Session i's row ks[i], vs[i] stored at pos[i], then qs[i] attends keys 0 .. pos[i];
    returns the list of outputs."""
    n = len(caches)
    ks = [np.ascontiguousarray(a, dtype=np.float32) for a in ks]
    vs = [np.ascontiguousarray(a, dtype=np.float32) for a in vs]
    qs = [np.ascontiguousarray(a, dtype=np.float32) for a in qs]
    outs = [np.empty_like(q) for q in qs]
    kvp = (_vp * n)(*[c.h for c in caches])
    pp = (_u32 * n)(*[int(p) for p in pos])

    def arr(xs):
        return (_vp * n)(*[_ptr(x) for x in xs])

    _check(lib().wr_hip_attn_append_decode_batched(n, kvp, layer, pp, arr(ks), arr(vs), arr(qs),
                                                   arr(outs), qs[0].shape[0], scale_override,
                                                   window), "append_decode_batched")
    return outs


class DeviceBuffer:
    """Device memory owned through the library's allocator."""

    def __init__(self, nbytes: int):
        init()
        self.nbytes = nbytes
        self.p = lib().wr_hip_attn_dev_alloc(nbytes)
        if not self.p:
            raise HipAttnError(ERR_NOMEM, "dev_alloc")

    @classmethod
    def from_host(cls, a: np.ndarray) -> "DeviceBuffer":
        a = np.ascontiguousarray(a)
        b = cls(a.nbytes)
        _check(lib().wr_hip_attn_h2d(b.p, _ptr(a), a.nbytes), "h2d")
        return b

    def to_host(self, shape, dtype=np.float32) -> np.ndarray:
        out = np.empty(shape, dtype=dtype)
        assert out.nbytes <= self.nbytes
        _check(lib().wr_hip_attn_d2h(_ptr(out), self.p, out.nbytes), "d2h")
        return out

    def free(self) -> None:
        if self.p:
            lib().wr_hip_attn_dev_free(self.p)
            self.p = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def decode_batched_dev(caches, layer: int, seq_k, q_dev: DeviceBuffer, out_dev: DeviceBuffer,
                       nq: int, scale_override: float = 0.0, window: int = 0) -> None:
    n = len(caches)
    kvp = (_vp * n)(*[c.h for c in caches])
    sk = (_u32 * n)(*[int(s) for s in seq_k])
    _check(lib().wr_hip_attn_decode_batched_dev(n, kvp, layer, sk, q_dev.p, out_dev.p, nq,
                                                scale_override, window), "decode_batched_dev")


def decode_batched_dev_noalloc(caches, layer: int, seq_k, q_dev: DeviceBuffer,
                               out_dev: DeviceBuffer, nq: int, scale_override: float = 0.0,
                               window: int = 0) -> int:
    """The form that allocates nothing; returns the wr_status."""
    n = len(caches)
    kvp = (_vp * n)(*[c.h for c in caches])
    sk = (_u32 * n)(*[int(s) for s in seq_k])
    return lib().wr_hip_attn_decode_batched_dev_noalloc(n, kvp, layer, sk, q_dev.p, out_dev.p, nq,
                                                        scale_override, window)


def prefill_dev(cache: KVCache, layer: int, p0: int, T: int, q_dev: DeviceBuffer,
                out_dev: DeviceBuffer, nq: int, scale_override: float = 0.0,
                window: int = 0) -> None:
    _check(lib().wr_hip_attn_prefill_dev(cache.h, layer, p0, T, q_dev.p, out_dev.p, nq,
                                         scale_override, window), "prefill_dev")


def append_dev(cache: KVCache, layer: int, pos: int, n_rows: int, k_dev: DeviceBuffer,
               v_dev: DeviceBuffer) -> None:
    _check(lib().wr_hip_attn_append_dev(cache.h, layer, pos, n_rows, k_dev.p, v_dev.p),
           "append_dev")


def rope_dev(x_dev: DeviceBuffer, cos_sin_dev: DeviceBuffer, rows: int, heads: int, hd: int,
             n_rot: int) -> None:
    _check(lib().wr_hip_attn_rope_dev(x_dev.p, cos_sin_dev.p, rows, heads, hd, n_rot), "rope_dev")


def rope_table_dev(rows: int, hd: int, theta: float, n_rot_pairs: int = 0, pos0: int = 0,
                   pos=None) -> np.ndarray:
    """The rotary table made on the device (wr_hip_attn_rope_table_dev), brought
    down: float32 [rows, n_rot, 2] of (cos, sin) for positions pos0 + r, or the
    listed ones."""
    n_rot = n_rot_pairs if 1 <= n_rot_pairs < hd // 2 else hd // 2
    buf = DeviceBuffer(rows * n_rot * 8)
    try:
        plist = None
        if pos is not None:
            plist = (_u32 * len(pos))(*[int(p) for p in pos])
        _check(lib().wr_hip_attn_rope_table_dev(buf.p, rows, pos0, plist, hd, theta, n_rot_pairs),
               "rope_table_dev")
        return buf.to_host((rows, n_rot, 2))
    finally:
        buf.free()


class Weight:
    """A projection weight on the device (wr_hip_weight): row blocks of F16 bit
    patterns [rows_i, n_in], stacked in order."""

    def __init__(self, parts):
        init()
        parts = [np.ascontiguousarray(p, dtype=np.uint16) for p in parts]
        n_in = parts[0].shape[1]
        assert all(p.ndim == 2 and p.shape[1] == n_in for p in parts)
        ptrs = (_vp * len(parts))(*[_ptr(p) for p in parts])
        rows = (_u32 * len(parts))(*[p.shape[0] for p in parts])
        self.h = _vp()
        _check(lib().wr_hip_proj_weight_create(len(parts), ptrs, rows, n_in, C.byref(self.h)),
               "proj_weight_create")
        self.n_out = int(lib().wr_hip_proj_weight_rows(self.h))
        self.n_in = int(lib().wr_hip_proj_weight_cols(self.h))

    def rows(self, x: np.ndarray) -> np.ndarray:
        """y = x . W^T for host F32 rows [R, n_in]."""
        x = np.ascontiguousarray(x, dtype=np.float32)
        y = np.empty((x.shape[0], self.n_out), dtype=np.float32)
        _check(lib().wr_hip_proj_rows(self.h, x.shape[0], _ptr(x), _ptr(y)), "proj_rows")
        return y

    def rows_dev(self, rows: int, x_dev, ldx: int, y_dev, ldy: int, add_dev=None) -> None:
        _check(lib().wr_hip_proj_rows_dev(self.h, rows, x_dev.p, ldx,
                                          add_dev.p if add_dev is not None else None, y_dev.p, ldy),
               "proj_rows_dev")

    def close(self) -> None:
        if self.h:
            lib().wr_hip_proj_weight_destroy(self.h)
            self.h = _vp()


def sync() -> None:
    _check(lib().wr_hip_attn_sync(), "sync")


def set_tuning(decode_keys_per_wg: int = 0, force_generic: bool = False) -> None:
    lib().wr_hip_attn_set_tuning(decode_keys_per_wg, 1 if force_generic else 0)


def set_prefill_one_wave(on: bool) -> None:
    lib().wr_hip_attn_set_prefill_one_wave(1 if on else 0)


def profile_begin(max_launches: int) -> None:
    _check(lib().wr_hip_attn_profile_begin(max_launches), "profile_begin")


def profile_end():
    ms = C.c_double(0.0)
    n = _u32(0)
    _check(lib().wr_hip_attn_profile_end(C.byref(ms), C.byref(n)), "profile_end")
    return ms.value, n.value


def device_name() -> str:
    return lib().wr_hip_attn_device_name().decode()
