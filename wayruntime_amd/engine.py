"""ctypes binding of the host engine's wr_* API (engine, model, session,
prefill, step, batched step) — used by the tests and the end-to-end runs.

``Engine(lib_path)`` loads either the shipped library
(``wayruntime_amd/libwayruntime_amd.so``, attention on the device) or, for
CPU-only tests of the host logic, the test build that links the CPU test double
(``oracle/libwayruntime_cpuattn.so``).  The default is always the device
library; nothing falls back silently.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

PKG = os.path.dirname(os.path.abspath(__file__))
HOST_SO = os.path.join(PKG, "libwayruntime_amd.so")

WR_OK, WR_ERR_IO, WR_ERR_FORMAT, WR_ERR_UNSUPPORTED, WR_ERR_INVAL = 0, -1, -2, -3, -4
WR_ERR_NOMEM, WR_ERR_CTX_FULL, WR_ERR_STATE, WR_ERR_LIMIT = -5, -6, -7, -8
WR_ERR_BUSY, WR_ERR_INTERNAL = -9, -10
WR_BATCH_MAX = 16
WR_SWA_ENABLED, WR_SWA_DISABLED = 0, 1
WR_CTR_ATTENTION_CALLS = 3


class ModelParams(C.Structure):
    _fields_ = [("max_context", C.c_uint32), ("keep_quantized", C.c_int32),
                ("swa_mode", C.c_int32), ("use_mmap", C.c_int32)]


class SessionParams(C.Structure):
    _fields_ = [("max_context", C.c_uint32)]


class ModelInfo(C.Structure):
    _fields_ = ([("arch", C.c_char * 32), ("quant", C.c_char * 16)] +
                [(n, C.c_uint32) for n in ("n_layers", "n_q_heads", "n_kv_heads", "head_dim",
                                           "head_dim_swa", "hidden_dim", "ffn_dim", "vocab_size",
                                           "train_context", "max_context")] +
                [("rope_freq_base", C.c_float), ("rms_eps", C.c_float),
                 ("logit_softcap", C.c_float), ("sliding_window", C.c_uint32),
                 ("is_gemma", C.c_uint8), ("has_qk_norm", C.c_uint8),
                 ("tied_lm_head", C.c_uint8), ("has_swa", C.c_uint8)])


class EngineError(RuntimeError):
    def __init__(self, rc, what):
        super().__init__(f"{what} failed with wr_status {rc}")
        self.rc = rc


def _bind(lib):
    vp, u32 = C.c_void_p, C.c_uint32
    lib.wr_engine_create.argtypes = [vp, C.POINTER(vp)]
    lib.wr_engine_destroy.argtypes = [vp]
    lib.wr_engine_destroy.restype = None
    lib.wr_engine_counters.argtypes = [vp, C.POINTER(C.c_uint64)]
    lib.wr_model_load.argtypes = [vp, C.c_char_p, C.POINTER(ModelParams), C.POINTER(vp)]
    lib.wr_model_free.argtypes = [vp]
    lib.wr_model_free.restype = None
    lib.wr_model_get_info.argtypes = [vp, C.POINTER(ModelInfo)]
    lib.wr_session_create.argtypes = [vp, C.POINTER(SessionParams), C.POINTER(vp)]
    lib.wr_session_destroy.argtypes = [vp]
    lib.wr_session_destroy.restype = None
    lib.wr_prefill.argtypes = [vp, C.POINTER(u32), u32]
    lib.wr_step.argtypes = [vp, u32]
    lib.wr_step.restype = C.POINTER(C.c_float)
    lib.wr_batch_step.argtypes = [C.POINTER(vp), C.POINTER(u32), u32, C.POINTER(C.POINTER(C.c_float))]
    lib.wr_session_pos.argtypes = [vp]
    lib.wr_session_pos.restype = u32
    lib.wr_session_max_context.argtypes = [vp]
    lib.wr_session_max_context.restype = u32
    lib.wr_session_status.argtypes = [vp]
    lib.wr_status_str.argtypes = [C.c_int]
    lib.wr_status_str.restype = C.c_char_p
    lib.wr_version.restype = C.c_char_p
    lib.wrh_debug_fail_attention_at.argtypes = [C.c_int]
    lib.wrh_debug_fail_attention_at.restype = None
    return lib


class Engine:
    def __init__(self, lib_path: str = HOST_SO, threads: int = 0):
        if not os.path.exists(lib_path):
            raise FileNotFoundError(f"{lib_path} is not built")
        self.lib = _bind(C.CDLL(lib_path, mode=C.RTLD_GLOBAL))
        self.h = C.c_void_p()
        cfg = (C.c_uint32 * 8)()            # wr_engine_config, zeroed; n_threads first
        cfg[0] = threads
        rc = self.lib.wr_engine_create(C.cast(cfg, C.c_void_p), C.byref(self.h))
        if rc != WR_OK:
            raise EngineError(rc, "wr_engine_create")

    def close(self):
        if self.h:
            self.lib.wr_engine_destroy(self.h)
            self.h = None

    def counters(self):
        out = (C.c_uint64 * 12)()
        assert self.lib.wr_engine_counters(self.h, out) == WR_OK
        return list(out)

    def load(self, path: str, max_context: int = 0, swa_mode: int = WR_SWA_ENABLED) -> "Model":
        return Model(self, path, max_context, swa_mode)


class Model:
    def __init__(self, eng: Engine, path: str, max_context: int = 0, swa_mode: int = WR_SWA_ENABLED):
        self.eng, self.lib = eng, eng.lib
        self.h = C.c_void_p()
        p = ModelParams(max_context, 0, swa_mode, 0)
        rc = self.lib.wr_model_load(eng.h, path.encode(), C.byref(p), C.byref(self.h))
        if rc != WR_OK:
            raise EngineError(rc, "wr_model_load")
        self.info = ModelInfo()
        assert self.lib.wr_model_get_info(self.h, C.byref(self.info)) == WR_OK
        self.vocab = self.info.vocab_size

    def close(self):
        if self.h:
            self.lib.wr_model_free(self.h)
            self.h = None

    def session(self, max_context: int = 0) -> "Session":
        return Session(self, max_context)


class Session:
    def __init__(self, model: Model, max_context: int = 0):
        self.model, self.lib = model, model.lib
        self.h = C.c_void_p()
        sp = SessionParams(max_context)
        rc = self.lib.wr_session_create(model.h, C.byref(sp), C.byref(self.h))
        if rc != WR_OK:
            raise EngineError(rc, "wr_session_create")

    def close(self):
        if self.h:
            self.lib.wr_session_destroy(self.h)
            self.h = None

    @property
    def pos(self) -> int:
        return self.lib.wr_session_pos(self.h)

    @property
    def status(self) -> int:
        return self.lib.wr_session_status(self.h)

    def prefill(self, ids) -> int:
        ids = [int(t) for t in ids]
        arr = (C.c_uint32 * max(len(ids), 1))(*ids)
        return self.lib.wr_prefill(self.h, arr, len(ids))

    def step(self, token: int):
        """Logits as a numpy COPY, or None on error (see .status)."""
        p = self.lib.wr_step(self.h, int(token))
        if not p:
            return None
        return np.ctypeslib.as_array(p, shape=(self.model.vocab,)).copy()


def batch_step(sessions, tokens):
    """Returns (rc, [logits copies])."""
    lib = sessions[0].lib
    n = len(sessions)
    hs = (C.c_void_p * n)(*[s.h for s in sessions])
    toks = (C.c_uint32 * n)(*[int(t) for t in tokens])
    outs = (C.POINTER(C.c_float) * n)()
    rc = lib.wr_batch_step(hs, toks, n, outs)
    if rc < 0:
        return rc, None
    v = sessions[0].model.vocab
    return rc, [np.ctypeslib.as_array(outs[i], shape=(v,)).copy() for i in range(n)]
