"""The reference's own attention self-test fixtures, run on the device path
through the C ABI.

Sources: wri_self_test_flash_attn cases (a)-(d), src/core/kernels.c:1907-2036
(literal Q, closed-form K/V fills, scale override 0.25, sliding window 4, and a
GROWABLE cache read at valid_rows 64 / 256 / 1024 / 4096), and ops_test_gqa,
src/core/kernels.c:2185-2208 (head mapping, exact).  The reference checks its
op against a materialised softmax at 1e-4 (kernels.c:1941-1946); the same bound
is used here.  Each seq_q = 2 fixture is two decode calls.  The device cache
holds binary16, as the reference's session cache does, so the expected values
are computed over the truncated K/V the cache holds (bits checked first)."""
import numpy as np
import pytest

from tests import util
from wayruntime_amd import hipattn, synth

pytestmark = pytest.mark.gpu

TOL = 1e-4            # src/core/kernels.c:1941-1946


@pytest.fixture(scope="module", autouse=True)
def _device():
    hipattn.init()
    yield


def _materialised_f64(q, k, v, scale, key_lo=0):
    """Textbook softmax attention in float64, one KV head: q [rows, d], k, v [keys, d]."""
    s = (q.astype(np.float64) @ k.astype(np.float64).T) * scale
    s[:, :key_lo] = -np.inf
    s -= s.max(axis=1, keepdims=True)
    p = np.exp(s)
    p /= p.sum(axis=1, keepdims=True)
    return p @ v.astype(np.float64)


def _f16_values(bits):
    return bits.view(np.float16).astype(np.float32)


def _cache_with(k32, v32):
    rows, nkv, hd = k32.shape
    kv = hipattn.KVCache(1, hd, nkv, rows)
    assert kv.append(0, 0, k32, v32) == hipattn.OK
    k16, v16 = synth.f32_to_f16_trunc(k32), synth.f32_to_f16_trunc(v32)
    gk, gv = kv.read_f16(0, 0, rows)
    assert np.array_equal(gk, k16) and np.array_equal(gv, v16)
    return kv, k16, v16


def test_flash_attn_fixture_small_default_scale_override_window():
    # kernels.c:1909-1974: SQ = 2, SK = 8, D = 4
    q = np.array([[0.1, 0.2, 0.3, 0.4], [0.5, 0.6, 0.7, 0.8]], dtype=np.float32).reshape(2, 1, 4)
    i = np.arange(32)
    k = (((i * 7 + 3) % 13).astype(np.float32) * np.float32(0.1)).reshape(8, 1, 4)
    v = (((i * 5 + 1) % 11).astype(np.float32) * np.float32(0.1)).reshape(8, 1, 4)
    kv, k16, v16 = _cache_with(k, v)
    kf, vf = _f16_values(k16)[:, 0], _f16_values(v16)[:, 0]
    for sc, win in ((0.0, 0), (0.25, 0), (0.0, 4)):
        print("fixture small: scale_override", sc, "window", win, flush=True)
        scale = sc if sc > 0 else 0.5                     # 1 / sqrt(4)
        want = _materialised_f64(q[:, 0], kf, vf, scale, key_lo=(8 - win) if win else 0)
        for row in range(2):
            got = kv.decode(0, 8, q[row], sc, win)
            assert np.max(np.abs(got[0] - want[row])) < TOL, (sc, win, row)
            oracle_row = util.oracle_decode(q[row], k16, v16, 8, sc, win)
            assert np.max(np.abs(got - oracle_row)) < TOL
    kv.close()


def test_flash_attn_fixture_long_growable_cursor():
    # kernels.c:1979-2036: LQ = 2, LD = 8, integer-hash fills, the cursor at
    # 64 / 256 / 1024 / 4096 of a cache that holds 4096 rows
    LQ, LD, SK_MAX = 2, 8, 4096
    qi = np.arange(LQ * LD)
    q = (((qi * 11 + 3) % 17).astype(np.float32) * np.float32(0.05)).reshape(LQ, 1, LD)
    with np.errstate(over="ignore"):
        s = np.arange(SK_MAX * LD, dtype=np.uint32) * np.uint32(2654435761) + np.uint32(0x9E3779B9)
    k = (((s & 0xFFFF).astype(np.int32).astype(np.float32) / np.float32(32768.0) - np.float32(1.0))
         * np.float32(0.3)).reshape(SK_MAX, 1, LD)
    v = ((((s >> 16) & 0xFFFF).astype(np.int32).astype(np.float32) / np.float32(32768.0)
          - np.float32(1.0)) * np.float32(0.3)).reshape(SK_MAX, 1, LD)
    kv, k16, v16 = _cache_with(k, v)
    kf, vf = _f16_values(k16)[:, 0], _f16_values(v16)[:, 0]
    for sk in (64, 256, 1024, 4096):
        print("fixture long: valid_rows", sk, flush=True)
        want = _materialised_f64(q[:, 0], kf[:sk], vf[:sk], 1.0 / np.sqrt(LD))
        for row in range(LQ):
            got = kv.decode(0, sk, q[row])
            assert np.max(np.abs(got[0] - want[row])) < TOL, (sk, row)
            assert np.max(np.abs(got - util.oracle_decode(q[row], k16, v16, sk))) < TOL
    # the same two rows as one causal-free pair of batched sessions is not a
    # thing the fixture has; prefill rows are: row i of a chunk appended at
    # p0 = sk - 2 sees sk - 1 + i keys
    got = kv.prefill(0, 4094, q)
    for row in range(LQ):
        want = _materialised_f64(q[row:row + 1, 0], kf[:4095 + row], vf[:4095 + row], 1.0 / np.sqrt(LD))
        assert np.max(np.abs(got[row, 0] - want[0])) < TOL
    kv.close()


def test_ops_test_gqa_head_map_exact():
    # kernels.c:2185-2208: one key, so each output row is the V row of KV head qh // group
    q = np.ones((4, 2), dtype=np.float32)
    k = np.ones((1, 2, 2), dtype=np.float32)
    v = np.array([10, 20, 30, 40], dtype=np.float32).reshape(1, 2, 2)
    kv, _k16, _v16 = _cache_with(k, v)
    got = kv.decode(0, 1, q)
    assert np.array_equal(got.reshape(-1), [10, 20, 10, 20, 30, 40, 30, 40])
    got = kv.prefill(0, 0, q[None])
    assert np.array_equal(got.reshape(-1), [10, 20, 10, 20, 30, 40, 30, 40])
    kv.close()


@pytest.mark.parametrize("hd,nq,nkv", [(128, 16, 8), (64, 8, 8), (256, 8, 4)])
def test_fixture_fills_on_the_matrix_core_kernels(hd, nq, nkv):
    # the fixtures' head dims (4, 8) run on the generic kernels; the same
    # closed-form fills at the head dims the MFMA kernels serve, scale override
    # and window included, against the materialised softmax at the same bound
    SK = 300
    with np.errstate(over="ignore"):
        s = np.arange(SK * nkv * hd, dtype=np.uint32) * np.uint32(2654435761) + np.uint32(0x9E3779B9)
    k = (((s & 0xFFFF).astype(np.int32).astype(np.float32) / np.float32(32768.0) - np.float32(1.0))
         * np.float32(0.3)).reshape(SK, nkv, hd)
    v = ((((s >> 16) & 0xFFFF).astype(np.int32).astype(np.float32) / np.float32(32768.0)
          - np.float32(1.0)) * np.float32(0.3)).reshape(SK, nkv, hd)
    qi = np.arange(nq * hd)
    q = (((qi * 11 + 3) % 17).astype(np.float32) * np.float32(0.05)).reshape(nq, hd)
    kv, k16, v16 = _cache_with(k, v)
    kf, vf = _f16_values(k16), _f16_values(v16)
    g = nq // nkv
    for sc, win, sk in ((0.0, 0, 300), (0.25, 0, 257), (0.0, 4, 300), (0.0, 70, 129)):
        print("fixture fills hd", hd, "scale", sc, "window", win, "seq_k", sk, flush=True)
        scale = sc if sc > 0 else 1.0 / np.sqrt(hd)
        got = kv.decode(0, sk, q, sc, win)
        for h in range(nq):
            want = _materialised_f64(q[h:h + 1], kf[:sk, h // g], vf[:sk, h // g], scale,
                                     key_lo=max(sk - win, 0) if win else 0)
            assert np.max(np.abs(got[h] - want[0])) < TOL, (sc, win, sk, h)
    kv.close()
