"""Row steps on the device (RMSNorm, Q/K/V split with per-head norm and rotary
embedding, gated activation) against the CPU oracle, through the C ABI.

Sums over a row are tree reductions on the device and sequential loops in the
reference, and the device's exp is not the reference's polynomial, so these
agree to F32 rounding: |got - want| <= 4e-6 * max|want| per call (the largest
term is the polynomial exp's own 2e-6).  Where no sum or exp is involved
(rotation without the norm, the V copy) the bits are equal."""
import numpy as np
import pytest

import oracle
from wayruntime_amd import hipattn, synth

pytestmark = pytest.mark.gpu

TOL = 4e-6


@pytest.fixture(scope="module", autouse=True)
def _device():
    hipattn.init()
    yield


def _dev(a):
    return hipattn.DeviceBuffer.from_host(np.ascontiguousarray(a, dtype=np.float32))


def _close(got, want):
    assert not np.isnan(got).any()
    assert np.max(np.abs(got.astype(np.float64) - want)) <= TOL * np.max(np.abs(want))


@pytest.mark.parametrize("rows,dim,wn,eps", [(3, 1024, 1024, 1e-6), (16, 4096, 4096, 1e-5),
                                             (1, 96, 0, 1e-6), (2, 300, 4, 1e-6)])
def test_rmsnorm_rows(rows, dim, wn, eps):
    print("rmsnorm", rows, dim, wn, flush=True)
    ldx, ldo = dim + 8, dim + 4
    x = synth.normal(dim + rows, (rows, ldx), std=2.0)
    w = synth.normal(dim, (wn,)) + np.float32(1.0) if wn else None
    xd, od = _dev(x), _dev(np.full((rows, ldo), 9.0))
    wd = _dev(w) if wn else None
    rc = hipattn.lib().wr_hip_rows_rmsnorm_dev(xd.p, ldx, wd.p if wn else None, wn, od.p, ldo, rows,
                                               dim, eps)
    assert rc == hipattn.OK
    hipattn.sync()
    got = od.to_host((rows, ldo))
    _close(got[:, :dim], oracle.rmsnorm(np.ascontiguousarray(x[:, :dim]), w, eps).astype(np.float64))
    assert np.all(got[:, dim:] == 9.0)


@pytest.mark.parametrize("rows,nq,nkv,hd,norm,theta,n_rot_pairs,pos", [
    (1, 16, 8, 128, True, 1e6, 0, 77),          # Qwen3: per-head norm, full rotation
    (5, 32, 8, 128, False, 5e5, 0, 4000),       # Llama: no norm
    (3, 8, 4, 256, True, 1e6, 0, 0),
    (2, 4, 2, 64, False, 1e4, 10, 9),           # partial rotation, pairs across lanes
    (2, 2, 1, 32, True, 1e4, 0, 3),
])
def test_qkv_prep(rows, nq, nkv, hd, norm, theta, n_rot_pairs, pos):
    print("qkv_prep", rows, nq, nkv, hd, norm, flush=True)
    width = (nq + 2 * nkv) * hd
    ld = width + 16
    qkv = synth.normal(hd + rows, (rows, ld), std=1.5)
    qn = synth.normal(1, (hd,)) * np.float32(0.1) + np.float32(1.0)
    kn = synth.normal(2, (hd,)) * np.float32(0.1) + np.float32(1.0)
    tab = oracle.rope_table(rows, hd, pos, theta, n_rot_pairs)
    n_rot = tab.shape[1]
    qd, kd = nq * hd, nkv * hd
    bufs = [_dev(qkv), _dev(qn), _dev(kn), _dev(tab), _dev(np.zeros((rows, qd))),
            _dev(np.zeros((rows, kd))), _dev(np.zeros((rows, kd)))]
    xd, qnd, knd, td, qo, ko, vo = bufs
    eps = 1e-6
    rc = hipattn.lib().wr_hip_rows_qkv_prep_dev(xd.p, ld, rows, nq, nkv, hd,
                                                qnd.p if norm else None, knd.p if norm else None,
                                                eps, td.p, n_rot, qo.p, ko.p, vo.p)
    assert rc == hipattn.OK
    hipattn.sync()
    q_in = np.ascontiguousarray(qkv[:, :qd]).reshape(rows, nq, hd)
    k_in = np.ascontiguousarray(qkv[:, qd:qd + kd]).reshape(rows, nkv, hd)
    v_in = np.ascontiguousarray(qkv[:, qd + kd:width]).reshape(rows, nkv, hd)
    if norm:
        q_in = oracle.rmsnorm(q_in, qn, eps)
        k_in = oracle.rmsnorm(k_in, kn, eps)
    want_q = oracle.rope(q_in, pos, theta, n_rot_pairs)
    want_k = oracle.rope(k_in, pos, theta, n_rot_pairs)
    got_q, got_k, got_v = qo.to_host((rows, nq, hd)), ko.to_host((rows, nkv, hd)), vo.to_host((rows, nkv, hd))
    assert np.array_equal(got_v, v_in)
    if norm:
        _close(got_q, want_q.astype(np.float64))
        _close(got_k, want_k.astype(np.float64))
    else:
        assert got_q.tobytes() == want_q.tobytes()
        assert got_k.tobytes() == want_k.tobytes()
    for b in bufs:
        b.free()


def test_swiglu_rows():
    rows, ffn = 3, 3072
    ld, ldo = 2 * ffn + 8, ffn + 4
    gu = synth.normal(5, (rows, ld), std=3.0)
    gu[0, :8] = [-100.0, -60.0, -20.0, 0.0, 20.0, 60.0, 80.0, 100.0]
    gd, ad = _dev(gu), _dev(np.full((rows, ldo), 9.0))
    assert hipattn.lib().wr_hip_rows_swiglu_dev(gd.p, ld, ad.p, ldo, rows, ffn) == hipattn.OK
    hipattn.sync()
    got = ad.to_host((rows, ldo))
    want = oracle.silu_mul(np.ascontiguousarray(gu[:, :ffn]), np.ascontiguousarray(gu[:, ffn:2 * ffn]))
    _close(got[:, :ffn], want.astype(np.float64))
    assert np.all(got[:, ffn:] == 9.0)
    gd.free()
    ad.free()


def test_error_contract():
    lib = hipattn.lib()
    d = _dev(np.zeros(4096))
    assert lib.wr_hip_rows_rmsnorm_dev(None, 8, None, 0, d.p, 8, 1, 8, 1e-6) == hipattn.ERR_INVAL
    assert lib.wr_hip_rows_rmsnorm_dev(d.p, 4, None, 0, d.p, 8, 1, 8, 1e-6) == hipattn.ERR_INVAL   # stride < dim
    assert lib.wr_hip_rows_rmsnorm_dev(d.p, 8, None, 3, d.p, 8, 1, 8, 1e-6) == hipattn.ERR_INVAL   # weight missing
    # odd head_dim, stride too small, one norm vector without the other, table missing
    assert lib.wr_hip_rows_qkv_prep_dev(d.p, 64, 1, 1, 1, 7, None, None, 1e-6, d.p, 3, d.p, d.p, d.p) == hipattn.ERR_INVAL
    assert lib.wr_hip_rows_qkv_prep_dev(d.p, 8, 1, 1, 1, 8, None, None, 1e-6, d.p, 4, d.p, d.p, d.p) == hipattn.ERR_INVAL
    assert lib.wr_hip_rows_qkv_prep_dev(d.p, 24, 1, 1, 1, 8, d.p, None, 1e-6, d.p, 4, d.p, d.p, d.p) == hipattn.ERR_INVAL
    assert lib.wr_hip_rows_qkv_prep_dev(d.p, 24, 1, 1, 1, 8, None, None, 1e-6, None, 4, d.p, d.p, d.p) == hipattn.ERR_INVAL
    assert lib.wr_hip_rows_swiglu_dev(d.p, 8, d.p, 8, 1, 8) == hipattn.ERR_INVAL                    # stride < 2 ffn
    d.free()


import ctypes as C


@pytest.mark.parametrize("rows,nq,nkv,hd,norm,pos,batch,rot_pairs,pad", [
    (70, 16, 8, 128, True, 13, False, 0, 16),      # three cache blocks, both ends partial
    (1, 16, 8, 128, True, 77, False, 0, 16),       # one decode row
    (33, 4, 2, 64, False, 0, False, 0, 16),        # no norm; head_dim 64 (the pair sits in two lanes)
    (5, 8, 4, 256, True, 31, False, 0, 16),        # crosses a block boundary after one row
    (5, 16, 8, 128, True, 0, True, 0, 16),         # batched step: row i to session i at its own position
    (16, 32, 8, 128, False, 0, True, 0, 16),
    # head dims 128 and 256 take the eight-lanes-per-position path when rows,
    # tables and vectors are 16-byte aligned and the rotated pairs come in
    # eights; the cases below sit on both sides of each condition
    (70, 8, 4, 128, True, 13, False, 24, 16),      # partial rotation, pairs in eights
    (40, 8, 4, 128, True, 5, False, 20, 16),       # partial rotation, not in eights: one wave per position
    (40, 8, 4, 128, True, 5, False, 0, 3),         # row stride not a multiple of four floats: likewise
    (67, 4, 2, 256, False, 30, False, 40, 8),      # head_dim 256, no norm, partial rotation
    (7, 4, 2, 256, True, 0, True, 0, 4),           # head_dim 256, batched step
])
def test_qkv_append_equals_prep_then_append(rows, nq, nkv, hd, norm, pos, batch, rot_pairs, pad):
    # the fused launch against the two-step path: Q rows and the cache contents, bit for bit
    print("qkv_append", rows, nq, nkv, hd, norm, pos, batch, rot_pairs, pad, flush=True)
    lib = hipattn.lib()
    width = (nq + 2 * nkv) * hd
    ld = width + pad
    qkv = synth.normal(7 * hd + rows, (rows, ld), std=1.5)
    qn = synth.normal(1, (hd,)) * np.float32(0.1) + np.float32(1.0)
    kn = synth.normal(2, (hd,)) * np.float32(0.1) + np.float32(1.0)
    qd, kd = nq * hd, nkv * hd
    eps = 1e-6
    n_kv = rows if batch else 1
    positions = [3 + 37 * i for i in range(rows)] if batch else [pos]
    if batch:
        tab = np.concatenate([oracle.rope_table(1, hd, p, 1e6, rot_pairs) for p in positions])
    else:
        tab = oracle.rope_table(rows, hd, pos, 1e6, rot_pairs)
    n_rot = tab.shape[1]
    assert n_rot == (rot_pairs or hd // 2)
    ctx = 1024
    two_step = [hipattn.KVCache(1, hd, nkv, ctx) for _ in range(n_kv)]
    fused = [hipattn.KVCache(1, hd, nkv, ctx) for _ in range(n_kv)]
    bufs = [_dev(qkv), _dev(qn), _dev(kn), _dev(tab), _dev(np.zeros((rows, qd))), _dev(np.zeros((rows, kd))),
            _dev(np.zeros((rows, kd))), _dev(np.full((rows, qd), 5.0))]
    xd, qnd, knd, td, qo, ko, vo, qo2 = bufs
    qnp, knp = (qnd.p, knd.p) if norm else (None, None)
    assert lib.wr_hip_rows_qkv_prep_dev(xd.p, ld, rows, nq, nkv, hd, qnp, knp, eps, td.p, n_rot,
                                        qo.p, ko.p, vo.p) == hipattn.OK
    if batch:
        kvp = (C.c_void_p * n_kv)(*[c.h for c in two_step])
        pp = (C.c_uint32 * n_kv)(*positions)
        assert lib.wr_hip_attn_append_batched_dev(n_kv, kvp, 0, pp, ko.p, vo.p) == hipattn.OK
    else:
        hipattn.append_dev(two_step[0], 0, pos, rows, ko, vo)
    kvp = (C.c_void_p * n_kv)(*[c.h for c in fused])
    pp = (C.c_uint32 * n_kv)(*positions)
    assert lib.wr_hip_rows_qkv_append_dev(xd.p, ld, rows, nq, qnp, knp, eps, td.p, n_rot, n_kv, kvp, 0, pp,
                                          qo2.p, 0) == hipattn.OK
    hipattn.sync()
    assert qo.to_host((rows, qd)).tobytes() == qo2.to_host((rows, qd)).tobytes()
    for a, b, p in zip(two_step, fused, positions if batch else [pos]):
        n = 1 if batch else rows
        lo = max(0, p - 40)
        ka, va = a.read_f16(0, lo, p + n - lo + 40)      # neighbours too: nothing else may be written
        kb, vb = b.read_f16(0, lo, p + n - lo + 40)
        assert ka.tobytes() == kb.tobytes() and va.tobytes() == vb.tobytes()
    # contracts: all or nothing past the end of a cache; one cache or one per row; distinct caches
    pp_bad = (C.c_uint32 * n_kv)(*([ctx - (0 if batch else rows - 1)] * n_kv))
    assert lib.wr_hip_rows_qkv_append_dev(xd.p, ld, rows, nq, qnp, knp, eps, td.p, n_rot, n_kv, kvp, 0, pp_bad,
                                          qo2.p, 0) == hipattn.ERR_CTX_FULL
    if rows > 2:
        assert lib.wr_hip_rows_qkv_append_dev(xd.p, ld, rows, nq, qnp, knp, eps, td.p, n_rot, 2, kvp, 0, pp,
                                              qo2.p, 0) == hipattn.ERR_INVAL
    for c in two_step + fused:
        c.close()
    for b in bufs:
        b.free()


def test_rmsnorm_add_accumulates_into_the_residual():
    rows, dim = 5, 1024
    x = synth.normal(81, (rows, dim), std=3.0)
    w = synth.normal(82, (dim,)) * np.float32(0.1) + np.float32(1.0)
    acc = synth.normal(83, (rows, dim + 8))
    xd, wd, ad = _dev(x), _dev(w), _dev(acc)
    assert hipattn.lib().wr_hip_rows_rmsnorm_add_dev(xd.p, dim, wd.p, dim, ad.p, dim + 8, rows, dim, 1e-6) == hipattn.OK
    hipattn.sync()
    got = ad.to_host((rows, dim + 8))
    want = acc[:, :dim].astype(np.float64) + oracle.rmsnorm(x, w, 1e-6).astype(np.float64)
    _close(got[:, :dim], want)
    assert np.array_equal(got[:, dim:], acc[:, dim:])     # padding columns untouched
    for b in (xd, wd, ad):
        b.free()


def _f16_ulps(a16, b16):
    # distance in binary16 steps between two arrays of bit patterns of the same sign
    return np.abs(a16.astype(np.int32) - b16.astype(np.int32))


@pytest.mark.parametrize("hd", [64, 128, 256])
def test_qkv_append_gemma_flags(hd):
    # V_NORM: the V heads get a weightless RMSNorm before they are truncated into
    # the cache; Q_ONLY: rows of Q heads only, nothing is appended (a layer that
    # reads another layer's cache)
    print("qkv_append flags", hd, flush=True)
    lib = hipattn.lib()
    rows, nq, nkv, pos = 9, 4, 2, 30
    width = (nq + 2 * nkv) * hd
    qkv = synth.normal(91, (rows, width), std=1.5)
    qn = synth.normal(1, (hd,)) * np.float32(0.1) + np.float32(1.0)
    kn = synth.normal(2, (hd,)) * np.float32(0.1) + np.float32(1.0)
    tab = oracle.rope_table(rows, hd, pos, 1e6, 0)
    n_rot = tab.shape[1]
    qd, kd = nq * hd, nkv * hd
    eps = 1e-6
    kv = hipattn.KVCache(1, hd, nkv, 256)
    bufs = [_dev(qkv), _dev(qn), _dev(kn), _dev(tab), _dev(np.zeros((rows, qd))), _dev(np.zeros((rows, qd))),
            _dev(np.zeros((rows, kd))), _dev(np.zeros((rows, kd)))]
    xd, qnd, knd, td, q1, q2, ko, vo = bufs
    kvp = (C.c_void_p * 1)(kv.h)
    pp = (C.c_uint32 * 1)(pos)
    assert lib.wr_hip_rows_qkv_append_dev(xd.p, width, rows, nq, qnd.p, knd.p, eps, td.p, n_rot, 1, kvp, 0, pp,
                                          q1.p, hipattn.QKV_V_NORM) == hipattn.OK
    hipattn.sync()
    k16, v16 = kv.read_f16(0, pos, rows)
    v_in = np.ascontiguousarray(qkv[:, qd + kd:]).reshape(rows, nkv, hd)
    want_v = synth.f32_to_f16_trunc(oracle.rmsnorm(v_in, None, eps))
    assert _f16_ulps(v16, want_v).max() <= 1              # a last-bit difference in F32 can move the truncation
    assert (_f16_ulps(v16, want_v) > 0).mean() < 0.01
    # K is what the unflagged call stores
    kv2 = hipattn.KVCache(1, hd, nkv, 256)
    kvp2 = (C.c_void_p * 1)(kv2.h)
    assert lib.wr_hip_rows_qkv_append_dev(xd.p, width, rows, nq, qnd.p, knd.p, eps, td.p, n_rot, 1, kvp2, 0, pp,
                                          q2.p, 0) == hipattn.OK
    hipattn.sync()
    k16b, _ = kv2.read_f16(0, pos, rows)
    assert k16.tobytes() == k16b.tobytes()
    assert q1.to_host((rows, qd)).tobytes() == q2.to_host((rows, qd)).tobytes()
    # Q_ONLY on rows that hold the Q heads alone: the same Q, and the cache stays as it is
    q_rows = np.ascontiguousarray(qkv[:, :qd])
    qx = _dev(q_rows)
    before = kv2.read_f16(0, 0, 256)
    assert lib.wr_hip_rows_qkv_append_dev(qx.p, qd, rows, nq, qnd.p, None, eps, td.p, n_rot, 1, kvp2, 0, pp,
                                          q1.p, hipattn.QKV_Q_ONLY) == hipattn.OK
    hipattn.sync()
    assert q1.to_host((rows, qd)).tobytes() == q2.to_host((rows, qd)).tobytes()
    after = kv2.read_f16(0, 0, 256)
    assert before[0].tobytes() == after[0].tobytes() and before[1].tobytes() == after[1].tobytes()
    assert lib.wr_hip_rows_qkv_append_dev(qx.p, qd, rows, nq, qnd.p, None, eps, td.p, n_rot, 1, kvp2, 0, pp,
                                          q1.p, 8) == hipattn.ERR_INVAL
    for c in (kv, kv2):
        c.close()
    for b in bufs + [qx]:
        b.free()


# The table the rotation takes, made on the device.  The reference reduces an
# angle by one subtraction of 2*pi per turn, each rounded, and evaluates its own
# polynomials (kernels.c:1384-1404, mathx.c:37-57, :72-86, :112-147); the device
# restates them operation for operation, so the BYTES must be equal: every
# position a 32768-token context can hold, for the bases of the three families
# (Llama 5e5, Qwen3 1e6, Gemma's sliding-window layers 1e4) and a partial
# rotation.
@pytest.mark.parametrize("hd,theta,rot_pairs", [(128, 1e6, 0), (128, 5e5, 0), (256, 1e4, 0),
                                                (64, 1e6, 0), (128, 1e6, 24), (96, 0.5, 0)])
def test_rope_table_on_device_is_the_oracles_bytes(hd, theta, rot_pairs):
    print("rope table", hd, theta, rot_pairs, flush=True)
    n = 32768
    want = oracle.rope_table(n, hd, 0, theta, rot_pairs)
    got = hipattn.rope_table_dev(n, hd, theta, rot_pairs, pos0=0)
    assert got.shape == want.shape
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # a window that does not start at zero, and a ragged row count
    got = hipattn.rope_table_dev(77, hd, theta, rot_pairs, pos0=31000)
    assert np.array_equal(got.view(np.uint32), want[31000:31077].view(np.uint32))


def test_rope_table_on_device_listed_positions():
    positions = [0, 32767, 5, 4096, 4095, 1, 77, 20000, 31, 32, 33, 9999, 16384, 2, 3, 12345]
    for n in (1, 7, 16):
        got = hipattn.rope_table_dev(n, 128, 1e6, 0, pos=positions[:n])
        want = np.concatenate([oracle.rope_table(1, 128, p, 1e6, 0) for p in positions[:n]])
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    lib = hipattn.lib()
    buf = hipattn.DeviceBuffer(17 * 64 * 8)
    import ctypes as C
    plist = (C.c_uint32 * 17)(*range(17))
    assert lib.wr_hip_attn_rope_table_dev(buf.p, 17, 0, plist, 128, 1e6, 0) == hipattn.ERR_INVAL
    assert lib.wr_hip_attn_rope_table_dev(buf.p, 1, 0, None, 127, 1e6, 0) == hipattn.ERR_INVAL
    assert lib.wr_hip_attn_rope_table_dev(None, 1, 0, None, 128, 1e6, 0) == hipattn.ERR_INVAL
    assert lib.wr_hip_attn_rope_table_dev(buf.p, 0, 0, None, 128, 1e6, 0) == hipattn.ERR_INVAL
    buf.free()


def test_rope_table_on_device_refuses_positions_beyond_the_sequence_limit():
    # The range reduction subtracts 2 pi in a loop that does not end for angles
    # beyond 2^27: the entry point takes positions below WR_HIP_ATTN_MAX_SEQ only
    # and refuses the rest before any kernel runs (nothing is launched here).
    import ctypes as C
    lib = hipattn.lib()
    buf = hipattn.DeviceBuffer.from_host(np.full((4, 64, 2), 9.0, dtype=np.float32))
    lim = hipattn.ATTN_MAX_SEQ
    assert lib.wr_hip_attn_rope_table_dev(buf.p, 4, lim - 3, None, 128, 1e6, 0) == hipattn.ERR_LIMIT
    assert lib.wr_hip_attn_rope_table_dev(buf.p, 1, 2 ** 31, None, 128, 1e6, 0) == hipattn.ERR_LIMIT
    assert lib.wr_hip_attn_rope_table_dev(buf.p, 4, 2 ** 32 - 2, None, 128, 1e6, 0) == hipattn.ERR_LIMIT
    plist = (C.c_uint32 * 3)(5, lim, 7)
    assert lib.wr_hip_attn_rope_table_dev(buf.p, 3, 0, plist, 128, 1e6, 0) == hipattn.ERR_LIMIT
    plist = (C.c_uint32 * 2)(2 ** 32 - 1, 1)
    assert lib.wr_hip_attn_rope_table_dev(buf.p, 2, 0, plist, 128, 1e6, 0) == hipattn.ERR_LIMIT
    hipattn.sync()
    assert np.all(buf.to_host((4, 64, 2)) == 9.0)            # nothing written
    # the last positions inside the limit are served
    got = hipattn.rope_table_dev(2, 128, 1e6, 0, pos0=lim - 2)
    assert np.isfinite(got).all()
    buf.free()


def test_row_step_without_rotation_ignores_the_table_pointer():
    # n_rot = 0 with a table pointer given: the eight-lane path must not read a
    # table that holds zero pairs per row (head dim 128, aligned operands)
    import ctypes as C
    lib = hipattn.lib()
    nq, nkv, hd, rows = 16, 8, 128, 40
    width = (nq + 2 * nkv) * hd
    x = synth.normal(8700, (rows, width))
    xd = hipattn.DeviceBuffer.from_host(x)
    tiny = hipattn.DeviceBuffer.from_host(np.zeros(4, dtype=np.float32))   # far smaller than a table would be
    outs = []
    for tab in (tiny.p, None):
        kv = hipattn.KVCache(1, hd, nkv, rows)
        q = hipattn.DeviceBuffer.from_host(np.full((rows, nq, hd), 2.0, dtype=np.float32))
        kvs = (C.c_void_p * 1)(kv.h)
        pos = (C.c_uint32 * 1)(0)
        assert lib.wr_hip_rows_qkv_append_dev(xd.p, width, rows, nq, None, None, 1e-6, tab, 0, 1, kvs, 0, pos,
                                              q.p, 0) == hipattn.OK
        hipattn.sync()
        outs.append((q.to_host((rows, nq, hd)),) + tuple(kv.read_f16(0, 0, rows)))
        q.free()
        kv.close()
    for a, b in zip(outs[0], outs[1]):
        assert np.array_equal(a, b)
    assert np.array_equal(outs[0][0], x[:, :nq * hd].reshape(rows, nq, hd))   # Q passes through unrotated
    xd.free()
    tiny.free()
