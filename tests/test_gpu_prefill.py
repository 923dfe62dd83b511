"""Causal prefill on the device against the CPU oracle (a loop of seq_q = 1
attention calls, the reference's prefill semantics), through the C ABI.
Tolerance: max-abs 2e-3, rel-L2 1e-3."""
import numpy as np
import pytest

import oracle
from tests import util
from wayruntime_amd import hipattn, synth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _device():
    hipattn.init()
    oracle.set_attn_max_seq(1 << 20)
    yield
    hipattn.set_tuning(0, False)


def _setup(nq, nkv, hd, p0, T, seed, theta=None, extra_rows=0):
    """Cache with p0 + T appended rows (through the F32 append path), q [T,nq,hd]."""
    rows = p0 + T
    k32 = synth.normal(seed, (rows, nkv, hd))
    v32 = synth.normal(seed + 1, (rows, nkv, hd))
    q = synth.normal(seed + 2, (T, nq, hd))
    if theta:
        # inputs "after RoPE": rotate K at positions 0.. and Q at p0..
        k32 = oracle.rope(k32, 0, theta)
        q = oracle.rope(q, p0, theta)
    kv = hipattn.KVCache(1, hd, nkv, rows + extra_rows)
    assert kv.append(0, 0, k32, v32) == hipattn.OK
    return kv, q, synth.f32_to_f16_trunc(k32), synth.f32_to_f16_trunc(v32)


@pytest.mark.parametrize("nq,nkv,hd,p0,T,win", [
    (16, 8, 128, 0, 512, 0),        # Qwen3 shape, empty cache
    (32, 8, 128, 0, 512, 0),        # Llama-3 shape
    (32, 8, 128, 100, 300, 0),      # chunk appended to a non-empty cache, ragged sizes
    (8, 4, 256, 0, 200, 0),         # Gemma-class
    (4, 4, 64, 7, 130, 0),          # MHA
    (8, 1, 64, 0, 97, 0),           # group of 8: two head chunks per KV head
    (16, 8, 128, 0, 1, 0),          # a single row
    (16, 8, 128, 31, 2, 0),
    (16, 8, 128, 0, 33, 0),
    (16, 8, 128, 0, 400, 64),       # sliding window
    (32, 8, 128, 50, 300, 33),
    (8, 4, 256, 0, 300, 100),
    (16, 8, 256, 40, 700, 0),       # head_dim 256 behind a non-empty cache: blocks of 2 to 24 tiles, odd and even
    (4, 4, 256, 5, 131, 0),         # head_dim 256, MHA: four 32-row blocks per workgroup
    (16, 2, 256, 0, 97, 0),         # head_dim 256, group of 8: two head chunks per KV head
    (16, 4, 256, 33, 260, 70),      # head_dim 256, group of 4, window, chunk that starts inside a tile
    (8, 4, 256, 0, 1, 0),           # head_dim 256, a single row
    (8, 4, 256, 63, 2, 0),
    (8, 4, 256, 0, 33, 0),
])
def test_prefill_matches_serial_stepping_oracle(nq, nkv, hd, p0, T, win):
    print("prefill", nq, nkv, hd, p0, T, win, flush=True)
    # the two workload shapes at T = 512 take their inputs after RoPE, as the
    # workload says (base 1e6 for the Qwen3 shape, 5e5 for the Llama-3 shape)
    theta = {(16, 512): 1e6, (32, 512): 5e5}.get((nq, T)) if (hd == 128 and p0 == 0 and win == 0) else None
    kv, q, k16, v16 = _setup(nq, nkv, hd, p0, T, seed=1000 + T + p0, theta=theta)
    got = kv.prefill(0, p0, q, 0.0, win)
    want = oracle.causal_prefill(q, k16, v16, p0=p0, window=win, threads=8)
    print("  errors", util.assert_close(got, want), flush=True)
    kv.close()


def _drawn_shapes(n, seed):
    """n (nq, nkv, hd, p0, T, win) tuples drawn from a fixed seed: matrix-core head dims and
    group sizes, chunks that start and end anywhere in a tile, windows shorter and longer
    than the chunk."""
    r = synth.splitmix64(seed, 6 * n).reshape(n, 6)
    out = []
    for a in r:
        hd = (64, 128, 256, 256)[int(a[0] % 4)]
        group = (1, 2, 4, 8)[int(a[1] % 4)]
        nkv = (1, 2, 4)[int(a[2] % 3)]
        p0 = int(a[3] % 150)
        T = 1 + int(a[4] % 260)
        win = (0, 0, 1 + int(a[5] % 40), 40 + int(a[5] % 300))[int((a[5] >> 20) % 4)]
        out.append((group * nkv, nkv, hd, p0, T, win))
    return out


@pytest.mark.parametrize("nq,nkv,hd,p0,T,win", _drawn_shapes(16, 20260))
def test_prefill_drawn_shapes_against_the_oracle(nq, nkv, hd, p0, T, win):
    print("prefill drawn", nq, nkv, hd, p0, T, win, flush=True)
    kv, q, k16, v16 = _setup(nq, nkv, hd, p0, T, seed=3000 + 7 * T + p0)
    got = kv.prefill(0, p0, q, 0.0, win)
    want = oracle.causal_prefill(q, k16, v16, p0=p0, window=win, threads=8)
    util.assert_close(got, want)
    kv.close()


@pytest.mark.parametrize("nq,nkv,hd,p0,T,win", [
    (4, 2, 32, 3, 70, 0),           # head_dim 32: generic kernel
    (6, 2, 64, 0, 40, 0),           # group of 3
    (3, 3, 20, 0, 25, 8),
])
def test_prefill_generic_shapes(nq, nkv, hd, p0, T, win):
    print("prefill generic", nq, nkv, hd, p0, T, win, flush=True)
    kv, q, k16, v16 = _setup(nq, nkv, hd, p0, T, seed=77 + T)
    got = kv.prefill(0, p0, q, 0.0, win)
    want = oracle.causal_prefill(q, k16, v16, p0=p0, window=win)
    util.assert_close(got, want)
    kv.close()


def test_prefill_row_equals_decode_call_and_last_row_sees_everything():
    nq, nkv, hd, p0, T = 16, 8, 128, 40, 100
    kv, q, k16, v16 = _setup(nq, nkv, hd, p0, T, seed=5)
    got = kv.prefill(0, p0, q)
    for i in (0, 1, 31, 32, 63, 99):
        dec = kv.decode(0, p0 + i + 1, q[i])             # definition: row i == decode at seq_k = p0+i+1
        assert util.errors(got[i], dec)[0] < 2e-3
        util.assert_close(got[i], util.oracle_decode(q[i], k16, v16, p0 + i + 1), f"row {i}")
    # the last row equals the reference op (non-causal) over the whole cache
    util.assert_close(got[-1], oracle.attention(q[-1:], k16, v16)[0])
    kv.close()


def test_prefill_mfma_and_generic_kernels_agree():
    nq, nkv, hd, p0, T = 32, 8, 128, 10, 150
    kv, q, k16, v16 = _setup(nq, nkv, hd, p0, T, seed=9)
    a = kv.prefill(0, p0, q)
    hipattn.set_tuning(0, True)
    b = kv.prefill(0, p0, q)
    hipattn.set_tuning(0, False)
    assert util.errors(a, b)[0] < 2e-3
    util.assert_close(b, oracle.causal_prefill(q, k16, v16, p0=p0, threads=8), "generic")
    kv.close()


@pytest.mark.parametrize("nq,nkv,hd", [(16, 8, 128), (8, 4, 256), (8, 4, 64)])
def test_prefill_ignores_rows_that_were_never_appended(nq, nkv, hd):
    T = 70
    kv, q, k16, v16 = _setup(nq, nkv, hd, 0, T, seed=21, extra_rows=58)
    bad = np.full((58, nkv, hd), 0x7E00, dtype=np.uint16)       # NaN patterns above the chunk
    kv.write_f16(0, T, bad, bad)
    got = kv.prefill(0, 0, q)
    util.assert_close(got, oracle.causal_prefill(q, k16, v16, threads=8))
    kv.close()


@pytest.mark.parametrize("nq,nkv,theta,T,hd", [
    (16, 8, 1e6, 2048, 128),        # Qwen3: one position block per workgroup (the pairs would not fill the chip)
    (32, 8, 5e5, 2048, 128),        # Llama-3: a long and a short block per workgroup
    (32, 8, 5e5, 4096, 128),
    (32, 8, 5e5, 2048, 64),         # paired blocks at the other head dims
    (32, 8, 5e5, 2048, 256),
])
def test_prefill_workload_sizes_after_rope_sampled_rows(nq, nkv, theta, T, hd):
    # the prefill workload: Q/K/V N(0,1), rotated (theta 1e6 Qwen3, 5e5 Llama-3),
    # appended to an empty cache; the CPU loop is quadratic, so the oracle checks a
    # spread of rows and properties cover the rest
    print("prefill workload", nq, nkv, T, hd, flush=True)
    kv, q, k16, v16 = _setup(nq, nkv, hd, 0, T, seed=synth.config_seed(4, nq + T % 97), theta=theta)
    got = kv.prefill(0, 0, q)
    assert not np.isnan(got).any()
    rows = sorted(set([0, 1, 31, 32, 33, 63, 64, 127, 128, 500, 1023, 1024, T // 2 + 17, T - 2, T - 1]))
    want = oracle.causal_prefill(q, k16, v16, rows=rows, threads=8)
    print("  errors", util.assert_close(got[rows], want[rows]), flush=True)
    # row 0 sees one key: its output is V row 0 of the matching KV head
    v0 = v16[0].view(np.float16).astype(np.float32)
    assert np.allclose(got[0], np.repeat(v0, nq // nkv, axis=0), atol=1e-5)
    # every output is a convex combination of V rows: bounded by the per-dim extremes
    v = v16.view(np.float16).astype(np.float32)
    vmax = np.repeat(np.maximum.accumulate(v, axis=0), nq // nkv, axis=1)
    vmin = np.repeat(np.minimum.accumulate(v, axis=0), nq // nkv, axis=1)
    assert np.all(got <= vmax + 1e-3) and np.all(got >= vmin - 1e-3)
    kv.close()


@pytest.mark.parametrize("nq,nkv,theta,T", [
    (32, 8, 5e5, 2048),             # Llama-3: the paired-block launch form
    (16, 8, 1e6, 2048),             # Qwen3: the one-block-per-workgroup form
    (16, 8, 1e6, 4096),             # Qwen3 at the longest chunk of the workload
    (32, 8, 5e5, 4096),             # Llama-3 at the longest chunk: two rounds of paired workgroups
])
def test_prefill_workload_sizes_after_rope_every_row(nq, nkv, theta, T):
    # the prefill workload at full size with EVERY row checked against the serial
    # stepping oracle (rows spread over 16 host threads): a wrong row anywhere in
    # either launch form cannot hide between samples
    hd = 128
    print("prefill workload, all rows", nq, nkv, T, flush=True)
    kv, q, k16, v16 = _setup(nq, nkv, hd, 0, T, seed=synth.config_seed(4, 50 + nq + T % 97), theta=theta)
    got = kv.prefill(0, 0, q)
    assert not np.isnan(got).any()
    want = oracle.causal_prefill(q, k16, v16, threads=16)
    print("  errors over all rows", util.assert_close(got, want), flush=True)
    # per row as well: one bad row must not drown in the aggregate norm
    err = np.max(np.abs(got - want).reshape(T, -1), axis=1)
    assert float(err.max()) <= util.MAX_ABS, (int(err.argmax()), float(err.max()))
    kv.close()


@pytest.mark.parametrize("nq,nkv,hd,p0,T,win", [
    (32, 8, 128, 100, 2048, 500),   # a long and a short block per workgroup, behind a non-empty cache, windowed
    (32, 8, 64, 37, 2048, 0),
    (32, 8, 256, 64, 2048, 300),
])
def test_prefill_paired_blocks_with_offset_and_window_sampled_rows(nq, nkv, hd, p0, T, win):
    # launches large enough for the paired form (256 workgroups and more), with
    # the options the small cases above exercise on the one-block form
    print("prefill paired", nq, nkv, hd, p0, T, win, flush=True)
    kv, q, k16, v16 = _setup(nq, nkv, hd, p0, T, seed=4000 + hd + p0)
    got = kv.prefill(0, p0, q, 0.0, win)
    assert not np.isnan(got).any()
    rows = sorted(set([0, 1, 30, 31, 32, 33, 63, 64, 65, 127, 128, 400, 500, 501, 1023, 1024, T // 2 + 17,
                       T - 33, T - 32, T - 2, T - 1]))
    want = oracle.causal_prefill(q, k16, v16, p0=p0, window=win, rows=rows, threads=8)
    print("  errors", util.assert_close(got[rows], want[rows]), flush=True)
    kv.close()


@pytest.mark.parametrize("every", [1, 3])
@pytest.mark.parametrize("nq,nkv,hd,p0", [(16, 8, 256, 0), (8, 4, 256, 70), (32, 8, 128, 0), (4, 2, 64, 0)])
def test_prefill_with_a_softmax_reference_that_moves_from_tile_to_tile(nq, nkv, hd, p0, every):
    # scores that climb by 8 (11.5 in log2 units, above the 2^8 the lazy reference
    # tolerates) every `every` tiles of 32 keys: each row's reference moves again
    # and again, at every tile or with plain tiles between the moves.  In the
    # head-dim-256 kernel a move finds the next tile's score chain already
    # started from the old reference.
    T = 330
    rows = p0 + T
    print("prefill moving reference", nq, nkv, hd, p0, every, flush=True)
    k32 = synth.normal(5100 + hd, (rows, nkv, hd), std=0.05)
    v32 = synth.normal(5101 + hd, (rows, nkv, hd))
    q = synth.normal(5102 + hd, (T, nq, hd), std=0.05)
    k32[:, :, 0] = (np.arange(rows) // (32 * every) * (8.0 * every))[:, None]
    q[:, :, 0] = np.sqrt(hd)                             # score = ramp(key) + noise
    kv = hipattn.KVCache(1, hd, nkv, rows)
    assert kv.append(0, 0, k32, v32) == hipattn.OK
    k16, v16 = synth.f32_to_f16_trunc(k32), synth.f32_to_f16_trunc(v32)
    got = kv.prefill(0, p0, q)
    want = oracle.causal_prefill(q, k16, v16, p0=p0, threads=8)
    print("  errors", util.assert_close(got, want), flush=True)
    again = kv.prefill(0, p0, q)
    assert np.array_equal(got, again)
    kv.close()


@pytest.mark.parametrize("nq,nkv,hd", [(4, 2, 64), (32, 8, 128), (16, 8, 128), (8, 4, 256)])
def test_prefill_is_bit_identical_from_launch_to_launch(nq, nkv, hd):
    # The same chunk through caches at different addresses and launch after launch
    # must give the same bits: the batched step equals serial steps only if it does
    # (src/core/batch.c:15-19), and a kernel whose result depends on timing (a
    # result read before it is complete, a slot refilled while still being read)
    # shows up here long before it leaves the tolerance.
    for T in (39, 65, 130, 300, 2048):
        print("prefill determinism", nq, nkv, hd, T, flush=True)
        k32 = synth.normal(1, (T, nkv, hd))
        v32 = synth.normal(2, (T, nkv, hd))
        q = synth.normal(3, (T, nq, hd))
        kvs = [hipattn.KVCache(1, hd, nkv, T + 17 * i) for i in range(3)]
        for kv in kvs:
            assert kv.append(0, 0, k32, v32) == hipattn.OK
        first = kvs[0].prefill(0, 0, q)
        for rep in range(1, 7):
            again = kvs[rep % 3].prefill(0, 0, q)
            assert np.array_equal(first, again), f"T={T}: launch {rep} differs from the first"
        for kv in kvs:
            kv.close()


def test_prefill_error_contract():
    lib = hipattn.lib()
    kv = hipattn.KVCache(1, 128, 8, 64)
    q = np.zeros((4, 16, 128), dtype=np.float32)
    out = np.zeros_like(q)
    pre = lambda p0, T, nq=16: lib.wr_hip_attn_prefill(kv.h, 0, p0, T, q.ctypes.data,   # noqa: E731
                                                        out.ctypes.data, nq, 0.0, 0)
    assert pre(0, 0) == hipattn.ERR_INVAL
    assert pre(62, 4) == hipattn.ERR_INVAL                 # runs past the allocation
    assert pre(hipattn.ATTN_MAX_SEQ, 4) == hipattn.ERR_LIMIT
    calls = lib.wr_hip_attn_calls()
    assert pre(0, 4, nq=12) == hipattn.ERR_INVAL
    # refused for its shape, yet counted: the reference counts each of the four
    # calls before it looks at shapes (kernels.c:1418-1423)
    assert lib.wr_hip_attn_calls() == calls + 4
    assert lib.wr_hip_attn_prefill(kv.h, 0, 0, 4, None, out.ctypes.data, 16, 0.0, 0) == hipattn.ERR_INVAL
    assert lib.wr_hip_attn_calls() == calls + 4            # a null pointer is refused before the count
    calls = lib.wr_hip_attn_calls()
    assert pre(0, 4) == hipattn.OK
    assert lib.wr_hip_attn_calls() == calls + 4            # one per token, as the serial loop counts
    kv.close()


@pytest.mark.parametrize("nq,nkv,T,p0,norm,scale,window", [
    (16, 8, 600, 0, True, 0.0, 0),       # Qwen3 shape: per-head norms, one block per workgroup
    (32, 8, 2048, 0, False, 0.0, 0),     # Llama shape: paired blocks
    (16, 8, 300, 500, True, 0.25, 0),    # a later chunk of a prompt, scale override
    (32, 8, 700, 0, False, 0.0, 256),    # sliding window
])
def test_prefill_from_f16_query_rows_equals_the_f32_form(nq, nkv, T, p0, norm, scale, window):
    # wr_hip_rows_qkv_append_q16_dev + wr_hip_attn_prefill_q16_dev against
    # wr_hip_rows_qkv_append_dev + wr_hip_attn_prefill_dev on twin caches: the
    # kernel rounds Q to binary16 once in either form, so the outputs must agree
    # byte for byte, as must the caches; the F16 rows themselves are checked against
    # the F32 rows times the scale, rounded to nearest
    import ctypes as C
    hd, eps, theta = 128, 1e-6, 1e6
    lib = hipattn.lib()
    print("prefill q16", nq, nkv, T, p0, norm, scale, window, flush=True)
    width = (nq + 2 * nkv) * hd
    x = synth.normal(8800 + T, (T, width), std=1.5)
    qw = synth.normal(8801, (hd,), std=1.0) if norm else None
    kw = synth.normal(8802, (hd,), std=1.0) if norm else None
    tab = oracle.rope_table(T, hd, p0, theta, 0)
    n_rot = tab.shape[1]
    xd = hipattn.DeviceBuffer.from_host(x)
    td = hipattn.DeviceBuffer.from_host(tab)
    qwd = hipattn.DeviceBuffer.from_host(qw) if norm else None
    kwd = hipattn.DeviceBuffer.from_host(kw) if norm else None
    qn = qwd.p if norm else None
    kn = kwd.p if norm else None
    _a, _b, k16, v16 = util.make_kv(8810, p0 + T, nkv, hd)
    twins = []
    for _ in range(2):
        kv = hipattn.KVCache(1, hd, nkv, p0 + T)
        kv.write_f16(0, 0, k16, v16)
        twins.append(kv)
    pp = (C.c_uint32 * 1)(p0)
    q32 = hipattn.DeviceBuffer(T * nq * hd * 4)
    q16 = hipattn.DeviceBuffer(T * nq * hd * 2)
    o32 = hipattn.DeviceBuffer.from_host(np.full((T, nq, hd), 3.0, dtype=np.float32))
    o16 = hipattn.DeviceBuffer.from_host(np.full((T, nq, hd), -4.0, dtype=np.float32))
    kva = (C.c_void_p * 1)(twins[0].h)
    kvb = (C.c_void_p * 1)(twins[1].h)
    assert lib.wr_hip_rows_qkv_append_dev(xd.p, width, T, nq, qn, kn, eps, td.p, n_rot, 1, kva, 0, pp,
                                          q32.p, 0) == hipattn.OK
    assert lib.wr_hip_attn_prefill_dev(twins[0].h, 0, p0, T, q32.p, o32.p, nq, scale, window) == hipattn.OK
    assert lib.wr_hip_rows_qkv_append_q16_dev(xd.p, width, T, nq, qn, kn, eps, td.p, n_rot, 1, kvb, 0, pp,
                                              q16.p, scale, 0) == hipattn.OK
    assert lib.wr_hip_attn_prefill_q16_dev(twins[1].h, 0, p0, T, q16.p, o16.p, nq, scale, window) == hipattn.OK
    hipattn.sync()
    a, b = o32.to_host((T, nq, hd)), o16.to_host((T, nq, hd))
    rows_off = np.argwhere(np.abs(a - b).reshape(T, -1).max(axis=1) > 0)[:, 0]
    assert a.tobytes() == b.tobytes(), f"rows that differ: {rows_off[:8].tolist()} of {len(rows_off)}"
    ka, va = twins[0].read_f16(0, 0, p0 + T)
    kb, vb = twins[1].read_f16(0, 0, p0 + T)
    assert ka.tobytes() == kb.tobytes() and va.tobytes() == vb.tobytes()
    qs = np.float32((scale if scale > 0 else 1.0 / np.sqrt(np.float32(hd))) * np.float32(1.4426950408889634))
    want = (q32.to_host((T, nq, hd)) * qs).astype(np.float16)
    got = q16.to_host((T, nq, hd), dtype=np.float16)
    assert got.tobytes() == want.tobytes()
    # shapes the form does not take are refused before anything is written
    assert lib.wr_hip_rows_qkv_append_q16_dev(xd.p, width + 2, T, nq, qn, kn, eps, td.p, n_rot, 1, kvb, 0, pp,
                                              q16.p, scale, 0) == hipattn.ERR_UNSUPPORTED
    for kv in twins:
        kv.close()
    for buf in (xd, td, qwd, kwd, q32, q16, o32, o16):
        if buf is not None:
            buf.free()
