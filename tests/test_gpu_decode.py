"""Device decode attention and cache append against the CPU oracle, through
the C ABI.  Tolerance: max-abs 2e-3 and rel-L2 1e-3 on the attention outputs
(float32 accumulate), bit-exact on the cache contents."""
import numpy as np
import pytest

import oracle
from tests import util
from tests.golden import cases
from wayruntime_amd import hipattn, synth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _device():
    hipattn.init()
    print("device:", hipattn.device_name(), flush=True)
    yield
    hipattn.set_tuning(0, False)


# ------------------------------------------------------------------ append --

@pytest.mark.parametrize("nkv,hd,max_ctx,chunks", [
    (8, 128, 200, [1, 1, 1, 30, 1, 64, 33, 69]),      # crosses 32-position blocks at every offset
    (4, 256, 70, [70]),
    (2, 32, 40, [5, 35]),
    (1, 20, 9, [1] * 9),                               # head_dim that is no multiple of 16
])
def test_append_is_bit_exact_and_leaves_neighbours_alone(nkv, hd, max_ctx, chunks):
    kv = hipattn.KVCache(2, hd, nkv, max_ctx)
    k32 = synth.normal(100, (max_ctx, nkv, hd), std=3.0)
    v32 = synth.normal(101, (max_ctx, nkv, hd), std=3.0)
    # values that exercise the codec edges: overflow, subnormal range, signed zero, NaN
    k32.reshape(-1)[:6] = [1e6, -1e6, 3e-6, -3e-6, -0.0, np.nan]
    v32.reshape(-1)[:4] = [65504.0, 65520.0, 6.1e-5, 6.0e-5]
    pos = 0
    for n in chunks:
        print("append", nkv, hd, "pos", pos, "n", n, flush=True)
        assert kv.append(1, pos, k32[pos:pos + n], v32[pos:pos + n]) == hipattn.OK
        pos += n
        gk, gv = kv.read_f16(1, 0, pos)
        assert np.array_equal(gk, synth.f32_to_f16_trunc(k32[:pos]))
        assert np.array_equal(gv, synth.f32_to_f16_trunc(v32[:pos]))
    # the other layer is untouched (zero-filled at creation)
    zk, zv = kv.read_f16(0, 0, max_ctx)
    assert not zk.any() and not zv.any()
    # a full cache refuses and writes nothing
    before = kv.read_f16(1, 0, max_ctx)
    assert kv.append(1, max_ctx, k32[:1], v32[:1]) == hipattn.ERR_CTX_FULL
    assert kv.append(1, max_ctx - 1, k32[:2], v32[:2]) == hipattn.ERR_CTX_FULL
    after = kv.read_f16(1, 0, max_ctx)
    assert np.array_equal(before[0], after[0]) and np.array_equal(before[1], after[1])
    kv.close()


def test_append_matches_oracle_append_row():
    import ctypes as C
    nkv, hd, cap = 2, 64, 37
    kv = hipattn.KVCache(1, hd, nkv, cap)
    rows_k = synth.normal(7, (cap, nkv * hd), std=2.0)
    rows_v = synth.normal(8, (cap, nkv * hd), std=2.0)
    ok = np.zeros((cap, nkv, hd), dtype=np.uint16)
    ov = np.zeros((cap, nkv, hd), dtype=np.uint16)
    tk, tv = oracle.wrap(ok, flags=oracle.GROWABLE), oracle.wrap(ov, flags=oracle.GROWABLE)
    for i in range(cap):
        assert oracle.lib().wro_kv_append_row(C.byref(tk), rows_k[i], nkv, hd) == 0
        assert oracle.lib().wro_kv_append_row(C.byref(tv), rows_v[i], nkv, hd) == 0
        assert kv.append(0, i, rows_k[i].reshape(1, nkv, hd), rows_v[i].reshape(1, nkv, hd)) == 0
    gk, gv = kv.read_f16(0, 0, cap)
    assert np.array_equal(gk, ok) and np.array_equal(gv, ov)
    kv.close()



@pytest.mark.parametrize("nkv,hd,theta,n_rot_pairs,pos0,chunks", [
    (8, 128, 1e6, 0, 0, [1, 1, 31, 40, 1]),          # Qwen3-like, block boundaries
    (8, 128, 5e5, 0, 32760, [1, 7]),                 # long positions: thousands of range-reduction steps
    (4, 256, 1e6, 0, 5, [33]),
    (2, 64, 1e4, 10, 0, [3, 30]),                    # partial rotary: only 10 of 32 pairs rotate
])
def test_append_rope_cache_bits_equal_rotate_then_truncate(nkv, hd, theta, n_rot_pairs, pos0, chunks):
    """K rotated on the device inside the append must leave the same cache bits
    as the reference order of operations: wri_op_rope on the host, then the
    truncating append.  V is untouched by the rotation."""
    total = sum(chunks)
    kv = hipattn.KVCache(1, hd, nkv, pos0 + total)
    k32 = synth.normal(300 + hd, (total, nkv, hd), std=2.0)
    v32 = synth.normal(301 + hd, (total, nkv, hd), std=2.0)
    at = 0
    for n in chunks:
        print("append_rope", nkv, hd, "pos", pos0 + at, "n", n, flush=True)
        tab = oracle.rope_table(n, hd, pos0 + at, theta, n_rot_pairs)
        assert kv.append_rope(0, pos0 + at, k32[at:at + n], v32[at:at + n], tab) == hipattn.OK
        at += n
    want_k = synth.f32_to_f16_trunc(oracle.rope(k32, pos0, theta, n_rot_pairs))
    want_v = synth.f32_to_f16_trunc(v32)
    got_k, got_v = kv.read_f16(0, pos0, total)
    assert got_k.tobytes() == want_k.tobytes()
    assert got_v.tobytes() == want_v.tobytes()
    kv.close()


def test_rope_dev_equals_reference_rotation_and_error_contract():
    rows, heads, hd = 5, 16, 128
    x = synth.normal(310, (rows, heads, hd))
    tab = oracle.rope_table(rows, hd, 1000, 1e6)
    xd = hipattn.DeviceBuffer.from_host(x)
    td = hipattn.DeviceBuffer.from_host(tab)
    hipattn.rope_dev(xd, td, rows, heads, hd, tab.shape[1])
    hipattn.sync()
    got = xd.to_host((rows, heads, hd))
    assert got.tobytes() == oracle.rope(x, 1000, 1e6).tobytes()
    lib = hipattn.lib()
    assert lib.wr_hip_attn_rope_dev(None, td.p, rows, heads, hd, 64) == hipattn.ERR_INVAL
    assert lib.wr_hip_attn_rope_dev(xd.p, td.p, rows, heads, hd, 65) == hipattn.ERR_INVAL
    assert lib.wr_hip_attn_rope_dev(xd.p, td.p, rows, heads, 127, 10) == hipattn.ERR_INVAL
    kv = hipattn.KVCache(1, hd, 2, 4)
    k = synth.normal(311, (2, 2, hd))
    assert kv.append_rope(0, 3, k, k, tab[:2]) == hipattn.ERR_CTX_FULL      # writes nothing
    assert lib.wr_hip_attn_append_rope(kv.h, 0, 0, 1, k.ctypes.data, k.ctypes.data, None, 4) == hipattn.ERR_INVAL
    kv.close(); xd.free(); td.free()

# ------------------------------------------------------------------ decode --

def _run_decode(nq, nkv, hd, ctx, sc=0.0, win=0, seed=1, rows=None, generic=False, keys_per_wg=0):
    rows = rows or ctx
    q = synth.normal(seed, (nq, hd))
    if sc >= 1.0:
        q *= np.float32(0.125)      # keep the score range below the reference exp's defect band
    _k32, _v32, k16, v16 = util.make_kv(seed + 10, rows, nkv, hd)
    kv = hipattn.KVCache(1, hd, nkv, rows)
    kv.write_f16(0, 0, k16, v16)
    hipattn.set_tuning(keys_per_wg, generic)
    got = kv.decode(0, ctx, q, sc, win)
    hipattn.set_tuning(0, False)
    want = util.oracle_decode(q, k16, v16, ctx, sc, win)
    kv.close()
    return got, want


@pytest.mark.parametrize("ctx", [128, 512, 2048, 8192])
def test_decode_qwen3_shape_context_sweep(ctx):
    print("decode 16/8/128 ctx", ctx, flush=True)
    got, want = _run_decode(16, 8, 128, ctx, seed=synth.config_seed(2, ctx % 251))
    print("  errors", util.assert_close(got, want, f"ctx={ctx}"), flush=True)


@pytest.mark.parametrize("nq,nkv,hd,ctx,sc,win", [
    (32, 8, 128, 4096, 0.0, 0),        # Llama-3-8B shape
    (32, 8, 128, 1000, 0.0, 0),        # ragged: not a multiple of the 32-key tile
    (8, 4, 256, 3000, 0.0, 0),         # Gemma-class shape
    (8, 4, 256, 3000, 1.0, 1024),      # explicit scale 1.0 and sliding window
    (4, 4, 64, 777, 0.0, 0),           # MHA, head_dim 64
    (8, 1, 64, 300, 0.0, 0),           # group of 8
    (16, 8, 128, 1, 0.0, 0),           # a single key: output is the V row
    (16, 8, 128, 33, 0.0, 0),
    (16, 8, 128, 2048, 0.0, 100),      # window inside one workgroup's span
    (16, 8, 128, 2048, 0.0, 1999),
    (16, 8, 128, 2048, 0.0, 5000),     # window larger than the context: no masking
    (16, 8, 128, 700, 0.25, 0),        # scale override
])
def test_decode_shapes_windows_scales(nq, nkv, hd, ctx, sc, win):
    print("decode", nq, nkv, hd, ctx, sc, win, flush=True)
    got, want = _run_decode(nq, nkv, hd, ctx, sc, win, seed=ctx + win)
    print("  errors", util.assert_close(got, want), flush=True)


@pytest.mark.parametrize("nq,nkv,hd,ctx,sc,win", [
    (4, 2, 32, 200, 0.0, 16),          # head_dim 32: generic kernel
    (2, 1, 16, 96, 0.0, 0),
    (4, 1, 4, 8, 0.0, 4),              # the reference self-test's tiny shape
    (3, 3, 20, 50, 0.0, 0),            # odd head_dim
    (32, 2, 128, 500, 0.0, 0),         # group of 16: beyond the MFMA kernel's group limit
    (2, 1, 1024, 70, 0.0, 0),          # largest head_dim
])
def test_decode_generic_shapes(nq, nkv, hd, ctx, sc, win):
    print("decode generic", nq, nkv, hd, ctx, sc, win, flush=True)
    got, want = _run_decode(nq, nkv, hd, ctx, sc, win, seed=ctx)
    print("  errors", util.assert_close(got, want), flush=True)


@pytest.mark.parametrize("keys_per_wg", [32, 128, 4096, 1 << 20])
def test_split_k_partition_does_not_change_the_result(keys_per_wg):
    # any partition of the keys must give the unsplit result within tolerance;
    # one split (direct write) and many splits (partials + combine) both covered
    print("split-K keys_per_wg", keys_per_wg, flush=True)
    got, want = _run_decode(32, 8, 128, 3001, seed=5, keys_per_wg=keys_per_wg)
    util.assert_close(got, want)
    got_g, _ = _run_decode(32, 8, 128, 3001, seed=5, keys_per_wg=keys_per_wg, generic=True)
    util.assert_close(got_g, want, "generic")
    # the two device implementations agree far inside the tolerance
    assert util.errors(got, got_g)[0] < 2e-4


def test_rows_above_the_cursor_are_never_trusted():
    nq, nkv, hd, rows, ctx = 16, 8, 128, 512, 300
    q = synth.normal(3, (nq, hd))
    _a, _b, k16, v16 = util.make_kv(30, rows, nkv, hd)
    k_bad, v_bad = k16.copy(), v16.copy()
    k_bad[ctx:] = 0x7E00          # NaN bit patterns above the cursor
    v_bad[ctx:] = 0x7C00          # +inf
    kv = hipattn.KVCache(1, hd, nkv, rows)
    kv.write_f16(0, 0, k_bad, v_bad)
    got = kv.decode(0, ctx, q)
    util.assert_close(got, util.oracle_decode(q, k16, v16, ctx))
    kv.close()


@pytest.mark.parametrize("case", [c for c in cases.ATTN_CASES if c[9] == "f16" and c[1] == 1],
                         ids=lambda c: c[0])
def test_decode_against_reference_golden_outputs(case):
    # expected outputs written by the compiled reference (tests/golden)
    name, _sq, nq, nkv, hd, rows, seq_k, sc, win, _dt = case
    print("golden", name, flush=True)
    import os
    gold = np.load(os.path.join(os.path.dirname(__file__), "golden", "attn_golden.npz"))[name]
    q, k16, v16 = cases.attn_inputs(case)
    kv = hipattn.KVCache(1, hd, nkv, rows)
    kv.write_f16(0, 0, k16, v16)
    got = kv.decode(0, seq_k or rows, q[0], sc, win)
    util.assert_close(got, gold[0], name)
    kv.close()


# ----------------------------------------------------------------- batched --

def test_batched_ragged_llama_shape_equals_serial_and_oracle():
    nq, nkv, hd, S = 32, 8, 128, 16
    ctxs = synth.ragged_contexts(synth.config_seed(3, 0), S, 256, 4096)
    print("batched ctx", ctxs.tolist(), flush=True)
    caches, qs, kvs = [], [], []
    for i, ctx in enumerate(ctxs):
        q = synth.normal(synth.config_seed(3, 10 + i), (nq, hd))
        _a, _b, k16, v16 = util.make_kv(synth.config_seed(3, 40 + 2 * i), int(ctx), nkv, hd)
        kv = hipattn.KVCache(1, hd, nkv, int(ctx))
        kv.write_f16(0, 0, k16, v16)
        caches.append(kv); qs.append(q); kvs.append((k16, v16))
    outs = hipattn.decode_batched(caches, 0, ctxs, qs)
    for i in range(S):
        want = util.oracle_decode(qs[i], kvs[i][0], kvs[i][1], int(ctxs[i]))
        util.assert_close(outs[i], want, f"session {i}")
    # serial per-session stepping is bit-identical: the key partition of a
    # session depends on that session alone, and sessions never share arithmetic
    for i in range(S):
        single = caches[i].decode(0, int(ctxs[i]), qs[i])
        assert np.array_equal(single, outs[i]), f"session {i}"
    # ... also under a forced finer partition (many splits, in-kernel merge)
    hipattn.set_tuning(256, False)
    outs_fine = hipattn.decode_batched(caches, 0, ctxs, qs)
    for i in range(S):
        single = caches[i].decode(0, int(ctxs[i]), qs[i])
        assert np.array_equal(single, outs_fine[i]), f"session {i}"
        assert util.errors(outs_fine[i], outs[i])[0] < 1e-5
    hipattn.set_tuning(0, False)
    for kv in caches:
        kv.close()


def test_decode_step_loop_append_then_attend():
    # eight decode steps, each appending one position per session and then
    # attending (the long-context workload's step shape, at a short context)
    nq, nkv, hd, S, base = 8, 4, 256, 3, 250
    caches, k16s, v16s = [], [], []
    for i in range(S):
        kv = hipattn.KVCache(1, hd, nkv, base + 8)
        _a, _b, k16, v16 = util.make_kv(900 + i, base + 8, nkv, hd)
        kv.write_f16(0, 0, k16[:base], v16[:base])
        caches.append(kv); k16s.append(k16); v16s.append(v16)
    for step in range(8):
        qs = [synth.normal(1000 + 10 * step + i, (nq, hd)) for i in range(S)]
        for i in range(S):
            kn = synth.normal(2000 + 10 * step + i, (1, nkv, hd))
            vn = synth.normal(3000 + 10 * step + i, (1, nkv, hd))
            assert caches[i].append(0, base + step, kn, vn) == hipattn.OK
            k16s[i][base + step] = synth.f32_to_f16_trunc(kn)[0]
            v16s[i][base + step] = synth.f32_to_f16_trunc(vn)[0]
        outs = hipattn.decode_batched(caches, 0, [base + step + 1] * S, qs)
        for i in range(S):
            util.assert_close(outs[i], util.oracle_decode(qs[i], k16s[i], v16s[i], base + step + 1),
                              f"step {step} session {i}")
    for kv in caches:
        kv.close()


# ---------------------------------------------------------- error contract --

def test_error_contract():
    import ctypes as C
    lib = hipattn.lib()
    kv = hipattn.KVCache(2, [128, 0], 8, 64)      # layer 1 has no storage (shared layer)
    q = np.zeros((16, 128), dtype=np.float32)
    out = np.zeros_like(q)
    calls0 = lib.wr_hip_attn_calls()
    dec = lambda layer, seq_k, nq=16, qq=q: lib.wr_hip_attn_decode(      # noqa: E731
        kv.h, layer, seq_k, qq.ctypes.data, out.ctypes.data, nq, 0.0, 0)
    assert dec(0, 0) == hipattn.ERR_INVAL                    # empty sequence
    assert dec(0, 65) == hipattn.ERR_INVAL                   # beyond the allocation
    assert dec(0, hipattn.ATTN_MAX_SEQ + 1) == hipattn.ERR_LIMIT     # cap: refused, never clamped
    assert dec(1, 10) == hipattn.ERR_INVAL                   # layer without storage
    assert dec(2, 10) == hipattn.ERR_INVAL
    assert dec(0, 10, nq=12) == hipattn.ERR_INVAL            # nq % nkv != 0
    # calls refused for their shapes count, as in the reference, where the counter
    # sits between the pointer checks and the shape checks (kernels.c:1418-1423) ...
    assert lib.wr_hip_attn_calls() == calls0 + 6
    assert lib.wr_hip_attn_decode(kv.h, 0, 10, None, out.ctypes.data, 16, 0.0, 0) == hipattn.ERR_INVAL
    assert lib.wr_hip_attn_decode(None, 0, 10, q.ctypes.data, out.ctypes.data, 16, 0.0, 0) == hipattn.ERR_INVAL
    assert lib.wr_hip_attn_calls() == calls0 + 6             # ... calls refused for a null pointer do not
    calls = lib.wr_hip_attn_calls()
    assert dec(0, 10) == hipattn.OK
    assert lib.wr_hip_attn_calls() == calls + 1              # one count per session-layer call
    h = C.c_void_p()
    hd = (C.c_uint32 * 1)(128)
    assert lib.wr_hip_attn_kv_create(1, hd, 8, hipattn.ATTN_MAX_SEQ + 1, C.byref(h)) == hipattn.ERR_LIMIT
    assert lib.wr_hip_attn_kv_create(65, hd, 8, 16, C.byref(h)) == hipattn.ERR_LIMIT
    assert lib.wr_hip_attn_kv_create(1, hd, 0, 16, C.byref(h)) == hipattn.ERR_INVAL
    big = (C.c_uint32 * 1)(2048)
    assert lib.wr_hip_attn_kv_create(1, big, 8, 16, C.byref(h)) == hipattn.ERR_LIMIT
    # batch limits: 0 and 17 sessions are refused (reference batch.c:129)
    kvp = (C.c_void_p * 17)(*([kv.h] * 17))
    sk = (C.c_uint32 * 17)(*([10] * 17))
    ptrs = (C.c_void_p * 17)(*([q.ctypes.data] * 17))
    outs = (C.c_void_p * 17)(*([out.ctypes.data] * 17))
    assert lib.wr_hip_attn_decode_batched(0, kvp, 0, sk, ptrs, outs, 16, 0.0, 0) == hipattn.ERR_LIMIT
    assert lib.wr_hip_attn_decode_batched(17, kvp, 0, sk, ptrs, outs, 16, 0.0, 0) == hipattn.ERR_LIMIT
    # the same session twice in one batch is refused (reference batch.c:135-136)
    assert lib.wr_hip_attn_decode_batched(2, kvp, 0, sk, ptrs, outs, 16, 0.0, 0) == hipattn.ERR_INVAL
    assert lib.wr_hip_attn_init(0) == hipattn.ERR_STATE      # single engine per process
    kv.close()


def test_batched_append_writes_the_same_bits_as_single_appends():
    # one row per session in one launch, sessions at different positions and
    # capacities; the cache must hold what per-session appends put there, and
    # neighbouring rows must be untouched
    import ctypes as C
    nkv, hd, n = 4, 128, 5
    caps = [40, 64, 33, 100, 70]
    pos = [0, 31, 32, 63, 69]
    k = synth.normal(501, (n, nkv, hd), std=3.0)
    v = synth.normal(502, (n, nkv, hd), std=3.0)
    batch = [hipattn.KVCache(2, hd, nkv, c) for c in caps]
    single = [hipattn.KVCache(2, hd, nkv, c) for c in caps]
    kd, vd = hipattn.DeviceBuffer.from_host(k), hipattn.DeviceBuffer.from_host(v)
    lib = hipattn.lib()
    hs = (C.c_void_p * n)(*[c.h for c in batch])
    ps = (C.c_uint32 * n)(*pos)
    assert lib.wr_hip_attn_append_batched_dev(n, hs, 1, ps, kd.p, vd.p) == hipattn.OK
    hipattn.sync()
    for i in range(n):
        assert single[i].append(1, pos[i], k[i:i + 1], v[i:i + 1]) == 0
        gk, gv = batch[i].read_f16(1, 0, caps[i])
        wk, wv = single[i].read_f16(1, 0, caps[i])
        assert np.array_equal(gk, wk) and np.array_equal(gv, wv), i
        assert np.array_equal(gk[pos[i]], synth.f32_to_f16_trunc(k[i]))
    # a full cache anywhere in the batch refuses the whole call
    ps_full = (C.c_uint32 * n)(*[0, 31, 33, 63, 69])
    assert lib.wr_hip_attn_append_batched_dev(n, hs, 1, ps_full, kd.p, vd.p) == hipattn.ERR_CTX_FULL
    assert lib.wr_hip_attn_append_batched_dev(0, hs, 1, ps, kd.p, vd.p) == hipattn.ERR_LIMIT
    hs_dup = (C.c_void_p * 2)(batch[0].h, batch[0].h)
    assert lib.wr_hip_attn_append_batched_dev(2, hs_dup, 1, ps, kd.p, vd.p) == hipattn.ERR_INVAL
    for c in batch + single:
        c.close()
    kd.free()
    vd.free()


def test_work_list_at_its_largest():
    # 16 sessions, each cut into the maximum of 64 key splits: 1024 work-list
    # entries (the list's capacity), merged in-kernel; the longest-first order
    # and the per-session results must be unaffected by the other sessions
    nq, nkv, hd, S = 8, 2, 64, 16
    ctxs = [2048 - 31 * i for i in range(S)]
    caches, qs, wants = [], [], []
    for i, ctx in enumerate(ctxs):
        q = synth.normal(600 + i, (nq, hd))
        _a, _b, k16, v16 = util.make_kv(700 + 2 * i, ctx, nkv, hd)
        kv = hipattn.KVCache(1, hd, nkv, ctx)
        kv.write_f16(0, 0, k16, v16)
        caches.append(kv); qs.append(q)
        wants.append(util.oracle_decode(q, k16, v16, ctx))
    hipattn.set_tuning(32, False)                 # one 32-key tile per workgroup -> 64 splits each
    outs = hipattn.decode_batched(caches, 0, ctxs, qs)
    for i in range(S):
        util.assert_close(outs[i], wants[i], f"session {i}")
        assert np.array_equal(caches[i].decode(0, ctxs[i], qs[i]), outs[i]), f"session {i}"
    hipattn.set_tuning(0, False)
    for kv in caches:
        kv.close()


def test_threads_that_come_and_go_get_a_working_stream():
    # Every calling thread submits through a stream of its own in the library;
    # a thread that ends hands its stream and buffers on to the next new thread.
    # Thirty threads one after another, then eight at once, each attend the
    # same session: all must produce the main thread's bits.
    import threading
    nq, nkv, hd, ctx = 32, 8, 128, 3000
    _a, _b, k16, v16 = util.make_kv(9100, ctx, nkv, hd)
    kvs = []
    for _ in range(8):                            # one cache per concurrent thread (a cache is not shared)
        kv = hipattn.KVCache(1, hd, nkv, ctx)
        kv.write_f16(0, 0, k16, v16)
        kvs.append(kv)
    q = synth.normal(9101, (nq, hd))
    want = kvs[0].decode(0, ctx, q)
    util.assert_close(want, util.oracle_decode(q, k16, v16, ctx), "main thread")
    bad = []

    def job(i):
        try:
            got = kvs[i % 8].decode(0, ctx, q)
            if not np.array_equal(got, want):
                bad.append(i)
        except Exception as e:
            bad.append(repr(e))
    for i in range(30):
        th = threading.Thread(target=job, args=(i,))
        th.start()
        th.join()
    ths = [threading.Thread(target=job, args=(100 + i,)) for i in range(8)]
    for th in ths:
        th.start()
    for th in ths:
        th.join()
    for kv in kvs:
        kv.close()
    assert not bad, bad


# ---------------------------------------------- row step inside the attention launch --

@pytest.mark.parametrize("nq,nkv,norm,rot_pairs,window,kpw,base", [
    (16, 8, True, 0, 0, 0, 0),       # Qwen3: per-head norms, full rotation
    (32, 8, False, 0, 0, 0, 0),      # Llama: no norms
    (32, 8, True, 24, 0, 0, 0),      # partial rotation
    (16, 8, True, 0, 300, 0, 0),     # sliding window
    (16, 8, True, 0, 0, 64, 0),      # forced fine key splits: the new row's tile is the last split's
    (16, 8, True, 0, 0, 0, 8150),    # long sessions: a workgroup of the batch works through two splits,
                                     # one of the lone session through one; the new row's tile is in the second
])
def test_append_and_decode_in_one_launch_equals_the_two_calls(nq, nkv, norm, rot_pairs, window, kpw, base):
    # wr_hip_attn_append_decode_batched_dev against wr_hip_rows_qkv_append_dev +
    # wr_hip_attn_decode_batched_dev on twin caches: the same output bits and
    # the same cache bytes, for one session and for a ragged batch, at positions
    # on every side of a 32-key tile edge; both also against the oracle.
    import ctypes as C
    hd, eps, theta = 128, 1e-6, 1e6
    lib = hipattn.lib()
    positions = [base + p for p in (0, 1, 31, 32, 33, 63, 64, 500, 1023, 1024, 2047, 2500, 95, 96, 1999, 7)]
    cap = base + 2600
    n_rot = rot_pairs if rot_pairs else hd // 2
    width = (nq + 2 * nkv) * hd
    qw = synth.normal(9300, (hd,), std=1.0) if norm else None
    kw = synth.normal(9301, (hd,), std=1.0) if norm else None
    qwd = hipattn.DeviceBuffer.from_host(qw) if norm else None
    kwd = hipattn.DeviceBuffer.from_host(kw) if norm else None
    for n in (1, 16):
        pos = positions[:n] if n > 1 else [base + 777]
        print("fused step", nq, nkv, norm, rot_pairs, window, kpw, base, "n", n, flush=True)
        twins = []
        for i in range(n):
            _a, _b, k16, v16 = util.make_kv(9400 + 2 * i, cap, nkv, hd)
            pair = []
            for _ in range(2):
                kv = hipattn.KVCache(1, hd, nkv, cap)
                kv.write_f16(0, 0, k16, v16)          # rows at and above pos hold other data: they must not matter
                pair.append(kv)
            twins.append(pair)
        x = synth.normal(9500 + n, (n, width), std=1.5)
        xd = hipattn.DeviceBuffer.from_host(x)
        tab = np.concatenate([oracle.rope_table(1, hd, p, theta, rot_pairs) for p in pos])
        td = hipattn.DeviceBuffer.from_host(tab)
        pp = (C.c_uint32 * n)(*pos)
        sk = (C.c_uint32 * n)(*[p + 1 for p in pos])
        qn = qwd.p if norm else None
        kn = kwd.p if norm else None
        hipattn.set_tuning(kpw, False)
        # two calls, on the first twin of every session
        kv_a = (C.c_void_p * n)(*[t[0].h for t in twins])
        q_dev = hipattn.DeviceBuffer(n * nq * hd * 4)
        o_a = hipattn.DeviceBuffer.from_host(np.full((n, nq, hd), 3.0, dtype=np.float32))
        assert lib.wr_hip_rows_qkv_append_dev(xd.p, width, n, nq, qn, kn, eps, td.p, n_rot, n, kv_a, 0, pp,
                                              q_dev.p, 0) == hipattn.OK
        assert lib.wr_hip_attn_decode_batched_dev(n, kv_a, 0, sk, q_dev.p, o_a.p, nq, 0.0, window) == hipattn.OK
        # one call, on the second twin
        kv_b = (C.c_void_p * n)(*[t[1].h for t in twins])
        o_b = hipattn.DeviceBuffer.from_host(np.full((n, nq, hd), -4.0, dtype=np.float32))
        calls = int(hipattn.lib().wr_hip_attn_calls())
        assert lib.wr_hip_attn_append_decode_batched_dev(n, kv_b, 0, pp, xd.p, width, nq, qn, kn, eps, td.p, n_rot,
                                                         o_b.p, 0.0, window) == hipattn.OK
        assert int(hipattn.lib().wr_hip_attn_calls()) == calls + n
        hipattn.sync()
        hipattn.set_tuning(0, False)
        got_a, got_b = o_a.to_host((n, nq, hd)), o_b.to_host((n, nq, hd))
        differ = [(i, pos[i], float(np.abs(got_a[i] - got_b[i]).max()),
                   [int(h) for h in np.argwhere(np.abs(got_a[i] - got_b[i]).max(axis=1) > 0)[:, 0]])
                  for i in range(n) if not np.array_equal(got_a[i], got_b[i])]
        assert differ == [], f"outputs differ from the two-call path: (session, position, max diff, heads) {differ}"
        for i in range(n):
            ka, va = twins[i][0].read_f16(0, 0, pos[i] + 1)
            kb, vb = twins[i][1].read_f16(0, 0, pos[i] + 1)
            assert np.array_equal(ka, kb) and np.array_equal(va, vb), f"cache of session {i} differs"
            util.assert_close(got_b[i], util.oracle_decode(q_dev.to_host((n, nq, hd))[i], ka, va, pos[i] + 1, 0.0, window),
                              f"session {i}")
        # refusals: a full cache (nothing written), a shape the one-launch form does not take
        full = (C.c_uint32 * n)(*([cap] + list(pos[1:])))
        assert lib.wr_hip_attn_append_decode_batched_dev(n, kv_b, 0, full, xd.p, width, nq, qn, kn, eps, td.p, n_rot,
                                                         o_b.p, 0.0, window) == hipattn.ERR_CTX_FULL
        calls = int(hipattn.lib().wr_hip_attn_calls())
        assert lib.wr_hip_attn_append_decode_batched_dev(n, kv_b, 0, pp, xd.p, width + 2, nq, qn, kn, eps, td.p, n_rot,
                                                         o_b.p, 0.0, window) == hipattn.ERR_UNSUPPORTED
        assert int(hipattn.lib().wr_hip_attn_calls()) == calls
        hipattn.sync()
        assert np.array_equal(o_b.to_host((n, nq, hd)), got_b)
        for b in (xd, td, q_dev, o_a, o_b):
            b.free()
        for pair in twins:
            for kv in pair:
                kv.close()
    for b in (qwd, kwd):
        if b is not None:
            b.free()


def test_append_and_decode_in_one_launch_with_sixteen_short_sessions_paired_splits():
    # Sixteen sessions of 500 to 640 keys at the Llama shape: a launch that fills
    # the device, so a workgroup of a short session takes two consecutive splits,
    # and the one that makes the new row runs a body split followed by the tail
    # split.  Same output bits and cache bytes as the two-call path, and the oracle.
    import ctypes as C
    nq, nkv, hd, eps, theta, n = 32, 8, 128, 1e-6, 5e5, 16
    lib = hipattn.lib()
    pos = [500 + 9 * i + (i % 3) for i in range(n)]           # 500 .. 637, on both sides of tile edges
    cap = 700
    width = (nq + 2 * nkv) * hd
    twins = []
    for i in range(n):
        _a, _b, k16, v16 = util.make_kv(9800 + 2 * i, cap, nkv, hd)
        pair = []
        for _ in range(2):
            kv = hipattn.KVCache(1, hd, nkv, cap)
            kv.write_f16(0, 0, k16, v16)
            pair.append(kv)
        twins.append(pair)
    x = synth.normal(9850, (n, width), std=1.5)
    xd = hipattn.DeviceBuffer.from_host(x)
    td = hipattn.DeviceBuffer.from_host(np.concatenate([oracle.rope_table(1, hd, p, theta, 0) for p in pos]))
    pp = (C.c_uint32 * n)(*pos)
    sk = (C.c_uint32 * n)(*[p + 1 for p in pos])
    kv_a = (C.c_void_p * n)(*[t[0].h for t in twins])
    kv_b = (C.c_void_p * n)(*[t[1].h for t in twins])
    q_dev = hipattn.DeviceBuffer(n * nq * hd * 4)
    o_a = hipattn.DeviceBuffer.from_host(np.full((n, nq, hd), 3.0, dtype=np.float32))
    o_b = hipattn.DeviceBuffer.from_host(np.full((n, nq, hd), -4.0, dtype=np.float32))
    assert lib.wr_hip_rows_qkv_append_dev(xd.p, width, n, nq, None, None, eps, td.p, hd // 2, n, kv_a, 0, pp,
                                          q_dev.p, 0) == hipattn.OK
    assert lib.wr_hip_attn_decode_batched_dev(n, kv_a, 0, sk, q_dev.p, o_a.p, nq, 0.0, 0) == hipattn.OK
    assert lib.wr_hip_attn_append_decode_batched_dev(n, kv_b, 0, pp, xd.p, width, nq, None, None, eps, td.p, hd // 2,
                                                     o_b.p, 0.0, 0) == hipattn.OK
    hipattn.sync()
    got_a, got_b = o_a.to_host((n, nq, hd)), o_b.to_host((n, nq, hd))
    differ = [(i, pos[i], float(np.abs(got_a[i] - got_b[i]).max())) for i in range(n)
              if not np.array_equal(got_a[i], got_b[i])]
    assert differ == [], f"outputs differ from the two-call path: (session, position, max diff) {differ}"
    qh = q_dev.to_host((n, nq, hd))
    for i in range(n):
        ka, va = twins[i][0].read_f16(0, 0, pos[i] + 1)
        kb, vb = twins[i][1].read_f16(0, 0, pos[i] + 1)
        assert np.array_equal(ka, kb) and np.array_equal(va, vb), f"cache of session {i} differs"
        util.assert_close(got_b[i], util.oracle_decode(qh[i], ka, va, pos[i] + 1, 0.0, 0), f"session {i}")
    for b in (xd, td, q_dev, o_a, o_b):
        b.free()
    for pair in twins:
        for kv in pair:
            kv.close()


def test_append_and_decode_in_one_launch_refuses_what_it_must():
    # argument contract of wr_hip_attn_append_decode_batched_dev: pointers, counts,
    # head shapes and strides are checked before anything is counted or written
    import ctypes as C
    lib = hipattn.lib()
    nq, nkv, hd, cap = 16, 8, 128, 96
    width = (nq + 2 * nkv) * hd
    kv = hipattn.KVCache(1, hd, nkv, cap)
    D = hipattn.DeviceBuffer
    x = D.from_host(synth.normal(9701, (1, width)))
    w = D.from_host(np.ones(hd, dtype=np.float32))
    tab = D.from_host(oracle.rope_table(1, hd, 5, 1e6, 0))
    out = D.from_host(np.full((1, nq, hd), 3.0, dtype=np.float32))
    kvs = (C.c_void_p * 1)(kv.h)
    pos = (C.c_uint32 * 1)(5)
    call = lambda n=1, k=kvs, p=pos, xp=x.p, ld=width, q=nq, qn=w.p, kn=w.p, cs=tab.p, nr=hd // 2, o=out.p, layer=0: \
        lib.wr_hip_attn_append_decode_batched_dev(n, k, layer, p, xp, ld, q, qn, kn, 1e-6, cs, nr, o, 0.0, 0)   # noqa: E731
    calls = int(lib.wr_hip_attn_calls())
    assert call(k=None) == hipattn.ERR_INVAL
    assert call(p=None) == hipattn.ERR_INVAL
    assert call(xp=None) == hipattn.ERR_INVAL
    assert call(o=None) == hipattn.ERR_INVAL
    assert call(n=0) == hipattn.ERR_LIMIT
    assert call(n=17) == hipattn.ERR_LIMIT
    assert call(layer=1) == hipattn.ERR_INVAL               # the cache has one layer
    assert call(q=12) == hipattn.ERR_INVAL                  # 12 query heads over 8 KV heads
    assert call(qn=None) == hipattn.ERR_INVAL               # one norm vector without the other
    assert call(cs=None) == hipattn.ERR_INVAL               # a rotation without its table
    assert call(nr=hd) == hipattn.ERR_INVAL                 # more pairs than half the head
    assert call(ld=width - 4) == hipattn.ERR_INVAL          # rows shorter than Q + K + V
    assert call(nr=4) == hipattn.ERR_UNSUPPORTED            # pairs not a multiple of eight: the two calls take it
    assert int(lib.wr_hip_attn_calls()) == calls            # nothing counted
    hipattn.sync()
    assert np.all(out.to_host((1, nq, hd)) == 3.0)          # nothing written
    k_now, v_now = kv.read_f16(0, 0, 6)
    assert not k_now.any() and not v_now.any()
    # and the call itself, for the record
    assert call() == hipattn.OK
    assert int(lib.wr_hip_attn_calls()) == calls + 1
    for b in (x, w, tab, out):
        b.free()
    kv.close()


# ---------------------- append + decode in one call, rows from host memory --

@pytest.mark.parametrize("nq,nkv,hd,base,steps,sc,win", [
    (32, 8, 128, 700, 3, 0.0, 0),        # one launch (head dim 128, group 4)
    (16, 8, 128, 0, 4, 0.0, 0),          # from an empty cache: the first key is the row itself
    (64, 8, 128, 333, 2, 0.07, 100),     # group 8, scale override, sliding window
    (8, 8, 128, 31, 3, 0.0, 0),          # group 1, across a 32-position block edge
    (8, 4, 256, 250, 2, 0.0, 0),         # two launches back to back: head dim 256
    (8, 2, 64, 95, 3, 0.0, 16),          # head dim 64
    (6, 2, 80, 17, 2, 0.0, 0),           # a shape the generic kernels take
])
def test_append_decode_from_host_rows_equals_the_two_calls(nq, nkv, hd, base, steps, sc, win):
    cap = base + steps
    _a, _b, k16, v16 = util.make_kv(7100 + nq + hd, cap, nkv, hd)
    one = hipattn.KVCache(1, hd, nkv, cap)
    two = hipattn.KVCache(1, hd, nkv, cap)
    if base:
        one.write_f16(0, 0, k16[:base], v16[:base])
        two.write_f16(0, 0, k16[:base], v16[:base])
    calls0 = hipattn.lib().wr_hip_attn_calls()
    for s in range(steps):
        pos = base + s
        print("append+decode", nq, nkv, hd, "pos", pos, flush=True)
        kn = synth.normal(7200 + 3 * s, (nkv, hd), std=2.0)
        vn = synth.normal(7201 + 3 * s, (nkv, hd), std=2.0)
        q = synth.normal(7202 + 3 * s, (nq, hd))
        got = one.append_decode(0, pos, kn, vn, q, sc, win)
        assert two.append(0, pos, kn[None], vn[None]) == hipattn.OK
        want = two.decode(0, pos + 1, q, sc, win)
        assert np.array_equal(got, want), f"step {s}"
        k16[pos] = synth.f32_to_f16_trunc(kn)
        v16[pos] = synth.f32_to_f16_trunc(vn)
        util.assert_close(got, util.oracle_decode(q, k16, v16, pos + 1, sc, win), f"step {s}")
    gk, gv = one.read_f16(0, 0, cap)
    assert np.array_equal(gk, k16) and np.array_equal(gv, v16)
    # one attention call counted per step by each form
    assert hipattn.lib().wr_hip_attn_calls() == calls0 + 2 * steps
    one.close(); two.close()


@pytest.mark.parametrize("nq,nkv,hd", [(32, 8, 128), (8, 4, 256)])
def test_append_decode_batched_from_host_rows_equals_the_two_calls(nq, nkv, hd):
    S = 16 if hd == 128 else 5
    ctxs = synth.ragged_contexts(synth.config_seed(5, 1), S, 1, 3000)
    ctxs[0] = 1                                   # a session whose cache is empty before the step
    print("append+decode batched", nq, nkv, hd, ctxs.tolist(), flush=True)
    ones, twos, ks, vs, qs, kv16 = [], [], [], [], [], []
    for i, ctx in enumerate(int(c) for c in ctxs):
        _a, _b, k16, v16 = util.make_kv(7300 + i, ctx, nkv, hd)
        a = hipattn.KVCache(1, hd, nkv, ctx)
        b = hipattn.KVCache(1, hd, nkv, ctx)
        if ctx > 1:
            a.write_f16(0, 0, k16[:ctx - 1], v16[:ctx - 1])
            b.write_f16(0, 0, k16[:ctx - 1], v16[:ctx - 1])
        kn = synth.normal(7400 + i, (nkv, hd))
        vn = synth.normal(7500 + i, (nkv, hd))
        k16[ctx - 1] = synth.f32_to_f16_trunc(kn)
        v16[ctx - 1] = synth.f32_to_f16_trunc(vn)
        ones.append(a); twos.append(b); ks.append(kn); vs.append(vn); kv16.append((k16, v16))
        qs.append(synth.normal(7600 + i, (nq, hd)))
    got = hipattn.append_decode_batched(ones, 0, [int(c) - 1 for c in ctxs], ks, vs, qs)
    for i, ctx in enumerate(int(c) for c in ctxs):
        assert twos[i].append(0, ctx - 1, ks[i][None], vs[i][None]) == hipattn.OK
    want = hipattn.decode_batched(twos, 0, ctxs, qs)
    for i, ctx in enumerate(int(c) for c in ctxs):
        assert np.array_equal(got[i], want[i]), f"session {i}"
        util.assert_close(got[i], util.oracle_decode(qs[i], kv16[i][0], kv16[i][1], ctx), f"session {i}")
        gk, gv = ones[i].read_f16(0, 0, ctx)
        assert np.array_equal(gk, kv16[i][0]) and np.array_equal(gv, kv16[i][1]), f"session {i}"
    for kv in ones + twos:
        kv.close()


def test_append_decode_from_host_rows_refuses_what_it_must():
    import ctypes as C
    lib = hipattn.lib()
    nq, nkv, hd, cap = 16, 8, 128, 12
    kv = hipattn.KVCache(2, [hd, 0], nkv, cap)
    other = hipattn.KVCache(1, hd, nkv, 4)
    _a, _b, k16, v16 = util.make_kv(7700, cap, nkv, hd)
    kv.write_f16(0, 0, k16, v16)
    k = synth.normal(7701, (nkv, hd)); v = synth.normal(7702, (nkv, hd))
    q = synth.normal(7703, (nq, hd)); out = np.zeros_like(q)
    p = lambda a: a.ctypes.data                                        # noqa: E731
    call = lambda layer, pos, nq_=nq, kk=p(k), qq=p(q), oo=p(out): lib.wr_hip_attn_append_decode(   # noqa: E731
        kv.h, layer, pos, kk, p(v), qq, oo, nq_, 0.0, 0)
    calls0 = lib.wr_hip_attn_calls()
    assert call(0, cap) == hipattn.ERR_CTX_FULL                        # a full cache: refused ...
    assert call(0, cap + 5) == hipattn.ERR_CTX_FULL
    assert call(1, 3) == hipattn.ERR_INVAL                             # layer without storage
    assert call(2, 3) == hipattn.ERR_INVAL
    assert call(0, 3, nq_=12) == hipattn.ERR_INVAL                     # nq % nkv != 0
    assert call(0, 3, kk=None) == hipattn.ERR_INVAL
    assert call(0, 3, qq=None) == hipattn.ERR_INVAL
    assert call(0, 3, oo=None) == hipattn.ERR_INVAL
    assert lib.wr_hip_attn_append_decode(None, 0, 3, p(k), p(v), p(q), p(out), nq, 0.0, 0) == hipattn.ERR_INVAL
    assert lib.wr_hip_attn_calls() == calls0                           # ... none of them counted
    gk, gv = kv.read_f16(0, 0, cap)
    assert np.array_equal(gk, k16) and np.array_equal(gv, v16)         # ... and nothing written
    # batch: 0 and 17 sessions, the same session twice, one full session among good ones
    kvp = (C.c_void_p * 17)(*([kv.h] * 17))
    pos = (C.c_uint32 * 17)(*([3] * 17))
    arr = lambda a: (C.c_void_p * 17)(*([p(a)] * 17))                  # noqa: E731
    bat = lambda n, kvs=kvp, ps=pos: lib.wr_hip_attn_append_decode_batched(     # noqa: E731
        n, kvs, 0, ps, arr(k), arr(v), arr(q), arr(out), nq, 0.0, 0)
    assert bat(0) == hipattn.ERR_LIMIT
    assert bat(17) == hipattn.ERR_LIMIT
    assert bat(2) == hipattn.ERR_INVAL
    two = (C.c_void_p * 17)(kv.h, other.h, *([None] * 15))
    assert bat(2, two, (C.c_uint32 * 17)(3, 4, *([0] * 15))) == hipattn.ERR_CTX_FULL
    gk, gv = kv.read_f16(0, 0, cap)
    assert np.array_equal(gk, k16) and np.array_equal(gv, v16)         # the good session's row was not written
    assert bat(2, two, (C.c_uint32 * 17)(3, 3, *([0] * 15))) == hipattn.OK
    gk, _gv = kv.read_f16(0, 3, 1)
    assert np.array_equal(gk[0], synth.f32_to_f16_trunc(k))
    kv.close(); other.close()
