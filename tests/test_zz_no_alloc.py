"""The decode entry point that allocates nothing
(wr_hip_attn_decode_batched_dev_noalloc) against the ordinary one
(wr_hip_attn_decode_batched_dev), through the C ABI: same kernels, same key
partition, so the outputs must be equal bit for bit; both are also checked
against the CPU oracle (max-abs 2e-3, rel-L2 1e-3).  Two calls in a row share
the fixed scratch array, the second with a smaller input."""
import numpy as np
import pytest

from tests import util
from wayruntime_amd import hipattn, synth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _device():
    hipattn.init()
    yield
    hipattn.set_tuning(0, False)


def _sessions(seed, ctxs, nkv, hd):
    caches, kvs = [], []
    for i, ctx in enumerate(ctxs):
        _a, _b, k16, v16 = util.make_kv(seed + 2 * i, int(ctx), nkv, hd)
        kv = hipattn.KVCache(1, hd, nkv, int(ctx))
        kv.write_f16(0, 0, k16, v16)
        caches.append(kv)
        kvs.append((k16, v16))
    return caches, kvs


def _both(caches, ctxs, q, nq, hd):
    """Outputs of the ordinary and of the no-alloc entry point for one step."""
    n = len(caches)
    q_dev = hipattn.DeviceBuffer.from_host(q)
    # the two outputs start from different garbage so that a launch that wrote
    # nothing cannot pass
    o_ref = hipattn.DeviceBuffer.from_host(np.full((n, nq, hd), 7.0, dtype=np.float32))
    o_new = hipattn.DeviceBuffer.from_host(np.full((n, nq, hd), -9.0, dtype=np.float32))
    hipattn.decode_batched_dev(caches, 0, ctxs, q_dev, o_ref, nq)
    rc = hipattn.decode_batched_dev_noalloc(caches, 0, ctxs, q_dev, o_new, nq)
    assert rc == hipattn.OK, rc
    hipattn.sync()
    ref = o_ref.to_host((n, nq, hd))
    new = o_new.to_host((n, nq, hd))
    for b in (q_dev, o_ref, o_new):
        b.free()
    return ref, new


def test_no_alloc_decode_equals_the_ordinary_entry_point_twice_in_a_row():
    nq, nkv, hd = 32, 8, 128
    # first call: 16 ragged sessions, several key splits each (in-kernel merge
    # through the scratch array); second call: fewer, shorter sessions, so the
    # array still holds the first call's partials and tickets
    ctx_a = [4096, 300, 2500, 1111, 4000, 257, 3333, 2048, 1025, 777, 3900, 1500, 2222, 640, 3071, 999]
    ctx_b = [1000, 2000, 45]
    caches, kvs = _sessions(7100, ctx_a, nkv, hd)
    try:
        for call, (idx, seed) in enumerate([(list(range(16)), 7200), ([3, 7, 5], 7300)]):
            use = [caches[i] for i in idx]
            ctxs = [ctx_a[i] for i in idx] if call == 0 else ctx_b
            q = synth.normal(seed, (len(use), nq, hd))
            print("no-alloc call", call, "ctx", ctxs, flush=True)
            ref, new = _both(use, ctxs, q, nq, hd)
            assert np.array_equal(ref, new), f"call {call}: outputs differ from the ordinary entry point"
            for j, i in enumerate(idx):
                want = util.oracle_decode(q[j], kvs[i][0], kvs[i][1], int(ctxs[j]))
                util.assert_close(new[j], want, f"call {call} session {j}")
    finally:
        for kv in caches:
            kv.close()


def test_no_alloc_decode_with_the_finest_partition_and_a_window():
    # 64 key splits per session (forced), head_dim 256, sliding window: the
    # largest ticket / partial footprint per head, then a one-split call
    nq, nkv, hd = 8, 4, 256
    ctxs = [2048, 2048, 1999]
    caches, kvs = _sessions(7400, ctxs, nkv, hd)
    try:
        hipattn.set_tuning(32, False)
        q = synth.normal(7500, (3, nq, hd))
        n = len(caches)
        q_dev = hipattn.DeviceBuffer.from_host(q)
        o_ref = hipattn.DeviceBuffer(q.nbytes)
        o_new = hipattn.DeviceBuffer(q.nbytes)
        hipattn.decode_batched_dev(caches, 0, ctxs, q_dev, o_ref, nq, 0.0, 1500)
        assert hipattn.decode_batched_dev_noalloc(caches, 0, ctxs, q_dev, o_new, nq, 0.0, 1500) == hipattn.OK
        hipattn.sync()
        assert np.array_equal(o_ref.to_host((n, nq, hd)), o_new.to_host((n, nq, hd)))
        hipattn.set_tuning(0, False)
        small = [20, 31, 7]                     # one split each: no scratch use at all
        hipattn.decode_batched_dev(caches, 0, small, q_dev, o_ref, nq)
        assert hipattn.decode_batched_dev_noalloc(caches, 0, small, q_dev, o_new, nq) == hipattn.OK
        hipattn.sync()
        got = o_new.to_host((n, nq, hd))
        assert np.array_equal(o_ref.to_host((n, nq, hd)), got)
        for j in range(n):
            util.assert_close(got[j], util.oracle_decode(q[j], kvs[j][0], kvs[j][1], small[j]),
                              f"session {j}")
        for b in (q_dev, o_ref, o_new):
            b.free()
    finally:
        hipattn.set_tuning(0, False)
        for kv in caches:
            kv.close()


def test_no_alloc_decode_of_long_sessions_whose_workgroups_take_two_splits():
    # sessions of 8K keys and more are cut into sixteen splits; in a launch that
    # fills the device a workgroup works through two of them and the merging
    # workgroup is the last of eight, not of sixteen, to draw its ticket from the
    # array.  Then one of them alone (a workgroup per split) on the same array.
    nq, nkv, hd = 16, 8, 128
    ctxs = [8192, 9000, 12288, 16384, 8223, 10000, 8255, 11111]
    caches, kvs = _sessions(7400, ctxs, nkv, hd)
    q = synth.normal(7450, (len(ctxs), nq, hd))
    ref, new = _both(caches, ctxs, q, nq, hd)
    assert np.array_equal(ref, new)
    util.assert_close(new[3], util.oracle_decode(q[3], kvs[3][0], kvs[3][1], ctxs[3]), "session 3")
    ref1, new1 = _both(caches[4:5], ctxs[4:5], q[4:5], nq, hd)
    assert np.array_equal(ref1, new1)
    assert np.array_equal(new1[0], new[4])            # alone or in the full launch: the same bits
    for kv in caches:
        kv.close()


def test_no_alloc_decode_refuses_what_does_not_fit():
    # 16 sessions x 32 heads x 64 splits x (256 + 2) floats = 33.8 MB of partials:
    # more than the fixed array; refused with WR_HIP_ERR_LIMIT, nothing launched,
    # and the ordinary entry point still serves the same call
    nq, nkv, hd, S = 32, 8, 256, 16
    ctxs = [2048] * S
    caches = [hipattn.KVCache(1, hd, nkv, 2048) for _ in range(S)]   # zero-filled caches
    try:
        hipattn.set_tuning(32, False)
        q = synth.normal(7600, (S, nq, hd))
        q_dev = hipattn.DeviceBuffer.from_host(q)
        o_dev = hipattn.DeviceBuffer.from_host(np.full((S, nq, hd), 5.0, dtype=np.float32))
        assert hipattn.decode_batched_dev_noalloc(caches, 0, ctxs, q_dev, o_dev, nq) == hipattn.ERR_LIMIT
        hipattn.sync()
        assert np.all(o_dev.to_host((S, nq, hd)) == 5.0)             # untouched
        hipattn.decode_batched_dev(caches, 0, ctxs, q_dev, o_dev, nq)
        hipattn.sync()
        assert np.all(o_dev.to_host((S, nq, hd)) == 0.0)             # V is all zero
        # more heads than the fixed ticket array holds
        assert hipattn.decode_batched_dev_noalloc(caches[:1], 0, [8], q_dev, o_dev, 2048) == hipattn.ERR_LIMIT
        q_dev.free()
        o_dev.free()
    finally:
        hipattn.set_tuning(0, False)
        for kv in caches:
            kv.close()


def test_partials_of_one_launch_are_never_read_from_the_launch_before():
    # Two batches of different shape take turns on the one scratch array, back
    # to back without a host wait in between, so the partial rows a launch
    # finds there belong to the other batch: a workgroup that merged before
    # every partial of its own launch had landed would write a row that is
    # wrong, not merely old.  (A workgroup draws its ticket only after its own
    # partial stores have been acknowledged.)
    nq, nkv, hd = 32, 8, 128
    ctx_sets = [[1300, 3500, 2200, 2900], [4096, 2049, 600]]
    groups = [_sessions(7900 + 40 * t, ctxs, nkv, hd) for t, ctxs in enumerate(ctx_sets)]
    qs = [synth.normal(7950 + t, (len(ctxs), nq, hd)) for t, ctxs in enumerate(ctx_sets)]
    try:
        want, q_dev, outs = [], [], []
        for t, ctxs in enumerate(ctx_sets):
            q_dev.append(hipattn.DeviceBuffer.from_host(qs[t]))
            o = hipattn.DeviceBuffer(qs[t].nbytes)
            hipattn.decode_batched_dev(groups[t][0], 0, ctxs, q_dev[t], o, nq)
            hipattn.sync()
            want.append(o.to_host(qs[t].shape))
            o.free()
        rounds = 40
        for t in range(2):
            outs.append([hipattn.DeviceBuffer(qs[t].nbytes) for _ in range(rounds)])
        for r in range(rounds):
            for t, ctxs in enumerate(ctx_sets):
                assert hipattn.decode_batched_dev_noalloc(groups[t][0], 0, ctxs, q_dev[t], outs[t][r], nq) == hipattn.OK
        hipattn.sync()
        wrong = [(t, r) for t in range(2) for r in range(rounds)
                 if not np.array_equal(outs[t][r].to_host(qs[t].shape), want[t])]
        assert wrong == []
        for b in q_dev + outs[0] + outs[1]:
            b.free()
    finally:
        for caches, _ in groups:
            for kv in caches:
                kv.close()


def test_no_alloc_decode_from_several_threads_shares_the_one_array():
    # Every calling thread has its own stream in the library, but the scratch
    # array is one per device: launches that use it are chained by an event
    # whatever thread they come from.  Four threads each step their own
    # sessions twenty times through the no-alloc entry point; every output must
    # equal the ordinary entry point's (which uses per-thread partial buffers).
    import threading
    nq, nkv, hd = 32, 8, 128
    ctx_sets = [[3000, 1500, 2600], [4096, 2049], [1300, 3500, 2200, 2900], [2500]]
    groups = [_sessions(7700 + 40 * t, ctxs, nkv, hd) for t, ctxs in enumerate(ctx_sets)]
    qs = [synth.normal(7800 + t, (len(ctxs), nq, hd)) for t, ctxs in enumerate(ctx_sets)]
    # reference outputs, one thread, ordinary entry point
    want = []
    for t, ctxs in enumerate(ctx_sets):
        q_dev = hipattn.DeviceBuffer.from_host(qs[t])
        o = hipattn.DeviceBuffer(qs[t].nbytes)
        hipattn.decode_batched_dev(groups[t][0], 0, ctxs, q_dev, o, nq)
        hipattn.sync()
        want.append(o.to_host(qs[t].shape))
        q_dev.free(); o.free()
    bad = [None] * 4

    def job(t):
        try:
            ctxs = ctx_sets[t]
            q_dev = hipattn.DeviceBuffer.from_host(qs[t])
            o = hipattn.DeviceBuffer(qs[t].nbytes)
            wrong = []
            for it in range(20):
                assert hipattn.decode_batched_dev_noalloc(groups[t][0], 0, ctxs, q_dev, o, nq) == hipattn.OK
                hipattn.sync()
                got = o.to_host(qs[t].shape)
                if not np.array_equal(got, want[t]):
                    d = np.abs(got - want[t]).max(axis=2)              # [session][head]
                    wrong.append((it, [(int(a), int(b), float(d[a, b])) for a, b in np.argwhere(d > 0)][:8]))
            q_dev.free(); o.free()
            bad[t] = wrong or 0
        except Exception as e:
            bad[t] = repr(e)
    threads = [threading.Thread(target=job, args=(t,)) for t in range(4)]
    try:
        for th in threads:
            th.start()
        for th in threads:
            th.join()
        assert bad == [0] * 4, bad
    finally:
        for caches, _ in groups:
            for kv in caches:
                kv.close()


def test_no_alloc_decode_refuses_to_be_a_threads_first_library_call():
    # A thread's first call into the library creates its stream and staging
    # buffers (that allocates); the no-alloc entry point must not be that call:
    # WR_HIP_ERR_STATE, nothing launched, the output untouched.  After any other
    # call from the same thread it runs and equals the ordinary entry point.
    import threading
    nq, nkv, hd = 16, 8, 128
    ctxs = [700, 130]
    caches, _ = _sessions(7950, ctxs, nkv, hd)
    q = synth.normal(7951, (len(ctxs), nq, hd))
    q_dev = hipattn.DeviceBuffer.from_host(q)
    o_ref = hipattn.DeviceBuffer(q.nbytes)
    o_new = hipattn.DeviceBuffer.from_host(np.full(q.shape, 5.0, dtype=np.float32))
    hipattn.decode_batched_dev(caches, 0, ctxs, q_dev, o_ref, nq)
    hipattn.sync()
    want = o_ref.to_host(q.shape)
    seen = {}

    def job():
        try:
            seen["first"] = hipattn.decode_batched_dev_noalloc(caches, 0, ctxs, q_dev, o_new, nq)
            hipattn.sync()                                    # this thread's context is made here
            seen["untouched"] = bool((o_new.to_host(q.shape) == 5.0).all())
            seen["second"] = hipattn.decode_batched_dev_noalloc(caches, 0, ctxs, q_dev, o_new, nq)
            hipattn.sync()
            seen["equal"] = bool(np.array_equal(o_new.to_host(q.shape), want))
        except Exception as e:                                # noqa: BLE001
            seen["error"] = repr(e)
    th = threading.Thread(target=job)
    th.start()
    th.join()
    try:
        assert seen == {"first": hipattn.ERR_STATE, "untouched": True, "second": hipattn.OK, "equal": True}, seen
    finally:
        for b in (q_dev, o_ref, o_new):
            b.free()
        for kv in caches:
            kv.close()
