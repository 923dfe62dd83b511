"""The long-context decode workload at its real size on the device: 16 sessions
at 32768 cached positions each, one cache layer, eight steps that each append one
position per session (src/core/session.c:139-154) and then attend over everything
(src/core/kernels.c:1437-1445: cursor, hard cap), for the Gemma-class head shape
(8 Q / 4 KV heads, head_dim 256) and the Llama-3-8B one (32 / 8 / 128).  Through
the C ABI.  Every session is checked against the CPU oracle on the first and on the
last step (max-abs 2e-3, rel-L2 1e-3; sessions spread over host threads), the
batched launch against serial decode calls bit for bit, and the eight appended rows
of every cache by bits."""
from concurrent.futures import ThreadPoolExecutor

import numpy as np
import pytest

from tests import util
from wayruntime_amd import hipattn, synth

pytestmark = pytest.mark.gpu

S, BASE, STEPS = 16, 32768, 8


@pytest.fixture(scope="module", autouse=True)
def _device():
    hipattn.init()
    yield
    hipattn.set_tuning(0, False)


@pytest.mark.parametrize("nq,nkv,hd", [(8, 4, 256), (32, 8, 128)])
def test_long_context_step_loop_at_full_size(nq, nkv, hd):
    cap = BASE + STEPS
    # one pool of N(0,1) rows; session i reads it rotated by 1999 * i positions, so
    # the sessions differ row by row without generating 2 x 10^9 normals
    # (V reads the same pool 12345 rows further on: half the generation time)
    pk16 = synth.f32_to_f16_trunc(synth.normal(synth.config_seed(5, hd), (cap, nkv, hd)))
    pv16 = np.roll(pk16, 12345, axis=0)
    caches, k16s, v16s = [], [], []
    for i in range(S):
        k16 = np.roll(pk16, 1999 * i, axis=0)
        v16 = np.roll(pv16, 1999 * i + 7, axis=0)
        kv = hipattn.KVCache(1, hd, nkv, cap)
        kv.write_f16(0, 0, k16[:BASE], v16[:BASE])
        caches.append(kv); k16s.append(k16); v16s.append(v16)
    print("long context: %d sessions x %d rows, %d/%d/%d, %.2f GB of cache" % (
        S, BASE, nq, nkv, hd, sum(c.bytes for c in caches) / 1e9), flush=True)
    try:
        for step in range(STEPS):
            seq_k = BASE + step + 1
            qs = [synth.normal(synth.config_seed(5, 1000 + 16 * step + i), (nq, hd)) for i in range(S)]
            for i in range(S):
                kn = synth.normal(synth.config_seed(5, 3000 + 16 * step + i), (1, nkv, hd))
                vn = synth.normal(synth.config_seed(5, 5000 + 16 * step + i), (1, nkv, hd))
                assert caches[i].append(0, BASE + step, kn, vn) == hipattn.OK
                k16s[i][BASE + step] = synth.f32_to_f16_trunc(kn)[0]
                v16s[i][BASE + step] = synth.f32_to_f16_trunc(vn)[0]
            outs = hipattn.decode_batched(caches, 0, [seq_k] * S, qs)
            assert not any(np.isnan(o).any() for o in outs)
            if step in (0, STEPS - 1):
                with ThreadPoolExecutor(16) as ex:
                    wants = list(ex.map(lambda i: util.oracle_decode(qs[i], k16s[i], v16s[i], seq_k), range(S)))
                worst = max(util.assert_close(outs[i], wants[i], f"step {step} session {i}")[0] for i in range(S))
                print("  step %d: all %d sessions within tolerance (worst max-abs %.2e)" % (step, S, worst),
                      flush=True)
                # the batched launch equals serial calls bit for bit (src/core/batch.c:15-19)
                for i in (0, 7, 15):
                    assert np.array_equal(caches[i].decode(0, seq_k, qs[i]), outs[i]), f"session {i}"
            else:
                # cheap property on the other steps: a session's output changes when its
                # own new row does, and only then (sessions never share arithmetic)
                again = hipattn.decode_batched(caches, 0, [seq_k] * S, qs)
                assert all(np.array_equal(a, b) for a, b in zip(again, outs))
        for i in range(S):
            gk, gv = caches[i].read_f16(0, BASE, STEPS)
            assert np.array_equal(gk, k16s[i][BASE:cap]) and np.array_equal(gv, v16s[i][BASE:cap]), f"session {i}"
            # and a stretch of the bulk rows, for the upload path
            gk, gv = caches[i].read_f16(0, 1000 * i, 64)
            assert np.array_equal(gk, k16s[i][1000 * i:1000 * i + 64])
            assert np.array_equal(gv, v16s[i][1000 * i:1000 * i + 64])
        # a full cache refuses the next append and keeps its rows
        kn = np.zeros((1, nkv, hd), dtype=np.float32)
        assert caches[0].append(0, cap, kn, kn) == hipattn.ERR_CTX_FULL
    finally:
        for kv in caches:
            kv.close()


def test_long_sessions_keep_their_bits_whatever_launch_they_are_in():
    # From 8K keys up a session is cut into twice as many splits as it gets
    # workgroups in a launch that fills the device: a workgroup there works through
    # two consecutive splits, in a small launch every split has a workgroup of its
    # own.  The split is the unit of arithmetic, so the three launches below must
    # agree byte for byte (reference contract: src/core/batch.c:15-19).
    nq, nkv, hd = 16, 8, 128
    ctxs = [8192, 8193, 8223, 8224, 9000, 10000, 12288, 16384, 8255, 11111, 13000, 15000, 8500, 9999, 14000, 16000]
    caches, qs, kvs = [], [], []
    for i, ctx in enumerate(ctxs):
        q = synth.normal(7700 + i, (nq, hd))
        _a, _b, k16, v16 = util.make_kv(7800 + 2 * i, ctx, nkv, hd)
        kv = hipattn.KVCache(1, hd, nkv, ctx)
        kv.write_f16(0, 0, k16, v16)
        caches.append(kv); qs.append(q); kvs.append((k16, v16))
    print("long sessions: batch of 16", flush=True)
    outs = hipattn.decode_batched(caches, 0, ctxs, qs)
    for i in (0, 7):
        util.assert_close(outs[i], util.oracle_decode(qs[i], kvs[i][0], kvs[i][1], ctxs[i]), f"session {i}")
    print("long sessions: alone", flush=True)
    for i in range(len(ctxs)):
        single = caches[i].decode(0, ctxs[i], qs[i])
        assert np.array_equal(single, outs[i]), f"session {i} alone"
    print("long sessions: pairs", flush=True)
    for i in range(0, len(ctxs), 2):
        two = hipattn.decode_batched(caches[i:i + 2], 0, ctxs[i:i + 2], qs[i:i + 2])
        assert np.array_equal(two[0], outs[i]) and np.array_equal(two[1], outs[i + 1]), f"sessions {i}, {i + 1}"
    for kv in caches:
        kv.close()


def test_long_sessions_at_head_dim_64_keep_their_bits_too():
    # head_dim 64 keeps two tiles per wave in registers and has its own form of
    # the step from one split to the next inside a workgroup; its sessions are
    # "long" from 16K keys up (64 tiles per workgroup otherwise)
    nq, nkv, hd = 16, 8, 64
    ctxs = [16384, 16385, 17000, 20000]
    caches, qs, kvs = [], [], []
    for i, ctx in enumerate(ctxs):
        q = synth.normal(7900 + i, (nq, hd))
        _a, _b, k16, v16 = util.make_kv(7950 + 2 * i, ctx, nkv, hd)
        kv = hipattn.KVCache(1, hd, nkv, ctx)
        kv.write_f16(0, 0, k16, v16)
        caches.append(kv); qs.append(q); kvs.append((k16, v16))
    print("long sessions, head_dim 64: four in one launch", flush=True)
    outs = hipattn.decode_batched(caches, 0, ctxs, qs)
    util.assert_close(outs[2], util.oracle_decode(qs[2], kvs[2][0], kvs[2][1], ctxs[2]), "session 2")
    print("long sessions, head_dim 64: alone", flush=True)
    for i in range(len(ctxs)):
        single = caches[i].decode(0, ctxs[i], qs[i])
        assert np.array_equal(single, outs[i]), f"session {i} alone"
    for kv in caches:
        kv.close()


def test_sixteen_sessions_with_the_whole_models_cache_footprint():
    # The cache of the long-context workload's model as a serving process holds it
    # (src/core/session.c:640-733): Llama-3-8B geometry, 32 layers x 8 KV heads x
    # head_dim 128 at 32768 positions = 4 GiB per session, 16 sessions = 64 GiB of
    # ordinary device allocations on one 288 GB device.  Appends and decode calls
    # on the first and the last layer of the first and the last session against the
    # CPU oracle at a short cursor, the byte count of every slab, then everything
    # is destroyed and allocated once more (a leak of 64 GiB per round would not
    # fit a third time; no allocation here runs the device out of memory).
    layers, nq, nkv, hd, ctx, n = 32, 32, 8, 128, 32768, 16
    per_session = 2 * layers * nkv * ctx * hd * 2
    assert per_session == 4 << 30
    for round_ in range(2):
        caches = [hipattn.KVCache(layers, hd, nkv, ctx) for _ in range(n)]
        try:
            total = sum(c.bytes for c in caches)
            print("footprint round %d: %d sessions, %.1f GiB" % (round_, n, total / 2.0 ** 30), flush=True)
            assert all(c.bytes >= per_session for c in caches)
            assert total < 1.02 * n * per_session            # alignment only, no hidden copies
            rows = 77
            for si in (0, n - 1):
                for layer in (0, layers - 1):
                    seed = synth.config_seed(5, 9000 + 100 * round_ + 10 * si + layer)
                    k32 = synth.normal(seed, (rows, nkv, hd))
                    v32 = synth.normal(seed + 1, (rows, nkv, hd))
                    q = synth.normal(seed + 2, (nq, hd))
                    assert caches[si].append(layer, 0, k32, v32) == hipattn.OK
                    got = caches[si].decode(layer, rows, q)
                    k16, v16 = synth.f32_to_f16_trunc(k32), synth.f32_to_f16_trunc(v32)
                    util.assert_close(got, util.oracle_decode(q, k16, v16, rows), f"session {si} layer {layer}")
                    kb, vb = caches[si].read_f16(layer, 0, rows)
                    assert np.array_equal(kb, k16) and np.array_equal(vb, v16)
            # the slabs are zero-filled at creation: an untouched layer of an untouched
            # session reads back zeros, also at the far end of the context
            kz, vz = caches[5].read_f16(17, ctx - 64, 64)
            assert not kz.any() and not vz.any()
            # the two sessions in one batched launch, last layer
            qs = [synth.normal(synth.config_seed(5, 9900 + i), (nq, hd)) for i in range(2)]
            outs = hipattn.decode_batched([caches[0], caches[n - 1]], layers - 1, [rows, rows], qs)
            for o, c, qq in zip(outs, (caches[0], caches[n - 1]), qs):
                assert np.array_equal(o, c.decode(layers - 1, rows, qq))
        finally:
            for c in caches:
                c.close()
