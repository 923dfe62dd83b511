"""End to end on the device: the C11 host engine (wr_engine / wr_model /
wr_session API) against the greedy token stream the compiled reference produced
for the same random-init model (tests/golden/e2e_*_golden.npz, written by
tests/golden/make_e2e_golden.py).  Every test runs twice: with the whole layer
walk on the device (weights uploaded at load, the default for F16 models) and
with the host walk that sends only the cache append and attention to the GPU
(WAYRT_HOST_LAYERS=1 while the model loads)."""
import os

import numpy as np
import pytest

from tests.golden.make_e2e_golden import (GEMMA_SEED, GEMMA_STD, GEMMA_TOY, SMALL16, TINY, file_crc,
                                          workload)
from wayruntime_amd import engine as E, gguf_writer as gw, hipattn

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden")


@pytest.fixture(scope="module")
def eng():
    hipattn.shutdown()              # the engine owns the device library in this module
    e = E.Engine(E.HOST_SO)
    yield e
    e.close()


@pytest.fixture(params=["device_walk", "host_walk"])
def walk(request, monkeypatch):
    if request.param == "host_walk":
        monkeypatch.setenv("WAYRT_HOST_LAYERS", "1")
    else:
        monkeypatch.delenv("WAYRT_HOST_LAYERS", raising=False)
    return request.param


def _run_stream(model, g, n_prompt):
    prompt = workload(gw.ModelShape(vocab=model.vocab), n_prompt)
    assert np.array_equal(prompt, g["prompt"])
    n_steps = len(g["tokens"])
    probe_idx = np.linspace(0, model.vocab - 1, 8).astype(int)
    # free-running greedy: step for step against the reference's stream
    s = model.session(n_prompt + n_steps - 1)
    assert s.prefill(prompt[:-1]) == n_prompt - 1
    tok, got, worst_probe = int(prompt[-1]), [], 0.0
    for step in range(n_steps):
        logits = s.step(tok)
        assert logits is not None, f"step {step}: status {s.status}"
        worst_probe = max(worst_probe, float(np.max(np.abs(logits[probe_idx] - g["probes"][step]))))
        tok = int(np.argmax(logits))            # first maximum: ties keep the lower id
        got.append(tok)
    s.close()
    # teacher-forced: feed the reference's own tokens, compare the argmax at each step
    t = model.session(n_prompt + n_steps - 1)
    assert t.prefill(prompt[:-1]) == n_prompt - 1
    feed, forced = int(prompt[-1]), 0
    for step in range(n_steps):
        logits = t.step(feed)
        forced += int(np.argmax(logits)) == int(g["tokens"][step])
        feed = int(g["tokens"][step])
    t.close()
    return np.array(got), forced, worst_probe


def test_tiny_model_stream_on_device(eng, tmp_path, walk):
    g = np.load(os.path.join(GOLD, "e2e_tiny_golden.npz"))
    p = str(tmp_path / "tiny.gguf")
    gw.write_model(p, TINY)
    m = eng.load(p)
    got, forced, probe = _run_stream(m, g, len(g["prompt"]))
    print("tiny", walk, ": forced", forced, "probe err", probe, flush=True)
    assert forced == len(g["tokens"]) and np.array_equal(got, g["tokens"]) and probe < 1e-4
    m.close()


def test_small16_model_stream_on_device(eng, tmp_path, walk):
    # the smallest shape the device walk takes (TINY's vocabulary of 300 keeps it on the host walk)
    g = np.load(os.path.join(GOLD, "e2e_small16_golden.npz"))
    p = str(tmp_path / "small16.gguf")
    gw.write_model(p, SMALL16)
    if file_crc(p) != int(g["model_crc"][0]):
        pytest.skip("random-init model file differs from the one the golden stream was made with")
    m = eng.load(p)
    got, forced, probe = _run_stream(m, g, len(g["prompt"]))
    print("small16", walk, ": forced", forced, "probe err", probe, flush=True)
    assert forced == len(g["tokens"]) and np.array_equal(got, g["tokens"]) and probe < 1e-3
    m.close()


def test_gemma_family_stream_on_device(eng, tmp_path, walk):
    # The reference's Gemma block, on the device walk and on the host walk with the device's attention:
    # head_dim 64 on global layers and 32 on sliding-window layers (16-key
    # window, skipped tiles), scale_override 1.0, two layers that read an earlier
    # layer's cache, partial rotary, logit soft cap.  Probe tolerance: scale-1.0
    # attention over normalised Q and K (scores of +-30 and more) amplifies
    # rounding; the reference's own SIMD variants differ by 3e-4 in these logits
    # (tests/test_host_cpu.py), and the device adds the prefill kernel's single
    # F16 rounding of Q, which is relative to such scores: measured 2.5e-3.
    g = np.load(os.path.join(GOLD, "e2e_gemma_golden.npz"))
    p = str(tmp_path / "gemma.gguf")
    gw.write_model(p, GEMMA_TOY, seed=GEMMA_SEED, std=GEMMA_STD)
    if file_crc(p) != int(g["model_crc"][0]):
        pytest.skip("random-init model file differs from the one the golden stream was made with")
    m = eng.load(p)
    got, forced, probe = _run_stream(m, g, len(g["prompt"]))
    print("gemma", walk, ": forced", forced, "probe err", probe, flush=True)
    assert forced == len(g["tokens"]) and np.array_equal(got, g["tokens"]) and probe < 5e-3
    m.close()


def test_qwen3_0_6b_greedy_stream_matches_reference(eng, tmp_path, walk):
    # 28 layers, hidden 1024, 16/8 heads, head_dim 128, F16 weights N(0, 0.02):
    # 127-token prefill, then 129 greedy steps
    g = np.load(os.path.join(GOLD, "e2e_qwen3_golden.npz"))
    p = str(tmp_path / "qwen3.gguf")
    print("writing model ...", flush=True)
    gw.write_model(p, gw.QWEN3_0_6B)
    if file_crc(p) != int(g["model_crc"][0]):
        pytest.skip("random-init model file differs from the one the golden stream was made with "
                    "(different numpy build?): inputs differ, nothing to compare")
    m = eng.load(p, max_context=512)
    before = eng.counters()[E.WR_CTR_ATTENTION_CALLS]
    got, forced, probe = _run_stream(m, g, 128)
    n = len(g["tokens"])
    print(f"qwen3 ({walk}): teacher-forced {forced}/{n}, probe logit err {probe:.2e}, "
          f"min reference top-2 gap {float(g['gaps'].min()):.4f}", flush=True)
    assert forced == n                                   # argmax agrees at every step
    assert np.array_equal(got, g["tokens"])              # and the free-running stream is identical
    assert probe < 1e-3
    # one attention per session-layer-token, as the reference counts them: two runs of 127 + 129
    assert eng.counters()[E.WR_CTR_ATTENTION_CALLS] - before == 2 * 28 * (127 + 129)
    m.close()
    os.remove(p)


@pytest.mark.parametrize("family", ["qwen3", "qwen3-hd128", "gemma"])
def test_batched_step_equals_serial_on_device(eng, tmp_path, walk, family):
    p = str(tmp_path / "model.gguf")
    if family == "gemma":       # sliding-window layers, shared caches, per-layer head_dim in the batched walk
        gw.write_model(p, GEMMA_TOY, seed=GEMMA_SEED, std=GEMMA_STD)
    elif family == "qwen3-hd128":   # the head_dim of the real models: the wide-access row kernels
        gw.write_model(p, gw.ModelShape(n_layers=2, hidden=256, ffn=512, n_q=4, n_kv=2, head_dim=128,
                                        vocab=320, context=512))
    else:
        gw.write_model(p, SMALL16)
    m = eng.load(p)
    n = 12                                  # more than eight rows: two row groups in the projections
    prompts = [workload(gw.ModelShape(vocab=m.vocab), 4 + 7 * i) for i in range(n)]
    batch = [m.session(128) for _ in range(n)]
    serial = [m.session(128) for _ in range(n)]
    for i in range(n):
        assert batch[i].prefill(prompts[i]) == len(prompts[i])
        assert serial[i].prefill(prompts[i]) == len(prompts[i])
    toks = list(range(10, 10 + n))
    for _ in range(6):
        rc, lb = E.batch_step(batch, toks)
        assert rc == n
        ls = [serial[i].step(toks[i]) for i in range(n)]
        for i in range(n):
            assert lb[i].tobytes() == ls[i].tobytes(), f"session {i}"
        toks = [int(np.argmax(x)) for x in lb]
    # context full in one session refuses the whole batch; nobody advances
    small = m.session(2)
    assert small.prefill([1, 2]) == 2
    pos = [s.pos for s in batch]
    assert E.batch_step(batch + [small], toks + [1])[0] == E.WR_ERR_CTX_FULL
    assert [s.pos for s in batch] == pos
    # injected failure mid-stack: rollback, then the retry equals the serial twins
    eng.lib.wrh_debug_fail_attention_at(1)
    assert E.batch_step(batch, toks)[0] == E.WR_ERR_INTERNAL
    assert [s.pos for s in batch] == pos
    rc, lb = E.batch_step(batch, toks)
    ls = [serial[i].step(toks[i]) for i in range(n)]
    assert rc == n and all(lb[i].tobytes() == ls[i].tobytes() for i in range(n))
    for s in batch + serial + [small]:
        s.close()
    m.close()


def test_concurrent_calls_on_one_model(eng, tmp_path, walk):
    # Two threads drive disjoint groups of sessions of one model at the same time
    # (batched steps, a prefill, single steps).  The model keeps one scratch set
    # per kind of call; the call that finds it taken allocates its own.  Results
    # must equal the same calls made one after another.
    import threading
    p = str(tmp_path / "small16.gguf")
    gw.write_model(p, SMALL16)
    m = eng.load(p)
    shape = gw.ModelShape(vocab=m.vocab)

    def run(group_seed, out):
        ss = [m.session(256) for _ in range(5)]
        for i, s in enumerate(ss):
            assert s.prefill(workload(shape, 9 + 5 * i + group_seed)) == 9 + 5 * i + group_seed
        toks = [3 + group_seed + i for i in range(5)]
        trace = []
        for step in range(8):
            rc, lb = E.batch_step(ss, toks)
            assert rc == 5
            toks = [int(np.argmax(x)) for x in lb]
            trace.append(list(toks))
            if step == 3:                                   # a single step and a longer prefill in between
                trace.append(int(np.argmax(ss[0].step(toks[0]))))
                extra = m.session(256)
                assert extra.prefill(workload(shape, 70 + group_seed)) == 70 + group_seed
                trace.append(int(np.argmax(extra.step(1))))
                extra.close()
                toks[0] = trace[-2]
        for s in ss:
            s.close()
        out.append(trace)

    serial = []
    for seed in (0, 1):
        run(seed, serial)
    for _ in range(3):                                      # a few rounds: the interleaving differs every time
        a, b = [], []
        ta = threading.Thread(target=run, args=(0, a))
        tb = threading.Thread(target=run, args=(1, b))
        ta.start(); tb.start(); ta.join(); tb.join()
        assert a and b and a[0] == serial[0] and b[0] == serial[1]
    m.close()


def test_eight_threads_then_a_batch_beside_a_single_session(eng, tmp_path, walk):
    # The reference's concurrency case (test/sdk_gen.c:799-904): four prompts,
    # their greedy chains computed one after another as the reference; then
    # eight threads each run one of the chains on a session of their own, and
    # every step's logits must equal the sequential ones byte for byte; then a
    # batched step over two sessions runs while a third session steps in
    # another thread, same bar.  Each thread submits through its own stream in
    # the device library, so the launches of different sessions overlap.
    import threading
    p = str(tmp_path / "small16.gguf")
    gw.write_model(p, SMALL16)
    m = eng.load(p)
    shape = gw.ModelShape(vocab=m.vocab)
    prompts = [workload(shape, n) for n in (5, 11, 23, 40)]
    STEPS = 6

    def chain(prompt, ref=None):
        """logits bytes of STEPS greedy steps after the prompt; with ref, the count of steps that differ"""
        s = m.session(len(prompt) + STEPS)
        assert s.prefill(prompt[:-1]) == len(prompt) - 1
        tok, out, bad = int(prompt[-1]), [], 0
        for k in range(STEPS):
            lg = s.step(tok)
            assert lg is not None, s.status
            out.append(lg.tobytes())
            bad += ref is not None and out[-1] != ref[k]
            tok = int(np.argmax(lg))
        s.close()
        return out, bad

    refs = [chain(pr)[0] for pr in prompts]

    results = [None] * 8
    def job(t):
        try:
            results[t] = chain(prompts[t % 4], refs[t % 4])[1]
        except Exception as e:                    # an assert in a thread would otherwise pass silently
            results[t] = repr(e)
    threads = [threading.Thread(target=job, args=(t,)) for t in range(8)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert results == [0] * 8, results

    side = [None]
    def side_job():
        try:
            side[0] = chain(prompts[2], refs[2])[1]
        except Exception as e:
            side[0] = repr(e)
    st = threading.Thread(target=side_job)
    st.start()
    ab = [m.session(len(prompts[i]) + STEPS) for i in range(2)]
    for i in range(2):
        assert ab[i].prefill(prompts[i][:-1]) == len(prompts[i]) - 1
    cur = [int(prompts[0][-1]), int(prompts[1][-1])]
    mism = 0
    for k in range(STEPS):
        rc, lo = E.batch_step(ab, cur)
        assert rc == 2
        for i in range(2):
            mism += lo[i].tobytes() != refs[i][k]
            cur[i] = int(np.argmax(lo[i]))
    st.join()
    for s in ab:
        s.close()
    assert mism == 0 and side[0] == 0, (mism, side[0])
    m.close()
