"""Wall-clock timings of the host engine on a random-init model: prompt
processing, single-session decode and a 16-session batched step, with the whole
layer on the device (default) or with the host walk (--host).

    python -m wayruntime_amd.e2e_timing [--host] [--prompt 2047] [--skip-decode]

The model is Qwen3-0.6B-shaped (28 layers, hidden 1024, 16/8 heads of 128,
vocabulary 151 936, F16 weights drawn N(0, 0.02)); it is written once to
--model (default: the system's temporary directory) and reused."""
from __future__ import annotations

import argparse
import os
import sys
import tempfile
import time

import numpy as np

from wayruntime_amd import engine as E, gguf_writer as gw


def prompt_tokens(vocab: int, n: int) -> np.ndarray:
    return ((np.arange(n, dtype=np.uint64) * 2654435761 + 12345) % vocab).astype(np.uint32)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--host", action="store_true", help="host walk: only append and attention on the device")
    ap.add_argument("--prompt", type=int, nargs="*", default=[511, 2047, 4095])
    ap.add_argument("--reps", type=int, default=3)
    ap.add_argument("--skip-decode", action="store_true")
    ap.add_argument("--json", action="store_true", help="one JSON line with the figures at the end")
    ap.add_argument("--model", default=os.path.join(tempfile.gettempdir(), "wayruntime_amd_qwen3_0_6b.gguf"))
    args = ap.parse_args()
    if args.host:
        os.environ["WAYRT_HOST_LAYERS"] = "1"
    if not os.path.exists(args.model):
        gw.write_model(args.model, gw.QWEN3_0_6B)
    eng = E.Engine(E.HOST_SO)
    ctx = max(args.prompt + [1024]) + 128
    t = time.perf_counter()
    m = eng.load(args.model, max_context=ctx)
    walk = "host walk" if args.host else "device walk"
    print(f"{walk}: load {time.perf_counter() - t:.2f} s", flush=True)
    figures = {"model": "Qwen3-0.6B shape, random init, F16", "walk": walk}
    for n in args.prompt:
        toks = prompt_tokens(m.vocab, n)
        best = None
        for _ in range(args.reps):
            s = m.session(ctx)
            t = time.perf_counter()
            assert s.prefill(toks) == n
            dt = time.perf_counter() - t
            best = dt if best is None else min(best, dt)
            s.close()
        print(f"{walk}: prefill {n} tokens: {best * 1e3:.1f} ms ({n / best:.0f} tok/s)", flush=True)
        figures[f"prefill_{n}_ms"] = round(best * 1e3, 2)
        figures[f"prefill_{n}_tok_s"] = round(n / best)
    if not args.skip_decode:
        toks = prompt_tokens(m.vocab, 512)
        s = m.session(ctx)
        assert s.prefill(toks[:-1]) == 511
        tok, steps = int(toks[-1]), (16 if args.host else 64)
        for _ in range(4):
            tok = int(np.argmax(s.step(tok)))
        per_step = []                             # the engine call alone: the greedy pick over 150 000
        for _ in range(steps):                    # logits in numpy costs 50 us a row and is not the engine's
            t = time.perf_counter()
            logits = s.step(tok)
            per_step.append(time.perf_counter() - t)
            tok = int(np.argmax(logits))
        dt = sum(per_step) / steps
        med = float(np.median(per_step))
        print(f"{walk}: decode step at context ~520: {dt * 1e3:.2f} ms/token ({1 / dt:.0f} tok/s), "
              f"median {med * 1e3:.2f}, slowest {max(per_step) * 1e3:.2f}", flush=True)
        figures["decode_ms_per_token"] = round(dt * 1e3, 3)
        figures["decode_ms_per_token_median"] = round(med * 1e3, 3)
        ss = [m.session(1024) for _ in range(16)]
        for i, x in enumerate(ss):
            assert x.prefill(toks[:100 + i]) == 100 + i
        feed = list(range(16))
        for _ in range(2):
            rc, lb = E.batch_step(ss, feed)
            feed = [int(np.argmax(x)) for x in lb]
        steps = 4 if args.host else 32
        import ctypes as C
        hs = (C.c_void_p * 16)(*[x.h for x in ss])
        outs = (C.POINTER(C.c_float) * 16)()
        dt = 0.0
        for _ in range(steps):                    # the C call alone, as for the single step
            toks_c = (C.c_uint32 * 16)(*feed)
            t = time.perf_counter()
            rc = ss[0].lib.wr_batch_step(hs, toks_c, 16, outs)
            dt += time.perf_counter() - t
            assert rc == 16
            feed = [int(np.argmax(np.ctypeslib.as_array(outs[i], shape=(m.vocab,)))) for i in range(16)]
        dt /= steps
        print(f"{walk}: batched step, 16 sessions: {dt * 1e3:.2f} ms/step ({16 / dt:.0f} tok/s aggregate)",
              flush=True)
        figures["batch16_ms_per_step"] = round(dt * 1e3, 3)
        figures["batch16_tok_s"] = round(16 / dt)
        for x in ss + [s]:
            x.close()
    m.close()
    eng.close()
    if args.json:
        import json
        print(json.dumps(figures), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
