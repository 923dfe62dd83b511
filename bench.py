#!/usr/bin/env python3
"""Benchmark of the attention path on one MI355X.

Headline workload (the configuration the metric is quoted on): batched decode
attention, Llama-3-8B head shape (32 query / 8 KV heads, head_dim 128),
16 sessions, every session at 4096 cached positions, F16 cache resident in HBM,
F32 queries resident in HBM.  One "step" is one batched attention launch over
one layer of all 16 caches; successive steps walk through `--layers` distinct
layers so the working set (268 MB per layer) cannot sit in the last-level
cache.

Prints ONE JSON line.  `value` is algorithmic K/V bytes per step divided by
wall time per step (whole step: split-K kernel + combine).  `roofline` is for
the split-K kernel alone, timed with per-launch events.  `cpu_baseline` is the
CPU oracle (a bit-exact restatement of the reference op) on the same data, one
core, on a bounded sample.  `prefill` reports causal prefill attention
(the metric's T = 2048 launch checked against the oracle on sampled rows;
`other_shapes`: the same launch timed at other head shapes and lengths),
`decode_configs` the other decode workloads (16 ragged sessions, 16 x 32768 at
both long-context head shapes, one session at 128 / 512 / 2048 / 8192 keys),
each with its kernel time, rate, fraction of the HBM peak and an oracle check of
one session; `projection` the row projections either side of the path: 16 rows
(proj_rows_kernel, HBM-bound on the F16 weight bytes) and a 1024-row prefill
pass (proj_gemm_lds_kernel, MFMA-bound); `end_to_end` the host engine on a
random-init Qwen3-0.6B-shaped model (python -m wayruntime_amd.e2e_timing in a
child process): every layer on the device, and (`host_walk_*`) the layers on
the host with only the cache append and the attention on the device, plus what
that pair of calls costs per layer as two calls and as one
(`host_rows_append_then_decode_us`, `host_rows_append_decode_us`).
`mfma_probe` is what back-to-back MFMAs alone sustain on this device with
operands of zeros, of ones and of N(0, 1) samples (wayruntime_amd/calib_mfma):
the clock the device grants depends on the data, and
`prefill.frac_of_mfma_probe_normal_operands` prices the prefill launch against
the last of the three beside the published peak.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0           # MI355X HBM3E
MFMA_F16_PEAK_TFLOPS = 2500.0   # MI355X dense f16

TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "decode_prefill_traffic_pmc.txt")
DECODE_KERNEL_SRC = os.path.join(ROOT, "wayruntime_amd", "csrc", "kernels_decode.hip.h")


def pmc_traffic_bytes(sessions: int, ctx: int):
    """HBM bytes one launch of the decode kernel moves on the default workload:
    rocprofv3 FETCH_SIZE + WRITE_SIZE per dispatch, each scaled by what the same
    counter reads for a plain copy kernel of known size.  Counters cannot be read
    from inside this process, so the figure is read from the committed counter
    summary, which names the workload and the SHA-1 of the kernel source it was
    measured on (line `bench.traffic decode SxCTX fetch_bytes=.. write_bytes=..
    kernel_sha1=..`).  Another workload, or a kernel source that has changed
    since, gives None rather than a stale number."""
    import hashlib
    try:
        sha = hashlib.sha1(open(DECODE_KERNEL_SRC, "rb").read()).hexdigest()
        for ln in open(TRAFFIC_PROFILE):
            f = ln.split()
            if len(f) >= 6 and f[0] == "bench.traffic" and f[1] == "decode" and f[2] == "%dx%d" % (sessions, ctx):
                kv = dict(x.split("=", 1) for x in f[3:])
                if kv.get("kernel_sha1") == sha:
                    return int(kv["fetch_bytes"]) + int(kv["write_bytes"])
    except (OSError, ValueError, KeyError):
        pass
    return None


def pooled16(pool16: np.ndarray, salt: int, n: int) -> np.ndarray:
    """n F16 bit patterns drawn from a pool of truncated N(0,1) samples at a
    salted offset, sign-flipped for odd salts: distinct per (session, layer),
    still N(0,1), and cheap to make."""
    if n > pool16.size // 2:                      # long contexts: the pool repeated, rotated by the salt
        x = np.resize(np.roll(pool16, -((salt * 40503) % pool16.size)), n)
    else:
        off = (salt * 2654435761) % (pool16.size - n)
        x = pool16[off:off + n].copy()
    if salt & 1:
        x ^= np.uint16(0x8000)
    return x


def batch1_rotation(ctx: int):
    """(layers, replicas) for a one-session workload of `ctx` keys (4096 bytes per
    key): enough distinct copies that the working set passes 600 MB."""
    layers = 64
    per_cache = 4096 * ctx * layers
    return layers, max(1, -(-600_000_000 // per_cache))


class _Off:                                         # device pointer at an offset
    def __init__(self, p):
        self.p = p


class DecodeWorkload:
    """S sessions of one head shape with the given context lengths, resident in
    HBM.  `replicas` independent copies of the session set with `layers` cache
    layers each are walked by successive steps, so that the bytes a step reads
    were last touched (replicas x layers) steps ago and cannot sit in the
    last-level cache (256 MB)."""

    def __init__(self, hipattn, synth, pool16, nq, nkv, hd, ctxs, layers, replicas=1, keep_host="first"):
        self.h, self.nq, self.nkv, self.hd = hipattn, nq, nkv, hd
        self.ctxs, self.L, self.R, self.S = list(ctxs), layers, replicas, len(ctxs)
        row = nkv * hd
        self.caches, self.host_kv = [], {}
        for r in range(replicas):
            group = []
            for s_i, c in enumerate(self.ctxs):
                kv = hipattn.KVCache(layers, hd, nkv, c)
                for layer in range(layers):
                    salt = 2 * ((r * self.S + s_i) * layers + layer)
                    k16 = pooled16(pool16, 1 + salt, c * row).reshape(c, nkv, hd)
                    v16 = pooled16(pool16, 2 + salt, c * row).reshape(c, nkv, hd)
                    kv.write_f16(layer, 0, k16, v16)
                    if r == 0 and layer == 0 and (s_i == 0 or keep_host == "all"):
                        self.host_kv[s_i] = (k16, v16)
                group.append(kv)
            self.caches.append(group)
        self.q_host = synth.normal(synth.config_seed(3, 1), (layers, self.S, nq, hd))
        self.q_dev = hipattn.DeviceBuffer.from_host(self.q_host)
        self.out_dev = hipattn.DeviceBuffer(self.S * nq * hd * 4)
        self.step_q_bytes = self.S * nq * hd * 4
        self.bytes_per_step = 2 * 2 * nkv * hd * sum(self.ctxs)      # K and V, two bytes each

    def step(self, i: int) -> None:
        group = self.caches[i % self.R]
        layer = (i // self.R) % self.L
        self.h.decode_batched_dev(group, layer, self.ctxs, _Off(self.q_dev.p + layer * self.step_q_bytes),
                                  self.out_dev, self.nq)

    def check(self, oracle):
        """Session 0, layer 0 of replica 0 against the oracle: (max_abs, rel_l2)."""
        self.step(0)
        self.h.sync()
        got = self.out_dev.to_host((self.S, self.nq, self.hd))
        k16, v16 = self.host_kv[0]
        want0 = oracle.attention(self.q_host[0, 0][None], k16, v16)[0]
        return (float(np.max(np.abs(got[0] - want0))),
                float(np.linalg.norm(got[0] - want0) / np.linalg.norm(want0)))

    def time_steps(self, steps: int, warmup: int) -> float:
        """ms per step, wall clock around `steps` launches (stream drained on both sides)."""
        for i in range(warmup):
            self.step(i)
        self.h.sync()
        t = time.perf_counter()
        for i in range(steps):
            self.step(i)
        self.h.sync()
        return (time.perf_counter() - t) * 1e3 / steps

    def time_kernel(self, n: int) -> float:
        """mean duration (ms) of the split-K kernel alone, per-launch events on the library stream"""
        self.h.profile_begin(n)
        for i in range(n):
            self.step(i)
        ms, timed = self.h.profile_end()
        return ms / max(timed, 1)

    def close(self):
        for group in self.caches:
            for kv in group:
                kv.close()
        self.q_dev.free()
        self.out_dev.free()


def decode_config(hipattn, synth, oracle, pool16, name, nq, nkv, hd, ctxs, layers, replicas, steps, warmup):
    """One secondary decode workload: kernel time, rate, fraction of peak, oracle check."""
    w = DecodeWorkload(hipattn, synth, pool16, nq, nkv, hd, ctxs, layers, replicas)
    try:
        max_abs, rel_l2 = w.check(oracle)
        ok = max_abs <= 2e-3 and rel_l2 <= 1e-3
        ms = w.time_steps(steps, warmup)
        kern_ms = w.time_kernel(min(steps, 256))
        gbs = w.bytes_per_step / (kern_ms * 1e-3) / 1e9
        return {"workload": name, "shape": "%d/%d/%d" % (nq, nkv, hd), "sessions": len(ctxs),
                "ctx": ctxs[0] if len(set(ctxs)) == 1 else [min(ctxs), max(ctxs)],
                "bytes_per_launch": w.bytes_per_step, "kernel_us": round(kern_ms * 1e3, 2),
                "GB/s": round(gbs, 1), "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4),
                "wall_us_per_step": round(ms * 1e3, 2),
                "working_set_MB": round(w.bytes_per_step * layers * replicas / 1e6, 1),
                "check_session0": {"max_abs": max_abs, "rel_l2": rel_l2, "ok": ok}}
    finally:
        w.close()


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--layers", type=int, default=8,
                    help="distinct cache layers walked by successive steps")
    ap.add_argument("--sessions", type=int, default=16)
    ap.add_argument("--ctx", type=int, default=4096)
    ap.add_argument("--cpu-seconds", type=float, default=12.0,
                    help="budget for the CPU baseline sample (0 disables it)")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--no-proj", action="store_true")
    ap.add_argument("--no-e2e", action="store_true")
    ap.add_argument("--no-decode-configs", action="store_true")
    ap.add_argument("--keys-per-wg", type=int, default=0)
    ap.add_argument("--workload", default="headline",
                    choices=["headline", "ragged16", "long16", "long16-hd256", "batch1"],
                    help="headline: 16 sessions x --ctx, 32/8/128 (the metric's configuration), with "
                         "the other decode workloads as secondary keys; "
                         "ragged16: 16 sessions with contexts drawn from [256, 4096]; "
                         "long16 / long16-hd256: 16 sessions x 32768 at 32/8/128 / 8/4/256; "
                         "batch1: one session, 16/8/128, --ctx keys.  Other than headline they "
                         "run that one workload as the timed steps and report the decode figures only")
    args = ap.parse_args()

    if args.gpus != 1:
        print("bench.py: this build measures one GPU; --gpus %d is not supported "
              "(nothing here uses a second device)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    from wayruntime_amd import hipattn, synth

    hipattn.init(0)
    nq, nkv, hd = 32, 8, 128
    S, ctx, L, R = args.sessions, args.ctx, args.layers, 1
    ctxs = None
    if args.workload == "ragged16":
        S = 16
        ctxs = [int(c) for c in synth.ragged_contexts(synth.config_seed(3, 0), S, 256, 4096)]
    elif args.workload in ("long16", "long16-hd256"):
        S, ctx, L = 16, 32768, 2
        if args.workload == "long16-hd256":
            nq, nkv, hd = 8, 4, 256
    elif args.workload == "batch1":
        nq, S = 16, 1
        L, R = batch1_rotation(ctx)
    if ctxs is None:
        ctxs = [ctx] * S
    secondary = args.workload != "headline"
    if secondary:
        args.no_prefill = args.no_proj = args.no_e2e = args.no_decode_configs = True
        args.cpu_seconds = 0.0

    t0 = time.time()
    pool16 = synth.f32_to_f16_trunc(synth.normal(synth.config_seed(3, 0), (1 << 24,)))
    work = DecodeWorkload(hipattn, synth, pool16, nq, nkv, hd, ctxs, L, R,
                          keep_host="first" if secondary else "all")
    caches, host_kv, q_host = work.caches[0], work.host_kv, work.q_host
    setup_s = time.time() - t0

    if args.keys_per_wg:
        hipattn.set_tuning(args.keys_per_wg, False)

    # ---- correctness of what is being timed: session 0, layer 0 vs the oracle
    import oracle
    oracle.set_attn_max_seq(1 << 20)
    max_abs, rel_l2 = work.check(oracle)
    if not (max_abs <= 2e-3 and rel_l2 <= 1e-3):
        print("bench.py: device output outside tolerance: max_abs=%g rel_l2=%g" % (max_abs, rel_l2),
              file=sys.stderr)
        sys.exit(1)

    # ---- timed region
    ms_per_step = work.time_steps(args.steps, args.warmup)
    bytes_per_step = work.bytes_per_step
    value = bytes_per_step / (ms_per_step * 1e-3) / 1e9

    # ---- dominant kernel alone, per-launch events
    kern_avg_ms = work.time_kernel(min(max(args.steps, 100), 512))
    achieved = bytes_per_step / (kern_avg_ms * 1e-3) / 1e9
    roofline = {"bound": "hbm", "kernel": "decode_mfma_kernel<%d, false>" % hd, "achieved": round(achieved, 1),
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                "traffic": pmc_traffic_bytes(S, ctx) if not secondary and len(set(ctxs)) == 1 else None,
                "kernel_avg_us": round(kern_avg_ms * 1e3, 2),
                "bytes_per_launch": bytes_per_step}

    # ---- causal prefill (secondary figure of the metric)
    prefill = None
    if not args.no_prefill:
        T = 2048
        qp = synth.normal(synth.config_seed(4, 1), (T, nq, hd))
        qp_dev = hipattn.DeviceBuffer.from_host(qp)
        op_dev = hipattn.DeviceBuffer(qp.nbytes)
        reps = 60                                          # whatever --steps says: a stable mean
        hipattn.prefill_dev(caches[0], 0, 0, T, qp_dev, op_dev, nq)
        hipattn.profile_begin(reps)
        for _ in range(reps):
            hipattn.prefill_dev(caches[0], 0, 0, T, qp_dev, op_dev, nq)
        pms, pn = hipattn.profile_end()
        flops = 4.0 * nq * hd * T * (T + 1) / 2.0
        p_avg = pms / max(pn, 1)
        tfl = flops / (p_avg * 1e-3) / 1e12
        gotp = op_dev.to_host((T, nq, hd))
        rows = [0, 1, 31, 32, 777, 2047]
        wantp = oracle.causal_prefill(qp, host_kv[0][0], host_kv[0][1], p0=0, rows=rows)
        perr = float(np.max(np.abs(gotp[rows] - wantp[rows])))
        prefill = {"workload": "causal prefill, 32/8/128, T=2048, empty cache", "tflops": round(tfl, 2),
                   "ms": round(p_avg, 4), "frac_of_f16_mfma_peak": round(tfl / MFMA_F16_PEAK_TFLOPS, 4),
                   "max_abs_err_sampled_rows": perr}
        # the form for callers whose Q never leaves the device: Q as the binary16
        # operand the kernel would round it to (same output bits, half the Q bytes)
        qscale = np.float32(np.float32(1.0) / np.sqrt(np.float32(hd))) * np.float32(1.4426950408889634)
        q16_dev = hipattn.DeviceBuffer.from_host((qp * qscale).astype(np.float16))
        o16_dev = hipattn.DeviceBuffer(qp.nbytes)
        lib = hipattn.lib()
        def q16_launch():
            rc = lib.wr_hip_attn_prefill_q16_dev(caches[0].h, 0, 0, T, q16_dev.p, o16_dev.p, nq, 0.0, 0)
            if rc != hipattn.OK:
                raise RuntimeError("wr_hip_attn_prefill_q16_dev: %d" % rc)
        q16_launch()
        hipattn.profile_begin(reps)
        for _ in range(reps):
            q16_launch()
        qms, qn_ = hipattn.profile_end()
        q_avg = qms / max(qn_, 1)
        got16 = o16_dev.to_host((T, nq, hd))
        prefill["q16_dev"] = {"ms": round(q_avg, 4), "tflops": round(flops / (q_avg * 1e-3) / 1e12, 2),
                              "frac_of_f16_mfma_peak": round(flops / (q_avg * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS, 4),
                              "same_bits_as_f32_rows": bool(got16.tobytes() == gotp.tobytes())}
        # the other kernel for this head dim (one wave per SIMD, two units per wave),
        # kept for comparison: same workload, F32 rows
        hipattn.set_prefill_one_wave(True)
        try:
            hipattn.prefill_dev(caches[0], 0, 0, T, qp_dev, op_dev, nq)
            hipattn.profile_begin(reps)
            for _ in range(reps):
                hipattn.prefill_dev(caches[0], 0, 0, T, qp_dev, op_dev, nq)
            wms, wn = hipattn.profile_end()
            w_avg = wms / max(wn, 1)
            goto = op_dev.to_host((T, nq, hd))
            prefill["one_wave_kernel"] = {
                "ms": round(w_avg, 4), "tflops": round(flops / (w_avg * 1e-3) / 1e12, 2),
                "frac_of_f16_mfma_peak": round(flops / (w_avg * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS, 4),
                "max_abs_err_sampled_rows": float(np.max(np.abs(goto[rows] - wantp[rows])))}
        finally:
            hipattn.set_prefill_one_wave(False)
        q16_dev.free()
        o16_dev.free()
        qp_dev.free()
        op_dev.free()
        # the same launch at other head shapes and lengths (timing only: their
        # parity is the GPU tests'), caches written directly as F16 bit patterns
        others = []
        for onq, onkv, ohd, oT in ((32, 8, 128, 4096), (16, 8, 128, 2048), (16, 8, 256, 2048), (32, 8, 128, 512)):
            okv = hipattn.KVCache(1, ohd, onkv, oT)
            rngp = np.random.default_rng(oT + ohd)
            bits = rngp.integers(0x3000, 0x3C00, size=(2, oT, onkv, ohd), dtype=np.uint16)
            bits |= (rngp.integers(0, 2, size=bits.shape, dtype=np.uint16) << 15)
            okv.write_f16(0, 0, bits[0], bits[1])
            oq = synth.normal(synth.config_seed(4, 2), (oT, onq, ohd))
            oq_dev = hipattn.DeviceBuffer.from_host(oq)
            oo_dev = hipattn.DeviceBuffer(oq.nbytes)
            hipattn.prefill_dev(okv, 0, 0, oT, oq_dev, oo_dev, onq)
            oreps = 50
            hipattn.profile_begin(oreps)
            for _ in range(oreps):
                hipattn.prefill_dev(okv, 0, 0, oT, oq_dev, oo_dev, onq)
            oms, on = hipattn.profile_end()
            o_avg = oms / max(on, 1)
            otfl = 4.0 * onq * ohd * oT * (oT + 1) / 2.0 / (o_avg * 1e-3) / 1e12
            others.append({"shape": f"{onq}/{onkv}/{ohd}", "T": oT, "ms": round(o_avg, 4), "tflops": round(otfl, 1),
                           "frac_of_f16_mfma_peak": round(otfl / MFMA_F16_PEAK_TFLOPS, 4)})
            oq_dev.free()
            oo_dev.free()
            okv.close()
        prefill["other_shapes"] = others

    # ---- row projections either side of the attention path (secondary figure):
    # 16 rows through Llama-3-8B-sized F16 weights, HBM-bound on the weight
    # bytes; distinct copies are walked so the weights come from HBM.
    proj = None
    if not args.no_proj:
        proj = {}
        rng = np.random.default_rng(7)
        rows = 16
        for name, n_out, n_in, copies in (("qkv 6144x4096", 6144, 4096, 6),
                                          ("gate_up 28672x4096", 28672, 4096, 3),
                                          ("lm_head 128256x4096", 128256, 4096, 2)):
            ws = [hipattn.Weight([rng.integers(0, 0x3C00, size=(n_out, n_in), dtype=np.uint16)])
                  for _ in range(copies)]
            xd = hipattn.DeviceBuffer.from_host(synth.normal(9, (rows, n_in)))
            yd = hipattn.DeviceBuffer(rows * n_out * 4)
            reps = 24
            for i in range(3 * copies):
                ws[i % copies].rows_dev(rows, xd, n_in, yd, n_out)
            hipattn.profile_begin(reps)
            for i in range(reps):
                ws[i % copies].rows_dev(rows, xd, n_in, yd, n_out)
            pms, pn = hipattn.profile_end()
            us = pms / max(pn, 1) * 1e3
            gbs = 2.0 * n_out * n_in / (us * 1e-6) / 1e9
            proj[name] = {"rows": rows, "kernel_us": round(us, 2), "GB/s": round(gbs, 1),
                          "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4)}
            for w in ws:
                w.close()
            xd.free()
            yd.free()
        # the same weights against a prefill pass of 1024 rows: MFMA-bound.  The
        # activations travel as two half-precision terms, so the matrix cores do
        # twice the useful multiply-adds; both rates are given.
        rows = 1024
        for name, n_out, n_in in (("qkv 6144x4096", 6144, 4096), ("gate_up 28672x4096", 28672, 4096),
                                  ("down 4096x14336", 4096, 14336)):
            w = hipattn.Weight([rng.integers(0, 0x3C00, size=(n_out, n_in), dtype=np.uint16)])
            xd = hipattn.DeviceBuffer.from_host(synth.normal(10, (rows, n_in)))
            yd = hipattn.DeviceBuffer(rows * n_out * 4)
            reps = 10
            for _ in range(2):
                w.rows_dev(rows, xd, n_in, yd, n_out)
            hipattn.profile_begin(reps)
            for _ in range(reps):
                w.rows_dev(rows, xd, n_in, yd, n_out)
            pms, pn = hipattn.profile_end()
            us = pms / max(pn, 1) * 1e3
            tf = 2.0 * rows * n_out * n_in / (us * 1e-6) / 1e12
            proj[name + " x 1024 rows"] = {"rows": rows, "kernel_us": round(us, 2), "TFLOP/s": round(tf, 1),
                                           "mfma_TFLOP/s": round(2 * tf, 1),
                                           "frac_of_f16_peak": round(2 * tf / MFMA_F16_PEAK_TFLOPS, 4)}
            w.close()
            xd.free()
            yd.free()

    # ---- CPU baseline: the oracle on the same data, bounded sample.  The
    # reference runs one attention call on one core, so one core is the faithful
    # figure; sessions are independent, so one thread per session is the best a
    # caller of the reference could do, and is reported beside it.
    cpu = None
    if args.cpu_seconds > 0:
        # the compiled reference itself where its library has been built
        # (oracle/_ref, made from the reference's own sources by oracle/Makefile),
        # else the bit-exact restatement
        use_ref = oracle.have_ref()
        if use_ref:
            try:
                oracle.ref()
            except OSError:
                use_ref = False

        def cpu_attention(q1, k16, v16):
            if use_ref:
                rc, _ = oracle.ref_attention(q1, k16, v16)
                assert rc == 0, rc
            else:
                oracle.attention(q1, k16, v16)

        done_bytes, t_cpu, n_calls = 0, 0.0, 0
        s = 0
        while t_cpu < args.cpu_seconds * 0.6:
            k16, v16 = host_kv[s % S]
            tc = time.perf_counter()
            cpu_attention(q_host[0, s % S][None], k16, v16)
            t_cpu += time.perf_counter() - tc
            done_bytes += 2 * 2 * nkv * hd * ctx
            n_calls += 1
            s += 1
        per_call = t_cpu / n_calls
        # session-parallel: the foreign calls release the interpreter lock
        from concurrent.futures import ThreadPoolExecutor
        n_thr = min(S, os.cpu_count() or 1)
        rounds = max(1, int(args.cpu_seconds * 0.4 / per_call))

        def worker(i):
            k16, v16 = host_kv[i % S]
            for _ in range(rounds):
                cpu_attention(q_host[0, i % S][None], k16, v16)

        tp = time.perf_counter()
        with ThreadPoolExecutor(n_thr) as ex:
            list(ex.map(worker, range(n_thr)))
        t_par = time.perf_counter() - tp
        par_gbs = n_thr * rounds * 2 * 2 * nkv * hd * ctx / t_par / 1e9
        cpu_model = ""
        try:
            with open("/proc/cpuinfo") as f:
                for ln in f:
                    if ln.startswith("model name"):
                        cpu_model = ln.split(":", 1)[1].strip()
                        break
        except OSError:
            pass
        cpu = {"value": round(done_bytes / t_cpu / 1e9, 4), "unit": "GB/s", "cores": 1,
               "kind": "reference" if use_ref else "port",
               "sample": "%d single-session calls of the same workload (32/8/128, ctx %d), "
                         "%.1f s of CPU time" % (n_calls, ctx, t_cpu),
               "session_parallel": {"value": round(par_gbs, 4), "unit": "GB/s", "cores": n_thr,
                                    "sample": "%d threads x %d calls, %.1f s" % (n_thr, rounds, t_par)},
               "host": "%s, %d cpus visible" % (cpu_model, os.cpu_count() or 0)}

    # ---- the other decode workloads (secondary figures): same timing code as the
    # headline, fewer steps; each checks session 0 against the oracle first
    decode_configs = None
    if not args.no_decode_configs:
        work.close()
        caches = []
        decode_configs = []
        sec_steps, sec_warm = 60, 10
        ragged = [int(c) for c in synth.ragged_contexts(synth.config_seed(3, 0), 16, 256, 4096)]
        specs = [("ragged16", 32, 8, 128, ragged, 8, 1),
                 ("long16", 32, 8, 128, [32768] * 16, 2, 1),
                 ("long16-hd256", 8, 4, 256, [32768] * 16, 2, 1)]
        for c1 in (128, 512, 2048, 8192):
            l1, r1 = batch1_rotation(c1)
            specs.append(("batch1-ctx%d" % c1, 16, 8, 128, [c1], l1, r1))
        for name, cnq, cnkv, chd, cctx, cl, cr in specs:
            try:
                decode_configs.append(decode_config(hipattn, synth, oracle, pool16, name, cnq, cnkv, chd,
                                                    cctx, cl, cr, sec_steps, sec_warm))
            except Exception as exc:                  # reported, not fatal to the headline line
                decode_configs.append({"workload": name, "error": repr(exc)[:200]})

    # ---- what a kernel that only reads gets out of HBM on this device, for the
    # decode kernel's access pattern and for the friendliest one (secondary
    # figure: the roofline above stays priced against the published peak)
    read_probe = None
    probe_exe = os.path.join(ROOT, "wayruntime_amd", "calib_read")
    if not args.no_decode_configs and os.path.exists(probe_exe):
        import subprocess
        try:
            res = subprocess.run([probe_exe, "256", "24"], capture_output=True, text=True, timeout=120)
            read_probe = []
            for ln in res.stdout.splitlines():
                if " avg " in ln and "GB/s" in ln:
                    f = ln.split()
                    read_probe.append({"pattern": ln.split("  grid")[0].strip(), "workgroups": int(f[f.index("grid") + 1]),
                                       "kernel_us": float(f[f.index("avg") + 1]),
                                       "GB/s": float(f[f.index("GB/s") - 1])})
            if res.returncode != 0 or not read_probe:
                read_probe = {"error": "exit %d: %s" % (res.returncode, (res.stderr or res.stdout)[-200:])}
        except Exception as exc:
            read_probe = {"error": repr(exc)[:200]}

    # ---- what the matrix pipes sustain with nothing but MFMAs in flight, with
    # operands of zeros and with operands drawn from N(0, 1): the clock the device
    # grants depends on the data (secondary figure: the prefill fraction above stays
    # priced against the published peak)
    mfma_probe = None
    mfma_exe = os.path.join(ROOT, "wayruntime_amd", "calib_mfma")
    if not args.no_prefill and os.path.exists(mfma_exe):
        import subprocess
        try:
            res = subprocess.run([mfma_exe, "32"], capture_output=True, text=True, timeout=120)
            mfma_probe = []
            for ln in res.stdout.splitlines():
                f = ln.split()
                if ln.startswith("operands") and "TFLOP/s" in f:
                    mfma_probe.append({"operands": f[1], "launch_us": float(f[f.index("launch_us") + 1]),
                                       "TFLOP/s": float(f[f.index("TFLOP/s") + 1]),
                                       "shader_GHz": float(f[f.index("GHz") + 1])})
            if res.returncode != 0 or not mfma_probe:
                mfma_probe = {"error": "exit %d: %s" % (res.returncode, (res.stderr or res.stdout)[-200:])}
            elif isinstance(prefill, dict) and prefill.get("tflops"):
                normal = [m["TFLOP/s"] for m in mfma_probe if m["operands"] == "normal"]
                if normal:
                    prefill["frac_of_mfma_probe_normal_operands"] = round(prefill["tflops"] / normal[0], 4)
        except Exception as exc:
            mfma_probe = {"error": repr(exc)[:200]}

    # ---- what one launch costs inside a chain of dependent launches (the
    # device walk's decode step is such a chain): a floor, from kernels that
    # only read their predecessor's row, reduce it and store (secondary figure)
    chain_probe = None
    chain_exe = os.path.join(ROOT, "wayruntime_amd", "calib_chain")
    if not args.no_e2e and os.path.exists(chain_exe):
        import subprocess
        try:
            res = subprocess.run([chain_exe, "400"], capture_output=True, text=True, timeout=120)
            chain_probe = []
            for ln in res.stdout.splitlines():
                if "us per launch" in ln:
                    f = ln.split()
                    chain_probe.append({"kernel": ln.split("  grid")[0].strip(), "workgroups": int(f[f.index("grid") + 1]),
                                        "us_per_launch": float(f[-1])})
            if res.returncode != 0 or not chain_probe:
                chain_probe = {"error": "exit %d: %s" % (res.returncode, (res.stderr or res.stdout)[-200:])}
        except Exception as exc:
            chain_probe = {"error": repr(exc)[:200]}

    # ---- the host engine end to end on a random-init Qwen3-0.6B-shaped model
    # (secondary figures): a child process, so this process's device state and
    # the engine's do not meet.  A failure is reported, not fatal.
    e2e = None
    if not args.no_e2e:
        import subprocess
        try:
            res = subprocess.run([sys.executable, "-m", "wayruntime_amd.e2e_timing", "--json", "--reps", "2"],
                                 cwd=ROOT, capture_output=True, text=True, timeout=240)
            last = [ln for ln in res.stdout.splitlines() if ln.startswith("{")]
            e2e = json.loads(last[-1]) if res.returncode == 0 and last else {
                "error": "exit %d: %s" % (res.returncode, (res.stderr or res.stdout)[-200:])}
            # the same model on the host walk: the host does the layer, the library
            # only the cache append and the attention (what a reference build with
            # this library behind its two call sites does per layer)
            if "error" not in e2e:
                res = subprocess.run([sys.executable, "-m", "wayruntime_amd.e2e_timing", "--json", "--host",
                                      "--prompt", "511", "--reps", "1"],
                                     cwd=ROOT, capture_output=True, text=True, timeout=240)
                last = [ln for ln in res.stdout.splitlines() if ln.startswith("{")]
                if res.returncode == 0 and last:
                    hw = json.loads(last[-1])
                    for key in ("decode_ms_per_token", "batch16_ms_per_step", "prefill_511_ms"):
                        e2e["host_walk_" + key] = hw.get(key)
                else:
                    e2e["host_walk_error"] = "exit %d: %s" % (res.returncode, (res.stderr or res.stdout)[-200:])
        except Exception as exc:                      # timeout, missing model space, ...
            e2e = e2e if isinstance(e2e, dict) else {}
            e2e["error"] = repr(exc)[:200]

    # ---- what the two call sites cost a host-resident caller per layer of a decode
    # step (Qwen3 head shape, context 520): cache append then attention as two
    # synchronous calls, and the one call that does both
    if isinstance(e2e, dict):
        try:
            hkv = hipattn.KVCache(1, 128, 8, 1024)
            hkv.append(0, 0, synth.normal(11, (520, 8, 128)), synth.normal(12, (520, 8, 128)))
            hk, hv, hq = synth.normal(13, (8, 128)), synth.normal(14, (8, 128)), synth.normal(15, (16, 128))
            hout = np.empty_like(hq)
            hlib = hipattn.lib()

            def hop_two(pos):
                hlib.wr_hip_attn_append(hkv.h, 0, pos, 1, hk.ctypes.data, hv.ctypes.data)
                hlib.wr_hip_attn_decode(hkv.h, 0, pos + 1, hq.ctypes.data, hout.ctypes.data, 16, 0.0, 0)

            def hop_one(pos):
                hlib.wr_hip_attn_append_decode(hkv.h, 0, pos, hk.ctypes.data, hv.ctypes.data, hq.ctypes.data,
                                               hout.ctypes.data, 16, 0.0, 0)

            for key, fn in (("host_rows_append_then_decode_us", hop_two), ("host_rows_append_decode_us", hop_one)):
                ts = []
                for i in range(220):
                    t0 = time.perf_counter()
                    fn(520 + i)
                    ts.append(time.perf_counter() - t0)
                e2e[key] = round(float(np.median(ts[20:])) * 1e6, 1)
            hkv.close()
        except Exception as exc:
            e2e["host_rows_error"] = repr(exc)[:200]

    line = {
        "metric": "decode-attn HBM GB/s (% peak) at 16 sess x 4K ctx; prefill attn TFLOP/s",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16 cache, f32 accumulate",
        "data": "synthetic",
        "config": {"workload": ("batched decode attention, Llama-3-8B head shape 32/8/128, "
                                "%d sessions x %d ctx, %d cache layers walked" % (S, ctx, L))
                   if not secondary else
                   ("decode attention, head shape %d/%d/%d, %d session(s), contexts %d..%d "
                    "(%s), %d cache layers walked" % (nq, nkv, hd, S, min(ctxs), max(ctxs),
                                                      args.workload, L)),
                   "sessions": S, "ctx": ctx if len(set(ctxs)) == 1 else ctxs, "layers": L},
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
        "roofline": roofline, "cpu_baseline": cpu, "prefill": prefill, "decode_configs": decode_configs,
        "hbm_read_probe": read_probe,
        "launch_chain_probe": chain_probe,
        "mfma_probe": mfma_probe,
        "projection": proj,
        "end_to_end": e2e,
        "check": {"max_abs": max_abs, "rel_l2": rel_l2},
        "device": hipattn.device_name(), "setup_s": round(setup_s, 1),
    }
    print(json.dumps(line), flush=True)
    if caches:
        work.close()


if __name__ == "__main__":
    main()
