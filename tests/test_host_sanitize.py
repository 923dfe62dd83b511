"""The C11 host engine under AddressSanitizer and UndefinedBehaviorSanitizer, on
the CPU test double: every host source is compiled with the sanitizers together
with tests/host_sanitize.c and the oracle-backed stand-in for the device
library, and the exerciser runs over three toy models (two Qwen3 shapes and a
Gemma one).  A heap error, an undefined operation or a leaked allocation in the
host code fails the run."""
import glob
import os
import subprocess

import pytest

from tests.golden.make_e2e_golden import GEMMA_SEED, GEMMA_STD, GEMMA_TOY, SMALL16, TINY
from wayruntime_amd import gguf_writer as gw

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_host_engine_is_sanitizer_clean(tmp_path):
    exe = str(tmp_path / "host_sanitize")
    srcs = ([os.path.join(ROOT, "tests", "host_sanitize.c")]
            + sorted(glob.glob(os.path.join(ROOT, "wayruntime_amd", "host", "*.c")))
            + [os.path.join(ROOT, "oracle", "wr_hip_attn_cpu_shim.c"), os.path.join(ROOT, "oracle", "wr_oracle.c")])
    cmd = (["gcc", "-std=c11", "-O1", "-g", "-mavx2", "-mfma", "-mf16c", "-ffp-contract=off", "-fopenmp",
            "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-static-libasan",
            "-static-libubsan", "-fno-omit-frame-pointer",
            "-I" + os.path.join(ROOT, "wayruntime_amd", "host", "include"), "-I" + os.path.join(ROOT, "include"),
            "-I" + os.path.join(ROOT, "oracle"), "-o", exe] + srcs + ["-lpthread", "-lm"])
    built = subprocess.run(cmd, capture_output=True, text=True)
    if built.returncode != 0 and "asan" in built.stderr.lower() and "cannot find" in built.stderr.lower():
        pytest.skip("the sanitizer runtime is not installed")
    assert built.returncode == 0, built.stderr[-2000:]

    args = []
    for name, shape, kw in (("tiny", TINY, {}), ("small16", SMALL16, {}),
                            ("gemma", GEMMA_TOY, dict(seed=GEMMA_SEED, std=GEMMA_STD))):
        p = str(tmp_path / (name + ".gguf"))
        gw.write_model(p, shape, **kw)
        args += [p, str(shape.vocab)]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:verify_asan_link_order=0", OMP_NUM_THREADS="4")
    run = subprocess.run([exe] + args, capture_output=True, text=True, env=env, timeout=600)
    out = run.stdout + run.stderr
    assert run.returncode == 0, out[-3000:]
    assert out.count(" ok acc=") == 3
    assert "AddressSanitizer" not in out and ": runtime error:" not in out, out[-3000:]
