"""Builds the gfx950 shared library in-tree (``wayruntime_amd/libwr_hip_attn.so``).

    python -m wayruntime_amd.build            # compile
    python -m wayruntime_amd.build --temps    # also keep ISA / resource usage under build/temps
"""
from __future__ import annotations

import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
HIP_SO = os.path.join(PKG, "libwr_hip_attn.so")
HIP_SRC = os.path.join(PKG, "csrc", "wr_hip_attn.hip")

HIPCC_FLAGS = [
    "-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-shared",
    # no packed-FP32 VALU forms in device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def build_hip(keep_temps: bool = False) -> str:
    cmd = ["hipcc"] + HIPCC_FLAGS
    if keep_temps:
        tmp = os.path.join(ROOT, "build", "temps")
        os.makedirs(tmp, exist_ok=True)
        cmd += ["-save-temps=obj"]
    cmd += ["-o", HIP_SO, HIP_SRC]
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if err.strip():
        sys.stderr.write(err + "\n")
    if res.returncode != 0:
        raise RuntimeError("hipcc failed building " + HIP_SO)
    if keep_temps:
        for f in os.listdir(PKG):
            if f.startswith("wr_hip_attn-") or f.startswith("wr_hip_attn.hip-"):
                os.replace(os.path.join(PKG, f), os.path.join(ROOT, "build", "temps", f))
    return HIP_SO


HOST_SO = os.path.join(PKG, "libwayruntime_amd.so")
HOST_DIR = os.path.join(PKG, "host")
HOST_SRCS = ["wr_math.c", "wr_ops.c", "wr_model.c", "wr_session.c", "wr_device.c"]
# -ffp-contract=off: the scalar ops keep the reference's multiply-then-add
# rounding; the matmul uses explicit FMA intrinsics and is not affected.
HOST_CFLAGS = ["-std=c11", "-O3", "-mavx2", "-mfma", "-mf16c", "-ffp-contract=off", "-fopenmp",
               "-fPIC", "-shared", "-Wall", "-Wextra", "-Wshadow", "-Wvla"]


def build_host() -> str:
    """The C11 host engine, linked against the device library next to it."""
    cmd = (["gcc"] + HOST_CFLAGS + ["-I" + os.path.join(HOST_DIR, "include"), "-o", HOST_SO]
           + [os.path.join(HOST_DIR, f) for f in HOST_SRCS]
           + ["-L" + PKG, "-lwr_hip_attn", "-Wl,-rpath,$ORIGIN", "-lpthread"])
    subprocess.check_call(cmd)
    return HOST_SO


CALIB_BINS = {"calib_copy": "calib_copy.hip", "calib_read": "calib_read.hip", "calib_chain": "calib_chain.hip",
              "calib_mfma": "calib_mfma.hip"}
CALIB_BIN = os.path.join(PKG, "calib_copy")


def build_calib() -> str:
    """Measurement aids: the counter-calibration copy program, the read-only
    bandwidth probe, the launch-chain probe and the matrix-pipe probe (see
    csrc/calib_copy.hip, csrc/calib_read.hip, csrc/calib_chain.hip,
    csrc/calib_mfma.hip)."""
    for name, src in CALIB_BINS.items():
        out = os.path.join(PKG, name)
        res = subprocess.run(["hipcc", "-O3", "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang",
                              "-packed-fp32-ops", "-o", out,
                              os.path.join(PKG, "csrc", src)], capture_output=True, text=True)
        if res.returncode != 0:
            sys.stderr.write(res.stderr)
            raise RuntimeError("hipcc failed building " + out)
    return CALIB_BIN


def build_all(keep_temps: bool = False) -> None:
    build_hip(keep_temps)
    build_host()
    build_calib()


if __name__ == "__main__":
    build_all("--temps" in sys.argv)
    print("built", HIP_SO, HOST_SO)
