"""The one-wave-per-SIMD prefill kernel (head dim 128, selected with
wr_hip_attn_set_prefill_one_wave) through the same checks as the default kernel:
parity with the CPU oracle (max-abs 2e-3, rel-L2 1e-3), rows above the cursor,
the F16-query form byte for byte, bit identity from launch to launch."""
import numpy as np
import pytest

import oracle
from tests import test_gpu_prefill as base
from tests import util
from wayruntime_amd import hipattn

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _one_wave():
    hipattn.init()
    oracle.set_attn_max_seq(1 << 20)
    hipattn.set_prefill_one_wave(True)
    yield
    hipattn.set_prefill_one_wave(False)
    hipattn.set_tuning(0, False)


@pytest.mark.parametrize("nq,nkv,hd,p0,T,win", [
    (16, 8, 128, 0, 512, 0),        # Qwen3 shape: two units of a wave are two heads at one sub-block
    (32, 8, 128, 0, 512, 0),        # Llama-3 shape
    (32, 8, 128, 100, 300, 0),      # behind a non-empty cache, ragged sizes
    (8, 8, 128, 7, 130, 0),         # MHA: a wave's two units are two sub-blocks of one head
    (64, 8, 128, 0, 97, 0),         # group of 8: two head chunks per KV head
    (16, 8, 128, 0, 1, 0),
    (16, 8, 128, 31, 2, 0),
    (16, 8, 128, 0, 33, 0),
    (16, 8, 128, 0, 400, 64),       # sliding window
    (32, 8, 128, 50, 300, 33),
])
def test_one_wave_prefill_matches_serial_stepping_oracle(nq, nkv, hd, p0, T, win):
    base.test_prefill_matches_serial_stepping_oracle(nq, nkv, hd, p0, T, win)


@pytest.mark.parametrize("nq,nkv,theta,T", [(32, 8, 5e5, 2048), (16, 8, 1e6, 2048)])
def test_one_wave_prefill_workload_sizes_sampled_rows(nq, nkv, theta, T):
    print("one-wave prefill workload", nq, nkv, T, flush=True)
    kv, q, k16, v16 = base._setup(nq, nkv, 128, 0, T, seed=9100 + nq, theta=theta)
    got = kv.prefill(0, 0, q)
    rows = sorted(set([0, 1, 31, 32, 33, 63, 64, 65, 500, 1023, 1024, T - 33, T - 32, T - 1]))
    want = oracle.causal_prefill(q, k16, v16, rows=rows, threads=8)
    print("  errors", util.assert_close(got[rows], want[rows]), flush=True)
    kv.close()


def test_one_wave_prefill_paired_blocks_with_offset_and_window():
    base.test_prefill_paired_blocks_with_offset_and_window_sampled_rows(32, 8, 128, 100, 2048, 500)


@pytest.mark.parametrize("nq,nkv,T,p0,norm,scale,window", [
    (16, 8, 600, 0, True, 0.0, 0),
    (32, 8, 2048, 0, False, 0.0, 0),     # rows whose reference moves often: the rescale path
    (16, 8, 300, 500, True, 0.25, 0),
    (32, 8, 700, 0, False, 0.0, 256),
])
def test_one_wave_prefill_from_f16_query_rows_equals_the_f32_form(nq, nkv, T, p0, norm, scale, window):
    base.test_prefill_from_f16_query_rows_equals_the_f32_form(nq, nkv, T, p0, norm, scale, window)


@pytest.mark.parametrize("nq,nkv", [(32, 8), (16, 8)])
def test_one_wave_prefill_is_bit_identical_from_launch_to_launch(nq, nkv):
    base.test_prefill_is_bit_identical_from_launch_to_launch(nq, nkv, 128)


def test_one_wave_prefill_ignores_rows_that_were_never_appended():
    base.test_prefill_ignores_rows_that_were_never_appended(16, 8, 128)
