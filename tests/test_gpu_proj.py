"""Row projections on the device (y = x . W^T, F16 weights, F32 rows) against
the CPU oracle's restatement of the reference matmul, through the C ABI.

The device sums in a different order (matrix-core tiles of 32 inputs, F32
accumulation) and feeds each activation as two half-precision terms, so the
results agree to F32 rounding, not bit for bit.  Tolerance, per output: 3e-7 *
sqrt(n_in) * sum_k |x_k w_k| (a few F32 ulps of the magnitudes summed, growing
like a random walk with the length of the sum), which is also what separates
the reference's own SIMD variants from its scalar loop."""
import ctypes as C

import numpy as np
import pytest

import oracle
from wayruntime_amd import hipattn, synth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _device():
    hipattn.init()
    yield


def _w16(seed, n_out, n_in, std):
    return synth.f32_to_f16_trunc(synth.normal(seed, (n_out, n_in), std=std))


def _widen(w16):
    # IEEE binary16 -> float64, the same values the reference's decoder yields
    return np.ascontiguousarray(w16).view(np.float16).astype(np.float64)


def _check(got, x, w16, what):
    want = oracle.matmul_w16(x, w16)
    mag = np.abs(x.astype(np.float64)) @ np.abs(_widen(w16)).T
    tol = 3e-7 * np.sqrt(x.shape[1]) * mag + 1e-37
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    assert not np.isnan(got).any(), what
    assert np.all(err <= tol), f"{what}: worst err/tol = {np.max(err / tol):.3f}"


@pytest.mark.parametrize("rows,n_in,n_out,std", [
    (1, 1024, 4096, 0.02),        # Qwen3-0.6B: wq, wk, wv stacked
    (1, 2048, 1024, 0.02),        # wo
    (16, 1024, 3072, 0.02),       # a full batch through an FFN-sized weight
    (9, 96, 48, 0.5),             # three input tiles: no full batch of eight, tail loop only
    (3, 320, 16, 1.0),            # ten input tiles: one batch and a tail; a single output tile
    (8, 32, 64, 1.0),             # one input tile
    (17, 512, 80, 0.1),           # rows pad to four groups of eight; outputs not a multiple of 64
    (300, 256, 128, 0.1),         # prefill-sized rows: the register GEMM, 32 x 32 tiles, inputs split over four waves
    (64, 96, 48, 0.5),            # ... its smallest row count; three input tiles (a wave with none), three output tiles
    (100, 160, 80, 0.3),          # ... a last row group of four rows, five input tiles
    (300, 160, 2512, 0.2),        # ... 64 x 32 tiles, a partial last tile both ways
    (4102, 64, 32, 1.0),          # more rows than one launch takes: 4096 + a six-row launch
    (500, 96, 4112, 0.3),         # LDS-staged GEMM, 128 x 64 tiles, pipelined reads: partial panels, odd input tiles
    (500, 32, 4112, 0.5),         # ... a single input tile
    (500, 128, 4112, 0.3),        # ... an even number of them
    (1000, 1056, 4112, 0.02),     # ... the plain 128 x 64 tile (two workgroups per CU), 33 input tiles
    (1000, 96, 8208, 0.3),        # LDS-staged GEMM, 128 x 128 tiles: partial output and row panels, three input tiles
    (1536, 64, 6144, 0.3),        # ... 576 such tiles would fill 1.1 rounds: the 128 x 64 tile takes over
    (1000, 32, 8208, 0.5),        # ... a single input tile (the ring's prologue covers the whole product)
    (2040, 96, 4112, 0.3),        # LDS-staged GEMM, eight waves, 256 x 128 tiles: partial panels, three input tiles
    (2040, 32, 4112, 0.5),        # ... a single input tile
    (500, 1088, 4112, 0.02),      # ... 34 input tiles, partial panels
    (2047, 2048, 1024, 0.02),     # the output projection of a 2047-token prompt (Qwen3-0.6B): one 128 x 64 tile per CU,
                                  # two sets of waves halving the input range
    (2047, 3072, 1024, 0.02),     # ... its down projection, 96 input tiles
    (2000, 2112, 1040, 0.02),     # ... partial panels both ways, 66 input tiles
    (2000, 2080, 1040, 0.02),     # ... an odd number of input tiles: one set of waves takes the whole range
    (1000, 2048, 1040, 0.02),     # too few LDS tiles for the chip: the register GEMM with a long contraction
])
def test_projection_shapes_vs_oracle(rows, n_in, n_out, std):
    print("proj", rows, n_in, n_out, flush=True)
    x = synth.normal(rows * 7 + n_in, (rows, n_in))
    w16 = _w16(n_out + 3, n_out, n_in, std)
    w = hipattn.Weight([w16])
    _check(w.rows(x), x, w16, f"{rows}x{n_in}x{n_out}")
    w.close()


@pytest.mark.parametrize("rows,n_in,n_out", [(2047, 2048, 1024), (2000, 2112, 1040), (1000, 2048, 1040)])
def test_repeated_launches_give_the_same_bits(rows, n_in, n_out):
    # no sum in these kernels depends on the order in which waves or workgroups finish
    print("proj repeat", rows, n_in, n_out, flush=True)
    x = synth.normal(5, (rows, n_in))
    w16 = _w16(6, n_out, n_in, 0.02)
    w = hipattn.Weight([w16])
    first = w.rows(x)
    for _ in range(4):
        assert w.rows(x).tobytes() == first.tobytes()
    w.close()


def test_stacked_parts_equal_separate_weights():
    n_in = 1024
    parts = [_w16(11, 2048, n_in, 0.02), _w16(12, 1024, n_in, 0.02), _w16(13, 1024, n_in, 0.02)]
    x = synth.normal(14, (2, n_in))
    stacked = hipattn.Weight(parts)
    y = stacked.rows(x)
    assert y.shape == (2, 4096)
    off = 0
    for p in parts:
        single = hipattn.Weight([p])
        assert np.array_equal(single.rows(x), y[:, off:off + p.shape[0]])
        off += p.shape[0]
        single.close()
    stacked.close()


def test_small_integers_are_exact():
    # every product and partial sum is exact in F32 and the half-precision split
    # of a small integer has no low term: any correct implementation gives the
    # integer result bit for bit, a wrong tile or lane mapping cannot
    rng = np.random.default_rng(9)
    rows, n_in, n_out = 5, 160, 48
    xi = rng.integers(-8, 9, size=(rows, n_in))
    wi = rng.integers(-8, 9, size=(n_out, n_in))
    w16 = np.array([oracle.f32_to_f16(float(v)) for v in range(-8, 9)], dtype=np.uint16)[wi + 8]
    w = hipattn.Weight([w16])
    got = w.rows(xi.astype(np.float32))
    assert np.array_equal(got, (xi @ wi.T).astype(np.float32))
    w.close()


def test_row_magnitudes_do_not_matter():
    # rows of very different scale in one call, and one row whose entries span
    # fourteen orders of magnitude: the per-row power-of-two scaling and the
    # scaled low term keep F32-level accuracy (reference: float64)
    n_in, n_out = 256, 32
    x = synth.normal(21, (5, n_in))
    x[0] *= np.float32(1e-20)
    x[1] *= np.float32(1e20)
    x[2, 1:] *= np.float32(5e-5)         # one entry of order 1, the rest tiny
    x[3] = 0.0
    x[4, ::2] *= np.float32(1e-14)
    w16 = _w16(22, n_out, n_in, 0.5)
    w = hipattn.Weight([w16])
    got = w.rows(x).astype(np.float64)
    wf = _widen(w16)
    want = x.astype(np.float64) @ wf.T
    mag = np.abs(x.astype(np.float64)) @ np.abs(wf).T
    assert np.all(got[3] == 0.0)
    assert np.all(np.abs(got - want) <= 3e-7 * np.sqrt(n_in) * mag + 1e-37)
    w.close()


@pytest.mark.parametrize("rows,n_in,n_out", [
    (6, 128, 64), (70, 128, 64),    # the row kernel and the register-tiled one
    (1000, 2048, 1040),             # a GEMM-sized launch
])
def test_device_form_with_strides_and_residual_add(rows, n_in, n_out):
    ldx, ldy = n_in + 32, n_out + 8
    x = synth.normal(31, (rows, ldx))
    add = synth.normal(32, (rows, ldy))
    w16 = _w16(33, n_out, n_in, 0.2)
    w = hipattn.Weight([w16])
    xd = hipattn.DeviceBuffer.from_host(x)
    ad = hipattn.DeviceBuffer.from_host(add)
    yd = hipattn.DeviceBuffer.from_host(np.full((rows, ldy), 7.0, dtype=np.float32))
    w.rows_dev(rows, xd, ldx, yd, ldy, add_dev=ad)
    hipattn.sync()
    y = yd.to_host((rows, ldy))
    plain = w.rows(np.ascontiguousarray(x[:, :n_in]))
    assert np.array_equal(y[:, :n_out], plain + add[:, :n_out])
    assert np.all(y[:, n_out:] == 7.0)              # padding columns are not touched
    # in place: the residual is the output buffer (the device walk's h += W . x)
    w.rows_dev(rows, xd, ldx, ad, ldy, add_dev=ad)
    hipattn.sync()
    y2 = ad.to_host((rows, ldy))
    assert np.array_equal(y2[:, :n_out], y[:, :n_out]) and np.array_equal(y2[:, n_out:], add[:, n_out:])
    for b in (xd, ad, yd):
        b.free()
    w.close()


def test_error_contract():
    lib = hipattn.lib()
    h = C.c_void_p()
    good = _w16(41, 16, 32, 1.0)
    ptrs = (C.c_void_p * 1)(good.ctypes.data)

    def create(rows, n_in):
        return lib.wr_hip_proj_weight_create(1, ptrs, (C.c_uint32 * 1)(rows), n_in, C.byref(h))

    assert create(16, 31) == hipattn.ERR_INVAL           # inputs not a multiple of 32
    assert create(8, 32) == hipattn.ERR_INVAL            # outputs not a multiple of 16
    assert create(0, 32) == hipattn.ERR_INVAL
    assert lib.wr_hip_proj_weight_create(0, ptrs, (C.c_uint32 * 1)(16), 32, C.byref(h)) == hipattn.ERR_INVAL
    assert lib.wr_hip_proj_weight_create(1, None, (C.c_uint32 * 1)(16), 32, C.byref(h)) == hipattn.ERR_INVAL
    assert create(16, 32) == hipattn.OK
    x = np.zeros((1, 32), dtype=np.float32)
    y = np.zeros((1, 16), dtype=np.float32)
    assert lib.wr_hip_proj_rows(h, 1, None, y.ctypes.data) == hipattn.ERR_INVAL
    assert lib.wr_hip_proj_rows(None, 1, x.ctypes.data, y.ctypes.data) == hipattn.ERR_INVAL
    assert lib.wr_hip_proj_rows(h, 0, x.ctypes.data, y.ctypes.data) == hipattn.OK     # nothing to do
    lib.wr_hip_proj_weight_destroy(h)


def test_fused_sources_equal_the_separate_steps():
    # rmsnorm -> projection and swiglu -> projection in one call each must give
    # the bits of the separate row step followed by the plain projection
    lib = hipattn.lib()
    rows, n_in, n_out = 11, 256, 96
    x = synth.normal(51, (rows, n_in), std=2.0)
    nw = synth.normal(52, (n_in,)) * np.float32(0.2) + np.float32(1.0)
    gu = synth.normal(53, (rows, 2 * n_in), std=2.0)
    add = synth.normal(54, (rows, n_out))
    w16 = _w16(55, n_out, n_in, 0.1)
    w = hipattn.Weight([w16])
    D = hipattn.DeviceBuffer
    xd, nwd, gud, addd = D.from_host(x), D.from_host(nw), D.from_host(gu), D.from_host(add)
    tmp, y1, y2 = D(rows * n_in * 4), D(rows * n_out * 4), D(rows * n_out * 4)
    eps = 1e-6
    # norm
    assert lib.wr_hip_rows_rmsnorm_dev(xd.p, n_in, nwd.p, n_in, tmp.p, n_in, rows, n_in, eps) == hipattn.OK
    w.rows_dev(rows, tmp, n_in, y1, n_out, add_dev=addd)
    assert lib.wr_hip_proj_rows_norm_dev(w.h, rows, xd.p, n_in, nwd.p, eps, addd.p, y2.p, n_out) == hipattn.OK
    hipattn.sync()
    a, b = y1.to_host((rows, n_out)), y2.to_host((rows, n_out))
    assert a.tobytes() == b.tobytes()
    want = oracle.matmul_w16(oracle.rmsnorm(x, nw, eps), w16) + add
    assert np.max(np.abs(b - want)) <= 1e-5 * np.max(np.abs(want))
    # swiglu
    assert lib.wr_hip_rows_swiglu_dev(gud.p, 2 * n_in, tmp.p, n_in, rows, n_in) == hipattn.OK
    w.rows_dev(rows, tmp, n_in, y1, n_out)
    assert lib.wr_hip_proj_rows_swiglu_dev(w.h, rows, gud.p, 2 * n_in, None, y2.p, n_out) == hipattn.OK
    hipattn.sync()
    a, b = y1.to_host((rows, n_out)), y2.to_host((rows, n_out))
    assert a.tobytes() == b.tobytes()
    want = oracle.matmul_w16(oracle.silu_mul(np.ascontiguousarray(gu[:, :n_in]),
                                             np.ascontiguousarray(gu[:, n_in:])), w16)
    assert np.max(np.abs(b - want)) <= 1e-5 * np.max(np.abs(want))
    # contracts: missing norm vector, gate/up stride too small
    assert lib.wr_hip_proj_rows_norm_dev(w.h, rows, xd.p, n_in, None, eps, None, y2.p, n_out) == hipattn.ERR_INVAL
    assert lib.wr_hip_proj_rows_swiglu_dev(w.h, rows, gud.p, n_in, None, y2.p, n_out) == hipattn.ERR_INVAL
    for d in (xd, nwd, gud, addd, tmp, y1, y2):
        d.free()
    w.close()


@pytest.mark.parametrize("n_in", [256, 1056, 2080, 4128])
def test_fused_sources_with_many_rows(n_in):
    # 64 rows and more: the fragment kernel that takes a row group per workgroup
    # (values held in registers up to 4096 inputs, re-read beyond) and the GEMM
    # kernels.  The row sums of the norm are formed in another order than in the
    # separate row step, so the comparison is with the oracle, to rounding; the
    # gated activation has no sum and stays bit-identical to the separate steps.
    lib = hipattn.lib()
    rows, n_out = 77, 48
    x = synth.normal(61 + n_in, (rows, n_in), std=2.0)
    nw = synth.normal(62, (n_in,)) * np.float32(0.2) + np.float32(1.0)
    gu = synth.normal(63 + n_in, (rows, 2 * n_in), std=2.0)
    add = synth.normal(64, (rows, n_out))
    w16 = _w16(65, n_out, n_in, 0.1)
    w = hipattn.Weight([w16])
    D = hipattn.DeviceBuffer
    xd, nwd, gud, addd = D.from_host(x), D.from_host(nw), D.from_host(gu), D.from_host(add)
    tmp, y1, y2 = D(rows * n_in * 4), D(rows * n_out * 4), D(rows * n_out * 4)
    eps = 1e-6
    assert lib.wr_hip_proj_rows_norm_dev(w.h, rows, xd.p, n_in, nwd.p, eps, addd.p, y2.p, n_out) == hipattn.OK
    hipattn.sync()
    got = y2.to_host((rows, n_out))
    normed = oracle.rmsnorm(x, nw, eps)
    want = oracle.matmul_w16(normed, w16) + add
    mag = np.abs(normed.astype(np.float64)) @ np.abs(_widen(w16)).T + np.abs(add)
    assert np.all(np.abs(got - want) <= 1e-6 * np.sqrt(n_in) * mag)
    assert lib.wr_hip_rows_swiglu_dev(gud.p, 2 * n_in, tmp.p, n_in, rows, n_in) == hipattn.OK
    w.rows_dev(rows, tmp, n_in, y1, n_out)
    assert lib.wr_hip_proj_rows_swiglu_dev(w.h, rows, gud.p, 2 * n_in, None, y2.p, n_out) == hipattn.OK
    hipattn.sync()
    a, b = y1.to_host((rows, n_out)), y2.to_host((rows, n_out))
    assert a.tobytes() == b.tobytes()
    act = oracle.silu_mul(np.ascontiguousarray(gu[:, :n_in]), np.ascontiguousarray(gu[:, n_in:]))
    _check(b, act, w16, f"swiglu {n_in}")
    for d in (xd, nwd, gud, addd, tmp, y1, y2):
        d.free()
    w.close()


@pytest.mark.parametrize("n_in,n_out", [(1024, 4096), (3072, 1024), (2048, 48), (14336, 64), (96, 16)])
def test_one_row_equals_its_row_of_two(n_in, n_out):
    # A single row takes the kernel that builds its operand terms in LDS; two rows
    # take the fragment launch and then the product.  Same values, same order of
    # every sum: the row's bits must not depend on the company it keeps (the
    # reference's batch contract, src/core/batch.c:15-19).  All three sources.
    lib = hipattn.lib()
    x = synth.normal(71 + n_in, (2, n_in), std=2.0)
    nw = synth.normal(72, (n_in,)) * np.float32(0.2) + np.float32(1.0)
    gu = synth.normal(73 + n_in, (2, 2 * n_in), std=2.0)
    add = synth.normal(74, (2, n_out))
    w16 = _w16(75, n_out, n_in, 0.1)
    w = hipattn.Weight([w16])
    D = hipattn.DeviceBuffer
    xd, nwd, gud, addd = D.from_host(x), D.from_host(nw), D.from_host(gu), D.from_host(add)
    y1, y2 = D(n_out * 4), D(2 * n_out * 4)
    eps = 1e-6
    for what, one, two in (
        ("plain", lambda: w.rows_dev(1, xd, n_in, y1, n_out, add_dev=addd),
         lambda: w.rows_dev(2, xd, n_in, y2, n_out, add_dev=addd)),
        ("norm", lambda: lib.wr_hip_proj_rows_norm_dev(w.h, 1, xd.p, n_in, nwd.p, eps, None, y1.p, n_out),
         lambda: lib.wr_hip_proj_rows_norm_dev(w.h, 2, xd.p, n_in, nwd.p, eps, None, y2.p, n_out)),
        ("swiglu", lambda: lib.wr_hip_proj_rows_swiglu_dev(w.h, 1, gud.p, 2 * n_in, None, y1.p, n_out),
         lambda: lib.wr_hip_proj_rows_swiglu_dev(w.h, 2, gud.p, 2 * n_in, None, y2.p, n_out)),
    ):
        assert one() in (None, hipattn.OK) and two() in (None, hipattn.OK)
        hipattn.sync()
        a, b = y1.to_host((1, n_out)), y2.to_host((2, n_out))
        assert a[0].tobytes() == b[0].tobytes(), what
    _check(w.rows(x[:1]), x[:1], w16, "one row")
    for d in (xd, nwd, gud, addd, y1, y2):
        d.free()
    w.close()


@pytest.mark.parametrize("rows", [1, 11, 70])
def test_geglu_source(rows):
    # gelu_tanh(gate) * up feeding a projection (Gemma's FFN), against the closed
    # form in float64; one row, a few rows and a prefill-sized count take three
    # different fragment paths
    lib = hipattn.lib()
    n_in, n_out = 256, 48
    gu = synth.normal(95 + rows, (rows, 2 * n_in), std=2.0)
    w16 = _w16(96, n_out, n_in, 0.1)
    w = hipattn.Weight([w16])
    D = hipattn.DeviceBuffer
    gud, y = D.from_host(gu), D(rows * n_out * 4)
    assert lib.wr_hip_proj_rows_geglu_dev(w.h, rows, gud.p, 2 * n_in, None, y.p, n_out) == hipattn.OK
    hipattn.sync()
    g, u = gu[:, :n_in].astype(np.float64), gu[:, n_in:].astype(np.float64)
    act = 0.5 * g * (1.0 + np.tanh(0.7978845608 * (g + 0.044715 * g ** 3))) * u
    want = act @ _widen(w16).T
    got = y.to_host((rows, n_out)).astype(np.float64)
    mag = np.abs(act) @ np.abs(_widen(w16)).T
    assert np.all(np.abs(got - want) <= 2e-6 * np.sqrt(n_in) * mag + 1e-30)
    gud.free()
    y.free()
    w.close()


def test_projection_random_shapes():
    # a seeded sweep over row counts, input and output widths that crosses every
    # kernel-selection boundary (1 row, 2-63 rows, the four GEMM tilings, more
    # rows than a launch takes), checked against the oracle like the fixed cases
    rng = np.random.default_rng(20240607)
    row_choices = [1, 2, 7, 8, 9, 16, 17, 40, 63, 64, 65, 127, 128, 129, 500, 1023, 1025, 2047, 4096, 4100]
    done = 0
    for case in range(28):
        rows = int(rng.choice(row_choices))
        n_in = 32 * int(rng.integers(1, 40))
        budget = max(16, int(2.5e8 / (rows * n_in)) // 16 * 16)
        n_out = 16 * int(rng.integers(1, min(520, budget // 16) + 1))
        print("random proj", case, rows, n_in, n_out, flush=True)
        x = synth.normal(1000 + case, (rows, n_in), std=float(rng.choice([0.01, 1.0, 30.0])))
        w16 = _w16(2000 + case, n_out, n_in, 0.2)
        w = hipattn.Weight([w16])
        _check(w.rows(x), x, w16, f"case {case}: {rows}x{n_in}x{n_out}")
        w.close()
        done += 1
    assert done == 28
