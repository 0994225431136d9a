"""Pins for the oracle's fused BlockQ8 producers (CPU only).

The fused kernels are compared with the oracle bit for bit, so the oracle itself has
to be tied to something else: the reference's own CPU forms and their unit-test
values (src/cpu/ops.rs:14-76, 176-236), libm over the whole input range, and the
identity "fused output == quantize_q8 of the unfused fp32 result"."""
import numpy as np
import pytest

from oracle import orc


def test_exp_det_matches_exp_over_the_range():
    x = np.linspace(-87, 88, 1_000_003).astype(np.float32)
    got = orc.map_det("exp", x).astype(np.float64)
    want = np.exp(x.astype(np.float64))
    assert np.max(np.abs(got - want) / want) < 3e-7              # ~4 ulp
    # clamped outside: finite and monotone at the ends
    ends = orc.map_det("exp", np.array([-1e30, -88, -87, 88, 89, 1e30, np.inf, -np.inf], np.float32))
    assert ends[0] == ends[1] == ends[2] > 0 and ends[3] == ends[4] == ends[5] == ends[6] < np.inf and ends[7] == ends[0]
    assert orc.map_det("exp", np.zeros(1, np.float32))[0] == 1.0


def test_known_values_of_the_reference_unit_tests():
    # src/cpu/ops.rs:176-188
    silu = orc.map_det("silu", np.array([0.0, 1.0, -1.0], np.float32))
    assert silu[0] == 0.0
    assert abs(silu[1] - 0.7310585786) < 1e-6 and abs(silu[2] + 0.2689414213) < 1e-6
    sig = orc.map_det("sigmoid", np.array([0.0, 100.0, -100.0], np.float32))
    assert abs(sig[0] - 0.5) < 1e-7 and abs(sig[1] - 1.0) < 1e-6 and abs(sig[2]) < 1e-6
    # gelu: odd part and large arguments (ops.rs:33-36 is the closed form itself)
    g = orc.map_det("gelu", np.array([0.0, 10.0, -10.0, 1.0], np.float32))
    assert g[0] == 0.0 and abs(g[1] - 10.0) < 1e-5 and abs(g[2]) < 1e-5
    assert abs(g[3] - 0.5 * (1 + np.tanh(0.7978845608028654 * 1.044715))) < 1e-6


@pytest.mark.parametrize("which,tol", [("silu", 2e-6), ("sigmoid", 5e-7), ("gelu", 3e-5)])
def test_det_functions_agree_with_the_libm_forms(which, tol):
    x = np.concatenate([np.linspace(-30, 30, 600_001), np.random.default_rng(0).standard_normal(100_000) * 3]).astype(np.float32)
    d, r = orc.map_det(which, x).astype(np.float64), orc.map_ref(which, x).astype(np.float64)
    xx = x.astype(np.float64)
    true = {"silu": xx / (1 + np.exp(-xx)), "sigmoid": 1 / (1 + np.exp(-xx)),
            "gelu": xx / (1 + np.exp(np.minimum(-2 * 0.7978845608028654 * (xx + 0.044715 * xx ** 3), 700.0)))}[which]
    # against the exact function: relative, a handful of ulp (gelu: the fp32 rounding of
    # the cubic argument, up to ~20 in magnitude, is amplified by the exponential)
    assert np.max(np.abs(d - true) / np.maximum(np.abs(true), 1e-30)) < tol
    # against the reference's fp32 form with libm: absolute (its 1 + tanh cancels in the
    # negative tail of gelu, so a relative bound there would test libm, not this)
    assert np.max(np.abs(d - r)) < tol * 30


def test_sumsq_order_and_value():
    rng = np.random.default_rng(1)
    for n in (32, 64, 96, 2048, 5120, 8192, 32 * 67):
        x = rng.standard_normal(n).astype(np.float32)
        got = orc.sumsq_det(x)
        assert abs(got - float(np.sum(x.astype(np.float64) ** 2))) < 2e-6 * n
    # exactly representable case: all ones
    assert orc.sumsq_det(np.ones(5120, np.float32)) == 5120.0
    # restated with numpy: butterfly per sub-block, 64 strided running sums, butterfly
    x = rng.standard_normal(32 * 150).astype(np.float32)
    s = (x * x).reshape(-1, 32)
    for o in (16, 8, 4, 2, 1):
        s = s + s[:, np.arange(32) ^ o]
    part = s[:, 0]
    lane = np.zeros(64, np.float32)
    for sb, p in enumerate(part):
        lane[sb & 63] = np.float32(lane[sb & 63] + p)
    for o in (32, 16, 8, 4, 2, 1):
        lane = lane + lane[np.arange(64) ^ o]
    assert orc.sumsq_det(x) == float(lane[0])


def test_rmsnorm_closed_forms_of_the_reference():
    # src/cpu/ops.rs:199-236, padded to one 32-value sub-block with zeros (zeros add
    # nothing to the sum of squares; n enters through the mean, so scale eps-free cases)
    def run(x, w, z=None):
        n = 32
        xv, wv = np.zeros((1, n), np.float32), np.ones(n, np.float32)
        xv[0, : len(x)], wv[: len(w)] = x, w
        if z is None:
            return orc.add_rmsnorm(xv, None, wv, 0.0)[1][0]
        zv = np.zeros((1, n), np.float32)
        zv[0, : len(z)] = z
        return orc.rmsnorm_gated(xv, zv, wv, 0.0)[0]

    rms = np.sqrt(np.float32(25.0 / 32))
    out = run([3, 4], [1, 1])
    assert abs(out[0] - 3 / rms) < 1e-6 and abs(out[1] - 4 / rms) < 1e-6
    out = run([1] * 32, [2, 0.5])
    assert abs(out[0] - 2.0) < 1e-6 and abs(out[1] - 0.5) < 1e-6
    out = run([1] * 32, [1, 1], z=[0, 1])
    assert abs(out[0]) < 1e-6 and abs(out[1] - 0.7310585786) < 1e-6


@pytest.mark.parametrize("n", [2048, 5120, 8192, 2816])
def test_rmsnorm_matches_the_reference_cpu_form(n):
    rng = np.random.default_rng(n)
    x = rng.standard_normal((3, n)).astype(np.float32) * 2
    add = rng.standard_normal((3, n)).astype(np.float32)
    w = (1 + 0.1 * rng.standard_normal(n)).astype(np.float32)
    hid, y = orc.add_rmsnorm(x, add, w, 1e-6)
    assert np.array_equal(hid, x + add)
    for v in range(3):
        ref = orc.rmsnorm_ref(hid[v], w, 1e-6)
        assert np.max(np.abs(y[v] - ref)) < 2e-6 * np.max(np.abs(ref))        # summation order only
    z = rng.standard_normal((3, n)).astype(np.float32)
    yg = orc.rmsnorm_gated(x, z, w, 1e-6)
    for v in range(3):
        ref = orc.rmsnorm_gated_ref(x[v], z[v], w, 1e-6)
        assert np.max(np.abs(yg[v] - ref)) < 4e-6 * np.max(np.abs(ref))


def test_elementwise_producers_against_the_reference_forms():
    rng = np.random.default_rng(5)
    g, u = rng.standard_normal(4096).astype(np.float32) * 3, rng.standard_normal(4096).astype(np.float32)
    assert np.max(np.abs(orc.swiglu_det(g, u) - orc.swiglu_mul(g, u))) < 1e-5       # tolerance of kernels.rs:1468-1473
    assert np.max(np.abs(orc.sigmoid_mul_det(u, g) - u * orc.map_ref("sigmoid", g))) < 1e-6
    gu = rng.standard_normal((5, 2 * 768)).astype(np.float32) * 2
    want = orc.map_ref("gelu", gu[:, :768]) * gu[:, 768:]
    assert np.max(np.abs(orc.geglu_det(gu) - want)) < 1e-5


def test_fused_blocks_are_quantize_q8_of_the_fp32_result():
    # the BlockQ8 form of every producer is defined as quantize_q8 of its fp32 result;
    # special blocks: all-zero rows stay d = 1, q = 0
    x = np.zeros((1, 64), np.float32)
    _, y = orc.add_rmsnorm(x, None, np.ones(64, np.float32), 1e-6)
    blocks = orc.quantize_q8(y).reshape(-1, 40)
    assert np.all(blocks[:, 8:] == 0)
    assert np.all(blocks[:, :4].copy().view(np.float32) == 1.0)
