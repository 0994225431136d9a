"""GPU parity of the fp16 formulation of the Q4_K prefill MMQ GEMM (whole superblocks accumulated in
the matrix unit; selected with the option REIN_MMQ16 and a workspace), through the C ABI, against the CPU oracle.
The kernel is a study formulation that the default code object does not hold (`make MMQ16=1` in
reinstinct_amd/csrc builds it in); without it the module is skipped.

Bar: fp32 outputs within 1e-3 relative / 1e-4 absolute of the oracle's int8 path -- the same bar as the
other launches of rein_mmq_xq8_ws; the token operand carries 22 of the 24 bits of x * dx, the products
are exact and the sums are fp32.
"""
import numpy as np
import pytest

import reinstinct_amd as rein
from reinstinct_amd import hip, quant, runtime
from reinstinct_amd._lib import init, set_option
from oracle import orc
from helpers import assert_close_f32, random_raw_weights

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def gpu():
    init()
    hip.set_device(0)
    try:
        hip.Module.builtin().function("rein_mmq16_q4k")
    except Exception:
        pytest.skip("the code object was built without the fp16 study kernel (make MMQ16=1)")
    set_option("REIN_MMQ16", "1")
    yield
    hip.synchronize()
    set_option("REIN_MMQ16", None)


from helpers import dev  # noqa: E402  (uploads that stay alive until the test's last launch has finished)


def weights(in_dim, out_dim, seed, gaussian):
    if gaussian:
        w = (np.random.default_rng(seed).standard_normal((out_dim, in_dim)) * 0.02).astype(np.float32)
        raw = quant.quantize_weights(rein.Q4_K, w)
    else:
        raw = random_raw_weights(rein.Q4_K, in_dim, out_dim, seed)
    return quant.repack_for_matvec(rein.Q4_K, raw, in_dim, out_dim)


def run(packed, x, in_dim, out_dim):
    p_rows = x.shape[0]
    dq = hip.DeviceBuf(p_rows * (in_dim // 32) * 40)
    runtime.quantize_q8(dev(x), dq, in_dim, p_rows)
    ws_bytes = runtime.mmq_workspace_bytes(rein.Q4_K, in_dim, p_rows)
    assert runtime.mmq_form_ws(rein.Q4_K, in_dim, out_dim, p_rows, ws_bytes) == 4
    ws = hip.DeviceBuf(ws_bytes)
    dy = dev(np.full(p_rows * out_dim, np.nan, np.float32))
    runtime.mmq_xq8_ws(rein.Q4_K, dev(packed), dq, dy, in_dim, out_dim, p_rows, ws, ws_bytes)
    hip.synchronize()
    xq = dq.to_host(np.uint8)
    want = orc.matvec_q8(rein.Q4_K, packed, in_dim, out_dim, xq, p_rows)
    return dy.to_host(np.float32).reshape(p_rows, out_dim), want


# ragged token counts (the 64-token group and its 32-token tiles partly filled), row counts off the
# 256-row and 32-row grain, one to twenty superblocks, both weight recipes
@pytest.mark.parametrize("p_rows,in_dim,out_dim,gaussian", [
    (17, 256, 40, False), (70, 2048, 384, False), (33, 4096, 129, True), (100, 1024, 300, True),
    (128, 5120, 256, True), (257, 768, 520, False), (512, 512, 128, True), (64, 256, 256, True)])
def test_f16_launch_matches_oracle(p_rows, in_dim, out_dim, gaussian):
    print(f"mmq16 P {p_rows} K {in_dim} N {out_dim}", flush=True)
    packed = weights(in_dim, out_dim, seed=p_rows + in_dim, gaussian=gaussian)
    x = np.random.default_rng(in_dim + 1).standard_normal((p_rows, in_dim)).astype(np.float32)
    got, want = run(packed, x, in_dim, out_dim)
    assert_close_f32(got, want, what=f"mmq16 {p_rows}x{in_dim}x{out_dim}")


def test_f16_launch_token_rows_of_any_magnitude():
    # the per-row exponent keeps x * dx inside the fp16 range: rows from 1e-30 to 1e30, a zero row, a row
    # with one huge outlier block (its small blocks fall below the fp16 grain of the row and must only
    # cost what they weigh in the sum)
    in_dim, out_dim, p_rows = 1024, 200, 40
    packed = weights(in_dim, out_dim, seed=9, gaussian=True)
    rng = np.random.default_rng(10)
    x = rng.standard_normal((p_rows, in_dim)).astype(np.float32)
    x *= np.float32(10.0) ** rng.integers(-30, 31, (p_rows, 1)).astype(np.float32)
    x[3] = 0.0
    x[5] = rng.standard_normal(in_dim).astype(np.float32) * 1e-3
    x[5, 64:96] *= 1e7
    got, want = run(packed, x, in_dim, out_dim)
    assert np.all(np.isfinite(got))
    assert np.all(got[3] == 0.0)
    scale = np.maximum(np.abs(want).max(axis=1, keepdims=True), 1e-300)
    # per row relative to the row's largest output: the absolute part of the bar has no meaning at 1e-30
    assert np.all(np.abs(got - want) <= 1e-3 * np.abs(want) + 1e-4 * scale)
