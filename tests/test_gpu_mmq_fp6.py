"""GPU parity of the workspace launch of the prefill MMQ GEMM (Q4_K on the block-scaled fp6
matrix instruction), through the C ABI, against the CPU oracle.

Bars: the per-block dots out of the fp6 instruction are bit-exact int32; fp32 outputs within
1e-3 relative / 1e-4 absolute of the oracle's int8 path; every token-group split gives the same
bits (each output element adds the same terms in the same order whatever tile it sits in).
"""
import os

import numpy as np
import pytest

import reinstinct_amd as rein
from reinstinct_amd import hip, quant, runtime
from reinstinct_amd._lib import ReinError, init
from oracle import orc
from helpers import assert_close_f32, random_raw_weights

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def gpu():
    init()
    hip.set_device(0)
    # the library keeps small GEMMs on the int8 launch; these tests are about the fp6 one
    os.environ["REIN_MMQ6_FROM"] = "17"
    yield
    hip.synchronize()
    os.environ.pop("REIN_MMQ6_FROM", None)


from helpers import dev  # noqa: E402  (uploads that stay alive until the test's last launch has finished)


def weights(in_dim, out_dim, seed, gaussian):
    if gaussian:
        w = (np.random.default_rng(seed).standard_normal((out_dim, in_dim)) * 0.02).astype(np.float32)
        raw = quant.quantize_weights(rein.Q4_K, w)
    else:
        raw = random_raw_weights(rein.Q4_K, in_dim, out_dim, seed)
    return quant.repack_for_matvec(rein.Q4_K, raw, in_dim, out_dim)


def quantized(x):
    n, k = x.shape
    dx, dq = dev(x), hip.DeviceBuf(n * (k // 32) * 40)
    runtime.quantize_q8(dx, dq, k, n)
    hip.synchronize()
    return dq


def run_ws(dw, dq, in_dim, out_dim, p_rows, fill=np.nan):
    ws_bytes = runtime.mmq_workspace_bytes(rein.Q4_K, in_dim, p_rows)
    assert ws_bytes > 0
    ws = hip.DeviceBuf(ws_bytes)
    dy = dev(np.full(p_rows * out_dim, fill, np.float32))
    runtime.mmq_xq8_ws(rein.Q4_K, dw, dq, dy, in_dim, out_dim, p_rows, ws, ws_bytes)
    hip.synchronize()
    return dy.to_host(np.float32).reshape(p_rows, out_dim)


# ragged token counts, row counts off the 128-row and 32-row grain, padded (power-of-two) and
# unpadded contractions, both weight recipes
@pytest.mark.parametrize("p_rows,in_dim,out_dim,gaussian", [
    (17, 256, 40, False), (70, 2048, 384, False), (33, 4096, 129, True), (100, 1024, 300, True),
    (128, 5120, 256, True), (257, 768, 130, False), (512, 512, 128, True)])
def test_ws_launch_matches_oracle(p_rows, in_dim, out_dim, gaussian):
    print(f"mmq6 P {p_rows} K {in_dim} N {out_dim}", flush=True)
    packed = weights(in_dim, out_dim, seed=p_rows + in_dim, gaussian=gaussian)
    x = np.random.default_rng(in_dim + 1).standard_normal((p_rows, in_dim)).astype(np.float32)
    dw, dq = dev(packed), quantized(x)
    xq = dq.to_host(np.uint8)
    got = run_ws(dw, dq, in_dim, out_dim, p_rows)
    want = orc.matvec_q8(rein.Q4_K, packed, in_dim, out_dim, xq, p_rows)
    assert_close_f32(got, want, what=f"mmq6 {p_rows}x{in_dim}x{out_dim}")


@pytest.mark.parametrize("p_rows,in_dim,out_dim", [(40, 1024, 200), (65, 2048, 129)])
def test_fp6_block_dots_bit_exact(p_rows, in_dim, out_dim):
    print(f"mmq6 dots P {p_rows} K {in_dim} N {out_dim}", flush=True)
    packed = weights(in_dim, out_dim, seed=3, gaussian=False)
    x = np.random.default_rng(4).standard_normal((p_rows, in_dim)).astype(np.float32) * 3.0
    dw, dq = dev(packed), quantized(x)
    ws_bytes = max(runtime.mmq_workspace_bytes(rein.Q4_K, in_dim, p_rows), 1 << 20)
    ws = hip.DeviceBuf(ws_bytes)
    n_sub = in_dim // 32
    out = dev(np.full(p_rows * out_dim * n_sub, -1, np.int32))
    runtime.mmq_block_dots_ws(rein.Q4_K, dw, dq, out, in_dim, out_dim, p_rows, ws, ws_bytes)
    hip.synchronize()
    want = orc.block_dots(rein.Q4_K, packed, in_dim, out_dim, dq.to_host(np.uint8), p_rows)
    assert np.array_equal(out.to_host(np.int32).reshape(want.shape), want)


def test_every_token_split_gives_the_same_bits():
    p_rows, in_dim, out_dim = 300, 1024, 260
    packed = weights(in_dim, out_dim, seed=9, gaussian=True)
    x = np.random.default_rng(10).standard_normal((p_rows, in_dim)).astype(np.float32)
    dw, dq = dev(packed), quantized(x)
    outs = {}
    try:
        for n4, n2 in ((2, 1), (1, 3), (0, 5), (0, 0), (2, 0)):
            print(f"mmq6 split n4 {n4} n2 {n2}", flush=True)
            os.environ["REIN_MMQ6_N4"], os.environ["REIN_MMQ6_N2"] = str(n4), str(n2)
            assert runtime.mmq_tile_plan_ws(rein.Q4_K, out_dim, p_rows) == (n4, n2)
            outs[(n4, n2)] = run_ws(dw, dq, in_dim, out_dim, p_rows).view(np.uint32)
    finally:
        os.environ.pop("REIN_MMQ6_N4", None)
        os.environ.pop("REIN_MMQ6_N2", None)
    first = next(iter(outs.values()))
    for k, v in outs.items():
        assert np.array_equal(v, first), f"split {k} differs"


def test_workspace_contract():
    p_rows, in_dim, out_dim = 64, 512, 128
    packed = weights(in_dim, out_dim, seed=1, gaussian=True)
    x = np.random.default_rng(2).standard_normal((p_rows, in_dim)).astype(np.float32)
    dw, dq = dev(packed), quantized(x)
    need = runtime.mmq_workspace_bytes(rein.Q4_K, in_dim, p_rows)
    assert need > 0
    # formats and row counts without a workspace launch ask for none
    assert runtime.mmq_workspace_bytes(rein.Q6_K, in_dim, p_rows) == 0
    assert runtime.mmq_workspace_bytes(rein.Q4_K, in_dim, 16) == 0
    os.environ["REIN_MMQ6_FROM"] = "320"
    assert runtime.mmq_workspace_bytes(rein.Q4_K, in_dim, 256) == 0 and runtime.mmq_workspace_bytes(rein.Q4_K, in_dim, 320) > 0
    os.environ["REIN_MMQ6_FROM"] = "17"
    ws = hip.DeviceBuf(need)
    dy = dev(np.zeros(p_rows * out_dim, np.float32))
    with pytest.raises(ReinError):                           # too small: refused, nothing launched
        runtime.mmq_xq8_ws(rein.Q4_K, dw, dq, dy, in_dim, out_dim, p_rows, ws, need - 1)
    # no workspace: the int8 launch, same result within the bar
    runtime.mmq_xq8_ws(rein.Q4_K, dw, dq, dy, in_dim, out_dim, p_rows, None, 0)
    hip.synchronize()
    plain = dy.to_host(np.float32).reshape(p_rows, out_dim)
    with_ws = run_ws(dw, dq, in_dim, out_dim, p_rows)
    assert_close_f32(with_ws, plain, what="workspace launch vs int8 launch")
    # matmul_ws: quantize + GEMM out of one scratch buffer, the same bits as the two calls
    sb = runtime.matmul_scratch_bytes(rein.Q4_K, in_dim, p_rows)
    assert sb >= p_rows * (in_dim // 32) * 40 + need
    scratch = hip.DeviceBuf(sb)
    dy2 = dev(np.zeros(p_rows * out_dim, np.float32))
    runtime.matmul_ws(rein.Q4_K, dw, dev(x), dy2, in_dim, out_dim, p_rows, scratch, sb)
    hip.synchronize()
    assert np.array_equal(dy2.to_host(np.uint32).reshape(p_rows, out_dim), with_ws.view(np.uint32))


def test_two_launches_and_a_reused_workspace_agree():
    # the same workspace serves a larger and then a smaller GEMM; records of the first must not leak
    in_dim, out_dim = 1024, 256
    packed = weights(in_dim, out_dim, seed=5, gaussian=True)
    dw = dev(packed)
    ws_bytes = runtime.mmq_workspace_bytes(rein.Q4_K, in_dim, 200)
    ws = hip.DeviceBuf(ws_bytes)
    for p_rows in (200, 45):
        x = np.random.default_rng(p_rows).standard_normal((p_rows, in_dim)).astype(np.float32)
        dq = quantized(x)
        dy = dev(np.full(p_rows * out_dim, np.nan, np.float32))
        runtime.mmq_xq8_ws(rein.Q4_K, dw, dq, dy, in_dim, out_dim, p_rows, ws, ws_bytes)
        hip.synchronize()
        want = orc.matvec_q8(rein.Q4_K, packed, in_dim, out_dim, dq.to_host(np.uint8), p_rows)
        assert_close_f32(dy.to_host(np.float32).reshape(p_rows, out_dim), want, what=f"reused workspace P {p_rows}")
