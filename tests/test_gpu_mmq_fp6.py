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
from reinstinct_amd._lib import ReinError, init, set_option
from oracle import orc
from helpers import assert_close_f32, random_raw_weights

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def gpu():
    init()
    hip.set_device(0)
    # the library keeps small GEMMs on the int8 launch; these tests are about the fp6 one
    set_option("REIN_MMQ6_FROM", "17")
    yield
    hip.synchronize()
    set_option("REIN_MMQ6_FROM", None)


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
            set_option("REIN_MMQ6_N4", str(n4))
            set_option("REIN_MMQ6_N2", str(n2))
            assert runtime.mmq_tile_plan_ws(rein.Q4_K, out_dim, p_rows) == (n4, n2)
            outs[(n4, n2)] = run_ws(dw, dq, in_dim, out_dim, p_rows).view(np.uint32)
    finally:
        set_option("REIN_MMQ6_N4", None)
        set_option("REIN_MMQ6_N2", None)
    first = next(iter(outs.values()))
    for k, v in outs.items():
        assert np.array_equal(v, first), f"split {k} differs"


def test_workspace_contract():
    p_rows, in_dim, out_dim = 64, 512, 128
    packed = weights(in_dim, out_dim, seed=1, gaussian=True)
    x = np.random.default_rng(2).standard_normal((p_rows, in_dim)).astype(np.float32)
    dw, dq = dev(packed), quantized(x)
    need = runtime.mmq_workspace_min_bytes(rein.Q4_K, in_dim, p_rows)
    assert 0 < need <= runtime.mmq_workspace_bytes(rein.Q4_K, in_dim, p_rows)
    # formats and row counts off the fp6 launch need no workspace (what they can use is room for the partial
    # tiles of the int8 split-tail launch); up to 16 rows nothing uses one
    assert runtime.mmq_workspace_min_bytes(rein.Q6_K, in_dim, p_rows) == 0
    assert runtime.mmq_workspace_bytes(rein.Q4_K, in_dim, 16) == 0
    set_option("REIN_MMQ6_FROM", "320")
    assert runtime.mmq_workspace_min_bytes(rein.Q4_K, in_dim, 256) == 0 and runtime.mmq_workspace_min_bytes(rein.Q4_K, in_dim, 320) > 0
    set_option("REIN_MMQ6_FROM", "17")
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


# ---- split-tail launch: whole tiles in rounds over the resident workgroups, the tiles left over split along the
# contraction, their partial tiles summed in range order by whichever workgroup completes the tile
def run_split_tail(dw, dq, in_dim, out_dim, p_rows, grid):
    ws_bytes = runtime.mmq_workspace_bytes(rein.Q4_K, in_dim, p_rows)
    set_option("REIN_MMQ6_SK_GRID", str(grid))
    try:
        assert runtime.mmq_form_ws(rein.Q4_K, in_dim, out_dim, p_rows, ws_bytes) == 2, "shape does not take the split-tail launch"
        ws = hip.DeviceBuf(ws_bytes)
        dy = dev(np.full(p_rows * out_dim, np.nan, np.float32))
        outs = []
        for _ in range(2):                               # the second launch finds the first one's counters and partial tiles
            runtime.mmq_xq8_ws(rein.Q4_K, dw, dq, dy, in_dim, out_dim, p_rows, ws, ws_bytes)
            hip.synchronize()
            outs.append(dy.to_host(np.float32).reshape(p_rows, out_dim).copy())
    finally:
        set_option("REIN_MMQ6_SK_GRID", None)
    return outs


# (tokens, K, N, workgroups): 128 units on 512 workgroups (no whole round, four ranges per tile); 18 units on 64
# (three ranges over four chunks: uneven, ragged rows); 20 units on 8 (two whole rounds, then four tiles in two
# ranges each; ragged last token group and last tile); 8 units on 16; 15 units on 32 (two ranges over five chunks)
@pytest.mark.parametrize("p_rows,in_dim,out_dim,grid,gaussian", [
    (512, 2048, 4096, 512, True), (256, 1024, 1100, 64, False), (470, 768, 640, 8, True), (128, 2048, 1024, 16, True),
    (384, 1280, 520, 32, False)])
def test_split_tail_matches_oracle_and_repeats(p_rows, in_dim, out_dim, grid, gaussian):
    print(f"mmq6 split-tail P {p_rows} K {in_dim} N {out_dim} grid {grid}", flush=True)
    packed = weights(in_dim, out_dim, seed=p_rows + grid, gaussian=gaussian)
    x = np.random.default_rng(grid).standard_normal((p_rows, in_dim)).astype(np.float32)
    dw, dq = dev(packed), quantized(x)
    first, second = run_split_tail(dw, dq, in_dim, out_dim, p_rows, grid)
    want = orc.matvec_q8(rein.Q4_K, packed, in_dim, out_dim, dq.to_host(np.uint8), p_rows)
    assert_close_f32(first, want, what=f"split-tail {p_rows}x{in_dim}x{out_dim} grid {grid}")
    assert np.array_equal(first.view(np.uint32), second.view(np.uint32)), "split-tail result is not reproducible"


def test_split_tail_needs_the_full_workspace():
    p_rows, in_dim, out_dim = 512, 2048, 4096
    full, least = runtime.mmq_workspace_bytes(rein.Q4_K, in_dim, p_rows), runtime.mmq_workspace_min_bytes(rein.Q4_K, in_dim, p_rows)
    assert 0 < least < full
    assert runtime.mmq_form_ws(rein.Q4_K, in_dim, out_dim, p_rows, full) == 2
    assert runtime.mmq_form_ws(rein.Q4_K, in_dim, out_dim, p_rows, full - 1) == 1
    assert runtime.mmq_form_ws(rein.Q4_K, in_dim, out_dim, p_rows, least - 1) == 0
    # the two fp6 launches agree within the bar (different order of the fp32 additions across superblocks)
    packed = weights(in_dim, out_dim, seed=21, gaussian=True)
    x = np.random.default_rng(22).standard_normal((p_rows, in_dim)).astype(np.float32)
    dw, dq = dev(packed), quantized(x)
    outs = []
    for nbytes in (full, least):
        ws = hip.DeviceBuf(nbytes)
        dy = dev(np.full(p_rows * out_dim, np.nan, np.float32))
        runtime.mmq_xq8_ws(rein.Q4_K, dw, dq, dy, in_dim, out_dim, p_rows, ws, nbytes)
        hip.synchronize()
        outs.append(dy.to_host(np.float32).reshape(p_rows, out_dim))
    assert_close_f32(outs[0], outs[1], what="split-tail vs one group per workgroup")


def test_workspace_launches_at_the_benchmark_shape():
    # 5120 x 17408 at 512 tokens (one whole round + 32 tiles split eight ways), 1024 tokens (two rounds + 64 tiles
    # split four ways) and 2048 tokens (mixed launch):
    # every element against the int8 launch, sampled tokens against the oracle; the default row threshold applies
    set_option("REIN_MMQ6_FROM", None)
    try:
        in_dim, out_dim = 5120, 17408
        w = (np.random.default_rng(31).standard_normal((512, in_dim)) * 0.02).astype(np.float32)
        raw = np.tile(quant.quantize_weights(rein.Q4_K, w), out_dim // 512)
        packed = quant.repack_for_matvec(rein.Q4_K, raw, in_dim, out_dim)
        x = np.random.default_rng(32).standard_normal((2048, in_dim)).astype(np.float32)
        dw, dq = dev(packed), quantized(x)
        xq = dq.to_host(np.uint8).reshape(2048, -1)
        for m, form in ((512, 2), (1024, 2), (2048, 1)):
            print(f"mmq6 benchmark shape M {m}", flush=True)
            ws_bytes = runtime.mmq_workspace_bytes(rein.Q4_K, in_dim, m)
            assert runtime.mmq_form_ws(rein.Q4_K, in_dim, out_dim, m, ws_bytes) == form
            ws = hip.DeviceBuf(ws_bytes)
            dy, dy8 = dev(np.full(m * out_dim, np.nan, np.float32)), dev(np.full(m * out_dim, np.nan, np.float32))
            runtime.mmq_xq8_ws(rein.Q4_K, dw, dq, dy, in_dim, out_dim, m, ws, ws_bytes)
            runtime.mmq_xq8(rein.Q4_K, dw, dq, dy8, in_dim, out_dim, m)
            hip.synchronize()
            got = dy.to_host(np.float32).reshape(m, out_dim)
            assert_close_f32(got, dy8.to_host(np.float32).reshape(m, out_dim), what=f"workspace launch vs int8 launch, M {m}")
            toks = np.unique(np.r_[0, 127, 128, m - 129, m - 1, np.random.default_rng(m).integers(0, m, 8)])
            want = orc.matvec_q8(rein.Q4_K, packed, in_dim, out_dim, np.ascontiguousarray(xq[toks]).reshape(-1), len(toks))
            assert_close_f32(got[toks], want, what=f"workspace launch vs oracle, M {m}")
    finally:
        set_option("REIN_MMQ6_FROM", "17")
