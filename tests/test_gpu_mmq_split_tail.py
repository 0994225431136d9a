"""GPU parity of the split-tail launch of the int8 prefill MMQ GEMM (rein_mmq_<fmt>_sk / _sk32 +
rein_mmq_tail_sum_t64 / _t32: whole workgroup tiles in rounds, the tiles left over split along the
contraction into partial tiles that a second launch adds in range order), through the C ABI,
against the CPU oracle.

Bar: fp32 outputs within 1e-3 relative / 1e-4 absolute of the oracle; the same bits on every
repetition (the partial tiles are added in a fixed order).
"""
import os

import numpy as np
import pytest

import reinstinct_amd as rein
from reinstinct_amd import hip, quant, runtime
from reinstinct_amd._lib import init, set_option
from oracle import orc
from helpers import assert_close_f32, dev, random_raw_weights

pytestmark = pytest.mark.gpu

KNOBS = ("REIN_MMQ_SK", "REIN_MMQ_SK_GRID", "REIN_MMQ_SK_SPLIT", "REIN_MMQ_SK_TM")


@pytest.fixture(scope="module", autouse=True)
def gpu():
    init()
    hip.set_device(0)
    set_option("REIN_MMQ6", "0")                    # Q4_K on the int8 tile too
    yield
    hip.synchronize()
    for k in KNOBS + ("REIN_MMQ6",):
        set_option(k, None)


@pytest.fixture(autouse=True)
def clean_knobs():
    for k in KNOBS:
        set_option(k, None)
    yield
    for k in KNOBS:
        set_option(k, None)


def weights(fmt, in_dim, out_dim, seed):
    raw = random_raw_weights(fmt, in_dim, out_dim, seed)
    return quant.repack_for_matvec(fmt, raw, in_dim, out_dim)


def quantized(x):
    n, k = x.shape
    dx, dq = dev(x), hip.DeviceBuf(n * (k // 32) * 40)
    runtime.quantize_q8(dx, dq, k, n)
    hip.synchronize()
    return dq


def run(fmt, dw, dq, in_dim, out_dim, p_rows, want_form=3):
    ws_bytes = runtime.mmq_workspace_bytes(fmt, in_dim, p_rows)
    assert ws_bytes > 0
    assert runtime.mmq_form_ws(fmt, in_dim, out_dim, p_rows, ws_bytes) == want_form
    ws = dev(np.full(ws_bytes // 4, np.nan, np.float32))          # stale partial tiles must not matter
    outs = []
    for _ in range(2):
        dy = dev(np.full(p_rows * out_dim, np.nan, np.float32))
        runtime.mmq_xq8_ws(fmt, dw, dq, dy, in_dim, out_dim, p_rows, ws, ws_bytes)
        hip.synchronize()
        outs.append(dy.to_host(np.float32).reshape(p_rows, out_dim).copy())
    return outs


K_FORMATS = [rein.Q4_K, rein.Q5_K, rein.Q6_K]
B32_FORMATS = [rein.Q8_0, rein.Q4_0, rein.IQ4_XS, rein.IQ3_S]

# (tokens, K, N, grid, ranges per tail unit, unit width): whole rounds + a split tail, a tail only,
# 32-token units with ragged tokens, rows off the 128-row grain, ranges of a single chunk
CASES = [
    (40, 1024, 260, 8, 2, 0), (200, 768, 640, 8, 2, 0), (24, 2048, 1024, 0, 0, 0), (130, 1024, 300, 16, 3, 0),
    (64, 512, 136, 8, 4, 0), (96, 1280, 520, 8, 2, 64), (65, 768, 128, 0, 3, 32)]


@pytest.mark.parametrize("fmt", K_FORMATS + B32_FORMATS)
@pytest.mark.parametrize("p_rows,in_dim,out_dim,grid,split,tm", CASES)
def test_split_tail_matches_oracle_and_repeats(fmt, p_rows, in_dim, out_dim, grid, split, tm):
    print(f"int8 split-tail fmt {fmt} P {p_rows} K {in_dim} N {out_dim} grid {grid} split {split} tm {tm}", flush=True)
    if grid: set_option("REIN_MMQ_SK_GRID", str(grid))
    else: set_option("REIN_MMQ_SK", "2")
    if split: set_option("REIN_MMQ_SK_SPLIT", str(split))
    if tm: set_option("REIN_MMQ_SK_TM", str(tm))
    packed = weights(fmt, in_dim, out_dim, seed=p_rows + out_dim)
    x = np.random.default_rng(in_dim).standard_normal((p_rows, in_dim)).astype(np.float32)
    dw, dq = dev(packed), quantized(x)
    first, second = run(fmt, dw, dq, in_dim, out_dim, p_rows)
    want = orc.matvec_q8(fmt, packed, in_dim, out_dim, dq.to_host(np.uint8), p_rows)
    assert_close_f32(first, want, what=f"split-tail fmt {fmt} {p_rows}x{in_dim}x{out_dim}")
    assert np.array_equal(first.view(np.uint32), second.view(np.uint32)), "a repetition gave other bits"


@pytest.mark.parametrize("fmt,in_dim", [(rein.Q8_0, 352), (rein.Q4_0, 608), (rein.Q8_0, 96)])
def test_split_tail_with_a_ragged_last_chunk(fmt, in_dim):
    # contractions that are not whole 256-weight chunks: the last range ends inside a chunk
    p_rows, out_dim = 50, 200
    set_option("REIN_MMQ_SK_GRID", "8")
    set_option("REIN_MMQ_SK_SPLIT", "2")
    packed = weights(fmt, in_dim, out_dim, seed=in_dim)
    x = np.random.default_rng(3).standard_normal((p_rows, in_dim)).astype(np.float32)
    dw, dq = dev(packed), quantized(x)
    first, second = run(fmt, dw, dq, in_dim, out_dim, p_rows)
    want = orc.matvec_q8(fmt, packed, in_dim, out_dim, dq.to_host(np.uint8), p_rows)
    assert_close_f32(first, want, what=f"split-tail fmt {fmt} K {in_dim}")
    assert np.array_equal(first.view(np.uint32), second.view(np.uint32))


def test_the_library_takes_it_for_small_gemms_only_with_the_workspace():
    # 17408 -> 5120 at 64 tokens: 40 workgroup tiles as whole units, split twelve ways by the library itself
    fmt, p_rows, in_dim, out_dim = rein.Q8_0, 64, 17408, 5120
    full = runtime.mmq_workspace_bytes(fmt, in_dim, p_rows)
    assert full > 0 and runtime.mmq_workspace_min_bytes(fmt, in_dim, p_rows) == 0
    assert runtime.mmq_form_ws(fmt, in_dim, out_dim, p_rows, full) == 3
    assert runtime.mmq_form_ws(fmt, in_dim, out_dim, p_rows, full - 1) == 0       # no room for the partial tiles
    assert runtime.mmq_form_ws(fmt, in_dim, out_dim, 16, full) == 0               # the skinny kernel's rows
    assert runtime.mmq_form_ws(fmt, in_dim, 17408, 2048, full) == 0               # many rounds: the mixed launch
    w = (np.random.default_rng(4).standard_normal((256, in_dim)) * 0.02).astype(np.float32)
    raw = np.tile(quant.quantize_weights(fmt, w), out_dim // 256)
    packed = quant.repack_for_matvec(fmt, raw, in_dim, out_dim)
    x = np.random.default_rng(5).standard_normal((p_rows, in_dim)).astype(np.float32)
    dw, dq = dev(packed), quantized(x)
    first, second = run(fmt, dw, dq, in_dim, out_dim, p_rows)
    # without the workspace: the plain launch, same result within the bar
    dy = dev(np.full(p_rows * out_dim, np.nan, np.float32))
    runtime.mmq_xq8_ws(fmt, dw, dq, dy, in_dim, out_dim, p_rows, None, 0)
    hip.synchronize()
    plain = dy.to_host(np.float32).reshape(p_rows, out_dim)
    assert_close_f32(first, plain, what="split-tail vs plain launch")
    rows = np.arange(0, out_dim, 37)
    sub = quant.repack_for_matvec(fmt, raw.reshape(out_dim, -1)[rows].reshape(-1), in_dim, len(rows))
    want = orc.matvec_q8(fmt, sub, in_dim, len(rows), dq.to_host(np.uint8), p_rows)
    assert_close_f32(first[:, rows], want, what="split-tail at 17408 -> 5120, every 37th row")
    assert np.array_equal(first.view(np.uint32), second.view(np.uint32))


def test_matmul_ws_carries_the_partial_tile_room():
    # quantize + GEMM out of one scratch buffer: the scratch size includes the 16 MiB, and the GEMM takes the
    # same launch and gives the same bits as the two calls
    fmt, p_rows, in_dim, out_dim = rein.Q6_K, 40, 2048, 512
    packed = weights(fmt, in_dim, out_dim, seed=9)
    x = np.random.default_rng(10).standard_normal((p_rows, in_dim)).astype(np.float32)
    dw, dq = dev(packed), quantized(x)
    assert runtime.mmq_form_ws(fmt, in_dim, out_dim, p_rows, runtime.mmq_workspace_bytes(fmt, in_dim, p_rows)) == 3
    two_calls, _ = run(fmt, dw, dq, in_dim, out_dim, p_rows)
    sb = runtime.matmul_scratch_bytes(fmt, in_dim, p_rows)
    assert sb >= p_rows * (in_dim // 32) * 40 + runtime.mmq_workspace_bytes(fmt, in_dim, p_rows)
    scratch = hip.DeviceBuf(sb)
    dy = dev(np.full(p_rows * out_dim, np.nan, np.float32))
    runtime.matmul_ws(fmt, dw, dev(x), dy, in_dim, out_dim, p_rows, scratch, sb)
    hip.synchronize()
    assert np.array_equal(dy.to_host(np.uint32).reshape(p_rows, out_dim), two_calls.view(np.uint32))


def test_split_tail_replays_from_a_graph():
    # the two launches (GEMM with partial tiles, tail sum) captured once and replayed with the program's own
    # eager work between the replays: every replay gives the eager bits
    fmt, p_rows, in_dim, out_dim = rein.Q8_0, 48, 2048, 640
    packed = weights(fmt, in_dim, out_dim, seed=12)
    x = np.random.default_rng(13).standard_normal((p_rows, in_dim)).astype(np.float32)
    dw, dq = dev(packed), quantized(x)
    ws_bytes = runtime.mmq_workspace_bytes(fmt, in_dim, p_rows)
    assert runtime.mmq_form_ws(fmt, in_dim, out_dim, p_rows, ws_bytes) == 3
    eager, _ = run(fmt, dw, dq, in_dim, out_dim, p_rows)
    stream = hip.Stream()
    ws = hip.DeviceBuf(ws_bytes)
    dy = dev(np.zeros(p_rows * out_dim, np.float32))
    stream.begin_capture()
    runtime.mmq_xq8_ws(fmt, dw, dq, dy, in_dim, out_dim, p_rows, ws, ws_bytes, stream)
    graph = stream.end_capture()
    ex = graph.instantiate()
    for replay in range(3):
        dy.copy_from_host(np.zeros(p_rows * out_dim, np.float32))
        other, _ = run(fmt, dw, dq, in_dim, out_dim, p_rows)               # eager work between the replays
        assert np.array_equal(other.view(np.uint32), eager.view(np.uint32))
        ex.launch(stream)
        stream.synchronize()
        assert np.array_equal(dy.to_host(np.uint32).reshape(p_rows, out_dim), eager.view(np.uint32)), f"replay {replay}"
