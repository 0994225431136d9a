"""The entry point that allocates nothing (rein_mmq_xq8_noalloc) against the entry point it is a
variant of (rein_mmq_xq8_ws with a caller's workspace of the size the fixed array is used at: the
activation image, rein_mmq_workspace_min_bytes): the same bits, on two calls in a row, the second
with a smaller input; shapes beyond the fixed array are refused."""
import numpy as np
import pytest

import reinstinct_amd as rein
from reinstinct_amd import hip, quant, runtime
from reinstinct_amd._lib import ReinError, init
from helpers import dev, random_raw_weights

pytestmark = pytest.mark.gpu


def run_pair(fmt, p_rows, in_dim, out_dim, seed):
    print(f"no-alloc entry: fmt {fmt} P {p_rows} K {in_dim} N {out_dim}", flush=True)
    raw = random_raw_weights(fmt, in_dim, out_dim, seed)
    dw = dev(quant.repack_for_matvec(fmt, raw, in_dim, out_dim))
    x = np.random.default_rng(seed).standard_normal((p_rows, in_dim)).astype(np.float32)
    d_x, dq = dev(x), hip.DeviceBuf(p_rows * (in_dim // 32) * 40)
    runtime.quantize_q8(d_x, dq, in_dim, p_rows)
    need = runtime.mmq_workspace_min_bytes(fmt, in_dim, p_rows)
    ws = hip.DeviceBuf(max(need, 16))
    d_ref = dev(np.full(p_rows * out_dim, np.nan, np.float32))
    runtime.mmq_xq8_ws(fmt, dw, dq, d_ref, in_dim, out_dim, p_rows, ws if need else None, need)
    d_got = dev(np.full(p_rows * out_dim, np.nan, np.float32))
    runtime.mmq_xq8_noalloc(fmt, dw, dq, d_got, in_dim, out_dim, p_rows)
    hip.synchronize()
    ref, got = d_ref.to_host(np.uint32), d_got.to_host(np.uint32)
    assert not np.isnan(d_got.to_host(np.float32)).any()
    assert np.array_equal(got, ref), f"no-alloc entry differs at P {p_rows} K {in_dim} N {out_dim}"
    return need


def test_no_alloc_entry_matches_the_workspace_entry_twice_in_a_row():
    init()
    hip.set_device(0)
    # Q4_K from 320 rows up, three 32-token tiles per resident workgroup (here 112 row blocks x 16 and x 14 token
    # tiles) and 2 M N K of 2.8e10 and more runs out of the fixed array; the second call is smaller than the first
    big = (2304, 14336)
    assert run_pair(rein.Q4_K, 512, *big, seed=1) > 0
    assert runtime.mmq_form_ws(rein.Q4_K, *big, 512, runtime.mmq_workspace_min_bytes(rein.Q4_K, big[0], 512)) == 1
    assert run_pair(rein.Q4_K, 448, *big, seed=2) > 0
    assert runtime.mmq_form_ws(rein.Q4_K, *big, 448, runtime.mmq_workspace_min_bytes(rein.Q4_K, big[0], 448)) == 1
    # launches that use no scratch go straight through: other formats, few rows, GEMMs too small for the fp6 launch
    assert run_pair(rein.Q6_K, 64, 512, 136, seed=3) == 0
    assert run_pair(rein.Q4_K, 40, 512, 136, seed=4) == 0
    assert run_pair(rein.Q4_K, 448, 2048, 264, seed=6) > 0
    assert runtime.mmq_form_ws(rein.Q4_K, 2048, 264, 448, runtime.mmq_workspace_min_bytes(rein.Q4_K, 2048, 448)) == 0
    # and once more the larger shape, after the smaller ones
    assert run_pair(rein.Q4_K, 512, *big, seed=5) > 0


def test_no_alloc_entry_under_stream_capture_and_without_touching_device_memory():
    # rein_noalloc_prepare places the array outside any capture; after it a call may be recorded into a graph,
    # the replays give the bits of the eager call, and the free device memory the runtime reports does not move
    init()
    hip.set_device(0)
    runtime.noalloc_prepare()
    fmt, p_rows, in_dim, out_dim = rein.Q4_K, 512, 2304, 14336
    assert runtime.mmq_workspace_min_bytes(fmt, in_dim, p_rows) > 0
    raw = random_raw_weights(fmt, in_dim, out_dim, 9)
    dw = dev(quant.repack_for_matvec(fmt, raw, in_dim, out_dim))
    x = np.random.default_rng(9).standard_normal((p_rows, in_dim)).astype(np.float32)
    d_x, dq = dev(x), hip.DeviceBuf(p_rows * (in_dim // 32) * 40)
    runtime.quantize_q8(d_x, dq, in_dim, p_rows)
    d_eager = dev(np.full(p_rows * out_dim, np.nan, np.float32))
    d_graph = dev(np.full(p_rows * out_dim, np.nan, np.float32))
    stream = hip.Stream()
    runtime.mmq_xq8_noalloc(fmt, dw, dq, d_eager, in_dim, out_dim, p_rows, stream)      # warm-up, and the eager result
    stream.synchronize()
    hip.synchronize()
    eager = d_eager.to_host(np.uint32)
    free_before = hip.mem_info()[0]
    print("no-alloc entry: capture", flush=True)
    stream.begin_capture()
    runtime.mmq_xq8_noalloc(fmt, dw, dq, d_graph, in_dim, out_dim, p_rows, stream)
    graph = stream.end_capture()
    exe = graph.instantiate()
    zero = np.zeros(p_rows * out_dim, np.float32)
    for replay in range(3):
        d_graph.copy_from_host(zero)
        hip.synchronize()
        exe.launch(stream)
        stream.synchronize()
        assert np.array_equal(d_graph.to_host(np.uint32), eager), f"replay {replay} differs from the eager call"
        # eager work between the replays
        runtime.mmq_xq8_noalloc(fmt, dw, dq, d_eager, in_dim, out_dim, p_rows, stream)
        stream.synchronize()
        assert np.array_equal(d_eager.to_host(np.uint32), eager)
    del exe, graph
    hip.synchronize()
    free_mid = hip.mem_info()[0]
    for _ in range(8):
        runtime.mmq_xq8_noalloc(fmt, dw, dq, d_eager, in_dim, out_dim, p_rows, stream)
    stream.synchronize()
    free_after = hip.mem_info()[0]
    assert free_after == free_mid, f"free device memory moved across eight calls: {free_mid} -> {free_after}"
    assert free_mid >= free_before - (4 << 20), "the graph objects aside, nothing may have been allocated"


def test_no_alloc_entry_refuses_what_the_fixed_array_cannot_hold():
    init()
    hip.set_device(0)
    p_rows, in_dim, out_dim = 1024, 5120, 128
    assert runtime.mmq_workspace_min_bytes(rein.Q4_K, in_dim, p_rows) > (8 << 20)
    raw = random_raw_weights(rein.Q4_K, in_dim, out_dim, 6)
    dw = dev(quant.repack_for_matvec(rein.Q4_K, raw, in_dim, out_dim))
    dq = hip.DeviceBuf(p_rows * (in_dim // 32) * 40)
    dy = hip.DeviceBuf(p_rows * out_dim * 4)
    with pytest.raises(ReinError) as err:
        runtime.mmq_xq8_noalloc(rein.Q4_K, dw, dq, dy, in_dim, out_dim, p_rows)
    assert err.value.code == -6 and "fixed array" in str(err.value)
