"""The entry point that allocates nothing (rein_mmq_xq8_noalloc) against the entry point it is a
variant of (rein_mmq_xq8_ws with a caller's workspace of the fixed array's size, 48 MiB): the same
bits, on two calls in a row, the second with a smaller input, through every launch form a workspace
of that size selects; shapes beyond the fixed array are refused."""
import numpy as np
import pytest

import reinstinct_amd as rein
from reinstinct_amd import hip, quant, runtime
from reinstinct_amd._lib import ReinError, init
from helpers import dev, random_raw_weights

pytestmark = pytest.mark.gpu

SCRATCH_BYTES = 48 << 20        # the stated size of the library's fixed array


def run_pair(fmt, p_rows, in_dim, out_dim, seed):
    print(f"no-alloc entry: fmt {fmt} P {p_rows} K {in_dim} N {out_dim}", flush=True)
    raw = random_raw_weights(fmt, in_dim, out_dim, seed)
    dw = dev(quant.repack_for_matvec(fmt, raw, in_dim, out_dim))
    x = np.random.default_rng(seed).standard_normal((p_rows, in_dim)).astype(np.float32)
    d_x, dq = dev(x), hip.DeviceBuf(p_rows * (in_dim // 32) * 40)
    runtime.quantize_q8(d_x, dq, in_dim, p_rows)
    ws = hip.DeviceBuf(SCRATCH_BYTES)
    d_ref = dev(np.full(p_rows * out_dim, np.nan, np.float32))
    runtime.mmq_xq8_ws(fmt, dw, dq, d_ref, in_dim, out_dim, p_rows, ws, SCRATCH_BYTES)
    d_got = dev(np.full(p_rows * out_dim, np.nan, np.float32))
    runtime.mmq_xq8_noalloc(fmt, dw, dq, d_got, in_dim, out_dim, p_rows)
    hip.synchronize()
    ref, got = d_ref.to_host(np.uint32), d_got.to_host(np.uint32)
    assert not np.isnan(d_got.to_host(np.float32)).any()
    assert np.array_equal(got, ref), f"no-alloc entry differs at P {p_rows} K {in_dim} N {out_dim}"
    return runtime.mmq_form_ws(fmt, in_dim, out_dim, p_rows, SCRATCH_BYTES)


def test_no_alloc_entry_matches_the_workspace_entry_twice_in_a_row():
    init()
    hip.set_device(0)
    # launch forms of rein_mmq_form_ws: 1 the mixed fp6 launch (activation image only), 2 the fp6 split-tail launch
    # (image + one partial tile per workgroup), 3 the int8 split-tail launch, 0 the plain launch without scratch.
    # The second call of each pair is smaller than the first and finds the first one's contents in the array.
    big = (3072, 14336)
    assert run_pair(rein.Q4_K, 384, *big, seed=1) == 1
    assert run_pair(rein.Q4_K, 352, *big, seed=2) == 1
    tail = (5120, 6144)
    assert run_pair(rein.Q4_K, 512, *tail, seed=7) == 2
    assert run_pair(rein.Q4_K, 480, 4096, 8192, seed=8) == 2
    assert run_pair(rein.Q6_K, 384, 4096, 12288, seed=9) == 3
    assert run_pair(rein.Q4_K, 448, 2048, 264, seed=6) == 3
    assert run_pair(rein.Q6_K, 64, 512, 136, seed=3) == 0
    assert run_pair(rein.Q4_K, 40, 512, 136, seed=4) == 0
    # and once more the first shapes, after the others
    assert run_pair(rein.Q4_K, 512, *tail, seed=10) == 2
    assert run_pair(rein.Q4_K, 384, *big, seed=5) == 1


@pytest.mark.parametrize("shape, form", [((384, 3072, 14336), 1), ((512, 5120, 6144), 2), ((448, 2048, 264), 3)])
def test_no_alloc_entry_under_stream_capture_and_without_touching_device_memory(shape, form):
    # rein_noalloc_prepare places the array outside any capture; after it a call may be recorded into a graph,
    # the replays give the bits of the eager call, and the free device memory the runtime reports does not move
    init()
    hip.set_device(0)
    runtime.noalloc_prepare()
    fmt, (p_rows, in_dim, out_dim) = rein.Q4_K, shape
    assert runtime.mmq_workspace_min_bytes(fmt, in_dim, p_rows) > 0
    assert runtime.mmq_form_ws(fmt, in_dim, out_dim, p_rows, SCRATCH_BYTES) == form
    print(f"no-alloc entry under capture: P {p_rows} K {in_dim} N {out_dim} form {form}", flush=True)
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


@pytest.mark.parametrize("fmt,p_rows,in_dim,out_dim", [(rein.IQ3_S, 4, 1536, 1030), (rein.Q5_K, 12, 2304, 520), (rein.Q6_K, 24, 1280, 2052),
                                                        (rein.Q8_0, 2, 8192, 4100), (rein.Q4_0, 7, 1056, 16390)])
def test_no_alloc_entry_with_few_rows_under_stream_capture(fmt, p_rows, in_dim, out_dim):
    # up to 32 rows the entry point launches the few-row kernels (decode matvecs, skinny MMQ, the 4x4x4 kernels), whose
    # handles rein_noalloc_prepare has looked up as well: the first call of a shape may already be a recorded one
    init()
    hip.set_device(0)
    runtime.noalloc_prepare()
    print(f"no-alloc entry, few rows under capture: fmt {fmt} P {p_rows} K {in_dim} N {out_dim}", flush=True)
    dw = dev(quant.repack_for_matvec(fmt, random_raw_weights(fmt, in_dim, out_dim, 21), in_dim, out_dim))
    x = np.random.default_rng(21).standard_normal((p_rows, in_dim)).astype(np.float32)
    d_x, dq = dev(x), hip.DeviceBuf(p_rows * (in_dim // 32) * 40)
    runtime.quantize_q8(d_x, dq, in_dim, p_rows)
    hip.synchronize()
    d_graph = dev(np.full(p_rows * out_dim, np.nan, np.float32))
    stream = hip.Stream()
    stream.begin_capture()
    runtime.mmq_xq8_noalloc(fmt, dw, dq, d_graph, in_dim, out_dim, p_rows, stream)
    exe = stream.end_capture().instantiate()
    d_eager = dev(np.full(p_rows * out_dim, np.nan, np.float32))
    d_ws = dev(np.full(p_rows * out_dim, np.nan, np.float32))
    for replay in range(2):
        d_graph.copy_from_host(np.zeros(p_rows * out_dim, np.float32))
        hip.synchronize()
        exe.launch(stream)
        stream.synchronize()
        # the eager call of the same entry point, and rein_mmq_xq8_ws with a workspace of the array's size, between the replays
        runtime.mmq_xq8_noalloc(fmt, dw, dq, d_eager, in_dim, out_dim, p_rows, stream)
        ws = hip.DeviceBuf(SCRATCH_BYTES)
        runtime.mmq_xq8_ws(fmt, dw, dq, d_ws, in_dim, out_dim, p_rows, ws, SCRATCH_BYTES, stream)
        stream.synchronize()
        assert np.array_equal(d_graph.to_host(np.uint32), d_eager.to_host(np.uint32)), f"replay {replay} differs from the eager call"
        assert np.array_equal(d_graph.to_host(np.uint32), d_ws.to_host(np.uint32)), f"replay {replay} differs from rein_mmq_xq8_ws"


def test_no_alloc_entry_refuses_what_the_fixed_array_cannot_hold():
    init()
    hip.set_device(0)
    p_rows, in_dim, out_dim = 4864, 5120, 128
    assert runtime.mmq_workspace_min_bytes(rein.Q4_K, in_dim, p_rows) > SCRATCH_BYTES
    raw = random_raw_weights(rein.Q4_K, in_dim, out_dim, 6)
    dw = dev(quant.repack_for_matvec(rein.Q4_K, raw, in_dim, out_dim))
    dq = hip.DeviceBuf(p_rows * (in_dim // 32) * 40)
    dy = hip.DeviceBuf(p_rows * out_dim * 4)
    with pytest.raises(ReinError) as err:
        runtime.mmq_xq8_noalloc(rein.Q4_K, dw, dq, dy, in_dim, out_dim, p_rows)
    assert err.value.code == -6 and "fixed array" in str(err.value)
