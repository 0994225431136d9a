"""Drop-in boundary of the MoE prefill path and the stated sizes, on the GPU.

The reference host finds kernels by name in a code object and launches them with its own,
hard-coded geometry (src/runtime/qwen35.rs:2892-3064).  These tests do exactly that through
rein_launch_kernel -- sort chain, gather, the four reference-named grouped GEMM symbols,
scatter -- with the reference's grids and with `tile_off` built at both token counts the
reference's two runtimes use (MOE_GEMM_BN = 16, qwen35.rs:127; 32, gemma4.rs:109), and compare
with the oracle.  Also here: the dot4 batched kernels at 3..8 rows (the library's own dispatch
sends those row counts to matrix-core kernels), and BASELINE's first configuration at its
stated 4096 x 4096.
"""
import ctypes as C
import os

import numpy as np
import pytest

import reinstinct_amd as rein
from reinstinct_amd import hip, quant, runtime
from reinstinct_amd._lib import init
from oracle import orc
from helpers import assert_close_f32, random_raw_weights, rel_l2

pytestmark = pytest.mark.gpu

NAME = {rein.Q4_0: "q4_0", rein.Q8_0: "q8_0", rein.Q4_K: "q4k", rein.Q5_K: "q5k", rein.Q6_K: "q6k",
        rein.IQ4_XS: "iq4xs", rein.IQ3_S: "iq3s"}


@pytest.fixture(scope="module", autouse=True)
def gpu():
    init()
    hip.set_device(0)
    yield
    hip.synchronize()


from helpers import dev  # noqa: E402  (uploads that stay alive until the test's last launch has finished)


def vp(buf):
    return C.c_void_p(buf.ptr)


def u32(v):
    return C.c_uint(v)


def expert_slabs(fmt, in_dim, out_dim, n_expert, seed):
    slabs = []
    for e in range(n_expert):
        raw = random_raw_weights(fmt, in_dim, out_dim, seed + e)
        slabs.append(quant.repack_for_matvec(fmt, raw, in_dim, out_dim))
    return np.concatenate(slabs)


def reference_sort_chain(mod, d_ids, n_entries, n_expert, bn):
    """launch_moe_sort as qwen35.rs:2892-2938 issues it: zero, histogram, scan, zero, scatter"""
    count, cursor = hip.DeviceBuf(n_expert * 4), hip.DeviceBuf(n_expert * 4)
    perm = dev(np.full(n_entries, -1, np.int32))
    eoff, toff = hip.DeviceBuf((n_expert + 1) * 4), hip.DeviceBuf((n_expert + 1) * 4)
    ge, gn = (n_expert + 255) // 256, (n_entries + 255) // 256
    mod.function("moe_sort_zero").launch((ge, 1, 1), (256, 1, 1), 0, None, [vp(count), u32(n_expert)])
    mod.function("moe_sort_histogram").launch((gn, 1, 1), (256, 1, 1), 0, None,
                                              [vp(d_ids), vp(count), u32(n_entries), u32(n_expert)])
    mod.function("moe_sort_scan").launch((1, 1, 1), (64, 1, 1), 0, None,
                                         [vp(count), vp(eoff), vp(toff), u32(n_expert), u32(bn)])
    mod.function("moe_sort_zero").launch((ge, 1, 1), (256, 1, 1), 0, None, [vp(cursor), u32(n_expert)])
    mod.function("moe_sort_scatter").launch((gn, 1, 1), (256, 1, 1), 0, None,
                                            [vp(d_ids), vp(eoff), vp(cursor), vp(perm), u32(n_entries), u32(n_expert)])
    hip.synchronize()
    return perm, eoff, toff


# (format, contraction, tokens per tile the scan is given): the reference passes 16 for every
# format (qwen35.rs:127, 2917) and 32 from its other runtime (gemma4.rs:109)
@pytest.mark.parametrize("fmt,in_dim,bn", [(rein.Q4_K, 512, 16), (rein.Q4_K, 512, 32), (rein.Q5_K, 256, 16),
                                           (rein.Q6_K, 768, 16), (rein.Q6_K, 768, 32), (rein.Q8_0, 352, 16),
                                           (rein.Q8_0, 352, 32)])
def test_reference_named_moe_prefill_chain(fmt, in_dim, bn):
    print(f"grouped by name fmt {fmt} K {in_dim} bn {bn}", flush=True)
    out_dim, n_expert, n_tok, n_used = 200, 9, 70, 3
    n = n_tok * n_used
    rng = np.random.default_rng(fmt + bn)
    ids = rng.integers(0, n_expert, (n_tok, n_used)).astype(np.int32)
    ids[ids == 4] = 5                                        # an expert without tokens
    ids[:50, 0] = 1                                          # and one with more than a tile of them
    slab = expert_slabs(fmt, in_dim, out_dim, n_expert, seed=700 + fmt)
    bpe = quant.repacked_len(fmt, in_dim, out_dim)
    x = rng.standard_normal((n_tok, in_dim)).astype(np.float32)
    mod = hip.Module.builtin()

    d_ids = dev(ids)
    perm, eoff, toff = reference_sort_chain(mod, d_ids, n, n_expert, bn)
    h_perm, h_eoff, h_toff = perm.to_host(np.int32), eoff.to_host(np.int32), toff.to_host(np.int32)
    _, want_eoff, want_toff = orc.moe_sort(ids, n_expert, bn)
    assert np.array_equal(h_eoff, want_eoff) and np.array_equal(h_toff, want_toff)
    flat = ids.ravel()
    assert sorted(h_perm.tolist()) == list(range(n))         # every entry placed once (qwen35.rs:2956-2987)
    for e in range(n_expert):
        assert np.all(flat[h_perm[h_eoff[e]:h_eoff[e + 1]]] == e)

    # quantize (qwen35.rs:3202-3211) and gather (2996-3012) with the reference's grids
    nsub = in_dim // 32
    d_x, d_xq = dev(x), hip.DeviceBuf(n_tok * nsub * 40)
    mod.function("quantize_q8_f32").launch(((in_dim + 255) // 256, n_tok, 1), (256, 1, 1), 0, None,
                                           [vp(d_x), vp(d_xq), u32(in_dim)])
    d_gin = hip.DeviceBuf(n * nsub * 40)
    mod.function("moe_gather_xq").launch(((nsub + 255) // 256, n, 1), (256, 1, 1), 0, None,
                                         [vp(d_xq), vp(perm), vp(d_gin), u32(nsub), u32(n_used), u32(n)])
    # grouped GEMM (3036-3064): grid (ceil(out / 64), tile_ub) x 256 with the reference's bound
    d_slab = dev(slab)
    d_y = dev(np.full(n * out_dim, np.nan, np.float32))
    tile_ub = (n + bn - 1) // bn + n_expert
    mod.function(f"mmq_gemm_{NAME[fmt]}_grouped_f32").launch(
        ((out_dim + 63) // 64, tile_ub, 1), (256, 1, 1), 0, None,
        [vp(d_slab), u32(bpe), vp(eoff), vp(toff), u32(n_expert), vp(d_gin), vp(d_y), u32(in_dim), u32(out_dim)])
    # scatter back to entry order (3014-3030)
    d_back = dev(np.full(n * out_dim, np.nan, np.float32))
    mod.function("moe_scatter_rows").launch(((out_dim + 255) // 256, n, 1), (256, 1, 1), 0, None,
                                            [vp(d_y), vp(perm), vp(d_back), u32(out_dim), u32(n)])
    hip.synchronize()

    xq = d_xq.to_host(np.uint8)
    assert np.array_equal(xq, orc.quantize_q8(x))
    gin = d_gin.to_host(np.uint8)
    assert np.array_equal(gin, orc.moe_gather_xq(xq, h_perm, nsub, n_used))
    want = orc.grouped_gemm(fmt, slab, bpe, h_eoff, gin, in_dim, out_dim)
    got = d_y.to_host(np.float32).reshape(n, out_dim)
    assert_close_f32(got, want, what=f"mmq_gemm_{NAME[fmt]}_grouped_f32 bn {bn}")
    assert np.array_equal(d_back.to_host(np.float32).reshape(n, out_dim), orc.moe_scatter_rows(got, h_perm, out_dim))
    del d_slab, d_ids, d_x                                   # alive until the launches above have finished


def test_library_grouped_launch_on_the_reference_named_kernel(options):
    # rein_moe_grouped_gemm falls back to the reference-named, grid-striding kernel when the
    # tile bound exceeds grid.y; the switch below forces that launch at a small size
    options.set("REIN_GROUPED_STRIDED", "1")
    fmt, in_dim, out_dim, n_expert, n_tok, n_used = rein.Q6_K, 768, 264, 5, 40, 2
    n = n_tok * n_used
    rng = np.random.default_rng(77)
    ids = rng.integers(0, n_expert, (n_tok, n_used)).astype(np.int32)
    slab = expert_slabs(fmt, in_dim, out_dim, n_expert, seed=900)
    bpe = quant.repacked_len(fmt, in_dim, out_dim)
    bufs = [hip.DeviceBuf(n_expert * 4), hip.DeviceBuf(n_expert * 4), dev(np.full(n, -1, np.int32)),
            hip.DeviceBuf((n_expert + 1) * 4), hip.DeviceBuf((n_expert + 1) * 4)]
    d_ids = dev(ids)
    runtime.moe_sort(d_ids, n, n_expert, runtime.moe_gemm_bn(), *bufs)
    x = rng.standard_normal((n_tok, in_dim)).astype(np.float32)
    d_x, d_xq = dev(x), hip.DeviceBuf(n_tok * (in_dim // 32) * 40)
    runtime.quantize_q8(d_x, d_xq, in_dim, n_tok)
    d_gin = hip.DeviceBuf(n * (in_dim // 32) * 40)
    runtime.moe_gather_xq(d_xq, bufs[2], d_gin, in_dim // 32, n_used, n)
    d_slab = dev(slab)
    d_y = dev(np.full(n * out_dim, np.nan, np.float32))
    runtime.moe_grouped_gemm(fmt, d_slab, bpe, bufs[3], bufs[4], n_expert, d_gin, d_y, in_dim, out_dim, n)
    hip.synchronize()
    want = orc.grouped_gemm(fmt, slab, bpe, bufs[3].to_host(np.int32), d_gin.to_host(np.uint8), in_dim, out_dim)
    assert_close_f32(d_y.to_host(np.float32).reshape(n, out_dim), want, what="strided grouped launch")


# ---- the dot4 batched kernels at the row counts the library sends elsewhere ------------
@pytest.mark.parametrize("fmt", [rein.Q4_0, rein.Q8_0, rein.Q4_K, rein.Q5_K, rein.Q6_K, rein.IQ4_XS, rein.IQ3_S])
def test_dot4_batched_kernels_3_to_8_rows(fmt, options):
    # rein_mv_<fmt>_r*_b4 / _b8: with both switches out of reach every row count stays on v_dot4
    options.set("REIN_SKINNY_FROM", "99")
    options.set("REIN_QUAD_FROM", "99")
    in_dim, out_dim = 1024, 391
    raw = random_raw_weights(fmt, in_dim, out_dim, 40 + fmt)
    packed = quant.repack_for_matvec(fmt, raw, in_dim, out_dim)
    x = np.random.default_rng(41).standard_normal((8, in_dim)).astype(np.float32)
    d_x, dq = dev(x), hip.DeviceBuf(8 * (in_dim // 32) * 40)
    runtime.quantize_q8(d_x, dq, in_dim, 8)
    dw = dev(packed)
    hip.synchronize()
    xq = dq.to_host(np.uint8)
    for rows in (3, 4, 5, 6, 7, 8):
        print(f"dot4 fmt {fmt} rows {rows}", flush=True)
        dy = dev(np.full(rows * out_dim, np.nan, np.float32))
        runtime.matvec_batched_xq8(fmt, dw, dq, dy, in_dim, out_dim, rows)
        hip.synchronize()
        want = orc.matvec_q8(fmt, packed, in_dim, out_dim, xq[: rows * (in_dim // 32) * 40], rows)
        assert_close_f32(dy.to_host(np.float32).reshape(rows, out_dim), want, what=f"dot4 fmt {fmt} rows {rows}")


# ---- BASELINE configs[0] at its stated size -------------------------------------------
def test_config0_q4k_4096_by_4096():
    # 4096 x 4096 fp32 ~N(0, 0.02) -> Q4_K -> repacked v2 (pad path: 129 sub-blocks per row),
    # x ~N(0, 1) of length 4096 -> quantize_q8, y of length 4096: bytes and block dots bit-exact,
    # fp32 within 1e-3 / 1e-4 of the int8 oracle and within the reference's rel_l2 bar of the
    # dequantize -> f32 CPU path (5e-2 here: see test_matvec_gaussian_weights_config1_shape)
    in_dim = out_dim = 4096
    w = (np.random.default_rng(2024).standard_normal((out_dim, in_dim)) * 0.02).astype(np.float32)
    raw = quant.quantize_weights(rein.Q4_K, w)
    packed = quant.repack_for_matvec(rein.Q4_K, raw, in_dim, out_dim)
    assert packed.size == out_dim * (129 * 18 + 16 * 4)
    x = np.random.default_rng(2025).standard_normal((1, in_dim)).astype(np.float32)
    d_x, dq = dev(x), hip.DeviceBuf((in_dim // 32) * 40)
    runtime.quantize_q8(d_x, dq, in_dim, 1)
    dw, dy = dev(packed), dev(np.full(out_dim, np.nan, np.float32))
    runtime.matvec_xq8(rein.Q4_K, dw, dq, dy, in_dim, out_dim)
    dd = hip.DeviceBuf(out_dim * (in_dim // 32) * 4)
    runtime.block_dots(rein.Q4_K, dw, dq, dd, in_dim, out_dim, 1, False)
    hip.synchronize()
    xq = dq.to_host(np.uint8)
    assert np.array_equal(xq, orc.quantize_q8(x))
    want = orc.matvec_q8(orc.Q4_K, packed, in_dim, out_dim, xq, 1)
    got = dy.to_host(np.float32)[None, :]
    assert_close_f32(got, want, what="configs[0] Q4_K 4096x4096", strict=True)
    dots = orc.block_dots(orc.Q4_K, packed, in_dim, out_dim, xq, 1)
    assert np.array_equal(dd.to_host(np.int32).reshape(dots.shape), dots)
    f32 = orc.matvec_f32(x[0], orc.dequantize_to_f32(orc.Q4_K, raw, in_dim * out_dim).reshape(out_dim, in_dim))
    assert rel_l2(got[0], f32) < 5e-2


def test_barrier_measurement_kernel_always_ends():
    """rein_measure_barrier (bench.py --extras): with polls allowed every workgroup passes and the generation advances by
    one per launch; with none allowed every workgroup gives up, says so, and still ends"""
    import ctypes as C
    f = hip.Module.builtin().function("rein_measure_barrier")
    out = hip.DeviceBuf.from_host(np.zeros(2, np.uint32))
    stream = hip.Stream()

    def launch(mode, spins, grid=256, block=1024):
        f.launch((grid, 1, 1), (block, 1, 1), 0, stream, [C.c_uint(mode), C.c_uint(spins), C.c_void_p(out.ptr)])
        stream.synchronize()
        return out.to_host(np.uint32)

    first = int(launch(1, 1 << 16)[0])
    for i, mode in enumerate((2, 3, 1, 2), start=1):
        got = launch(mode, 1 << 16)
        assert int(got[0]) == first + i and int(got[1]) == 0
    got = launch(2, 0)                                   # no poll allowed: the wait gives up at once
    assert int(got[1]) == 1 and int(got[0]) == first + 4
    out.copy_from_host(np.zeros(2, np.uint32))
    # the flags of the launch that gave up hold the next generation already; the launch after it passes
    got = launch(1, 1 << 16, grid=64)
    assert int(got[1]) == 0
