"""GPU parity of the MoE decode expert matvecs (expert id read on the device):
moe_matvec_<fmt>_repacked, the short-contraction down kernels and the fused
gate+up+SwiGLU kernel, through the C ABI and under the reference's launch geometry.

Oracle: the int8 matvec of the chosen expert's slab per (token, slot); fp32 bar 1e-3
relative / 1e-4 absolute as everywhere."""
import ctypes as C

import numpy as np
import pytest

import reinstinct_amd as rein
from reinstinct_amd import hip, quant, runtime
from reinstinct_amd._lib import init, lib
from oracle import orc
from helpers import assert_close_f32, random_raw_weights

pytestmark = pytest.mark.gpu
FMTS = [rein.Q4_K, rein.Q5_K, rein.Q6_K, rein.Q8_0, rein.Q5_1]
NAME = {rein.Q4_K: "q4k", rein.Q5_K: "q5k", rein.Q6_K: "q6k", rein.Q8_0: "q8_0", rein.Q5_1: "q5_1"}


@pytest.fixture(scope="module", autouse=True)
def gpu():
    init()
    hip.set_device(0)
    yield
    hip.synchronize()


from helpers import dev  # noqa: E402  (uploads that stay alive until the test's last launch has finished)


def expert_slabs(fmt, in_dim, out_dim, n_expert, seed, gaussian=True, pad16=False):
    # out_dim a multiple of 8 keeps every expert's slab 16-byte aligned (the library checks it);
    # pad16 pads each slab to a multiple of 16 bytes instead (bytes_per_expert is a stride)
    slabs = []
    for e in range(n_expert):
        if gaussian and fmt != rein.Q5_1:               # no synthetic quantizer for Q5_1
            w = (np.random.default_rng(seed + e).standard_normal((out_dim, in_dim)) * 0.02).astype(np.float32)
            raw = quant.quantize_weights(fmt, w)
        else:
            raw = random_raw_weights(fmt, in_dim, out_dim, seed + e)
        slabs.append(quant.repack_for_matvec(fmt, raw, in_dim, out_dim))
        if pad16 and slabs[-1].nbytes % 16:
            slabs[-1] = np.concatenate([slabs[-1], np.zeros(16 - slabs[-1].nbytes % 16, np.uint8)])
    return np.concatenate(slabs), slabs[0].nbytes


def oracle_expert_matvec(fmt, slab, bpe, ids, xq_rows, in_dim, out_dim, slot_rows):
    """xq_rows [n_tok][rows][n_sub*40]; slot_rows: True = one activation row per slot"""
    n_tok, n_used = ids.shape
    y = np.empty((n_tok, n_used, out_dim), np.float32)
    for t in range(n_tok):
        for s in range(n_used):
            e = int(ids[t, s])
            row = xq_rows[t, s if slot_rows else 0]
            y[t, s] = orc.matvec_q8(fmt, slab[e * bpe:e * bpe + orc.repacked_len(fmt, in_dim, out_dim)], in_dim, out_dim, row, 1)[0]
    return y


def quantized_rows(rng, n_tok, rows, in_dim):
    x = rng.standard_normal((n_tok * rows, in_dim)).astype(np.float32)
    return orc.quantize_q8(x).reshape(n_tok, rows, -1)


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("in_dim,out_dim,n_tok", [(2048, 768, 1), (2048, 72, 3), (512, 136, 2)])
def test_expert_matvec_shared_activation(fmt, in_dim, out_dim, n_tok):
    # gate / up projections: every slot of a token reads the token's row (slot stride 0)
    n_expert, n_used = 16, 4
    rng = np.random.default_rng(in_dim + out_dim + fmt)
    slab, bpe = expert_slabs(fmt, in_dim, out_dim, n_expert, seed=fmt * 100)
    ids = np.stack([rng.permutation(n_expert)[:n_used] for _ in range(n_tok)]).astype(np.int32)
    xq = quantized_rows(rng, n_tok, 1, in_dim)
    dy = dev(np.full((n_tok, n_used, out_dim), np.nan, np.float32))
    runtime.moe_expert_matvec(fmt, dev(slab), dev(ids), dev(xq), dy, in_dim, out_dim, bpe, in_dim // 32, 0, n_used, n_tok)
    hip.synchronize()
    want = oracle_expert_matvec(fmt, slab, bpe, ids, xq, in_dim, out_dim, slot_rows=False)
    assert_close_f32(dy.to_host(np.float32).reshape(want.shape), want, what=f"moe matvec fmt {fmt}")


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("in_dim,out_dim,n_tok", [(768, 2048, 1), (768, 56, 2), (256, 40, 1), (1024, 104, 1), (2048, 64, 1)])
def test_down_matvec_per_slot_activation(fmt, in_dim, out_dim, n_tok):
    # down projection: one activation row per (token, slot); contractions of 8..32 sub-blocks
    # take the half-wavefront kernels, 2048 falls back to the full-wavefront one
    n_expert, n_used = 12, 8
    rng = np.random.default_rng(in_dim * 3 + out_dim + fmt)
    slab, bpe = expert_slabs(fmt, in_dim, out_dim, n_expert, seed=fmt * 100 + 50)
    ids = np.stack([rng.permutation(n_expert)[:n_used] for _ in range(n_tok)]).astype(np.int32)
    xq = quantized_rows(rng, n_tok, n_used, in_dim)
    n_sub = in_dim // 32
    dy = dev(np.full((n_tok, n_used, out_dim), np.nan, np.float32))
    runtime.moe_down(fmt, dev(slab), dev(ids), dev(xq), dy, in_dim, out_dim, bpe, n_used * n_sub, n_sub, n_used, n_tok)
    hip.synchronize()
    want = oracle_expert_matvec(fmt, slab, bpe, ids, xq, in_dim, out_dim, slot_rows=True)
    assert_close_f32(dy.to_host(np.float32).reshape(want.shape), want, what=f"moe down fmt {fmt}")


@pytest.mark.parametrize("in_dim,out_dim,n_tok", [(2048, 768, 1), (2048, 104, 2), (256, 40, 1)])
def test_gate_up_swiglu(in_dim, out_dim, n_tok):
    fmt, n_expert, n_used = rein.Q4_K, 10, 8
    rng = np.random.default_rng(in_dim + out_dim)
    gate, bpe = expert_slabs(fmt, in_dim, out_dim, n_expert, seed=7)
    up, _ = expert_slabs(fmt, in_dim, out_dim, n_expert, seed=70)
    ids = np.stack([rng.permutation(n_expert)[:n_used] for _ in range(n_tok)]).astype(np.int32)
    xq = quantized_rows(rng, n_tok, 1, in_dim)
    dy = dev(np.full((n_tok, n_used, out_dim), np.nan, np.float32))
    runtime.moe_gate_up_swiglu(fmt, dev(gate), dev(up), dev(ids), dev(xq), dy, in_dim, out_dim, bpe, in_dim // 32, 0,
                               n_used, n_tok)
    hip.synchronize()
    g = oracle_expert_matvec(fmt, gate, bpe, ids, xq, in_dim, out_dim, slot_rows=False)
    u = oracle_expert_matvec(fmt, up, bpe, ids, xq, in_dim, out_dim, slot_rows=False)
    want = orc.map_det("silu", g) * u
    assert_close_f32(dy.to_host(np.float32).reshape(want.shape), want, rel=2e-3, abs_=2e-4, what="gate_up_swiglu")
    # and equals the three-launch chain on the GPU to rounding
    dg, du = dev(np.zeros_like(want)), dev(np.zeros_like(want))
    runtime.moe_expert_matvec(fmt, dev(gate), dev(ids), dev(xq), dg, in_dim, out_dim, bpe, in_dim // 32, 0, n_used, n_tok)
    runtime.moe_expert_matvec(fmt, dev(up), dev(ids), dev(xq), du, in_dim, out_dim, bpe, in_dim // 32, 0, n_used, n_tok)
    hip.synchronize()
    chain = orc.map_det("silu", dg.to_host(np.float32)) * du.to_host(np.float32)
    assert np.array_equal(dy.to_host(np.float32).view(np.uint32), chain.view(np.uint32))


@pytest.mark.parametrize("fmt", FMTS)
def test_reference_symbols_and_launch_geometry(fmt):
    # grid = (ceil(out/8), n_used, n_tok) x 256 for the generic kernels, (ceil(out/rpb), ...) with
    # rpb = 256 / n_sub for the down kernels (qwen35.rs:3086-3099, 3121-3138)
    mod = hip.Module.builtin()
    u, p = C.c_uint, C.c_void_p
    n_expert, n_used, n_tok = 6, 3, 2
    rng = np.random.default_rng(fmt)
    for in_dim, out_dim, down in ((1024, 56, False), (768, 72, True)):
        name = f"moe_matvec_{NAME[fmt]}_repacked_f32"
        if down:
            if fmt == rein.Q4_K:
                continue                                   # the reference has no Q4_K down kernel
            name = "moe_matvec_q8_0_repacked_down_f32" if fmt == rein.Q8_0 else f"moe_matvec_{NAME[fmt]}_down_f32"
        slab, bpe = expert_slabs(fmt, in_dim, out_dim, n_expert, seed=3, gaussian=False)
        ids = rng.integers(0, n_expert, (n_tok, n_used)).astype(np.int32)
        rows = n_used if down else 1
        xq = quantized_rows(rng, n_tok, rows, in_dim)
        n_sub = in_dim // 32
        d_slab, d_ids, d_xq = dev(slab), dev(ids), dev(xq)
        dy = dev(np.full((n_tok, n_used, out_dim), np.nan, np.float32))
        rpb = max(1, 256 // n_sub) if down else 8
        args = [p(d_slab.ptr), p(d_ids.ptr), p(d_xq.ptr), p(dy.ptr), u(in_dim), u(out_dim), u(bpe),
                u(rows * n_sub), u(n_sub if down else 0), u(n_used)]
        mod.function(name).launch(((out_dim + rpb - 1) // rpb, n_used, n_tok), (256, 1, 1), 0, None, args)
        hip.synchronize()
        want = oracle_expert_matvec(fmt, slab, bpe, ids, xq, in_dim, out_dim, slot_rows=down)
        assert_close_f32(dy.to_host(np.float32).reshape(want.shape), want, what=name)


def test_moe_decode_ffn_chain_config4_shapes():
    # one token of the 128-expert top-8 configuration: fused gate+up+SwiGLU (Q4_K 2048 -> 768)
    # -> quantize -> down (Q6_K 768 -> 2048) -> combine, against the same chain on the CPU
    hidden, ff, n_expert, n_used = 2048, 768, 128, 8
    rng = np.random.default_rng(44)
    # 128 experts share 8 distinct weight sets (expert e uses set e % 8): the kernels index by expert id all the same
    g8, bpe_gu = expert_slabs(rein.Q4_K, hidden, ff, 8, seed=900)
    u8, _ = expert_slabs(rein.Q4_K, hidden, ff, 8, seed=950)
    d8, bpe_dn = expert_slabs(rein.Q6_K, ff, hidden, 8, seed=990)
    tile = lambda s, bpe: np.concatenate([s.reshape(8, bpe)] * (n_expert // 8)).reshape(-1)
    gate, up, down = tile(g8, bpe_gu), tile(u8, bpe_gu), tile(d8, bpe_dn)
    x = rng.standard_normal((1, hidden)).astype(np.float32)
    logits = rng.standard_normal((1, n_expert)).astype(np.float32)
    ones = np.ones(n_expert, np.float32)

    d_ids, d_wts = hip.DeviceBuf(n_used * 4), hip.DeviceBuf(n_used * 4)
    runtime.moe_topk(dev(logits), 1, n_expert, n_used, d_ids, d_wts)
    d_xq = hip.DeviceBuf(hidden // 32 * 40)
    runtime.quantize_q8(dev(x), d_xq, hidden, 1)
    d_act = dev(np.zeros((n_used, ff), np.float32))
    runtime.moe_gate_up_swiglu(rein.Q4_K, dev(gate), dev(up), d_ids, d_xq, d_act, hidden, ff, bpe_gu, hidden // 32, 0, n_used, 1)
    d_aq = hip.DeviceBuf(n_used * ff // 32 * 40)
    runtime.quantize_q8(d_act, d_aq, ff, n_used)
    d_eo = dev(np.zeros((n_used, hidden), np.float32))
    runtime.moe_down(rein.Q6_K, dev(down), d_ids, d_aq, d_eo, ff, hidden, bpe_dn, n_used * (ff // 32), ff // 32, n_used, 1)
    d_out = dev(np.zeros(hidden, np.float32))
    runtime.moe_combine(d_eo, d_ids, d_wts, dev(ones), d_out, 1, hidden, n_used)
    hip.synchronize()

    ids, wts = orc.moe_topk(logits, n_used)
    assert np.array_equal(d_ids.to_host(np.int32), ids.reshape(-1))
    xq = orc.quantize_q8(x).reshape(1, 1, -1)
    g = oracle_expert_matvec(rein.Q4_K, gate, bpe_gu, ids, xq, hidden, ff, False)
    u_ = oracle_expert_matvec(rein.Q4_K, up, bpe_gu, ids, xq, hidden, ff, False)
    act = orc.map_det("silu", g) * u_
    aq = orc.quantize_q8(act.reshape(n_used, ff)).reshape(1, n_used, -1)
    eo = oracle_expert_matvec(rein.Q6_K, down, bpe_dn, ids, aq, ff, hidden, True)
    want = orc.moe_combine(eo, ids, wts, ones)
    from helpers import rel_l2
    got = d_out.to_host(np.float32)
    assert rel_l2(got, want) < 2e-3
    assert_close_f32(got, want.reshape(-1), rel=2e-2, abs_=2e-3, what="moe decode ffn")


# ------------------------------------------------------------------ the two fused launches
@pytest.mark.parametrize("rows", [0, 2, 4])
@pytest.mark.parametrize("in_dim,out_dim,n_tok", [(2048, 768, 1), (2048, 96, 3), (256, 32, 2), (1024, 768, 3)])
def test_gate_up_swiglu_q8_equals_the_two_launches(in_dim, out_dim, n_tok, rows, options):
    # gate + up + SwiGLU + quantize in one launch: byte for byte what the fused matvec
    # followed by quantize_q8 writes, and that chain is what the oracle is compared with above;
    # with the library's choice of rows per wavefront (0; the last shape is large enough for four)
    # and with two and four forced
    if rows:
        options.set("REIN_MOE_GU_ROWS", str(rows))
    fmt, n_expert, n_used = rein.Q4_K, 10, 8
    rng = np.random.default_rng(in_dim * 7 + out_dim)
    gate, bpe = expert_slabs(fmt, in_dim, out_dim, n_expert, seed=17)
    up, _ = expert_slabs(fmt, in_dim, out_dim, n_expert, seed=170)
    ids = np.stack([rng.permutation(n_expert)[:n_used] for _ in range(n_tok)]).astype(np.int32)
    xq = quantized_rows(rng, n_tok, 1, in_dim)
    d_gate, d_up, d_ids, d_xq = dev(gate), dev(up), dev(ids), dev(xq)
    d_act = dev(np.full((n_tok, n_used, out_dim), np.nan, np.float32))
    runtime.moe_gate_up_swiglu(fmt, d_gate, d_up, d_ids, d_xq, d_act, in_dim, out_dim, bpe, in_dim // 32, 0, n_used, n_tok)
    n_bytes = n_tok * n_used * (out_dim // 32) * 40
    d_chain = dev(np.full(n_bytes, 0xAA, np.uint8))
    runtime.quantize_q8(d_act, d_chain, out_dim, n_tok * n_used)
    d_fused = dev(np.full(n_bytes, 0x55, np.uint8))
    runtime.moe_gate_up_swiglu_q8(fmt, d_gate, d_up, d_ids, d_xq, d_fused, in_dim, out_dim, bpe, in_dim // 32, 0, n_used, n_tok)
    hip.synchronize()
    assert np.array_equal(d_fused.to_host(np.uint8), d_chain.to_host(np.uint8))
    # and against the CPU chain: same quants up to the fp32 rounding of the sums in front of them
    g = oracle_expert_matvec(fmt, gate, bpe, ids, xq, in_dim, out_dim, slot_rows=False)
    u = oracle_expert_matvec(fmt, up, bpe, ids, xq, in_dim, out_dim, slot_rows=False)
    want = orc.quantize_q8((orc.map_det("silu", g) * u).reshape(n_tok * n_used, out_dim)).reshape(-1, 40)
    got = d_fused.to_host(np.uint8).reshape(-1, 40)
    dq = np.abs(got[:, 8:].view(np.int8).astype(np.int32) - want[:, 8:].view(np.int8).astype(np.int32))
    assert dq.max() <= 1 and np.mean(dq != 0) < 0.02
    assert np.allclose(got[:, :4].copy().view(np.float32), want[:, :4].copy().view(np.float32), rtol=2e-3)


@pytest.mark.parametrize("rows", [0, 4])
@pytest.mark.parametrize("fmt", [rein.Q5_K, rein.Q6_K, rein.Q8_0, rein.Q5_1])
@pytest.mark.parametrize("in_dim,out_dim,n_tok", [(2048, 768, 1), (1024, 96, 3), (768, 768, 3)])
def test_gate_up_swiglu_q8_other_formats(fmt, in_dim, out_dim, n_tok, rows, options):
    # the fused launch for the expert formats the reference has no fused kernel for: byte for byte what two
    # expert matvecs (gate, up) followed by swiglu_q8 write
    if rows:
        options.set("REIN_MOE_GU_ROWS", str(rows))
    n_expert, n_used = 10, 8
    rng = np.random.default_rng(in_dim * 3 + out_dim + fmt)
    gate, bpe = expert_slabs(fmt, in_dim, out_dim, n_expert, seed=fmt * 10 + 1, pad16=True)
    up, _ = expert_slabs(fmt, in_dim, out_dim, n_expert, seed=fmt * 10 + 2, pad16=True)
    ids = np.stack([rng.permutation(n_expert)[:n_used] for _ in range(n_tok)]).astype(np.int32)
    xq = quantized_rows(rng, n_tok, 1, in_dim)
    d_gate, d_up, d_ids, d_xq = dev(gate), dev(up), dev(ids), dev(xq)
    n = n_tok * n_used * out_dim
    d_g, d_u = dev(np.full(n, np.nan, np.float32)), dev(np.full(n, np.nan, np.float32))
    runtime.moe_expert_matvec(fmt, d_gate, d_ids, d_xq, d_g, in_dim, out_dim, bpe, in_dim // 32, 0, n_used, n_tok)
    runtime.moe_expert_matvec(fmt, d_up, d_ids, d_xq, d_u, in_dim, out_dim, bpe, in_dim // 32, 0, n_used, n_tok)
    d_chain = dev(np.full(n // 32 * 40, 0xAA, np.uint8))
    runtime.swiglu_q8(d_g, d_u, None, d_chain, n)
    d_fused = dev(np.full(n // 32 * 40, 0x55, np.uint8))
    runtime.moe_gate_up_swiglu_q8(fmt, d_gate, d_up, d_ids, d_xq, d_fused, in_dim, out_dim, bpe, in_dim // 32, 0, n_used, n_tok)
    hip.synchronize()
    assert np.array_equal(d_fused.to_host(np.uint8), d_chain.to_host(np.uint8))
    g = oracle_expert_matvec(fmt, gate, bpe, ids, xq, in_dim, out_dim, slot_rows=False)
    u = oracle_expert_matvec(fmt, up, bpe, ids, xq, in_dim, out_dim, slot_rows=False)
    want = orc.quantize_q8((orc.map_det("silu", g) * u).reshape(n_tok * n_used, out_dim)).reshape(-1, 40)
    got = d_fused.to_host(np.uint8).reshape(-1, 40)
    dq = np.abs(got[:, 8:].view(np.int8).astype(np.int32) - want[:, 8:].view(np.int8).astype(np.int32))
    assert dq.max() <= 1 and np.mean(dq != 0) < 0.02


@pytest.mark.parametrize("rows", [0, 2, 4, 8])
@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("in_dim,out_dim,n_tok", [(768, 2048, 1), (768, 56, 2), (768, 43, 1), (2048, 64, 1), (1280, 37, 2)])
def test_down_combine_equals_the_two_launches(fmt, in_dim, out_dim, n_tok, rows, options):
    # down projection + weighted combine in one launch: bit for bit the two-launch result
    # (both team widths: up to 32 sub-blocks half-wavefronts, 2048 the full wavefront; the odd
    # row counts end on a workgroup that owns fewer rows than the others -- their slabs are padded to
    # the 16-byte stride the library asks for); with the library's own choice of rows per workgroup
    # (0) and with each of 2, 4 and 8 forced
    if rows:
        options.set("REIN_MOE_DC_ROWS", str(rows))
    n_expert, n_used = 12, 8
    rng = np.random.default_rng(in_dim * 5 + out_dim + fmt)
    slab, bpe = expert_slabs(fmt, in_dim, out_dim, n_expert, seed=fmt * 100 + 77, pad16=True)
    assert bpe % 16 == 0
    ids = np.stack([rng.permutation(n_expert)[:n_used] for _ in range(n_tok)]).astype(np.int32)
    wts = rng.random((n_tok, n_used)).astype(np.float32)
    scales = (0.5 + rng.random(n_expert)).astype(np.float32)
    xq = quantized_rows(rng, n_tok, n_used, in_dim)
    n_sub = in_dim // 32
    d_slab, d_ids, d_wts, d_sc, d_xq = dev(slab), dev(ids), dev(wts), dev(scales), dev(xq)
    d_eo = dev(np.full((n_tok, n_used, out_dim), np.nan, np.float32))
    runtime.moe_down(fmt, d_slab, d_ids, d_xq, d_eo, in_dim, out_dim, bpe, n_used * n_sub, n_sub, n_used, n_tok)
    d_chain = dev(np.full((n_tok, out_dim), np.nan, np.float32))
    runtime.moe_combine(d_eo, d_ids, d_wts, d_sc, d_chain, n_tok, out_dim, n_used)
    d_fused = dev(np.full((n_tok, out_dim), np.nan, np.float32))
    runtime.moe_down_combine(fmt, d_slab, d_ids, d_wts, d_sc, d_xq, d_fused, in_dim, out_dim, bpe, n_used * n_sub, n_sub,
                             n_used, n_tok)
    hip.synchronize()
    got = d_fused.to_host(np.float32)
    assert np.array_equal(got.view(np.uint32), d_chain.to_host(np.float32).view(np.uint32))
    eo = oracle_expert_matvec(fmt, slab, bpe, ids, xq, in_dim, out_dim, slot_rows=True)
    want = orc.moe_combine(eo, ids, wts, scales)
    assert_close_f32(got.reshape(want.shape), want, what=f"down+combine fmt {fmt}")
