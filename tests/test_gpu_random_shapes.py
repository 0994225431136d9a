"""Seeded random shapes through the dispatching entry points against the oracle: the dense product
(rein_matmul / rein_matmul_ws: matvec, batched matvec on every kernel family, MMQ in its plain and
workspace forms; larger GEMMs through rein_mmq_xq8_ws in all four launch forms against rein_mmq_xq8) and the MoE expert FFN (decode launches, fused and unfused pipeline, strided grouped
GEMM).  The fixed-shape tests pin each kernel; these pin the launch choices in between."""
import os

import numpy as np
import pytest

import reinstinct_amd as rein
from reinstinct_amd import hip, quant, runtime
from reinstinct_amd._lib import init
from oracle import orc
from helpers import assert_close_f32, dev, random_raw_weights

pytestmark = pytest.mark.gpu

DENSE = [rein.Q4_0, rein.Q8_0, rein.Q4_K, rein.Q5_K, rein.Q6_K, rein.IQ4_XS, rein.IQ3_S]
EXPERT = [rein.Q4_K, rein.Q5_K, rein.Q6_K, rein.Q8_0]


@pytest.fixture(scope="module", autouse=True)
def gpu():
    init()
    hip.set_device(0)
    yield
    hip.synchronize()


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_dense_dispatch_on_random_shapes(seed):
    rng = np.random.default_rng(seed)
    for case in range(100):
        fmt = DENSE[rng.integers(len(DENSE))]
        whole_superblocks = fmt not in (rein.Q4_0, rein.Q8_0) or rng.random() < 0.5
        in_dim = int(rng.integers(1, 13)) * 256 if whole_superblocks else int(rng.integers(1, 60)) * 32
        out_dim = int(rng.choice([int(rng.integers(1, 300)), int(rng.integers(300, 3000)), int(rng.integers(3000, 9000))]))
        n_rows = int(rng.choice([1, int(rng.integers(2, 9)), int(rng.integers(9, 33)), int(rng.integers(33, 130)),
                                 int(rng.integers(130, 700))]))
        while in_dim * out_dim * n_rows > 3e8:
            n_rows = max(1, n_rows // 2)
        with_scratch = bool(rng.integers(2))
        print(f"seed {seed} case {case}: fmt {fmt} K {in_dim} N {out_dim} rows {n_rows} scratch {with_scratch}", flush=True)
        packed = quant.repack_for_matvec(fmt, random_raw_weights(fmt, in_dim, out_dim, seed=1000 * seed + case), in_dim, out_dim)
        x = rng.standard_normal((n_rows, in_dim)).astype(np.float32)
        dw, dx = dev(packed), dev(x)
        dy = dev(np.full(n_rows * out_dim, np.nan, np.float32))
        if with_scratch:
            nbytes = runtime.matmul_scratch_bytes(fmt, in_dim, n_rows)
            scratch = hip.DeviceBuf(nbytes)
            runtime.matmul_ws(fmt, dw, dx, dy, in_dim, out_dim, n_rows, scratch, nbytes)
        else:
            scratch = hip.DeviceBuf(n_rows * (in_dim // 32) * 40)
            runtime.matmul(fmt, dw, dx, dy, in_dim, out_dim, n_rows, scratch)
        hip.synchronize()
        got = dy.to_host(np.float32).reshape(n_rows, out_dim)
        assert not np.isnan(got).any(), f"case {case}: output not fully written"
        want = orc.matvec_q8(fmt, packed, in_dim, out_dim, orc.quantize_q8(x), n_rows)
        assert_close_f32(got, want, what=f"seed {seed} case {case}")


def test_workspace_gemm_matches_the_plain_gemm_on_random_large_shapes():
    # rein_mmq_xq8_ws in whichever of its four launch forms the library picks (ragged row counts, contractions and
    # widths around the thresholds) against rein_mmq_xq8, which the fixed-shape tests hold against the oracle
    rng = np.random.default_rng(9)
    seen = set()
    # the fp6 split-tail form wants few, even tiles: two shapes that take it, beside the random ones
    fixed = {36: (rein.Q4_K, 5120, 5120, 640), 37: (rein.Q4_K, 8192, 8192, 512)}
    for case in range(38):
        big = case % 3 != 0
        fmt = rein.Q4_K if big else DENSE[rng.integers(len(DENSE))]
        in_dim = int(rng.integers(8 if big else 2, 36)) * 256
        out_dim = int(rng.integers(3000, 36000)) if big else int(rng.integers(100, 9000))
        p_rows = int(rng.integers(320, 2100)) if big else int(rng.integers(17, 520))
        while in_dim * out_dim * 0.6 > 3.5e8:
            out_dim //= 2
        while p_rows * out_dim * 4 > 4e8:
            p_rows //= 2
        if case in fixed:
            fmt, in_dim, out_dim, p_rows = fixed[case]
        nbytes = runtime.mmq_workspace_bytes(fmt, in_dim, p_rows)
        form = runtime.mmq_form_ws(fmt, in_dim, out_dim, p_rows, nbytes)
        seen.add(form)
        print(f"workspace case {case}: fmt {fmt} K {in_dim} N {out_dim} rows {p_rows} form {form}", flush=True)
        packed = quant.repack_for_matvec(fmt, random_raw_weights(fmt, in_dim, out_dim, seed=case), in_dim, out_dim)
        x = rng.standard_normal((p_rows, in_dim)).astype(np.float32)
        dw, dx = dev(packed), dev(x)
        dq = hip.DeviceBuf(p_rows * (in_dim // 32) * 40)
        runtime.quantize_q8(dx, dq, in_dim, p_rows)
        ws = hip.DeviceBuf(max(nbytes, 16))
        d_ws = dev(np.full(p_rows * out_dim, np.nan, np.float32))
        d_plain = dev(np.full(p_rows * out_dim, np.nan, np.float32))
        runtime.mmq_xq8_ws(fmt, dw, dq, d_ws, in_dim, out_dim, p_rows, ws, nbytes)
        runtime.mmq_xq8(fmt, dw, dq, d_plain, in_dim, out_dim, p_rows)
        hip.synchronize()
        got, want = d_ws.to_host(np.float32), d_plain.to_host(np.float32)
        assert not np.isnan(got).any() and not np.isnan(want).any(), f"workspace case {case}: output not fully written"
        assert_close_f32(got, want, what=f"workspace case {case}")
    assert seen == {0, 1, 2, 3}, f"launch forms reached: {sorted(seen)}"


def gaussian_slab(fmt, in_dim, out_dim, n_expert, seed):
    out = []
    for e in range(n_expert):
        w = (np.random.default_rng(seed + e).standard_normal((out_dim, in_dim)) * 0.02).astype(np.float32)
        out.append(quant.repack_for_matvec(fmt, quant.quantize_weights(fmt, w), in_dim, out_dim))
    return np.concatenate(out)


def test_moe_ffn_on_random_shapes(options):
    rng = np.random.default_rng(4)
    for case in range(40):
        gu = EXPERT[rng.integers(4)] if rng.random() < 0.4 else rein.Q4_K
        dn = EXPERT[rng.integers(4)]
        hidden, ff = int(rng.integers(1, 5)) * 256, int(rng.integers(1, 4)) * 256
        n_expert = int(rng.choice([4, 8, 16, 33, 64]))
        n_used = int(rng.integers(1, min(8, n_expert) + 1))
        n_tok = int(rng.choice([1, 2, int(rng.integers(3, 17)), int(rng.integers(17, 80)), int(rng.integers(80, 260))]))
        fused, strided = str(int(rng.integers(2))), str(int(rng.random() < 0.2))
        options.set("REIN_MOE_FUSED", fused)
        options.set("REIN_GROUPED_STRIDED", strided)
        print(f"moe case {case}: gate/up {gu} down {dn} hidden {hidden} ff {ff} experts {n_expert} top-{n_used} tokens {n_tok} "
              f"fused {fused} strided {strided}", flush=True)
        x = rng.standard_normal((n_tok, hidden)).astype(np.float32)
        logits = rng.standard_normal((n_tok, n_expert)).astype(np.float32)
        gate = gaussian_slab(gu, hidden, ff, n_expert, 1000 * case)
        up = gaussian_slab(gu, hidden, ff, n_expert, 1000 * case + 100)
        down = gaussian_slab(dn, ff, hidden, n_expert, 1000 * case + 200)
        scal = rng.uniform(0.5, 1.5, n_expert).astype(np.float32)
        sh = runtime.moe_shape(n_tok, hidden, n_expert, n_used, ff, gu, dn)
        ws = hip.DeviceBuf(runtime.moe_workspace_bytes(sh))
        bufs = [dev(a) for a in (x, logits, gate, up, down, scal)]
        d_out = dev(np.full(n_tok * hidden, np.nan, np.float32))
        runtime.moe_ffn(sh, *bufs, ws, d_out)
        hip.synchronize()
        got = d_out.to_host(np.float32).reshape(n_tok, hidden)
        assert not np.isnan(got).any(), f"moe case {case}: output not fully written"
        ids, wts = orc.moe_topk(logits, n_used)
        perm, eoff, _ = orc.moe_sort(ids, n_expert, 32)
        gin = orc.moe_gather_xq(orc.quantize_q8(x), perm, hidden // 32, n_used)
        bg, bd = orc.repacked_len(gu, hidden, ff), orc.repacked_len(dn, ff, hidden)
        eg = orc.grouped_gemm(gu, gate, bg, eoff, gin, hidden, ff)
        eu = orc.grouped_gemm(gu, up, bg, eoff, gin, hidden, ff)
        gout = orc.grouped_gemm(dn, down, bd, eoff, orc.quantize_q8(orc.swiglu_mul(eg, eu)), ff, hidden)
        want = orc.moe_combine(orc.moe_scatter_rows(gout, perm, hidden).reshape(n_tok, n_used, hidden), ids, wts, scal)
        # the intermediate is re-quantized after SwiGLU: fp32 noise in gate / up can move a quant by one step
        rel = float(np.linalg.norm(got - want) / max(1e-30, np.linalg.norm(want)))
        assert rel < 2e-3, f"moe case {case}: rel_l2 {rel:.2e}"
        assert_close_f32(got, want, rel=2e-2, abs_=2e-3, what=f"moe case {case}")
