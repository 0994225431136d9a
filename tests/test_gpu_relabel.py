"""GPU parity of the two relabelled formats beyond what the per-format sweeps of the other
GPU test files cover: Q5_1's sub-block decode (bit-exact block dots), ragged contractions
(Q5_1 blocks are 32 weights, so in_dim need not be a multiple of 256), and an expert FFN with
Q5_1 down experts end to end."""
import numpy as np
import pytest

import reinstinct_amd as rein
from reinstinct_amd import hip, quant, runtime
from reinstinct_amd._lib import init
from oracle import orc
from helpers import assert_close_f32, random_raw_weights, rel_l2

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def gpu():
    init()
    hip.set_device(0)
    yield
    hip.synchronize()


from helpers import dev  # noqa: E402  (uploads that stay alive until the test's last launch has finished)


def slabs(fmt, in_dim, out_dim, n_expert, seed):
    parts = [quant.repack_for_matvec(fmt, random_raw_weights(fmt, in_dim, out_dim, seed + e), in_dim, out_dim)
             for e in range(n_expert)]
    return np.concatenate(parts), parts[0].nbytes


@pytest.mark.parametrize("in_dim,out_dim,n_rows", [(256, 40, 1), (352, 24, 3), (96, 7, 2), (32, 5, 1), (2048, 16, 2)])
def test_q5_1_block_dots_bit_exact(in_dim, out_dim, n_rows):
    print("q5_1 block dots", in_dim, out_dim, n_rows, flush=True)
    raw = random_raw_weights(rein.Q5_1, in_dim, out_dim, seed=in_dim)
    packed = quant.repack_for_matvec(rein.Q5_1, raw, in_dim, out_dim)
    x = np.random.default_rng(in_dim).standard_normal((n_rows, in_dim)).astype(np.float32)
    xq = orc.quantize_q8(x)
    want = orc.block_dots(orc.Q5_1, packed, in_dim, out_dim, xq, n_rows)
    dd = hip.DeviceBuf(want.nbytes)
    runtime.block_dots(rein.Q5_1, dev(packed), dev(xq), dd, in_dim, out_dim, n_rows, False)
    hip.synchronize()
    assert np.array_equal(dd.to_host(np.int32).reshape(want.shape), want)


@pytest.mark.parametrize("in_dim,out_dim,n_tok,down", [(352, 72, 2, False), (96, 40, 1, False), (352, 64, 2, True),
                                                       (96, 40, 3, True), (32, 16, 1, True), (1120, 24, 1, True)])
def test_q5_1_expert_matvecs_ragged_contraction(in_dim, out_dim, n_tok, down):
    print("q5_1 expert matvec", in_dim, out_dim, n_tok, down, flush=True)
    n_expert, n_used = 9, 4
    rng = np.random.default_rng(in_dim + out_dim)
    slab, bpe = slabs(rein.Q5_1, in_dim, out_dim, n_expert, seed=40)
    ids = np.stack([rng.permutation(n_expert)[:n_used] for _ in range(n_tok)]).astype(np.int32)
    rows = n_used if down else 1
    n_sub = in_dim // 32
    xq = orc.quantize_q8(rng.standard_normal((n_tok * rows, in_dim)).astype(np.float32)).reshape(n_tok, rows, -1)
    dy = dev(np.full((n_tok, n_used, out_dim), np.nan, np.float32))
    if down:
        runtime.moe_down(rein.Q5_1, dev(slab), dev(ids), dev(xq), dy, in_dim, out_dim, bpe, n_used * n_sub, n_sub, n_used, n_tok)
    else:
        runtime.moe_expert_matvec(rein.Q5_1, dev(slab), dev(ids), dev(xq), dy, in_dim, out_dim, bpe, n_sub, 0, n_used, n_tok)
    hip.synchronize()
    want = np.empty((n_tok, n_used, out_dim), np.float32)
    for t in range(n_tok):
        for s in range(n_used):
            e = int(ids[t, s])
            want[t, s] = orc.matvec_q8(orc.Q5_1, slab[e * bpe:(e + 1) * bpe], in_dim, out_dim, xq[t, s if down else 0], 1)[0]
    assert_close_f32(dy.to_host(np.float32).reshape(want.shape), want, what="q5_1 expert matvec")


def test_q5_1_minimum_term_alone():
    # d = 0 in every block: the output is sum_s m_s * xsum_s, the part that goes through the
    # split-bf16 MFMA of the grouped GEMM; minimums with all eleven significant bits in use
    in_dim, out_dim, n_expert, n_tok, n_used = 512, 136, 3, 70, 1
    rng = np.random.default_rng(8)
    parts = []
    for e in range(n_expert):
        raw = random_raw_weights(rein.Q5_1, in_dim, out_dim, seed=e).reshape(-1, 24)
        raw[:, 0:2] = 0
        m = (rng.integers(1024, 2048, raw.shape[0]) * rng.choice([-1.0, 1.0], raw.shape[0]) * 2.0 ** -12).astype(np.float16)
        raw[:, 2:4] = m.view(np.uint8).reshape(-1, 2)
        parts.append(quant.repack_for_matvec(rein.Q5_1, raw.reshape(-1), in_dim, out_dim))
    slab, bpe = np.concatenate(parts), parts[0].nbytes
    ids = rng.integers(0, n_expert, (n_tok, n_used)).astype(np.int32)
    perm, eoff, toff = orc.moe_sort(ids, n_expert, runtime.moe_gemm_bn())
    xq = orc.quantize_q8(rng.standard_normal((n_tok, in_dim)).astype(np.float32))
    gin = orc.moe_gather_xq(xq, perm, in_dim // 32, n_used)
    dy = dev(np.full(n_tok * out_dim, np.nan, np.float32))
    runtime.moe_grouped_gemm(rein.Q5_1, dev(slab), bpe, dev(eoff), dev(toff), n_expert, dev(gin), dy, in_dim, out_dim, n_tok)
    hip.synchronize()
    want = orc.grouped_gemm(orc.Q5_1, slab, bpe, eoff, gin, in_dim, out_dim)
    assert_close_f32(dy.to_host(np.float32).reshape(n_tok, out_dim), want, rel=1e-5, abs_=2e-5, what="q5_1 minimum term")


def test_moe_ffn_with_q5_1_down_experts():
    # the Gemma-style mix: Q4_K gate / up experts, Q5_1 down experts (src/runtime/gemma4.rs:239)
    n_tok, hidden, n_expert, n_used, ff = 40, 512, 8, 2, 352
    rng = np.random.default_rng(12)
    x = rng.standard_normal((n_tok, hidden)).astype(np.float32)
    logits = rng.standard_normal((n_tok, n_expert)).astype(np.float32)

    def gauss(fmt, in_dim, out_dim, seed):
        w = (np.random.default_rng(seed).standard_normal((out_dim, in_dim)) * 0.02).astype(np.float32)
        return quant.repack_for_matvec(fmt, quant.quantize_weights(fmt, w), in_dim, out_dim)

    gate = np.concatenate([gauss(rein.Q4_K, hidden, ff, 300 + e) for e in range(n_expert)])
    up = np.concatenate([gauss(rein.Q4_K, hidden, ff, 400 + e) for e in range(n_expert)])
    down, bpe_dn = slabs(rein.Q5_1, ff, hidden, n_expert, seed=500)
    ones = np.ones(n_expert, np.float32)
    sh = runtime.moe_shape(n_tok, hidden, n_expert, n_used, ff, rein.Q4_K, rein.Q5_1)
    ws = hip.DeviceBuf(runtime.moe_workspace_bytes(sh))
    d_out = dev(np.full(n_tok * hidden, np.nan, np.float32))
    runtime.moe_ffn(sh, dev(x), dev(logits), dev(gate), dev(up), dev(down), dev(ones), ws, d_out)
    hip.synchronize()
    got = d_out.to_host(np.float32).reshape(n_tok, hidden)

    ids, wts = orc.moe_topk(logits, n_used)
    perm, eoff, _ = orc.moe_sort(ids, n_expert, 32)
    gin = orc.moe_gather_xq(orc.quantize_q8(x), perm, hidden // 32, n_used)
    bpe_gu = orc.repacked_len(orc.Q4_K, hidden, ff)
    eg = orc.grouped_gemm(orc.Q4_K, gate, bpe_gu, eoff, gin, hidden, ff)
    eu = orc.grouped_gemm(orc.Q4_K, up, bpe_gu, eoff, gin, hidden, ff)
    act = orc.swiglu_mul(eg, eu)
    gout = orc.grouped_gemm(orc.Q5_1, down, bpe_dn, eoff, orc.quantize_q8(act), ff, hidden)
    eout = orc.moe_scatter_rows(gout, perm, hidden).reshape(n_tok, n_used, hidden)
    want = orc.moe_combine(eout, ids, wts, ones)
    assert rel_l2(got, want) < 2e-3
    assert_close_f32(got, want, rel=2e-2, abs_=2e-3, what="moe_ffn q5_1")


def test_dispatch_rules_on_the_device():
    w = hip.DeviceBuf(1 << 16)
    with pytest.raises(rein.ReinError) as e:
        runtime.matvec_xq8(rein.Q5_1, w, w, w, 256, 8)
    assert e.value.code == -2
    with pytest.raises(rein.ReinError) as e:
        runtime.moe_grouped_gemm(rein.IQ3_S, w, 4608, w, w, 1, w, w, 256, 8, 1)
    assert e.value.code == -2
