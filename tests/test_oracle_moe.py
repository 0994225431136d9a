"""Pins the oracle's MoE glue: textbook softmax/top-k, the sort invariants the
reference's own verifier checks (qwen35.rs:2956-2987), closed forms."""
import numpy as np

from oracle import orc
from helpers import random_raw_weights


def test_topk_matches_textbook():
    rng = np.random.default_rng(0)
    logits = rng.standard_normal((37, 128)).astype(np.float32)
    ids, w = orc.moe_topk(logits, 8)
    p = np.exp(logits.astype(np.float64) - logits.max(axis=1, keepdims=True))
    p /= p.sum(axis=1, keepdims=True)
    order = np.argsort(-p, axis=1, kind="stable")[:, :8]
    assert np.array_equal(ids, order)
    chosen = np.take_along_axis(p, order, axis=1)
    assert np.allclose(w, chosen / chosen.sum(axis=1, keepdims=True), rtol=1e-5, atol=1e-7)
    assert np.allclose(w.sum(axis=1), 1.0, atol=1e-6)


def test_topk_ties_nan_and_floor():
    # equal logits: strict '>' keeps the lower thread, so the first pick is index 0
    # (moe_topk.cpp:78-93); later picks follow the halving tree past the -1 sentinel,
    # so only distinctness and the weights are fixed
    ids, w = orc.moe_topk(np.zeros((1, 16), np.float32), 4)
    assert ids[0, 0] == 0 and len(set(ids[0].tolist())) == 4 and np.allclose(w, 0.25)
    # a strict maximum is found wherever it sits, and the runner-up after it
    lg = np.zeros((1, 200), np.float32)
    lg[0, 171], lg[0, 9] = 3.0, 2.0
    ids, w = orc.moe_topk(lg, 2)
    assert list(ids[0]) == [171, 9]
    # NaN -> -inf at load: never selected while finite logits remain (moe_topk.cpp:42-47)
    lg = np.zeros((1, 8), np.float32)
    lg[0, 0] = np.nan
    lg[0, 5] = 2.0
    ids, w = orc.moe_topk(lg, 3)
    assert ids[0, 0] == 5 and 0 not in ids[0]
    # renormalisation floor 2^-14 (moe_topk.cpp:101-107): one dominant logit, the
    # remaining picks underflow to 0 so weights are p/ max(sum, 2^-14)
    lg = np.full((1, 8), -200.0, np.float32)
    lg[0, 3] = 0.0
    ids, w = orc.moe_topk(lg, 2)
    assert ids[0, 0] == 3 and w[0, 0] == 1.0 and w[0, 1] == 0.0


def check_sort(ids, n_expert, bn, perm, eoff, toff):
    ids = ids.ravel()
    count = np.bincount(ids[(ids >= 0) & (ids < n_expert)], minlength=n_expert)
    assert np.array_equal(eoff, np.concatenate([[0], np.cumsum(count)]))
    assert np.array_equal(toff, np.concatenate([[0], np.cumsum((count + bn - 1) // bn)]))
    valid = perm[: eoff[-1]]
    assert len(set(valid.tolist())) == valid.size
    for e in range(n_expert):
        assert np.all(ids[perm[eoff[e]: eoff[e + 1]]] == e)


def test_sort_invariants_and_out_of_range():
    rng = np.random.default_rng(1)
    ids = rng.integers(0, 128, (512, 8)).astype(np.int32)
    perm, eoff, toff = orc.moe_sort(ids, 128, 16)
    check_sort(ids, 128, 16, perm, eoff, toff)
    assert eoff[-1] == 4096
    # out-of-range ids are dropped from the grouping (moe_expert_sort.cpp:38-40,71)
    ids2 = ids.copy()
    ids2[0, 0], ids2[3, 2] = -1, 128
    perm, eoff, toff = orc.moe_sort(ids2, 128, 32)
    check_sort(ids2, 128, 32, perm, eoff, toff)
    assert eoff[-1] == 4094
    # an expert with no tokens owns an empty range and no tile
    ids3 = np.zeros((4, 2), np.int32)
    perm, eoff, toff = orc.moe_sort(ids3, 4, 16)
    assert list(eoff) == [0, 8, 8, 8, 8] and list(toff) == [0, 1, 1, 1, 1]
    assert list(perm) == list(range(8))


def test_gather_scatter_combine_swiglu():
    rng = np.random.default_rng(2)
    n_tok, n_used, nsub, dim = 5, 3, 4, 7
    xq = rng.integers(0, 256, n_tok * nsub * 40, dtype=np.uint8)
    perm = rng.permutation(n_tok * n_used).astype(np.int32)
    g = orc.moe_gather_xq(xq, perm, nsub, n_used).reshape(-1, nsub * 40)
    src = xq.reshape(n_tok, nsub * 40)
    for p, e in enumerate(perm):
        assert np.array_equal(g[p], src[e // n_used])
    rows = rng.standard_normal((n_tok * n_used, dim)).astype(np.float32)
    sc = orc.moe_scatter_rows(rows, perm, dim)
    assert np.array_equal(sc[perm], rows)
    experts = rng.standard_normal((n_tok, n_used, dim)).astype(np.float32)
    ids = rng.integers(0, 6, (n_tok, n_used)).astype(np.int32)
    w = rng.random((n_tok, n_used)).astype(np.float32)
    s = rng.random(6).astype(np.float32)
    out = orc.moe_combine(experts, ids, w, s)
    want = np.einsum("tj,tjh->th", (w * s[ids]).astype(np.float64), experts.astype(np.float64))
    assert np.allclose(out, want, rtol=1e-5, atol=1e-6)
    gate = rng.standard_normal(100).astype(np.float32) * 4
    up = rng.standard_normal(100).astype(np.float32)
    g64 = gate.astype(np.float64)
    assert np.allclose(orc.swiglu_mul(gate, up), g64 / (1 + np.exp(-g64)) * up, rtol=1e-5, atol=1e-6)


def test_grouped_gemm_is_per_expert_matvec():
    fmt, in_dim, out_dim, n_expert = orc.Q4_K, 512, 8, 3
    bpe = orc.repacked_len(fmt, in_dim, out_dim)
    slabs = [orc.repack_for_matvec(fmt, random_raw_weights(fmt, in_dim, out_dim, seed=e), in_dim, out_dim)
             for e in range(n_expert)]
    slab = np.concatenate(slabs)
    eoff = np.array([0, 2, 2, 5], np.int32)
    x = np.random.default_rng(4).standard_normal((5, in_dim)).astype(np.float32)
    xq = orc.quantize_q8(x)
    y = orc.grouped_gemm(fmt, slab, bpe, eoff, xq, in_dim, out_dim)
    xqr = xq.reshape(5, -1)
    for e in range(n_expert):
        for t in range(eoff[e], eoff[e + 1]):
            assert np.array_equal(y[t], orc.matvec_q8(fmt, slabs[e], in_dim, out_dim, xqr[t])[0])
