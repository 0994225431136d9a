"""Pins the oracle's activation quantizer, per-block integer dots and fp32
combine: special cases, invariants, brute force in numpy from the *dequantized*
weights (an independent route), and the reference's own GPU-test tolerance."""
import numpy as np
import pytest

from oracle import orc
from helpers import Lcg, random_raw_weights, rel_l2

ALL = [orc.Q4_0, orc.Q8_0, orc.Q4_K, orc.Q5_K, orc.Q6_K, orc.IQ4_XS]


def unpack_xq(xq, n_vec, n_sub):
    b = xq.reshape(n_vec, n_sub, 40)
    d = b[:, :, 0:4].copy().view(np.float32)[..., 0]
    xsum = b[:, :, 4:8].copy().view(np.float32)[..., 0]
    qs = b[:, :, 8:].view(np.int8)
    return d, xsum, qs


def test_quantize_q8_special_cases():
    x = np.zeros((1, 96), np.float32)
    x[0, 32 + 5] = 3.0          # single +amax -> +127
    x[0, 64 + 7] = -0.25        # single -amax -> -127
    d, xsum, qs = unpack_xq(orc.quantize_q8(x), 1, 3)
    assert d[0, 0] == 1.0 and xsum[0, 0] == 0.0 and np.all(qs[0, 0] == 0)   # all-zero block
    assert qs[0, 1, 5] == 127 and d[0, 1] == np.float32(3.0) / np.float32(127.0) and xsum[0, 1] == 3.0
    assert qs[0, 2, 7] == -127 and xsum[0, 2] == -0.25
    assert np.count_nonzero(qs) == 2


def test_quantize_q8_invariants_and_tree():
    rng = np.random.default_rng(1)
    x = (rng.standard_normal((5, 512)) * rng.uniform(0.01, 30, (5, 1))).astype(np.float32)
    d, xsum, qs = unpack_xq(orc.quantize_q8(x), 5, 16)
    xb = x.reshape(5, 16, 32)
    amax = np.abs(xb).max(axis=2)
    assert np.array_equal(d, amax / np.float32(127.0))
    assert np.abs(qs.astype(np.int32)).max() <= 127
    # q = rint(v * (127/amax)) with both operations in fp32, ties-to-even
    inv = np.float32(127.0) / amax
    want = np.clip(np.rint(xb * inv[..., None]), -127, 127).astype(np.int8)
    assert np.array_equal(qs, want)
    # the element of largest magnitude always lands on +-127
    idx = np.abs(xb).argmax(axis=2)
    top = np.take_along_axis(qs, idx[..., None], axis=2)[..., 0]
    assert np.all(np.abs(top.astype(np.int32)) == 127)
    # xsum = the fixed butterfly: pair i with i^16, then ^8, ^4, ^2, ^1
    s = xb.copy()
    for o in (16, 8, 4, 2, 1):
        s = s + s[..., np.arange(32) ^ o]
    assert np.array_equal(xsum, s[..., 0])
    # ... which is a genuine fp32 tree, not a left-to-right sum, but stays close to the exact sum
    exact = xb.astype(np.float64).sum(axis=2)
    assert np.allclose(xsum, exact, rtol=0, atol=1e-4 * np.abs(xb).sum(axis=2).max())


def test_quantize_q8_ties_to_even():
    # amax = 127 -> inv == 1 exactly, so v*inv == v and .5 cases expose the rounding mode
    v = np.zeros((1, 32), np.float32)
    v[0, :6] = [127.0, 0.5, 1.5, 2.5, -0.5, -3.5]
    _, _, qs = unpack_xq(orc.quantize_q8(v), 1, 1)
    assert list(qs[0, 0, :6]) == [127, 0, 2, 2, 0, -4]


def int_weights_from_dequant(fmt, raw, in_dim, out_dim):
    """Independent route to the integer weights: dequantize with unit scales."""
    return orc.dequantize_to_f32(fmt, raw, in_dim * out_dim).reshape(out_dim, in_dim)


@pytest.mark.parametrize("fmt", ALL)
@pytest.mark.parametrize("in_dim,out_dim,n_rows", [(256, 3, 1), (768, 4, 2), (1024, 2, 3)])
def test_block_dots_brute_force(fmt, in_dim, out_dim, n_rows):
    """Per-block integer dots against numpy brute force computed from the raw
    on-disk blocks: set every scale to a power of two so dequantize_to_f32
    returns the integer weights exactly, then dot them with the int8 activations."""
    rng = np.random.default_rng(fmt * 1000 + in_dim)
    bs, bb = orc.block_size(fmt), orc.bytes_per_block(fmt)
    nblk = in_dim * out_dim // bs
    raw = rng.integers(0, 256, (nblk, bb), dtype=np.uint8)
    one = [0x00, 0x3C]
    if fmt in (orc.Q4_K, orc.Q5_K):
        raw[:, 0:2] = one            # d = 1
        raw[:, 2:4] = 0              # dmin = 0
        raw[:, 4:16] = 0
        raw[:, 4:8] = 1              # sc[0..3] = 1
        raw[:, 12:16] = 1            # sc[4..7] = 1, m = 0
    elif fmt == orc.Q6_K:
        raw[:, 192:208] = 1
        raw[:, 208:210] = one
    elif fmt == orc.IQ4_XS:
        raw[:, 0:2] = one
        raw[:, 2:4] = [0xAA, 0xAA]   # ls high bits = 2 -> ls = 32 + 1
        raw[:, 4:8] = 0x11
    else:
        raw[:, 0:2] = one
    raw = raw.reshape(-1)
    w = int_weights_from_dequant(fmt, raw, in_dim, out_dim)          # exact integers (Q4_0: q-8, Q6_K: q-32)
    assert np.array_equal(w, np.round(w))
    x = rng.standard_normal((n_rows, in_dim)).astype(np.float32)
    xq = orc.quantize_q8(x)
    _, _, qs = unpack_xq(xq, n_rows, in_dim // 32)
    packed = orc.repack_for_matvec(fmt, raw, in_dim, out_dim)
    got = orc.block_dots(fmt, packed, in_dim, out_dim, xq, n_rows)

    # which original positions form sub-block sb, in dot order
    n_sub = in_dim // 32
    pos = np.empty((n_sub, 32), np.int64)
    for sb in range(n_sub):
        blk, s = divmod(sb, 8)
        if fmt in (orc.Q4_K, orc.Q5_K):
            base = blk * 256 + (s // 2) * 64 + (s & 1) * 32
        elif fmt == orc.Q6_K:
            base = blk * 256 + (s // 4) * 128 + (s % 4) * 32
        else:
            base = sb * 32
        pos[sb] = base + np.arange(32)
    wi = w.astype(np.int64)[:, pos]                                    # [out, n_sub, 32]
    q = qs.astype(np.int64)                                            # [rows, n_sub, 32]
    if fmt == orc.Q6_K:
        lo = np.einsum("rsk,tsk->trs", wi[..., :16], q[..., :16])
        hi = np.einsum("rsk,tsk->trs", wi[..., 16:], q[..., 16:])
        want = np.stack([lo, hi], axis=-1)
    else:
        want = np.einsum("rsk,tsk->trs", wi, q)[..., None]
    # for Q4_0/Q6_K `w` already carries the -8/-32, i.e. the folded form
    # (idot - 8*sum q8, idot - 32*sum q8) must be integer-identical to it
    assert np.array_equal(got.astype(np.int64), want)


@pytest.mark.parametrize("fmt", ALL)
def test_int8_path_equals_f32_path_on_integer_activations(fmt):
    """With integer activations whose block amax is exactly 127, dx == 1 and
    q8 == x, so the int8 path must reproduce dequant -> f32 matvec up to fp32
    summation order."""
    in_dim, out_dim = 1024, 24
    raw = random_raw_weights(fmt, in_dim, out_dim, seed=7 + fmt)
    rng = np.random.default_rng(3)
    x = rng.integers(-127, 128, in_dim).astype(np.float32)
    x.reshape(-1, 32)[:, 0] = 127.0
    xq = orc.quantize_q8(x)
    d, _, qs = unpack_xq(xq, 1, in_dim // 32)
    assert np.all(d == 1.0) and np.array_equal(qs.reshape(-1).astype(np.float32), x)
    packed = orc.repack_for_matvec(fmt, raw, in_dim, out_dim)
    w = orc.dequantize_to_f32(fmt, raw, in_dim * out_dim).reshape(out_dim, in_dim)
    if fmt == orc.IQ4_XS:   # the repack folds d*(ls-32) into one fp16: compare against its own decode
        w = orc.decode_repacked_to_f32(fmt, packed, in_dim, out_dim)
    y8 = orc.matvec_q8(fmt, packed, in_dim, out_dim, xq)[0]
    yf = orc.matvec_f32(x, w)
    y64 = w.astype(np.float64) @ x.astype(np.float64)
    scale = np.abs(w.astype(np.float64)) @ np.abs(x.astype(np.float64))
    assert np.all(np.abs(y8 - y64) <= 2e-6 * scale)
    assert np.all(np.abs(yf - y64) <= 2e-6 * scale)


@pytest.mark.parametrize("fmt,seed,xseed", [(orc.Q4_K, 0xD4A40001, 0x13579BDF)])
def test_reference_gpu_test_recipe_q4k(fmt, seed, xseed):
    """The reference's Q4_K repacked-matvec GPU test (kernels.rs:3026-3061):
    LCG bytes, tame scales, 2048 -> 384, rel_l2 < 1.5e-2 vs dequant -> f32."""
    in_dim, out_dim = 2048, 384
    g = Lcg(seed)
    raw = g.bytes(out_dim * (in_dim // 256) * 144).reshape(-1, 144)
    for blk in range(raw.shape[0]):
        d = np.float32(((blk % 29) - 14)) * np.float32(0.003)
        dm = np.float32(((blk % 17) - 8)) * np.float32(0.0015)
        raw[blk, 0], raw[blk, 1] = orc.f32_to_f16(d) & 0xFF, orc.f32_to_f16(d) >> 8
        raw[blk, 2], raw[blk, 3] = orc.f32_to_f16(dm) & 0xFF, orc.f32_to_f16(dm) >> 8
    raw = raw.reshape(-1)
    x = Lcg(xseed).acts(in_dim)
    w = orc.dequantize_to_f32(fmt, raw, in_dim * out_dim).reshape(out_dim, in_dim)
    want = orc.matvec_f32(x, w)
    packed = orc.repack_for_matvec(fmt, raw, in_dim, out_dim)
    got = orc.matvec_q8(fmt, packed, in_dim, out_dim, orc.quantize_q8(x))[0]
    assert rel_l2(got, want) < 1.5e-2


@pytest.mark.parametrize("fmt", ALL)
def test_int8_path_within_reference_tolerance(fmt):
    in_dim, out_dim = 2048, 96
    raw = random_raw_weights(fmt, in_dim, out_dim, seed=100 + fmt)
    x = Lcg(0x2468ACE0 + fmt).acts(in_dim)
    w = orc.dequantize_to_f32(fmt, raw, in_dim * out_dim).reshape(out_dim, in_dim)
    packed = orc.repack_for_matvec(fmt, raw, in_dim, out_dim)
    got = orc.matvec_q8(fmt, packed, in_dim, out_dim, orc.quantize_q8(x))[0]
    assert rel_l2(got, orc.matvec_f32(x, w)) < 1.5e-2          # kernels.rs:1598-1601


def test_matvec_f32_matches_sequential_sum():
    rng = np.random.default_rng(5)
    w = rng.standard_normal((300, 512)).astype(np.float32)
    x = rng.standard_normal(512).astype(np.float32)
    want = np.empty(300, np.float32)
    for j in range(300):
        acc = np.float32(0)
        for i in range(512):
            acc = np.float32(acc + np.float32(x[i] * w[j, i]))
        want[j] = acc
    assert np.array_equal(orc.matvec_f32(x, w, n_threads=4), want)
    assert np.array_equal(orc.matvec_f32(x, w, n_threads=1), want)


def test_matvec_q8_batched_rows_independent():
    fmt, in_dim, out_dim = orc.Q5_K, 768, 16
    raw = random_raw_weights(fmt, in_dim, out_dim, seed=11)
    packed = orc.repack_for_matvec(fmt, raw, in_dim, out_dim)
    x = np.random.default_rng(2).standard_normal((3, in_dim)).astype(np.float32)
    xq = orc.quantize_q8(x)
    y = orc.matvec_q8(fmt, packed, in_dim, out_dim, xq, 3)
    for t in range(3):
        assert np.array_equal(y[t], orc.matvec_q8(fmt, packed, in_dim, out_dim, orc.quantize_q8(x[t]))[0])
