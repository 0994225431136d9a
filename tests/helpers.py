"""Shared input builders for the tests (mirrors of the reference tests' recipes)."""
import numpy as np

from oracle import orc

MASK64 = (1 << 64) - 1


class Lcg:
    """The reference tests' generator (src/runtime/kernels.rs:3030-3048):
    s = s*6364136223846793005 + inc; byte = s>>56; act = (s>>33)/u32::MAX - 0.5."""

    def __init__(self, seed, inc=1442695040888963407):
        self.s = seed & MASK64
        self.inc = inc

    def step(self):
        self.s = (self.s * 6364136223846793005 + self.inc) & MASK64
        return self.s

    def bytes(self, n):
        out = np.empty(n, np.uint8)
        for i in range(n):
            out[i] = self.step() >> 56
        return out

    def acts(self, n):
        out = np.empty(n, np.float32)
        umax = np.float32(4294967295.0)
        for i in range(n):
            v = np.float32((self.step() >> 33) & 0xFFFFFFFF)
            out[i] = v / umax - np.float32(0.5)
        return out


def f16_bytes(v):
    b = orc.f32_to_f16(v)
    return [b & 0xFF, b >> 8]


def random_raw_weights(fmt, in_dim, out_dim, seed):
    """Random on-disk blocks with tame fp16 scales, the way the reference GPU
    tests build them (kernels.rs:3030-3048, 3097-3104, 2965-2972, 1740-1745)."""
    rng = np.random.default_rng(seed)
    bs, bb = orc.block_size(fmt), orc.bytes_per_block(fmt)
    nblk = out_dim * in_dim // bs
    raw = rng.integers(0, 256, size=(nblk, bb), dtype=np.uint8)
    blk = np.arange(nblk)

    def put(col, vals):
        h = np.asarray(vals, np.float32).astype(np.float16).view(np.uint16)
        raw[:, col] = h & 0xFF
        raw[:, col + 1] = h >> 8

    if fmt in (orc.Q4_K, orc.Q5_K):
        put(0, ((blk % 29) - 14) * 0.003)
        put(2, ((blk % 17) - 8) * 0.0015)
    elif fmt == orc.Q6_K:
        put(208, ((blk % 23) - 11) * 0.004)
    elif fmt == orc.Q4_0:
        put(0, ((blk % 29) - 14) * 0.003)
    elif fmt == orc.Q8_0:
        put(0, ((blk % 29) - 14) * 0.0005)
    elif fmt == orc.IQ4_XS:
        put(0, ((blk % 23) - 11) * 0.005)
    return raw.reshape(-1)


def rel_l2(a, b):
    """kernels.rs:1588-1596"""
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def assert_close_f32(got, want, rel=1e-3, abs_=1e-4, what=""):
    """fp32 output bar: |got-want| <= abs*max(1, rms(want)) + rel*|want| element-wise.

    The absolute part is stated for outputs of unit scale (weights ~N(0,0.02),
    activations ~N(0,1) give rms(y) ~ 1).  The random-byte weights of the
    reference's GPU tests (kernels.rs:3026-3061) give sums of terms of magnitude
    ~40 and rms(y) in the hundreds; there the order of the fp32 additions alone
    moves an element by 1e-4, so the absolute part scales with rms(want)."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    err = np.abs(got - want)
    scale = max(1.0, float(np.sqrt(np.mean(want * want)))) if want.size else 1.0
    tol = abs_ * scale + rel * np.abs(want)
    bad = ~(err <= tol)
    if bad.any():
        i = int(np.argmax(np.where(np.isnan(err), np.inf, err - tol)))
        raise AssertionError(
            f"{what}: {int(bad.sum())}/{bad.size} outside {rel} rel / {abs_}*{scale:.3g} abs; worst at flat {i}: "
            f"got {got.ravel()[i]!r} want {want.ravel()[i]!r}")
