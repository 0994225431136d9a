"""Shared input builders for the tests (mirrors of the reference tests' recipes)."""
import numpy as np

from oracle import orc

MASK64 = (1 << 64) - 1

# Device uploads of the GPU tests.  Launches are asynchronous: a buffer passed straight into a
# launch as `dev(array)` would otherwise be freed when the call returns, while the kernel may
# still read it.  They are kept here and released by conftest's fixture after each test has
# synchronized.
_uploads = []


def dev(a):
    from reinstinct_amd import hip
    buf = hip.DeviceBuf.from_host(np.ascontiguousarray(a))
    _uploads.append(buf)
    return buf


def release_uploads():
    _uploads.clear()


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
    elif fmt == orc.IQ3_S:
        put(0, ((blk % 23) - 11) * 0.0008)
    elif fmt == orc.Q5_1:
        put(0, ((blk % 29) - 14) * 0.003)
        put(2, ((blk % 17) - 8) * 0.0123)
    return raw.reshape(-1)


def rel_l2(a, b):
    """kernels.rs:1588-1596"""
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def assert_close_f32(got, want, rel=1e-3, abs_=1e-4, what="", strict=False):
    """fp32 output bar, element-wise.

    strict=True: |got-want| <= abs + rel*|want|, the bar as stated (1e-3 relative / 1e-4 absolute).  Every
    test on the BASELINE recipe (weights ~N(0,0.02) quantized per format, activations ~N(0,1)) uses it.

    strict=False: |got-want| <= abs*max(1, rms(want)) + rel*|want|.  Only for the random-byte weights of
    the reference's GPU tests (kernels.rs:3026-3061): they give sums of terms of magnitude ~40 and rms(y)
    in the hundreds, where the order of the fp32 additions alone moves an element by 1e-4, so the absolute
    part scales with rms(want)."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    err = np.abs(got - want)
    scale = 1.0 if strict or not want.size else max(1.0, float(np.sqrt(np.mean(want * want))))
    tol = abs_ * scale + rel * np.abs(want)
    bad = ~(err <= tol)
    if bad.any():
        i = int(np.argmax(np.where(np.isnan(err), np.inf, err - tol)))
        raise AssertionError(
            f"{what}: {int(bad.sum())}/{bad.size} outside {rel} rel / {abs_}*{scale:.3g} abs; worst at flat {i}: "
            f"got {got.ravel()[i]!r} want {want.ravel()[i]!r}")


# ---- a GGUF v3 writer for the container tests (layout: src/gguf/mod.rs:4-18 of the reference)
GGUF_U8, GGUF_I8, GGUF_U16, GGUF_I16, GGUF_U32, GGUF_I32, GGUF_F32, GGUF_BOOL, GGUF_STRING, GGUF_ARRAY, \
    GGUF_U64, GGUF_I64, GGUF_F64 = range(13)
_GGUF_PACK = {GGUF_U8: "<B", GGUF_I8: "<b", GGUF_U16: "<H", GGUF_I16: "<h", GGUF_U32: "<I", GGUF_I32: "<i",
              GGUF_F32: "<f", GGUF_BOOL: "<B", GGUF_U64: "<Q", GGUF_I64: "<q", GGUF_F64: "<d"}


def gguf_string(s):
    import struct
    b = s if isinstance(s, bytes) else s.encode()
    return struct.pack("<Q", len(b)) + b


def gguf_value(vt, v):
    """payload of one metadata value; arrays are (element type, [values])"""
    import struct
    if vt == GGUF_STRING:
        return gguf_string(v)
    if vt == GGUF_ARRAY:
        et, items = v
        return struct.pack("<IQ", et, len(items)) + b"".join(gguf_value(et, x) for x in items)
    return struct.pack(_GGUF_PACK[vt], v)


def write_gguf(meta, tensors, version=3, magic=b"GGUF", pad_data=0):
    """meta: [(key, value type, value)]; tensors: [(name, dims, ggml type, payload bytes)].
    Returns (file bytes, {name: offset in the data section}).  The alignment is what a
    `general.alignment` entry of `meta` says, else 32."""
    import struct
    align = 32
    for k, vt, v in meta:
        if k == "general.alignment" and vt != GGUF_STRING:
            align = int(v)
    out = bytearray(magic + struct.pack("<IQQ", version, len(tensors), len(meta)))
    for k, vt, v in meta:
        out += gguf_string(k) + struct.pack("<I", vt) + gguf_value(vt, v)
    offs, at = {}, 0
    for name, dims, ty, payload in tensors:
        offs[name] = at
        out += gguf_string(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        out += struct.pack("<IQ", ty, at)
        at += len(payload)
        if align > 1:
            at = (at + align - 1) // align * align
    if align > 1:
        out += b"\0" * (-len(out) % align)
    data_at = len(out)
    for name, dims, ty, payload in tensors:
        out += b"\0" * (data_at + offs[name] - len(out)) + bytes(payload)
    out += b"\0" * pad_data
    return bytes(out), offs
