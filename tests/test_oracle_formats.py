"""Pins the CPU oracle's formats against the reference's own closed-form unit
tests (src/quant/*.rs `mod tests`) and against what the mathematics fixes."""
import numpy as np
import pytest

from oracle import orc
from helpers import Lcg, f16_bytes, random_raw_weights

ALL = [orc.Q4_0, orc.Q8_0, orc.Q4_K, orc.Q5_K, orc.Q6_K, orc.IQ4_XS]
KV = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], np.float32)


# ---------------------------------------------------------------- half.rs
def test_f16_known_values():  # half.rs:93-106
    cases = [(0x0000, 0.0), (0x8000, -0.0), (0x3C00, 1.0), (0xBC00, -1.0), (0x4000, 2.0),
             (0x4200, 3.0), (0x3800, 0.5), (0x7BFF, 65504.0), (0xFBFF, -65504.0),
             (0x7C00, np.inf), (0xFC00, -np.inf), (0x0001, 5.9604645e-8)]
    for bits, want in cases:
        got = np.float32(orc.f16_to_f32(bits))
        assert got.view(np.uint32) == np.float32(want).view(np.uint32), hex(bits)
    assert np.isnan(orc.f16_to_f32(0x7E00))  # half.rs:109-113


def test_f16_to_f32_exhaustive_vs_numpy():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32).view(np.uint32)
    got = np.array([np.float32(orc.f16_to_f32(int(b))).view(np.uint32) for b in bits], np.uint32)
    nan = np.isnan(bits.view(np.float16))
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all(np.isnan(got[nan].view(np.float32)))


def test_f32_to_f16_roundtrip_and_rne():
    for bits in [0x0000, 0x3C00, 0xBC00, 0x4200, 0x3800, 0x7BFF, 0xFBFF]:  # half.rs:132-135
        assert orc.f32_to_f16(orc.f16_to_f32(bits)) == bits
    # every finite half survives f16 -> f32 -> f16
    for bits in range(0, 65536, 7):
        if (bits & 0x7C00) == 0x7C00:
            continue
        assert orc.f32_to_f16(orc.f16_to_f32(bits)) == bits
    # normal-range results are round-to-nearest-even == numpy's conversion
    rng = np.random.default_rng(0)
    v = (rng.standard_normal(20000) * 10.0 ** rng.uniform(-4, 4, 20000)).astype(np.float32)
    v = v[(np.abs(v) >= 6.2e-5) & (np.abs(v) < 65000)]
    want = v.astype(np.float16).view(np.uint16)
    got = np.array([orc.f32_to_f16(x) for x in v], np.uint16)
    assert np.array_equal(got, want)
    # exact ties: 1 + 2^-11 rounds to even (down), 1 + 3*2^-11 rounds up
    assert orc.f32_to_f16(1.0 + 2.0 ** -11) == 0x3C00
    assert orc.f32_to_f16(1.0 + 3 * 2.0 ** -11) == 0x3C02
    assert orc.f32_to_f16(1e6) == 0x7C00 and orc.f32_to_f16(-1e6) == 0xFC00
    assert orc.f32_to_f16(1e-9) == 0x0000


# ---------------------------------------------------------------- q4_k.rs
def synth_q4k(d, dmin, sc, m, nib):  # q4_k.rs:184-212
    b = np.zeros(144, np.uint8)
    b[0:2], b[2:4] = f16_bytes(d), f16_bytes(dmin)
    for j in range(4):
        b[4 + j] = (sc & 0x3F) | (((sc >> 4) & 3) << 6)
        b[8 + j] = (m & 0x3F) | (((m >> 4) & 3) << 6)
        b[12 + j] = (sc & 0xF) | ((m & 0xF) << 4)
    b[16:] = nib | (nib << 4)
    return b


def test_get_scale_min_k4():
    # hand-packed 12 bytes: sub-blocks 0..3 use the low 6 bits, 4..7 the split form
    q = np.zeros(12, np.uint8)
    sc = [1, 17, 33, 63, 5, 21, 42, 62]
    mn = [2, 18, 34, 61, 9, 30, 55, 63]
    for j in range(4):
        q[j] = sc[j] | ((sc[j + 4] >> 4) << 6)
        q[j + 4] = mn[j] | ((mn[j + 4] >> 4) << 6)
        q[j + 8] = (sc[j + 4] & 0xF) | ((mn[j + 4] & 0xF) << 4)
    for j in range(8):
        assert orc.get_scale_min_k4(j, q) == (sc[j], mn[j])


def test_q4k_closed_forms():
    for k in [0, 1, 7, 15]:  # q4_k.rs:214-224
        assert np.all(orc.dequantize_to_f32(orc.Q4_K, synth_q4k(1, 0, 1, 0, k), 256) == k)
    assert np.all(orc.dequantize_to_f32(orc.Q4_K, synth_q4k(2, 1, 3, 4, 5), 256) == 26.0)  # :226-233
    assert np.all(orc.dequantize_to_f32(orc.Q4_K, synth_q4k(1, 1, 63, 63, 1), 256) == 0.0)  # :235-251
    assert np.all(orc.dequantize_to_f32(orc.Q4_K, synth_q4k(1, 0, 63, 0, 2), 256) == 126.0)
    b = synth_q4k(1, 0, 1, 0, 0)  # :307-325 low/high nibbles feed adjacent sub-blocks
    b[16:] = 3 | (12 << 4)
    out = orc.dequantize_to_f32(orc.Q4_K, b, 256).reshape(4, 2, 32)
    assert np.all(out[:, 0] == 3.0) and np.all(out[:, 1] == 12.0)


def test_q4k_repack_reference_case():  # q4_k.rs:253-305
    raw = []
    for blk in range(2):
        b = synth_q4k(2, 1, 3, 4, 0)
        for i in range(128):
            b[16 + i] = ((blk * 128 + i) * 5 + 1) & 0xFF
        raw.append(b)
    raw = np.concatenate(raw)
    ref = orc.dequantize_to_f32(orc.Q4_K, raw, 512)
    packed = orc.repack_for_matvec(orc.Q4_K, raw, 512, 1)
    assert orc.repacked_n_sub_padded(512) == 17
    assert packed.size == 17 * 16 + 17 * 2 + 2 * 4
    # decode by hand, as the reference test does
    nib_len, sm_len = 17 * 16, 17 * 2
    got = np.zeros(512, np.float32)
    for gsb in range(16):
        nib = packed[gsb * 16: gsb * 16 + 16]
        sc, m = packed[nib_len + gsb * 2], packed[nib_len + gsb * 2 + 1]
        ddo = nib_len + sm_len + (gsb // 8) * 4
        d = orc.f16_to_f32(int(packed[ddo]) | int(packed[ddo + 1]) << 8)
        dmin = orc.f16_to_f32(int(packed[ddo + 2]) | int(packed[ddo + 3]) << 8)
        blk, s = divmod(gsb, 8)
        base = blk * 256 + (s // 2) * 64 + (s & 1) * 32
        for k in range(32):
            q = (nib[k] & 0xF) if k < 16 else (nib[k - 16] >> 4)
            got[base + k] = np.float32(d * sc) * np.float32(q) - np.float32(dmin * m)
    assert np.array_equal(got, ref)
    assert np.array_equal(orc.decode_repacked_to_f32(orc.Q4_K, packed, 512, 1)[0], ref)


# ---------------------------------------------------------------- q5_k.rs
def synth_q5k(d, dmin, sc, m, nib, high):  # q5_k.rs:159-187
    b = np.zeros(176, np.uint8)
    b[0:2], b[2:4] = f16_bytes(d), f16_bytes(dmin)
    for j in range(4):
        b[4 + j] = (sc & 0x3F) | (((sc >> 4) & 3) << 6)
        b[8 + j] = (m & 0x3F) | (((m >> 4) & 3) << 6)
        b[12 + j] = (sc & 0xF) | ((m & 0xF) << 4)
    b[16:48] = 0xFF if high else 0
    b[48:] = nib | (nib << 4)
    return b


def test_q5k_closed_forms():
    q5 = orc.dequantize_to_f32(orc.Q5_K, synth_q5k(2, 1, 3, 4, 5, False), 256)  # :189-212
    q4 = orc.dequantize_to_f32(orc.Q4_K, synth_q4k(2, 1, 3, 4, 5), 256)
    assert np.array_equal(q5, q4)
    assert np.all(orc.dequantize_to_f32(orc.Q5_K, synth_q5k(1, 0, 1, 0, 2, True), 256) == 18.0)  # :214-221
    b = synth_q5k(1, 0, 1, 0, 0, False)  # :223-243
    b[16] = 1
    out = orc.dequantize_to_f32(orc.Q5_K, b, 256)
    assert out[0] == 16.0 and np.all(out[1:] == 0)
    b = synth_q5k(1, 0, 1, 0, 0, False)
    b[16 + 31] = 0x80
    out = orc.dequantize_to_f32(orc.Q5_K, b, 256)
    assert out[255] == 16.0 and np.all(out[:255] == 0)


# ---------------------------------------------------------------- q6_k.rs
def synth_q6k(d, scale, q):  # q6_k.rs:157-178
    b = np.zeros(210, np.uint8)
    b[:128] = (q & 0xF) | ((q & 0xF) << 4)
    pair = (q >> 4) & 3
    b[128:192] = pair | (pair << 2) | (pair << 4) | (pair << 6)
    b[192:208] = np.uint8(scale & 0xFF)
    b[208:210] = f16_bytes(d)
    return b


def test_q6k_closed_forms():
    assert np.all(orc.dequantize_to_f32(orc.Q6_K, synth_q6k(2.5, -7, 32), 256) == 0.0)  # :180-187
    for q in [0, 16, 31, 32, 33, 47, 63]:  # :189-201
        assert np.all(orc.dequantize_to_f32(orc.Q6_K, synth_q6k(1, 1, q), 256) == q - 32)
    assert np.all(orc.dequantize_to_f32(orc.Q6_K, synth_q6k(1, -3, 33), 256) == -3.0)  # :203-210
    b = synth_q6k(1, 0, 33)  # :212-237
    b[192:208] = np.arange(16, dtype=np.uint8)
    out = orc.dequantize_to_f32(orc.Q6_K, b, 256)
    for idx in range(256):
        chunk, inner = divmod(idx, 128)
        group, l = divmod(inner, 32)
        assert out[idx] == chunk * 8 + l // 16 + group * 2


# ---------------------------------------------------------------- q4_0.rs / q8_0.rs
def test_q4_0_closed_forms():
    b = np.zeros(18, np.uint8)  # q4_0.rs:114-128
    b[0:2] = f16_bytes(1.0)
    for k in range(16):
        b[2 + k] = k | ((15 - k) << 4)
    out = orc.dequantize_to_f32(orc.Q4_0, b, 32)
    assert np.array_equal(out[:16], np.arange(16) - 8.0)
    assert np.array_equal(out[16:], (15 - np.arange(16)) - 8.0)


def test_q4_0_repack_bytes():  # q4_0.rs:132-170
    in_dim, out_dim, nb = 96, 2, 3
    assert orc.repacked_n_sub_padded(in_dim) == nb
    raw = (np.arange(out_dim * nb * 18) % 251).astype(np.uint8)
    for blk in range(out_dim * nb):
        raw[blk * 18: blk * 18 + 2] = f16_bytes(blk + 1.0)
    packed = orc.repack_for_matvec(orc.Q4_0, raw, in_dim, out_dim)
    assert packed.size == orc.repacked_len(orc.Q4_0, in_dim, out_dim)
    nib_len = out_dim * nb * 16
    for i in range(out_dim * nb):
        assert np.array_equal(packed[i * 16: i * 16 + 16], raw[i * 18 + 2: i * 18 + 18])
        assert np.array_equal(packed[nib_len + i * 2: nib_len + i * 2 + 2], raw[i * 18: i * 18 + 2])
    assert orc.repacked_n_sub_padded(32 * 4) == 5 and orc.repacked_n_sub_padded(32 * 6) == 6


def test_q4_0_repack_lcg_case():  # q4_0.rs:172-212 (seed, scales and shape as there)
    in_dim, out_dim = 256, 3
    g = Lcg(0xA5A51234, inc=1)
    raw = np.zeros(out_dim * 8 * 18, np.uint8)
    for blk in range(out_dim * 8):
        raw[blk * 18: blk * 18 + 2] = f16_bytes(np.float32(0.01) * np.float32(blk + 1.0))
        raw[blk * 18 + 2: blk * 18 + 18] = g.bytes(16)
    direct = orc.dequantize_to_f32(orc.Q4_0, raw, out_dim * in_dim).reshape(out_dim, in_dim)
    packed = orc.repack_for_matvec(orc.Q4_0, raw, in_dim, out_dim)
    assert orc.repacked_n_sub_padded(in_dim) == 9
    assert np.array_equal(orc.decode_repacked_to_f32(orc.Q4_0, packed, in_dim, out_dim), direct)


def test_q8_0_closed_forms():
    b = np.zeros(34, np.uint8)  # q8_0.rs:126-138
    b[0:2] = f16_bytes(1.0)
    b[2:] = np.arange(32, dtype=np.uint8)
    assert np.array_equal(orc.dequantize_to_f32(orc.Q8_0, b, 32), np.arange(32, dtype=np.float32))
    b[0:2] = f16_bytes(-0.5)  # :140-152
    b[2:] = 4
    assert np.all(orc.dequantize_to_f32(orc.Q8_0, b, 32) == -2.0)
    two = np.zeros(68, np.uint8)  # :154-170
    two[0:2], two[34:36] = f16_bytes(1.0), f16_bytes(2.0)
    two[2:34], two[36:68] = 1, 1
    out = orc.dequantize_to_f32(orc.Q8_0, two, 64)
    assert np.all(out[:32] == 1.0) and np.all(out[32:] == 2.0)


def test_q8_0_quantizer():  # q8_0.rs:45-61: d = amax/127, q = round-half-away(x/d)
    v = np.zeros(64, np.float32)
    v[:32] = np.linspace(-127, 127, 32).astype(np.float32)  # amax 127 -> d = 1, q = round(x)
    v[32] = 2.5  # second block: amax 2.5; 2.5/d = 127
    v[33] = -1.25
    out = orc.q8_0_quantize_from_f32(v)
    assert int(out[0]) | (int(out[1]) << 8) == orc.f32_to_f16(1.0)
    want = np.where(v[:32] >= 0, np.floor(v[:32] + 0.5), np.ceil(v[:32] - 0.5)).astype(np.int8)
    assert np.array_equal(out[2:34].view(np.int8), want)
    q2 = out[36:68].view(np.int8)
    assert q2[0] == 127 and q2[1] in (-63, -64) and np.all(q2[2:] == 0)
    # half-away-from-zero, not ties-to-even: x = 0.5*d with d = 1 must give 1, and -0.5 -> -1
    t = np.zeros(32, np.float32)
    t[0], t[1], t[2], t[3] = 127.0, 0.5, -0.5, 2.5
    q = orc.q8_0_quantize_from_f32(t)[2:].view(np.int8)
    assert list(q[:4]) == [127, 1, -1, 3]
    assert np.all(orc.q8_0_quantize_from_f32(np.zeros(32, np.float32)) == 0)


# ---------------------------------------------------------------- iq4_xs.rs
def synth_iq4xs(d, ls, nib):  # iq4_xs.rs:189-216
    b = np.zeros(136, np.uint8)
    b[0:2] = f16_bytes(d)
    sh = 0
    for ib in range(8):
        sh |= ((ls >> 4) & 3) << (2 * ib)
    b[2], b[3] = sh & 0xFF, sh >> 8
    b[4:8] = (ls & 0xF) | ((ls & 0xF) << 4)
    b[8:] = nib | (nib << 4)
    return b


def test_iq4xs_closed_forms():
    assert np.all(orc.dequantize_to_f32(orc.IQ4_XS, synth_iq4xs(7.0, 32, 5), 256) == 0.0)  # :218-225
    for nib in range(16):  # :227-239
        assert np.all(orc.dequantize_to_f32(orc.IQ4_XS, synth_iq4xs(1.0, 33, nib), 256) == KV[nib])
    assert np.all(orc.dequantize_to_f32(orc.IQ4_XS, synth_iq4xs(1.0, 20, 8), 256) == -12.0)  # :241-250
    b = synth_iq4xs(1.0, 33, 0)  # :252-270
    b[8:] = 2 | (10 << 4)
    out = orc.dequantize_to_f32(orc.IQ4_XS, b, 256).reshape(8, 2, 16)
    assert np.all(out[:, 0] == KV[2]) and np.all(out[:, 1] == KV[10])
    b = synth_iq4xs(1.0, 32, 8)  # :272-296
    sh, sl = 0, [0, 0, 0, 0]
    for sb in range(8):
        ls = 33 + sb
        sh |= ((ls >> 4) & 3) << (2 * sb)
        sl[sb // 2] |= (ls & 0xF) << (4 * (sb & 1))
    b[2], b[3] = sh & 0xFF, sh >> 8
    b[4:8] = sl
    out = orc.dequantize_to_f32(orc.IQ4_XS, b, 256).reshape(8, 32)
    for sb in range(8):
        assert np.all(out[sb] == 1 + sb)


def test_iq4xs_repack_lcg_case():  # iq4_xs.rs:148-187
    in_dim, out_dim = 512, 3
    assert orc.repacked_n_sub_padded(in_dim) == 17
    g = Lcg(0x1A4A5EED, inc=1)
    raw = np.zeros(out_dim * 2 * 136, np.uint8)
    for blk in range(out_dim * 2):
        raw[blk * 136 + 2: blk * 136 + 136] = g.bytes(134)
        raw[blk * 136: blk * 136 + 2] = f16_bytes(np.float32(0.02) * np.float32(blk + 1.0))
    direct = orc.dequantize_to_f32(orc.IQ4_XS, raw, out_dim * in_dim).reshape(out_dim, in_dim)
    packed = orc.repack_for_matvec(orc.IQ4_XS, raw, in_dim, out_dim)
    assert packed.size == orc.repacked_len(orc.IQ4_XS, in_dim, out_dim)
    got = orc.decode_repacked_to_f32(orc.IQ4_XS, packed, in_dim, out_dim)
    rel = np.abs(got - direct) / np.maximum(np.abs(direct), 1e-30)
    assert rel.max() < 5e-4  # one extra fp16 rounding of the folded scale


# ---------------------------------------------------------------- repack invariants, all formats
@pytest.mark.parametrize("fmt", ALL)
@pytest.mark.parametrize("in_dim,out_dim", [(256, 1), (512, 3), (768, 2), (1024, 5), (2048, 2)])
def test_repack_roundtrip(fmt, in_dim, out_dim):
    raw = random_raw_weights(fmt, in_dim, out_dim, seed=in_dim * 31 + out_dim + fmt)
    direct = orc.dequantize_to_f32(fmt, raw, in_dim * out_dim).reshape(out_dim, in_dim)
    packed = orc.repack_for_matvec(fmt, raw, in_dim, out_dim)
    n_sub = in_dim // 32
    nsp = n_sub + 1 if (n_sub & (n_sub - 1)) == 0 else n_sub
    per_sub = {orc.Q4_K: 18, orc.Q5_K: 22, orc.Q6_K: 26, orc.Q8_0: 34, orc.Q4_0: 18, orc.IQ4_XS: 18}[fmt]
    per_sup = {orc.Q4_K: 4, orc.Q5_K: 4, orc.Q6_K: 2}.get(fmt, 0)
    assert orc.repacked_n_sub_padded(in_dim) == nsp
    assert packed.size == out_dim * nsp * per_sub + out_dim * (in_dim // 256) * per_sup
    got = orc.decode_repacked_to_f32(fmt, packed, in_dim, out_dim)
    if fmt == orc.IQ4_XS:
        assert np.allclose(got, direct, rtol=5e-4, atol=0)
    elif fmt == orc.Q6_K:
        # dequant multiplies (d*sc)*q, the kernel form is the same product order
        assert np.array_equal(got, direct)
    else:
        assert np.array_equal(got, direct)
    if nsp != n_sub:  # the pad sub-block of every row stays zero
        nib = packed[: out_dim * nsp * 16].reshape(out_dim, nsp, 16)
        assert np.all(nib[:, n_sub] == 0)


def test_per_row_bytes_at_baseline_shapes():
    # bytes per output row quoted for the bench roofline
    want = {orc.Q4_0: 2880, orc.IQ4_XS: 2880, orc.Q4_K: 2960, orc.Q5_K: 3600, orc.Q6_K: 4200, orc.Q8_0: 5440}
    for fmt, b in want.items():
        assert orc.repacked_len(fmt, 5120, 1) == b
    assert orc.repacked_len(orc.Q4_K, 17408, 1) == 10064
    assert orc.repacked_len(orc.Q6_K, 17408, 1) == 14280
    assert orc.repacked_len(orc.Q4_K, 4096, 1) == 129 * 18 + 64
    assert orc.repacked_len(orc.Q4_K, 2048, 1) == 1202
    assert orc.repacked_len(orc.Q6_K, 768, 1) == 630
    assert orc.repacked_len(orc.Q4_K, 5120, 5120) + 160 * 40 + 5120 * 4 == 15182080
