"""Pins of the oracle's Q5_1 and IQ3_S restatements (the two formats the reference runs on
the Q5_K / IQ4_XS kernels): the IQ3_S grid against checksums taken from the reference's
table, closed-form single-weight cases of both block formats, and the reference's own unit
tests (src/quant/q5_1.rs:111-157, src/quant/iq3_s.rs:210-261) restated on the oracle."""
import json
import os
import zlib

import numpy as np
import pytest

from oracle import orc
from helpers import Lcg

HERE = os.path.dirname(os.path.abspath(__file__))
GRID_CHECK = json.load(open(os.path.join(HERE, "golden", "iq3s_grid_check.json")))


def oracle_grid():
    return np.array([orc.iq3s_grid_entry(i) for i in range(512)], dtype="<u4")


def test_iq3s_grid_matches_the_reference_table_checksums():
    g = oracle_grid()
    assert g.size == GRID_CHECK["count"]
    assert zlib.crc32(g.tobytes()) == GRID_CHECK["crc32_le_bytes"]
    assert int(g.astype(np.uint64).sum()) == GRID_CHECK["sum"]
    assert int(np.bitwise_xor.reduce(g)) == GRID_CHECK["xor"]
    by = g.view(np.uint8)
    assert {str(v): int((by == v).sum()) for v in range(1, 16, 2)} == GRID_CHECK["byte_histogram"]
    assert bool(np.all(np.diff(g.astype(np.int64)) > 0)) == GRID_CHECK["strictly_increasing"]
    for i, v in GRID_CHECK["entries_at"].items():
        assert int(g[int(i)]) == v


def iq3s_block(d=1.0, qs=None, qh=None, signs=None, scales=None):
    b = np.zeros(110, np.uint8)
    b[0:2] = np.frombuffer(np.float16(d).tobytes(), np.uint8)
    if qs is not None:
        b[2:66] = qs
    if qh is not None:
        b[66:74] = qh
    if signs is not None:
        b[74:106] = signs
    if scales is not None:
        b[106:110] = scales
    return b


def test_iq3s_closed_forms():
    # all-zero payload: index 0 everywhere -> grid entry 0 = (1,1,1,1), scale nibble 0 -> db = d
    assert np.all(orc.dequantize_to_f32(orc.IQ3_S, iq3s_block(0.5), 256) == 0.5)
    # db = d * (1 + 2 * nibble): byte p of scales holds sub-blocks 2p (low) and 2p+1 (high)
    out = orc.dequantize_to_f32(orc.IQ3_S, iq3s_block(1.0, scales=[0x10, 0x32, 0x54, 0xF6]), 256).reshape(8, 32)
    assert [float(out[s, 0]) for s in range(8)] == [1 + 2 * n for n in (0, 1, 2, 3, 4, 5, 6, 15)]
    # sign bit j of sign byte l flips weight 8l + j (of the sub-block the byte belongs to)
    signs = np.zeros(32, np.uint8)
    signs[0] = 0x01
    signs[1] = 0x80
    signs[4 * 3 + 2] = 0x10
    out = orc.dequantize_to_f32(orc.IQ3_S, iq3s_block(1.0, signs=signs), 256)
    neg = np.flatnonzero(out < 0).tolist()
    assert neg == [0, 15, 3 * 32 + 2 * 8 + 4]
    # index byte i of a sub-block covers weights 4i..4i+3, weight 0 in the low byte of the entry;
    # bit i of the sub-block's qh byte is the index's 9th bit
    g = oracle_grid()
    qs = np.zeros(64, np.uint8)
    qh = np.zeros(8, np.uint8)
    qs[8 * 2 + 5] = 200                   # sub-block 2, index 5 -> weights 20..23
    qs[8 * 7 + 0] = 255
    qh[7] = 0x01                          # sub-block 7, index 0 -> entry 511
    qh[1] = 0x08                          # sub-block 1, index 3 -> entry 256
    out = orc.dequantize_to_f32(orc.IQ3_S, iq3s_block(1.0, qs=qs, qh=qh), 256).reshape(8, 32)
    assert out[2, 20:24].tolist() == [float(x) for x in np.array([g[200]], "<u4").view(np.uint8)]
    assert out[7, 0:4].tolist() == [float(x) for x in np.array([g[511]], "<u4").view(np.uint8)]
    assert out[1, 12:16].tolist() == [float(x) for x in np.array([g[256]], "<u4").view(np.uint8)]
    assert out[1, 12:16].tolist() == [7.0, 5.0, 9.0, 5.0]          # 0x05090507 read low byte first
    assert np.all(out[0] == 1.0) and np.all(out[2, :20] == 1.0)


def test_iq3s_repack_matches_direct_dequant_reference_test():     # iq3_s.rs:217-258
    in_dim, out_dim = 512, 3
    n_blocks = in_dim // 256
    nsp = orc.repacked_n_sub_padded(in_dim)
    assert nsp == 17
    rng = Lcg(0x1A350000, inc=1)
    raw = np.zeros(out_dim * n_blocks * 110, np.uint8)
    for b in range(out_dim * n_blocks):
        d = np.float32(10.0) ** (b % 4 - 2) * (np.float32(1.0) + np.float32(b) / np.float32(48.0))
        raw[b * 110:b * 110 + 2] = np.frombuffer(np.float16(d).tobytes(), np.uint8)
        raw[b * 110 + 2:(b + 1) * 110] = rng.bytes(108)
    direct = orc.dequantize_to_f32(orc.IQ3_S, raw, out_dim * in_dim).reshape(out_dim, in_dim)
    packed = orc.repack_for_matvec(orc.IQ3_S, raw, in_dim, out_dim)
    assert packed.size == orc.repacked_len(orc.IQ3_S, in_dim, out_dim) == out_dim * nsp * 18
    kv = np.arange(16) * 2 - 15                                    # KVALUES_IQ3S, iq3_s.rs:161-162
    nib_len = out_dim * nsp * 16
    max_rel = 0.0
    for row in range(out_dim):
        for sb in range(in_dim // 32):
            nib = packed[(row * nsp + sb) * 16:][:16]
            db = np.float32(packed[nib_len + (row * nsp + sb) * 2:][:2].copy().view(np.float16)[0])
            lo = db * kv[nib & 0x0F].astype(np.float32)
            hi = db * kv[nib >> 4].astype(np.float32)
            a = direct[row, sb * 32:sb * 32 + 16]
            b = direct[row, sb * 32 + 16:sb * 32 + 32]
            max_rel = max(max_rel, float(np.max(np.abs(lo - a) / np.maximum(np.abs(a), 1e-30))),
                          float(np.max(np.abs(hi - b) / np.maximum(np.abs(b), 1e-30))))
    assert max_rel < 5e-4
    # the oracle's own plane reader agrees with that reading
    dec = orc.decode_repacked_to_f32(orc.IQ3_S, packed, in_dim, out_dim)
    assert np.max(np.abs(dec - direct) / np.maximum(np.abs(direct), 1e-30)) < 5e-4
    # the codebook words the reference's kernel_source emits (iq3_s.rs:259-261)
    words = kv.astype(np.int8).view("<u4")
    assert int(words[0]) == 0xF7F5F3F1 and int(words[3]) == 0x0F0D0B09


def q5_1_block(d, m, qh, qs):
    b = np.zeros(24, np.uint8)
    b[0:2] = np.frombuffer(np.float16(d).tobytes(), np.uint8)
    b[2:4] = np.frombuffer(np.float16(m).tobytes(), np.uint8)
    b[4:8] = np.frombuffer(np.uint32(qh).tobytes(), np.uint8)
    b[8:24] = qs
    return b


def test_q5_1_closed_forms():
    # w = d*q5 + m; byte k: weight k low nibble, weight k+16 high nibble; qh bit i = 5th bit of weight i
    out = orc.dequantize_to_f32(orc.Q5_1, q5_1_block(2.0, -3.0, 0, np.zeros(16, np.uint8)), 32)
    assert np.all(out == -3.0)
    qs = np.zeros(16, np.uint8)
    qs[5] = 0xA7
    out = orc.dequantize_to_f32(orc.Q5_1, q5_1_block(0.5, 1.0, (1 << 5) | (1 << 30), qs), 32)
    want = np.full(32, 1.0, np.float32)
    want[5] = 0.5 * (7 + 16) + 1.0
    want[21] = 0.5 * 10 + 1.0
    want[30] = 0.5 * 16 + 1.0
    assert np.array_equal(out, want)
    assert orc.block_size(orc.Q5_1) == 32 and orc.bytes_per_block(orc.Q5_1) == 24
    assert orc.block_size(orc.IQ3_S) == 256 and orc.bytes_per_block(orc.IQ3_S) == 110


def test_q5_1_repack_is_bit_exact_reference_test():                # q5_1.rs:111-157
    in_dim, out_dim = 256, 5
    n_sub = in_dim // 32
    nsp = orc.repacked_n_sub_padded(in_dim)
    assert nsp == 9
    rng = Lcg(0x05100001, inc=1)
    raw = np.zeros(out_dim * n_sub * 24, np.uint8)
    for b in range(out_dim * n_sub):
        d = np.float32(0.01) * (np.float32(b) + np.float32(1.0))
        m = np.float32(-0.1) * np.float32(b % 7)
        raw[b * 24:b * 24 + 2] = np.frombuffer(np.float16(d).tobytes(), np.uint8)
        raw[b * 24 + 2:b * 24 + 4] = np.frombuffer(np.float16(m).tobytes(), np.uint8)
        raw[b * 24 + 4:(b + 1) * 24] = rng.bytes(20)
    direct = orc.dequantize_to_f32(orc.Q5_1, raw, out_dim * in_dim).reshape(out_dim, in_dim)
    packed = orc.repack_for_matvec(orc.Q5_1, raw, in_dim, out_dim)
    nib_len, qh_len = out_dim * nsp * 16, out_dim * nsp * 4
    assert packed.size == nib_len + qh_len + out_dim * nsp * 4 == orc.repacked_len(orc.Q5_1, in_dim, out_dim)
    for row in range(out_dim):
        for sb in range(n_sub):
            i = row * nsp + sb
            nib = packed[i * 16:i * 16 + 16]
            qh = int(packed[nib_len + i * 4:][:4].copy().view("<u4")[0])
            dm = nib_len + qh_len + i * 4
            dsc = np.float32(packed[dm:dm + 2].copy().view(np.float16)[0])
            deff = -np.float32(packed[dm + 2:dm + 4].copy().view(np.float16)[0])
            for w in range(32):
                g, b = w // 4, w % 4
                byte = int(nib[(g // 2) * 4 + b])
                n = byte & 0x0F if g % 2 == 0 else byte >> 4
                q5 = n | (((qh >> (4 * g + b)) & 1) << 4)
                widx = (g // 2) * 4 + b if g % 2 == 0 else 16 + (g // 2) * 4 + b
                assert dsc * np.float32(q5) - deff == direct[row, sb * 32 + widx], (row, sb, widx)
    assert np.array_equal(orc.decode_repacked_to_f32(orc.Q5_1, packed, in_dim, out_dim), direct)


@pytest.mark.parametrize("fmt", [orc.Q5_1, orc.IQ3_S])
def test_int8_path_equals_decoded_planes_times_dequantized_activation(fmt):
    """sum_k w_k * (dx * q_k) from the decoded planes, in float64, against the oracle's
    int8 matvec; Q5_1's minimum rides on the fp32 block sum like Q5_K's."""
    in_dim, out_dim = 768, 6
    rng = np.random.default_rng(fmt)
    bb, bs = orc.bytes_per_block(fmt), orc.block_size(fmt)
    raw = rng.integers(0, 256, out_dim * in_dim // bs * bb, dtype=np.uint8)
    for blk in range(out_dim * in_dim // bs):                      # finite fp16 scales
        raw[blk * bb:blk * bb + 2] = np.frombuffer(np.float16(rng.uniform(0.01, 0.1)).tobytes(), np.uint8)
        if fmt == orc.Q5_1:
            raw[blk * bb + 2:blk * bb + 4] = np.frombuffer(np.float16(rng.uniform(-0.5, 0.5)).tobytes(), np.uint8)
    packed = orc.repack_for_matvec(fmt, raw, in_dim, out_dim)
    w = orc.decode_repacked_to_f32(fmt, packed, in_dim, out_dim).astype(np.float64)
    x = rng.standard_normal(in_dim).astype(np.float32)
    xq = orc.quantize_q8(x)
    blocks = xq.reshape(-1, 40)
    dx = blocks[:, 0:4].copy().view(np.float32)[:, 0].astype(np.float64)
    q = blocks[:, 8:40].copy().view(np.int8).astype(np.float64)
    xsum = blocks[:, 4:8].copy().view(np.float32)[:, 0].astype(np.float64)
    y = orc.matvec_q8(fmt, packed, in_dim, out_dim, xq)
    if fmt == orc.Q5_1:
        # the kernels use the fp32 block sum for the minimum term: w = d*q5 + m -> d*dx*idot + m*xsum
        nsp = orc.repacked_n_sub_padded(in_dim)
        dmp = packed[out_dim * nsp * 20:].reshape(out_dim, nsp, 4)
        d = dmp[:, :in_dim // 32, 0:2].copy().view(np.float16)[..., 0].astype(np.float64)
        m = dmp[:, :in_dim // 32, 2:4].copy().view(np.float16)[..., 0].astype(np.float64)
        wq = (w.reshape(out_dim, -1, 32) - m[..., None]) / d[..., None]
        want = (d * dx[None] * np.einsum("rsk,sk->rs", wq, q) + m * xsum[None]).sum(1)
    else:
        want = (w.reshape(out_dim, -1, 32) * (dx[:, None] * q)[None]).sum((1, 2))
    assert np.allclose(y, want, rtol=2e-5, atol=2e-5)
