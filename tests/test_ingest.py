"""Load-time ingestion of GGUF tensor bytes (CPU): the relabelled types of
GpuMatvecTensor::from_bytes_matvec (src/runtime/qwen35.rs:251-331) against the
reference's own unit-test statements — the relabel is exact, so
decode(ingest(bytes)) == dequantize(bytes) bit for bit."""
import numpy as np
import pytest

import reinstinct_amd as rein
from reinstinct_amd import quant
from oracle import orc
from helpers import Lcg


def q3k_blocks(n_blocks, seed):
    # src/quant/q3_k.rs:199-211: random bytes, tame fp16 d
    g = Lcg(seed, inc=1)
    raw = g.bytes(n_blocks * 110).reshape(n_blocks, 110)
    for b in range(n_blocks):
        h = orc.f32_to_f16(np.float32(0.02 * (1.0 + b / 32.0)))
        raw[b, 108], raw[b, 109] = h & 0xFF, h >> 8
    return raw.reshape(-1)


def test_q3k_scale_unpack_and_zero_factor_block():
    # src/quant/q3_k.rs:176-191: sixteen scales of 32 are bytes 0..7 = 0, 8..11 = 0xAA; the
    # factor (32 - 32) makes the block dequantize to zeros whatever the quants are
    blk = np.full(110, 0xA5, np.uint8)
    blk[96:104], blk[104:108] = 0, 0xAA
    h = orc.f32_to_f16(np.float32(1.0))
    blk[108], blk[109] = h & 0xFF, h >> 8
    assert np.all(orc.q3_k_dequantize(blk, 256) == 0)
    q6 = quant.transcode_q3_k_to_q6_k(blk, 256)
    assert np.all(q6[192:208].view(np.int8) == 0)          # sc6 = sc3 - 32
    assert np.all(orc.dequantize_to_f32(rein.Q6_K, q6, 256) == 0)


def test_q3k_closed_form_single_weight():
    # one sub-block scale 33 (factor +1), every stored quant 0 except weight 0 = 7: w0 = d*(7-4),
    # the rest of the sub-block d*(0-4)
    blk = np.zeros(110, np.uint8)
    blk[96:104], blk[104:108] = 0, 0xAA                   # all scales 32
    blk[96] = 1                                            # scale 0 -> 33
    blk[32] = 3                                            # qs: weight 0 low bits = 3
    blk[0] = 1                                             # hmask: weight 0, level 0 -> third bit set
    h = orc.f32_to_f16(np.float32(0.5))
    blk[108], blk[109] = h & 0xFF, h >> 8
    w = orc.q3_k_dequantize(blk, 256)
    assert w[0] == 0.5 * 3 and np.all(w[1:16] == 0.5 * -4) and np.all(w[16:] == 0)


@pytest.mark.parametrize("n_blocks", [1, 32])
def test_q3k_transcode_to_q6k_is_bit_exact(n_blocks):
    # src/quant/q3_k.rs:193-213
    raw = q3k_blocks(n_blocks, 0x0A3E0000)
    q6 = quant.transcode_q3_k_to_q6_k(raw, n_blocks * 256)
    direct = orc.q3_k_dequantize(raw, n_blocks * 256)
    via = orc.dequantize_to_f32(rein.Q6_K, q6, n_blocks * 256)
    assert np.array_equal(direct.view(np.uint32), via.view(np.uint32))
    assert np.any(direct != 0)
    # every transcoded quant lies in 28..35 and every scale in -32..31
    assert np.all((q6.reshape(n_blocks, 210)[:, 192:208].view(np.int8) >= -32))
    assert np.all((q6.reshape(n_blocks, 210)[:, 192:208].view(np.int8) <= 31))


def test_ingest_q3k_lands_on_q6k_planes():
    in_dim, out_dim = 512, 6
    raw = q3k_blocks(in_dim * out_dim // 256, 77)
    slab, fmt = quant.ingest_for_matvec(quant.GGML_Q3_K, raw, in_dim, out_dim)
    assert fmt == rein.Q6_K and slab.size == quant.repacked_len(rein.Q6_K, in_dim, out_dim)
    got = orc.decode_repacked_to_f32(rein.Q6_K, slab, in_dim, out_dim)
    assert np.array_equal(got.reshape(-1).view(np.uint32), orc.q3_k_dequantize(raw, in_dim * out_dim).view(np.uint32))


def test_ingest_iq4_nl_runs_as_iq4_xs():
    # src/quant/iq4_nl.rs:79-118: in_dim 128 -> 4 sub-blocks, a power of two -> nsp = 5
    in_dim, out_dim = 128, 3
    g = Lcg(0x1A4A1000, inc=1)
    raw = g.bytes(out_dim * 4 * 18).reshape(-1, 18)
    for b in range(raw.shape[0]):
        h = orc.f32_to_f16(np.float32(0.01 * (b - 5.0)))
        raw[b, 0], raw[b, 1] = h & 0xFF, h >> 8
    slab, fmt = quant.ingest_for_matvec(quant.GGML_IQ4_NL, raw.reshape(-1), in_dim, out_dim)
    assert fmt == rein.IQ4_XS and quant.repacked_n_sub_padded(in_dim) == 5
    assert slab.size == out_dim * 5 * 18
    got = orc.decode_repacked_to_f32(rein.IQ4_XS, slab, in_dim, out_dim)
    want = orc.iq4_nl_dequantize(raw.reshape(-1), in_dim * out_dim)
    assert np.array_equal(got.reshape(-1).view(np.uint32), want.view(np.uint32))


def test_ingest_bf16_requantizes_to_q8_0():
    # src/quant/half.rs:120-128 values, then q8_0::quantize_from_f32 (q8_0.rs:45-61)
    vals = np.array([1.0, -1.0, 0.0, 256.0, -0.5], np.float32)
    bits = (vals.view(np.uint32) >> 16).astype(np.uint16)
    assert np.array_equal(orc.bf16_to_f32(bits), vals)
    in_dim, out_dim = 64, 4
    w = (np.random.default_rng(1).standard_normal(in_dim * out_dim) * 0.05).astype(np.float32)
    bf = (w.view(np.uint32) >> 16).astype(np.uint16)                     # truncation to bf16
    slab, fmt = quant.ingest_for_matvec(quant.GGML_BF16, bf.view(np.uint8), in_dim, out_dim)
    assert fmt == rein.Q8_0
    widened = orc.bf16_to_f32(bf)
    want = orc.repack_for_matvec(rein.Q8_0, orc.q8_0_quantize_from_f32(widened), in_dim, out_dim)
    assert np.array_equal(slab, want)
    got = orc.decode_repacked_to_f32(rein.Q8_0, slab, in_dim, out_dim).reshape(-1)
    assert np.max(np.abs(got - widened)) <= np.max(np.abs(widened)) / 254 * 1.01   # half a Q8_0 step


@pytest.mark.parametrize("fmt", [rein.Q4_0, rein.Q8_0, rein.Q4_K, rein.Q5_K, rein.Q6_K, rein.IQ4_XS])
def test_ingest_native_formats_is_the_repack(fmt):
    from helpers import random_raw_weights
    in_dim, out_dim = 512, 5
    raw = random_raw_weights(fmt, in_dim, out_dim, seed=fmt)
    slab, label = quant.ingest_for_matvec(fmt, raw, in_dim, out_dim)
    assert label == fmt and np.array_equal(slab, orc.repack_for_matvec(fmt, raw, in_dim, out_dim))


def test_ingest_errors():
    with pytest.raises(rein.ReinError) as e:
        quant.ingest_for_matvec(7, np.zeros(24, np.uint8), 32, 1)          # Q5_1: no layout here
    assert e.value.code == -2 and "Q3_K" in str(e.value)
    with pytest.raises(rein.ReinError) as e:
        quant.ingest_for_matvec(quant.GGML_Q3_K, np.zeros(110, np.uint8), 128, 2)
    assert e.value.code == -3
