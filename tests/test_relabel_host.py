"""Host side of the two relabelled formats (Q5_1 on the Q5_K kernels, IQ3_S on the IQ4_XS
kernels): the product's repack against the oracle's byte for byte, the ingestion labels,
the GGUF load path and the dispatch rules (Q5_1 experts only, IQ3_S dense only)."""
import numpy as np
import pytest

import reinstinct_amd as rein
from reinstinct_amd import _lib, gguf, quant
from oracle import orc
from helpers import random_raw_weights, write_gguf


def test_format_ids_and_geometry():                     # src/gguf/types.rs:41,52,64-66,77,88
    assert (rein.Q5_1, rein.IQ3_S) == (7, 21) == (orc.Q5_1, orc.IQ3_S)
    for fmt, bs, bb in ((rein.Q5_1, 32, 24), (rein.IQ3_S, 256, 110)):
        assert quant.block_size(fmt) == bs == orc.block_size(fmt)
        assert quant.bytes_per_block(fmt) == bb == orc.bytes_per_block(fmt)


@pytest.mark.parametrize("fmt,in_dim,out_dim", [(rein.Q5_1, 256, 5), (rein.Q5_1, 32, 3), (rein.Q5_1, 352, 8), (rein.Q5_1, 2048, 16),
                                                (rein.IQ3_S, 256, 1), (rein.IQ3_S, 512, 3), (rein.IQ3_S, 768, 5),
                                                (rein.IQ3_S, 5120, 4)])
def test_repack_matches_oracle_bytes(fmt, in_dim, out_dim):
    raw = random_raw_weights(fmt, in_dim, out_dim, seed=fmt + in_dim)
    got = quant.repack_for_matvec(fmt, raw, in_dim, out_dim)
    want = orc.repack_for_matvec(fmt, raw, in_dim, out_dim)
    assert quant.repacked_len(fmt, in_dim, out_dim) == want.size == orc.repacked_len(fmt, in_dim, out_dim)
    assert np.array_equal(got, want)


def test_iq3s_repack_reaches_every_grid_entry():
    # 512 grid entries x both signs of each weight, all through the product's packed table
    in_dim, out_dim = 256, 128
    raw = np.zeros((out_dim, 110), np.uint8)
    raw[:, 0:2] = np.frombuffer(np.float16(0.25).tobytes(), np.uint8)
    idx = np.arange(out_dim * 64) % 512                  # index i of row r: entry (64 r + i) % 512
    raw[:, 2:66] = (idx & 0xFF).reshape(out_dim, 64)
    hi = (idx >> 8).reshape(out_dim, 8, 8)
    raw[:, 66:74] = (hi << np.arange(8)).sum(2)
    raw[:, 74:106] = np.random.default_rng(0).integers(0, 256, (out_dim, 32), dtype=np.uint8)
    raw = raw.reshape(-1)
    assert np.array_equal(quant.repack_for_matvec(rein.IQ3_S, raw, in_dim, out_dim),
                          orc.repack_for_matvec(orc.IQ3_S, raw, in_dim, out_dim))
    # and the decoded planes are the dequantized blocks (scale nibble 0: db = d, exactly an fp16)
    dec = orc.decode_repacked_to_f32(orc.IQ3_S, quant.repack_for_matvec(rein.IQ3_S, raw, in_dim, out_dim), in_dim, out_dim)
    assert np.array_equal(dec.reshape(-1), orc.dequantize_to_f32(orc.IQ3_S, raw, in_dim * out_dim))


def test_repack_threaded_path():
    for fmt, in_dim, out_dim in ((rein.IQ3_S, 4096, 1100), (rein.Q5_1, 4096, 1100)):
        raw = random_raw_weights(fmt, in_dim, out_dim, seed=5)
        assert np.array_equal(quant.repack_for_matvec(fmt, raw, in_dim, out_dim), orc.repack_for_matvec(fmt, raw, in_dim, out_dim))


def test_ingest_labels():                               # qwen35.rs:283-284 (dense), 415-425 (experts)
    lib = _lib.load()
    assert lib.rein_ingest_format(rein.IQ3_S) == rein.IQ3_S
    assert lib.rein_ingest_format(rein.Q5_1) == 0        # a dense Q5_1 tensor keeps its on-disk layout there
    assert [lib.rein_ingest_expert_format(t) for t in (12, 13, 14, 8, 7)] == [12, 13, 14, 8, 7]
    assert [lib.rein_ingest_expert_format(t) for t in (2, 23, 21, 20, 11, 30, 0, 99)] == [0] * 8
    raw = random_raw_weights(rein.IQ3_S, 512, 4, seed=1)
    slab, label = quant.ingest_for_matvec(rein.IQ3_S, raw, 512, 4)
    assert label == rein.IQ3_S and np.array_equal(slab, orc.repack_for_matvec(orc.IQ3_S, raw, 512, 4))
    with pytest.raises(rein.ReinError) as e:
        quant.ingest_for_matvec(rein.Q5_1, np.zeros(24 * 8, np.uint8), 64, 4)
    assert e.value.code == -2


def test_gguf_load_iq3s_dense_and_q5_1_experts():
    in_dim, out_dim, n_expert = 512, 16, 3
    iq = random_raw_weights(rein.IQ3_S, in_dim, out_dim, seed=2)
    ex = [random_raw_weights(rein.Q5_1, 352, out_dim, seed=10 + e) for e in range(n_expert)]
    q51_dense = random_raw_weights(rein.Q5_1, 64, 4, seed=3)
    data, _ = write_gguf([], [("blk.0.attn_q.weight", [in_dim, out_dim], 21, iq.tobytes()),
                              ("blk.0.ffn_down_exps.weight", [352, out_dim, n_expert], 7, b"".join(r.tobytes() for r in ex)),
                              ("dense_q5_1", [64, 4], 7, q51_dense.tobytes()),
                              ("iq3s_experts", [256, 8, 2], 21, bytes(110 * 16))])
    with gguf.GgufFile.from_bytes(data) as g:
        slab, label, dims = g.load_for_matvec("blk.0.attn_q.weight")
        assert label == rein.IQ3_S and np.array_equal(slab, orc.repack_for_matvec(orc.IQ3_S, iq, in_dim, out_dim))
        slab, label, dims = g.load_for_matvec("blk.0.ffn_down_exps.weight")
        per = orc.repacked_len(orc.Q5_1, 352, out_dim)
        assert label == rein.Q5_1 and dims["bytes_per_expert"] == per and dims["n_expert"] == n_expert
        for e in range(n_expert):
            assert np.array_equal(slab[e * per:(e + 1) * per], orc.repack_for_matvec(orc.Q5_1, ex[e], 352, out_dim))
        for name in ("dense_q5_1", "iq3s_experts"):      # neither site exists in the reference
            with pytest.raises(rein.ReinError) as err:
                g.load_for_matvec(name)
            assert err.value.code == -2, name


def test_dispatch_rules_without_a_gpu():
    lib = _lib.load()
    if lib.rein_is_loaded():
        pytest.skip("a GPU runtime is loaded in this process")
    # argument checks run before anything touches the device
    assert lib.rein_matvec_xq8(rein.Q5_1, 16, 16, 16, 256, 8, None) == -2
    assert b"expert kernels only" in lib.rein_last_error()
    assert lib.rein_mmq_xq8(rein.Q5_1, 16, 16, 16, 256, 8, 32, None) == -2
    assert lib.rein_matvec_xq8(rein.IQ3_S, 16, 16, 16, 256, 8, None) == -1          # accepted, then: no runtime
    assert lib.rein_matvec_xq8(rein.IQ3_S, 16, 16, 16, 288, 8, None) == -3          # 256-weight blocks
    assert lib.rein_moe_grouped_gemm(rein.IQ3_S, 16, 16, 16, 16, 1, 16, 16, 256, 8, 1, None) == -2
    assert lib.rein_moe_grouped_gemm(rein.Q5_1, 16, 16, 16, 16, 1, 16, 16, 96, 8, 1, None) == -1
    assert lib.rein_moe_grouped_gemm(rein.Q5_1, 16, 16, 16, 16, 1, 16, 16, 100, 8, 1, None) == -3
