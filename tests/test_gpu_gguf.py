"""File to kernel: tensors of a GGUF container written here go through the library's reader
and load path (mapping -> repacked slab -> device) and run on the kernels their type lands
on; the expected outputs come from the oracle working on the raw tensor bytes."""
import numpy as np
import pytest

import reinstinct_amd as rein
from reinstinct_amd import gguf, hip, quant, runtime
from reinstinct_amd._lib import init
from oracle import orc
from helpers import GGUF_STRING, GGUF_U32, assert_close_f32, random_raw_weights, rel_l2, write_gguf

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def gpu():
    init()
    hip.set_device(0)
    yield
    hip.synchronize()


from helpers import dev  # noqa: E402  (uploads that stay alive until the test's last launch has finished)


def q3k_raw(n_blocks, seed):
    rng = np.random.default_rng(seed)
    raw = rng.integers(0, 256, (n_blocks, 110), dtype=np.uint8)
    raw[:, 108:110] = np.frombuffer(np.float16(0.004).tobytes(), np.uint8)
    return raw.reshape(-1)


def test_dense_tensors_from_a_file_run_on_their_kernels(tmp_path):
    in_dim, out_dim = 1024, 136
    tensors, raws = [], {}
    for name, ty in (("q4_0", 2), ("q8_0", 8), ("q4_k", 12), ("q5_k", 13), ("q6_k", 14), ("iq4_xs", 23), ("iq3_s", 21)):
        raws[name] = (ty, random_raw_weights(ty, in_dim, out_dim, seed=ty))
    raws["q3_k"] = (11, q3k_raw(in_dim * out_dim // 256, 5))
    nl = random_raw_weights(rein.Q4_0, in_dim, out_dim, seed=9)          # IQ4_NL blocks have Q4_0's shape
    raws["iq4_nl"] = (20, nl)
    bf = (np.random.default_rng(3).standard_normal(in_dim * out_dim).astype(np.float32) * 0.02).view(np.uint32) >> 16
    raws["bf16"] = (30, bf.astype(np.uint16).view(np.uint8))
    for name, (ty, raw) in raws.items():
        tensors.append((f"blk.0.{name}.weight", [in_dim, out_dim], ty, raw.tobytes()))
    data, _ = write_gguf([("general.architecture", GGUF_STRING, "qwen35"), ("qwen35.block_count", GGUF_U32, 1)], tensors)
    path = tmp_path / "model.gguf"
    path.write_bytes(data)

    x = np.random.default_rng(1).standard_normal((3, in_dim)).astype(np.float32)
    xq = orc.quantize_q8(x)
    dq = dev(xq)
    with gguf.GgufFile.open(path) as g:
        assert g.metadata_get("general.architecture") == "qwen35" and g.as_u64("qwen35.block_count") == 1
        for name, (ty, raw) in raws.items():
            print("gguf tensor", name, flush=True)
            slab, fmt, dims = g.load_for_matvec(f"blk.0.{name}.weight")
            assert (dims["in_dim"], dims["out_dim"], dims["n_expert"]) == (in_dim, out_dim, 1)
            dw = dev(slab)
            for n_rows in (1, 3):
                dy = dev(np.full(n_rows * out_dim, np.nan, np.float32))
                if n_rows == 1:
                    runtime.matvec_xq8(fmt, dw, dq, dy, in_dim, out_dim)
                else:
                    runtime.matvec_batched_xq8(fmt, dw, dq, dy, in_dim, out_dim, n_rows)
                hip.synchronize()
                got = dy.to_host(np.float32).reshape(n_rows, out_dim)
                # the oracle from the raw tensor bytes: its own repack of the landing format, int8 path
                if ty in (2, 8, 12, 13, 14, 23, 21):
                    want = orc.matvec_q8(ty, orc.repack_for_matvec(ty, raw, in_dim, out_dim), in_dim, out_dim,
                                         xq[:n_rows * (in_dim // 32) * 40], n_rows)
                    assert_close_f32(got, want, what=name)
                # and the reference's CPU path: dequantize the on-disk bytes, f32 matvec (rel_l2 bar of kernels.rs:1598-1601)
                if ty == 11:
                    w = orc.q3_k_dequantize(raw, in_dim * out_dim)
                elif ty == 20:
                    w = orc.iq4_nl_dequantize(raw, in_dim * out_dim)
                elif ty == 30:
                    w = orc.bf16_to_f32(raw.view(np.uint16))
                else:
                    w = orc.dequantize_to_f32(ty, raw, in_dim * out_dim)
                ref = x[:n_rows].astype(np.float64) @ w.reshape(out_dim, in_dim).astype(np.float64).T
                assert rel_l2(got, ref.astype(np.float32)) < 1.5e-2, name


def test_expert_tensors_from_a_file_run_the_moe_decode_kernels(tmp_path):
    in_dim, out_dim, n_expert, n_used = 512, 64, 6, 3
    tensors, raws = [], {}
    for name, ty in (("q4_k", 12), ("q5_k", 13), ("q6_k", 14), ("q8_0", 8), ("q5_1", 7)):
        ex = [random_raw_weights(ty, in_dim, out_dim, seed=ty * 10 + e) for e in range(n_expert)]
        raws[name] = (ty, ex)
        tensors.append((f"blk.1.ffn_{name}_exps.weight", [in_dim, out_dim, n_expert], ty, b"".join(r.tobytes() for r in ex)))
    data, _ = write_gguf([], tensors)
    path = tmp_path / "moe.gguf"
    path.write_bytes(data)
    rng = np.random.default_rng(2)
    ids = rng.permutation(n_expert)[:n_used].astype(np.int32)[None, :]
    xq = orc.quantize_q8(rng.standard_normal((1, in_dim)).astype(np.float32))
    with gguf.GgufFile.open(path) as g:
        for name, (ty, ex) in raws.items():
            print("gguf expert tensor", name, flush=True)
            slab, fmt, dims = g.load_for_matvec(f"blk.1.ffn_{name}_exps.weight")
            assert fmt == ty and dims["n_expert"] == n_expert
            dy = dev(np.full(n_used * out_dim, np.nan, np.float32))
            runtime.moe_expert_matvec(fmt, dev(slab), dev(ids), dev(xq), dy, in_dim, out_dim, dims["bytes_per_expert"],
                                      in_dim // 32, 0, n_used, 1)
            hip.synchronize()
            got = dy.to_host(np.float32).reshape(n_used, out_dim)
            for s in range(n_used):
                e = int(ids[0, s])
                want = orc.matvec_q8(ty, orc.repack_for_matvec(ty, ex[e], in_dim, out_dim), in_dim, out_dim, xq, 1)[0]
                assert_close_f32(got[s], want, what=f"{name} expert {e}")
