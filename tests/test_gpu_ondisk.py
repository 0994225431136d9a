"""GPU parity of the matvec call sites outside the repacked path: the on-disk-layout
dp4a matvecs (tied token_embd / output matrix) and the split-K Q8_0 matvec.

The on-disk kernels read GGUF blocks as they are; the oracle works on the repacked
planes of the same blocks, so agreement also re-checks the block layouts of
src/quant/{q4_k,q5_k,q6_k,q8_0}.rs from the device side.  fp32 bar 1e-3 / 1e-4."""
import ctypes as C

import numpy as np
import pytest

import reinstinct_amd as rein
from reinstinct_amd import hip, quant, runtime
from reinstinct_amd._lib import init
from oracle import orc
from helpers import assert_close_f32, random_raw_weights, rel_l2

pytestmark = pytest.mark.gpu
FMTS = [rein.Q4_K, rein.Q5_K, rein.Q6_K, rein.Q8_0]
KERNEL = {rein.Q4_K: "matvec_q4_k_dp4a_f32", rein.Q5_K: "matvec_q5_k_dp4a_f32", rein.Q6_K: "matvec_q6_k_dp4a_f32",
          rein.Q8_0: "matvec_q8_0_dp4a_f32"}


@pytest.fixture(scope="module", autouse=True)
def gpu():
    init()
    hip.set_device(0)
    yield
    hip.synchronize()


from helpers import dev  # noqa: E402  (uploads that stay alive until the test's last launch has finished)


def gpu_quantize(x):
    n_vec, k = x.shape
    dq = hip.DeviceBuf(n_vec * (k // 32) * 40)
    runtime.quantize_q8(dev(x), dq, k, n_vec)
    hip.synchronize()
    return dq


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("in_dim,out_dim,gaussian", [(2048, 384, False), (5120, 1001, True), (256, 3, False), (4096, 64, True),
                                                     (17408, 9, False), (768, 2051, False)])
def test_ondisk_matvec_parity(fmt, in_dim, out_dim, gaussian):
    if gaussian:
        w = (np.random.default_rng(fmt + in_dim).standard_normal((out_dim, in_dim)) * 0.02).astype(np.float32)
        raw = quant.quantize_weights(fmt, w)
    else:
        raw = random_raw_weights(fmt, in_dim, out_dim, seed=fmt + out_dim)
    x = np.random.default_rng(in_dim).standard_normal((1, in_dim)).astype(np.float32)
    dq = gpu_quantize(x)
    dy = dev(np.full(out_dim, np.nan, np.float32))
    runtime.matvec_ondisk_xq8(fmt, dev(raw), dq, dy, in_dim, out_dim)
    hip.synchronize()
    got = dy.to_host(np.float32)
    packed = orc.repack_for_matvec(fmt, raw, in_dim, out_dim)
    xq = dq.to_host(np.uint8)
    assert_close_f32(got, orc.matvec_q8(fmt, packed, in_dim, out_dim, xq, 1)[0], what=f"on-disk fmt {fmt}")
    # and the reference's own bar against its CPU path: dequantize -> f32 matvec
    wf = orc.dequantize_to_f32(fmt, raw, in_dim * out_dim).reshape(out_dim, in_dim)
    if out_dim >= 64:
        assert rel_l2(got, orc.matvec_f32(x[0], wf)) < (5e-2 if gaussian and fmt in (rein.Q4_K, rein.Q5_K) else 1.5e-2)
    # the repacked kernel on the same weights gives the same numbers to rounding
    dy2 = dev(np.zeros(out_dim, np.float32))
    runtime.matvec_xq8(fmt, dev(packed), dq, dy2, in_dim, out_dim)
    hip.synchronize()
    assert_close_f32(got, dy2.to_host(np.float32), rel=1e-5, abs_=1e-6, what="on-disk vs repacked kernel")


@pytest.mark.parametrize("in_dim,out_dim", [(32, 1), (96, 5), (352, 7), (2080, 3), (4128, 130)])
def test_ondisk_q8_0_rows_that_are_not_multiples_of_16_bytes(in_dim, out_dim):
    # 34-byte blocks: rows start at 2-byte alignment and the matrix ends inside a 16-byte piece
    fmt = rein.Q8_0
    raw = random_raw_weights(fmt, in_dim, out_dim, seed=in_dim)
    x = np.random.default_rng(in_dim).standard_normal((1, in_dim)).astype(np.float32)
    dq = gpu_quantize(x)
    dy = dev(np.full(out_dim, np.nan, np.float32))
    runtime.matvec_ondisk_xq8(fmt, dev(raw), dq, dy, in_dim, out_dim)
    hip.synchronize()
    packed = orc.repack_for_matvec(fmt, raw, in_dim, out_dim)
    assert_close_f32(dy.to_host(np.float32), orc.matvec_q8(fmt, packed, in_dim, out_dim, dq.to_host(np.uint8), 1)[0], what="Q8_0 ragged rows")


@pytest.mark.parametrize("fmt", FMTS)
def test_ondisk_reference_symbols_and_geometry(fmt):
    # Q4_K: 256 threads, 8 rows per workgroup; the others 64 threads, 2 rows (qwen35.rs:2217-2226)
    in_dim, out_dim = 1024, 77
    raw = random_raw_weights(fmt, in_dim, out_dim, seed=9)
    x = np.random.default_rng(1).standard_normal((1, in_dim)).astype(np.float32)
    dq, d_raw = gpu_quantize(x), dev(raw)
    dy = dev(np.full(out_dim, np.nan, np.float32))
    rows, block = (8, 256) if fmt == rein.Q4_K else (2, 64)
    args = [C.c_void_p(d_raw.ptr), C.c_void_p(dq.ptr), C.c_void_p(dy.ptr), C.c_uint(in_dim), C.c_uint(out_dim)]
    hip.Module.builtin().function(KERNEL[fmt]).launch(((out_dim + rows - 1) // rows, 1, 1), (block, 1, 1), 0, None, args)
    hip.synchronize()
    packed = orc.repack_for_matvec(fmt, raw, in_dim, out_dim)
    assert_close_f32(dy.to_host(np.float32), orc.matvec_q8(fmt, packed, in_dim, out_dim, dq.to_host(np.uint8), 1)[0],
                     what=KERNEL[fmt])


@pytest.mark.parametrize("in_dim,out_dim,n_split", [(5120, 96, 8), (5120, 96, 3), (2048, 7, 4), (256, 33, 16), (1024, 64, 1)])
def test_q8_0_splitk(in_dim, out_dim, n_split):
    fmt = rein.Q8_0
    raw = random_raw_weights(fmt, in_dim, out_dim, seed=in_dim + n_split)
    packed = quant.repack_for_matvec(fmt, raw, in_dim, out_dim)
    x = np.random.default_rng(2).standard_normal((1, in_dim)).astype(np.float32)
    dq = gpu_quantize(x)
    dy = dev(np.full((n_split, out_dim), np.nan, np.float32))
    runtime.matvec_q8_0_splitk(dev(packed), dq, dy, in_dim, out_dim, n_split)
    hip.synchronize()
    parts = dy.to_host(np.float32).reshape(n_split, out_dim)
    xq = dq.to_host(np.uint8).reshape(-1, 40)
    n_sub = in_dim // 32
    chunk = -(-n_sub // n_split)
    blocks = raw.reshape(out_dim, n_sub, 34)
    for p in range(n_split):
        lo, hi = p * chunk, min((p + 1) * chunk, n_sub)
        if lo >= hi:
            assert np.all(parts[p] == 0)
            continue
        sub = orc.repack_for_matvec(fmt, np.ascontiguousarray(blocks[:, lo:hi]).reshape(-1), (hi - lo) * 32, out_dim)
        want = orc.matvec_q8(fmt, sub, (hi - lo) * 32, out_dim, np.ascontiguousarray(xq[lo:hi]).reshape(-1), 1)[0]
        assert_close_f32(parts[p], want, what=f"split {p}")
    full = orc.matvec_q8(fmt, packed, in_dim, out_dim, dq.to_host(np.uint8), 1)[0]
    assert_close_f32(parts.sum(axis=0), full, what="sum of the partials")
    # the reference launch: one wavefront per row pair, grid.y = n_split
    dy2 = dev(np.full((n_split, out_dim), np.nan, np.float32))
    d_packed = dev(packed)
    args = [C.c_void_p(d_packed.ptr), C.c_void_p(dq.ptr), C.c_void_p(dy2.ptr), C.c_uint(in_dim), C.c_uint(out_dim), C.c_uint(n_split)]
    hip.Module.builtin().function("matvec_q8_0_repacked_splitk_f32").launch(((out_dim + 1) // 2, n_split, 1), (64, 1, 1), 0, None, args)
    hip.synchronize()
    assert np.array_equal(dy2.to_host(np.uint32), dy.to_host(np.uint32))


@pytest.mark.parametrize("ggml_type", ["q3_k", "iq4_nl", "bf16"])
def test_ingested_types_run_on_the_relabelled_kernels(ggml_type):
    # GGUF bytes of a type without kernels of its own -> rein_ingest_for_matvec -> decode matvec;
    # compared with the CPU path of the SOURCE format (dequantize -> f32 matvec, the reference's
    # rel_l2 < 1.5e-2 bar) and with the int8 oracle on the relabelled planes
    from helpers import Lcg
    in_dim, out_dim = 2048, 384
    n = in_dim * out_dim
    rng = np.random.default_rng(5)
    if ggml_type == "q3_k":
        raw = Lcg(0xD3A40001).bytes(n // 256 * 110).reshape(-1, 110)
        d = (((np.arange(raw.shape[0]) % 23) - 11) * 0.004).astype(np.float32).astype(np.float16).view(np.uint16)
        raw[:, 108], raw[:, 109] = d & 0xFF, d >> 8
        raw = raw.reshape(-1)
        wf = orc.q3_k_dequantize(raw, n)
        gg = quant.GGML_Q3_K
    elif ggml_type == "iq4_nl":
        raw = rng.integers(0, 256, (n // 32, 18), dtype=np.uint8)
        d = (((np.arange(raw.shape[0]) % 29) - 14) * 0.0003).astype(np.float32).astype(np.float16).view(np.uint16)
        raw[:, 0], raw[:, 1] = d & 0xFF, d >> 8
        raw = raw.reshape(-1)
        wf = orc.iq4_nl_dequantize(raw, n)
        gg = quant.GGML_IQ4_NL
    else:
        w = (rng.standard_normal(n) * 0.02).astype(np.float32)
        bits = (w.view(np.uint32) >> 16).astype(np.uint16)
        raw = bits.view(np.uint8)
        wf = orc.bf16_to_f32(bits)
        gg = quant.GGML_BF16
    slab, fmt = quant.ingest_for_matvec(gg, raw, in_dim, out_dim)
    x = (Lcg(0x13579BDF).acts(in_dim)).reshape(1, in_dim)
    dq = gpu_quantize(x)
    dy = dev(np.full(out_dim, np.nan, np.float32))
    runtime.matvec_xq8(fmt, dev(slab), dq, dy, in_dim, out_dim)
    hip.synchronize()
    got = dy.to_host(np.float32)
    assert_close_f32(got, orc.matvec_q8(fmt, slab, in_dim, out_dim, dq.to_host(np.uint8), 1)[0], what=ggml_type)
    assert rel_l2(got, orc.matvec_f32(x[0], wf.reshape(out_dim, in_dim))) < 1.5e-2
