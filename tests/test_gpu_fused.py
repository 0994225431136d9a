"""GPU parity of the fused BlockQ8 producers (the step in front of a quantized
matvec): rmsnorm_q8, add_rmsnorm_q8, swiglu_q8, sigmoid_mul_q8, rmsnorm_gated_q8,
moe_geglu_q8.  Through the C ABI and under the reference's own launch geometry.

Bar: BlockQ8 bytes and fp32 outputs bit-exact against the oracle (the device code
uses only correctly rounded operations in a fixed order, and the oracle restates
them); every BlockQ8 output equals quantize_q8 of the kernel's own fp32 output."""
import ctypes as C

import numpy as np
import pytest

import reinstinct_amd as rein
from reinstinct_amd import hip, runtime
from reinstinct_amd._lib import init
from oracle import orc

pytestmark = pytest.mark.gpu
EPS = 1e-6


@pytest.fixture(scope="module", autouse=True)
def gpu():
    init()
    hip.set_device(0)
    yield
    hip.synchronize()


from helpers import dev  # noqa: E402  (uploads that stay alive until the test's last launch has finished)


def blocks(n_values):
    return hip.DeviceBuf(n_values // 32 * 40)


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def gpu_q8_of(y):
    """quantize_q8 kernel on a host fp32 array -> bytes"""
    y = np.ascontiguousarray(y, np.float32).reshape(-1)
    dq = blocks(y.size)
    runtime.quantize_q8(dev(y), dq, y.size, 1)
    hip.synchronize()
    return dq.to_host(np.uint8)


@pytest.mark.parametrize("n,n_vec", [(5120, 1), (2048, 3), (8192, 2), (2816, 1), (32, 1), (96, 5), (32768, 1), (17408, 2)])
def test_rmsnorm_q8_bit_exact(n, n_vec):
    rng = np.random.default_rng(n + n_vec)
    x = (rng.standard_normal((n_vec, n)) * 3).astype(np.float32)
    w = (1 + 0.2 * rng.standard_normal(n)).astype(np.float32)
    dq = blocks(n_vec * n)
    runtime.rmsnorm_q8(dev(x), dev(w), dq, n, n_vec, EPS)
    hip.synchronize()
    _, y = orc.add_rmsnorm(x, None, w, EPS)
    assert np.array_equal(dq.to_host(np.uint8), orc.quantize_q8(y))


@pytest.mark.parametrize("n,n_vec,with_add,with_y", [(5120, 1, True, True), (5120, 1, False, True), (2048, 4, True, True),
                                                     (8192, 1, True, False), (1024, 2, False, False), (160, 3, True, True)])
def test_add_rmsnorm_q8_bit_exact(n, n_vec, with_add, with_y):
    rng = np.random.default_rng(n * 7 + n_vec)
    hidden = rng.standard_normal((n_vec, n)).astype(np.float32)
    add = rng.standard_normal((n_vec, n)).astype(np.float32) if with_add else None
    w = (1 + 0.2 * rng.standard_normal(n)).astype(np.float32)
    d_h, d_y, dq = dev(hidden), dev(np.full((n_vec, n), np.nan, np.float32)), blocks(n_vec * n)
    runtime.add_rmsnorm_q8(d_h, dev(add) if with_add else None, dev(w), d_y if with_y else None, dq, n, n_vec, EPS)
    hip.synchronize()
    want_h, want_y = orc.add_rmsnorm(hidden, add, w, EPS)
    assert np.array_equal(bits(d_h.to_host(np.float32)), bits(want_h).reshape(-1))
    got_q = dq.to_host(np.uint8)
    assert np.array_equal(got_q, orc.quantize_q8(want_y))
    if with_y:
        got_y = d_y.to_host(np.float32)
        assert np.array_equal(bits(got_y), bits(want_y).reshape(-1))
        assert np.array_equal(got_q, gpu_q8_of(got_y))            # fused == the two-kernel chain
    else:
        assert np.all(np.isnan(d_y.to_host(np.float32)))


def test_norm_zero_vector_and_eps():
    n = 256
    x = np.zeros((1, n), np.float32)
    dq = blocks(n)
    runtime.rmsnorm_q8(dev(x), dev(np.ones(n, np.float32)), dq, n, 1, EPS)
    hip.synchronize()
    b = dq.to_host(np.uint8).reshape(-1, 40)
    assert np.all(b[:, 8:] == 0) and np.all(b[:, :4].copy().view(np.float32) == 1.0) and np.all(b[:, 4:8] == 0)
    # eps matters when the vector is tiny
    x = np.full((1, n), 1e-4, np.float32)
    for eps in (1e-6, 1e-2):
        d_y = dev(np.zeros((1, n), np.float32))
        runtime.add_rmsnorm_q8(dev(x), None, dev(np.ones(n, np.float32)), d_y, blocks(n), n, 1, eps)
        hip.synchronize()
        assert np.array_equal(bits(d_y.to_host(np.float32)), bits(orc.add_rmsnorm(x, None, np.ones(n, np.float32), eps)[1]).reshape(-1))


@pytest.mark.parametrize("n", [32, 17408, 34816 * 3, 768 * 4096])
def test_swiglu_q8_bit_exact(n):
    rng = np.random.default_rng(n)
    gate, up = (rng.standard_normal(n) * 4).astype(np.float32), rng.standard_normal(n).astype(np.float32)
    gate[:8] = [0.0, -0.0, 100.0, -100.0, 1e-30, -1e30, 88.5, -87.5]
    d_out, dq = dev(np.zeros(n, np.float32)), blocks(n)
    runtime.swiglu_q8(dev(gate), dev(up), d_out, dq, n)
    hip.synchronize()
    want = orc.swiglu_det(gate, up)
    got = d_out.to_host(np.float32)
    assert np.array_equal(bits(got), bits(want))
    assert np.array_equal(dq.to_host(np.uint8), orc.quantize_q8(want.reshape(1, -1)))
    assert np.max(np.abs(got - orc.swiglu_mul(gate, up))) < 1e-5 * max(1.0, float(np.max(np.abs(got))))   # vs the libm form
    # in place (out aliases gate) and without the fp32 output
    d_g, dq2 = dev(gate), blocks(n)
    runtime.swiglu_q8(d_g, dev(up), d_g, dq2, n)
    dq3 = blocks(n)
    runtime.swiglu_q8(dev(gate), dev(up), None, dq3, n)
    hip.synchronize()
    assert np.array_equal(bits(d_g.to_host(np.float32)), bits(want))
    assert np.array_equal(dq2.to_host(np.uint8), dq.to_host(np.uint8))
    assert np.array_equal(dq3.to_host(np.uint8), dq.to_host(np.uint8))


def test_sigmoid_mul_q8_bit_exact():
    n = 6144
    rng = np.random.default_rng(3)
    x, gate = rng.standard_normal(n).astype(np.float32), (rng.standard_normal(n) * 5).astype(np.float32)
    d_x, dq = dev(x), blocks(n)
    runtime.sigmoid_mul_q8(d_x, dev(gate), dq, n)
    hip.synchronize()
    want = orc.sigmoid_mul_det(x, gate)
    assert np.array_equal(bits(d_x.to_host(np.float32)), bits(want))
    assert np.array_equal(dq.to_host(np.uint8), orc.quantize_q8(want.reshape(1, -1)))


@pytest.mark.parametrize("n_heads,head_dim", [(48, 128), (5, 64), (3, 2048), (1, 32)])
def test_rmsnorm_gated_q8_bit_exact(n_heads, head_dim):
    rng = np.random.default_rng(n_heads + head_dim)
    x = rng.standard_normal((n_heads, head_dim)).astype(np.float32)
    z = (rng.standard_normal((n_heads, head_dim)) * 2).astype(np.float32)
    w = (1 + 0.1 * rng.standard_normal(head_dim)).astype(np.float32)
    d_y, dq = dev(np.zeros((n_heads, head_dim), np.float32)), blocks(n_heads * head_dim)
    runtime.rmsnorm_gated_q8(dev(x), dev(z), dev(w), d_y, dq, n_heads, head_dim, EPS)
    hip.synchronize()
    want = orc.rmsnorm_gated(x, z, w, EPS)
    assert np.array_equal(bits(d_y.to_host(np.float32)), bits(want).reshape(-1))
    assert np.array_equal(dq.to_host(np.uint8), orc.quantize_q8(want.reshape(1, -1)))
    ref = np.stack([orc.rmsnorm_gated_ref(x[h], z[h], w, EPS) for h in range(n_heads)])
    assert np.max(np.abs(want - ref)) < 1e-5 * max(1.0, float(np.max(np.abs(ref))))


@pytest.mark.parametrize("ff,n_slot", [(768, 8), (704, 3), (32, 1), (2112, 64)])
def test_moe_geglu_q8_bit_exact(ff, n_slot):
    rng = np.random.default_rng(ff + n_slot)
    gu = (rng.standard_normal((n_slot, 2 * ff)) * 2).astype(np.float32)
    dq = blocks(n_slot * ff)
    runtime.moe_geglu_q8(dev(gu), dq, ff, n_slot)
    hip.synchronize()
    assert np.array_equal(dq.to_host(np.uint8), orc.quantize_q8(orc.geglu_det(gu)))


def test_reference_symbols_and_launch_geometry():
    # the unmodified reference host launches these by name with its own grids
    # (gemma4.rs:1303-1316, qwen35.rs:2036-2079, gemma4.rs:1781-1796)
    mod = hip.Module.builtin()
    rng = np.random.default_rng(9)
    u, f = C.c_uint, C.c_float
    keep = []                                   # device buffers must outlive the asynchronous launches

    def p(host_or_buf):
        buf = host_or_buf if isinstance(host_or_buf, hip.DeviceBuf) else dev(host_or_buf)
        keep.append(buf)
        return C.c_void_p(buf.ptr)

    n, n_vec = 2816, 2
    x, w = rng.standard_normal((n_vec, n)).astype(np.float32), rng.standard_normal(n).astype(np.float32)
    dq = blocks(n_vec * n)
    mod.function("rmsnorm_q8_f32").launch((1, n_vec, 1), (512, 1, 1), 512 * 4, None,
                                          [p(x), p(w), p(dq), u(n), f(EPS)])
    hip.synchronize()
    assert np.array_equal(dq.to_host(np.uint8), orc.quantize_q8(orc.add_rmsnorm(x, None, w, EPS)[1]))

    n = 5120
    h, a, w = (rng.standard_normal((1, n)).astype(np.float32) for _ in range(3))
    d_h, d_y, dq = dev(h), dev(np.zeros(n, np.float32)), blocks(n)
    mod.function("add_rmsnorm_q8_f32").launch((1, 1, 1), (1024, 1, 1), 0, None,
                                              [p(d_h), p(a), p(w), p(d_y), p(dq), u(n), f(EPS)])
    hip.synchronize()
    want_h, want_y = orc.add_rmsnorm(h, a, w[0], EPS)
    assert np.array_equal(bits(d_h.to_host(np.float32)), bits(want_h).reshape(-1))
    assert np.array_equal(bits(d_y.to_host(np.float32)), bits(want_y).reshape(-1))
    assert np.array_equal(dq.to_host(np.uint8), orc.quantize_q8(want_y))

    n = 17408
    g, up = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
    d_o, dq = dev(np.zeros(n, np.float32)), blocks(n)
    mod.function("swiglu_q8_f32").launch(((n + 255) // 256, 1, 1), (256, 1, 1), 0, None,
                                         [p(g), p(up), p(d_o), p(dq), u(n)])
    d_x, dq2 = dev(up), blocks(n)
    mod.function("sigmoid_mul_q8_f32").launch(((n + 255) // 256, 1, 1), (256, 1, 1), 0, None,
                                              [p(d_x), p(g), p(dq2), u(n)])
    hip.synchronize()
    assert np.array_equal(dq.to_host(np.uint8), orc.quantize_q8(orc.swiglu_det(g, up).reshape(1, -1)))
    assert np.array_equal(dq2.to_host(np.uint8), orc.quantize_q8(orc.sigmoid_mul_det(up, g).reshape(1, -1)))

    n_heads, hd = 48, 128
    x, z = (rng.standard_normal((n_heads, hd)).astype(np.float32) for _ in range(2))
    w = rng.standard_normal(hd).astype(np.float32)
    d_y, dq = dev(np.zeros(n_heads * hd, np.float32)), blocks(n_heads * hd)
    mod.function("rmsnorm_gated_q8_f32").launch((n_heads, 1, 1), (hd, 1, 1), (hd // 64) * 4, None,
                                                [p(x), p(z), p(w), p(d_y), p(dq),
                                                 u(n_heads), u(hd), f(EPS)])
    hip.synchronize()
    assert np.array_equal(dq.to_host(np.uint8), orc.quantize_q8(orc.rmsnorm_gated(x, z, w, EPS).reshape(1, -1)))

    ff, n_slot = 704, 8
    gu = rng.standard_normal((n_slot, 2 * ff)).astype(np.float32)
    dq = blocks(n_slot * ff)
    mod.function("moe_geglu_q8_f32").launch(((ff // 32 + 7) // 8, n_slot, 1), (256, 1, 1), 0, None,
                                            [p(gu), p(dq), u(ff)])
    hip.synchronize()
    assert np.array_equal(dq.to_host(np.uint8), orc.quantize_q8(orc.geglu_det(gu)))


def test_fused_producer_feeds_the_matvec():
    # add_rmsnorm_q8 -> Q4_K matvec equals the oracle chain on the same bytes
    from reinstinct_amd import quant
    from helpers import assert_close_f32, random_raw_weights
    n, out_dim = 5120, 512
    rng = np.random.default_rng(11)
    h, a = rng.standard_normal((1, n)).astype(np.float32), rng.standard_normal((1, n)).astype(np.float32)
    w = (1 + 0.1 * rng.standard_normal(n)).astype(np.float32)
    raw = random_raw_weights(rein.Q4_K, n, out_dim, 3)
    packed = quant.repack_for_matvec(rein.Q4_K, raw, n, out_dim)
    dq, dy = blocks(n), dev(np.zeros(out_dim, np.float32))
    runtime.add_rmsnorm_q8(dev(h), dev(a), dev(w), None, dq, n, 1, EPS)
    runtime.matvec_xq8(rein.Q4_K, dev(packed), dq, dy, n, out_dim)
    hip.synchronize()
    xq = orc.quantize_q8(orc.add_rmsnorm(h, a, w, EPS)[1])
    assert_close_f32(dy.to_host(np.float32), orc.matvec_q8(orc.Q4_K, packed, n, out_dim, xq, 1)[0], what="norm -> matvec")
