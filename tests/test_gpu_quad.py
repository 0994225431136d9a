"""The batched decode matvec on the 4x4x4 int8 matrix instruction (rein_mvq_*) against the
oracle, for every dense format, every row count 1..8, output row counts that are not
multiples of four and contractions that are not multiples of 16 sub-blocks.  The library
picks these kernels for some formats only; REIN_QUAD_FROM forces them here."""
import numpy as np
import pytest

import reinstinct_amd as rein
from reinstinct_amd import hip, quant, runtime
from reinstinct_amd._lib import init
from oracle import orc
from helpers import assert_close_f32, random_raw_weights

pytestmark = pytest.mark.gpu

DENSE = [rein.Q4_0, rein.Q8_0, rein.Q4_K, rein.Q5_K, rein.Q6_K, rein.IQ4_XS, rein.IQ3_S]


@pytest.fixture(scope="module", autouse=True)
def gpu():
    init()
    hip.set_device(0)
    yield
    hip.synchronize()


from helpers import dev  # noqa: E402  (uploads that stay alive until the test's last launch has finished)


def run(fmt, packed, xq, in_dim, out_dim, n_rows):
    dw, dq = dev(packed), dev(xq)
    dy = dev(np.full(n_rows * out_dim, np.nan, np.float32))
    if n_rows == 1:
        runtime.matvec_xq8(fmt, dw, dq, dy, in_dim, out_dim)
    else:
        runtime.matvec_batched_xq8(fmt, dw, dq, dy, in_dim, out_dim, n_rows)
    hip.synchronize()
    return dy.to_host(np.float32).reshape(n_rows, out_dim)


@pytest.mark.parametrize("fmt", DENSE)
@pytest.mark.parametrize("in_dim,out_dim", [(2048, 389), (512, 3), (256, 64), (5120, 130), (4096, 33)])
def test_quad_matvec_parity(fmt, in_dim, out_dim, options):
    options.set("REIN_QUAD_FROM", "1")
    raw = random_raw_weights(fmt, in_dim, out_dim, seed=fmt + in_dim)
    packed = quant.repack_for_matvec(fmt, raw, in_dim, out_dim)
    for n_rows in range(1, 9):
        print("quad", fmt, in_dim, out_dim, n_rows, flush=True)
        x = np.random.default_rng(n_rows).standard_normal((n_rows, in_dim)).astype(np.float32)
        xq = orc.quantize_q8(x)
        want = orc.matvec_q8(fmt, packed, in_dim, out_dim, xq, n_rows)
        assert_close_f32(run(fmt, packed, xq, in_dim, out_dim, n_rows), want, what=f"quad fmt {fmt} rows {n_rows}")


@pytest.mark.parametrize("fmt", [rein.Q4_0, rein.Q8_0])       # 32-weight blocks: any multiple of 32
@pytest.mark.parametrize("in_dim", [32, 96, 352, 544, 1056])
def test_quad_matvec_ragged_contraction(fmt, in_dim, options):
    options.set("REIN_QUAD_FROM", "1")
    out_dim = 37
    raw = random_raw_weights(fmt, in_dim, out_dim, seed=in_dim)
    packed = quant.repack_for_matvec(fmt, raw, in_dim, out_dim)
    for n_rows in (1, 4, 7):
        xq = orc.quantize_q8(np.random.default_rng(n_rows).standard_normal((n_rows, in_dim)).astype(np.float32))
        want = orc.matvec_q8(fmt, packed, in_dim, out_dim, xq, n_rows)
        assert_close_f32(run(fmt, packed, xq, in_dim, out_dim, n_rows), want, what=f"quad ragged {in_dim}")


@pytest.mark.parametrize("fmt,n_rows", [(rein.Q6_K, 3), (rein.Q6_K, 4), (rein.Q5_K, 4), (rein.IQ4_XS, 3)])
def test_default_dispatch_at_benchmark_width(fmt, n_rows, options):
    # the row counts the library sends to these kernels by itself: 3-4 rows against more than 8192 and fewer than
    # 14336 rows from 2^24 weights (narrower matrices and longer contractions go to the LDS-staged kernels, as do five
    # rows and more)
    in_dim, out_dim = 2048, 9004
    raw = random_raw_weights(fmt, in_dim, out_dim, seed=n_rows)
    packed = quant.repack_for_matvec(fmt, raw, in_dim, out_dim)
    xq = orc.quantize_q8(np.random.default_rng(fmt).standard_normal((n_rows, in_dim)).astype(np.float32))
    want = orc.matvec_q8(fmt, packed, in_dim, out_dim, xq, n_rows)
    got = run(fmt, packed, xq, in_dim, out_dim, n_rows)
    assert_close_f32(got, want, what="default dispatch")
    options.set("REIN_QUAD_FROM", "1")
    forced = run(fmt, packed, xq, in_dim, out_dim, n_rows)
    assert np.array_equal(np.ascontiguousarray(got).view(np.uint32), np.ascontiguousarray(forced).view(np.uint32))


def bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


@pytest.mark.parametrize("fmt", [rein.Q4_K, rein.Q8_0, rein.Q4_0])
def test_mid_width_matrices_take_these_kernels_at_3_and_4_rows(fmt, options):
    # 8192..20480 output rows: the library's own choice for the formats that otherwise run the skinny MMQ;
    # the same bits as with the kernels forced, and the oracle's values
    in_dim, out_dim = 2304, 8200
    raw = random_raw_weights(fmt, in_dim, out_dim, seed=fmt)
    packed = quant.repack_for_matvec(fmt, raw, in_dim, out_dim)
    for n_rows in (3, 4):
        print("quad by default", fmt, n_rows, flush=True)
        xq = orc.quantize_q8(np.random.default_rng(n_rows).standard_normal((n_rows, in_dim)).astype(np.float32))
        got = run(fmt, packed, xq, in_dim, out_dim, n_rows)
        assert_close_f32(got, orc.matvec_q8(fmt, packed, in_dim, out_dim, xq, n_rows), what=f"fmt {fmt} rows {n_rows}")
        options.set("REIN_QUAD_FROM", "1")
        forced = run(fmt, packed, xq, in_dim, out_dim, n_rows)
        options.unset("REIN_QUAD_FROM")
        assert np.array_equal(bits(got), bits(forced)), "the default launch is not the 4x4x4 kernel"


@pytest.mark.parametrize("fmt", DENSE)
def test_small_matrices_stay_on_dot4(fmt, options):
    # up to 2^24 weights at 3-4 rows and 6 * 2^20 at 5-8 the library keeps the dot4 kernels: the same bits as
    # with both matrix-core families switched off, and the oracle's values
    in_dim, out_dim = 2048, 1536
    raw = random_raw_weights(fmt, in_dim, out_dim, seed=fmt + 1)
    packed = quant.repack_for_matvec(fmt, raw, in_dim, out_dim)
    for n_rows in (3, 4, 8):
        print("dot4 by default", fmt, n_rows, flush=True)
        xq = orc.quantize_q8(np.random.default_rng(n_rows).standard_normal((n_rows, in_dim)).astype(np.float32))
        got = run(fmt, packed, xq, in_dim, out_dim, n_rows)
        assert_close_f32(got, orc.matvec_q8(fmt, packed, in_dim, out_dim, xq, n_rows), what=f"fmt {fmt} rows {n_rows}")
        options.set("REIN_QUAD_FROM", "99")
        options.set("REIN_SKINNY_FROM", "99")
        forced = run(fmt, packed, xq, in_dim, out_dim, n_rows)
        options.unset("REIN_QUAD_FROM")
        options.unset("REIN_SKINNY_FROM")
        assert np.array_equal(bits(got), bits(forced)), "the default launch is not a dot4 kernel"
