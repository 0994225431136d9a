"""rein_matvec_multi_xq8: the decode step's consecutive matvecs on the same activations (Q / K / V, gate / up;
src/runtime/qwen35.rs:2670-2672, 2702-2703) in one launch.  Every output is compared with the oracle and, bit for
bit, with the launch of that matrix alone (rein_matvec_xq8; at two to four rows the dot4 kernels behind
rein_matvec_batched_xq8): mixed formats, matrices of very different heights, row counts that do not divide by the
rows per wavefront, each rows-per-wavefront kernel, and the argument checks."""
import numpy as np
import pytest

import reinstinct_amd as rein
from reinstinct_amd import hip, quant, runtime
from reinstinct_amd._lib import ReinError, init
from oracle import orc
from helpers import assert_close_f32, dev, random_raw_weights

pytestmark = pytest.mark.gpu

DENSE = [rein.Q4_0, rein.Q8_0, rein.Q4_K, rein.Q5_K, rein.Q6_K, rein.IQ4_XS, rein.IQ3_S]


@pytest.fixture(scope="module", autouse=True)
def gpu():
    init()
    hip.set_device(0)
    yield
    hip.synchronize()


def bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


DOT4_ONLY = (("REIN_MV_LDS", "0"), ("REIN_QUAD_LDS", "0"), ("REIN_SKINNY_FROM", "99"), ("REIN_QUAD_FROM", "99"))


def check(fmts, in_dim, out_dims, seed=0, n_rows=1, options=None, one_by_one=False):
    print("multi matvec", fmts, in_dim, out_dims, n_rows, flush=True)
    packed = [quant.repack_for_matvec(f, random_raw_weights(f, in_dim, n, seed=seed + 7 * i + f), in_dim, n)
              for i, (f, n) in enumerate(zip(fmts, out_dims))]
    xq = orc.quantize_q8(np.random.default_rng(seed).standard_normal((n_rows, in_dim)).astype(np.float32))
    dq = dev(xq)
    dws = [dev(p) for p in packed]
    # one buffer for all outputs with a guard word behind each, so a write past a matrix's rows shows
    offs = np.concatenate([[0], np.cumsum([n_rows * n + 1 for n in out_dims])])
    host = np.full(int(offs[-1]), np.float32(-77.0), np.float32)
    dy = dev(host)
    runtime.matvec_multi_xq8(fmts, dws, [dy.ptr + 4 * int(o) for o in offs[:-1]], out_dims, dq, in_dim, n_rows)
    hip.synchronize()
    got = dy.to_host(np.float32)
    if n_rows > 1 and not one_by_one:    # the few-row launches of one matrix are compared in their dot4 form
        for name, value in DOT4_ONLY:
            options.set(name, value)
    for i, (f, n) in enumerate(zip(fmts, out_dims)):
        mine = got[int(offs[i]):int(offs[i]) + n_rows * n].reshape(n_rows, n)
        assert got[int(offs[i]) + n_rows * n] == np.float32(-77.0), f"matrix {i} wrote past its rows"
        want = orc.matvec_q8(f, packed[i], in_dim, n, xq, n_rows)
        assert_close_f32(mine, want, what=f"multi matrix {i} fmt {f} {in_dim}->{n} rows {n_rows}")
        d1 = dev(np.full(n_rows * n, np.nan, np.float32))
        runtime.matvec_batched_xq8(f, dws[i], dq, d1, in_dim, n, n_rows)
        hip.synchronize()
        assert np.array_equal(bits(mine), bits(d1.to_host(np.float32).reshape(n_rows, n))), \
            f"matrix {i} fmt {f} rows {n_rows}: not the bits of the launch of that matrix alone"
    if n_rows > 1 and not one_by_one:
        for name, _ in DOT4_ONLY:
            options.unset(name)


@pytest.mark.parametrize("fmts,in_dim,out_dims", [
    ([rein.Q4_K, rein.Q4_K, rein.Q6_K], 2048, [2048, 512, 512]),             # Q, K, V with a Q6_K value projection
    ([rein.Q4_K, rein.Q4_K], 1024, [2816, 2816]),                            # gate, up
    ([rein.Q8_0, rein.Q8_0], 2048, [96, 96]),                                # two tiny projections
    ([rein.Q5_K, rein.Q6_K, rein.Q8_0, rein.Q4_0], 512, [33, 1, 130, 67]),   # four formats, odd heights
    ([rein.IQ4_XS, rein.IQ3_S], 768, [259, 3]),
    ([rein.Q6_K], 2304, [517]),                                              # one matrix: the plain launch
])
def test_multi_matvec(fmts, in_dim, out_dims):
    check(fmts, in_dim, out_dims)


@pytest.mark.parametrize("rows", ["1", "2", "4"])
@pytest.mark.parametrize("fmt", DENSE)
def test_multi_matvec_each_rows_per_wavefront(fmt, rows, options):
    options.set("REIN_MV_ROWS", rows)
    check([fmt, rein.Q4_K, fmt], 1280 if fmt in (rein.Q4_0, rein.Q8_0) else 1536, [131, 66, 7], seed=3)
    options.unset("REIN_MV_ROWS")


@pytest.mark.parametrize("n_rows", [2, 3, 4])
@pytest.mark.parametrize("fmts,in_dim,out_dims", [
    ([rein.Q4_K, rein.Q4_K, rein.Q6_K], 2048, [1024, 256, 256]),
    ([rein.Q5_K, rein.Q8_0, rein.IQ4_XS, rein.Q4_0], 768, [67, 5, 130, 33]),
    ([rein.IQ3_S, rein.Q6_K], 1536, [259, 131]),
])
def test_multi_matvec_few_rows(fmts, in_dim, out_dims, n_rows, options):
    """the two to four rows of a speculative-decode verify step"""
    check(fmts, in_dim, out_dims, seed=n_rows, n_rows=n_rows, options=options)


def test_multi_matvec_decode_shapes():
    """the attention and FFN projections of the 27B-class decoder (hidden 5120, 40 / 8 heads of 128, FFN 17408)"""
    check([rein.Q4_K, rein.Q4_K, rein.Q6_K], 5120, [5120, 1024, 1024], seed=1)
    check([rein.Q4_K, rein.Q4_K], 5120, [17408, 17408], seed=2)


def test_multi_matvec_decode_shapes_four_rows(options):
    check([rein.Q4_K, rein.Q4_K, rein.Q6_K], 5120, [5120, 1024, 1024], seed=4, n_rows=4, options=options)


def test_multi_matvec_ffn_sized_matrices_at_four_rows():
    """three and four rows against matrices of an FFN's size go out as the launches of the matrices one by one"""
    check([rein.Q4_K, rein.Q4_K], 5120, [8192, 8192], seed=5, n_rows=4, one_by_one=True)
    check([rein.Q4_K, rein.Q6_K], 5120, [8192, 8192], seed=6, n_rows=3, one_by_one=True)


def test_multi_matvec_argument_checks():
    dq = dev(np.zeros(40 * 8, np.uint8))
    dw = dev(np.zeros(4096, np.uint8))
    dy = dev(np.zeros(64, np.float32))
    with pytest.raises(ReinError):
        runtime.matvec_multi_xq8([], [], [], [], dq, 256)
    with pytest.raises(ReinError):
        runtime.matvec_multi_xq8([rein.Q4_K] * 5, [dw] * 5, [dy] * 5, [4] * 5, dq, 256)
    with pytest.raises(ReinError):
        runtime.matvec_multi_xq8([rein.Q4_K, rein.Q5_1], [dw, dw], [dy, dy], [4, 4], dq, 256)
    with pytest.raises(ReinError):
        runtime.matvec_multi_xq8([rein.Q4_K, rein.Q4_K], [dw, dw], [dy, dy], [4, 0], dq, 256)
    with pytest.raises(ReinError):
        runtime.matvec_multi_xq8([rein.Q4_K, rein.Q4_K], [dw, 0], [dy, dy], [4, 4], dq, 256)
    with pytest.raises(ReinError):
        runtime.matvec_multi_xq8([rein.Q4_K, rein.Q4_K], [dw, dw], [dy, dy], [4, 4], dq, 200)
    for rows in (0, 5):
        with pytest.raises(ReinError):
            runtime.matvec_multi_xq8([rein.Q4_K, rein.Q4_K], [dw, dw], [dy, dy], [4, 4], dq, 256, rows)


@pytest.mark.parametrize("seed", [11, 12])
def test_multi_matvec_on_random_tables(seed, options):
    """seeded tables of two to four matrices, one to four rows, against the oracle and the launches one by one"""
    rng = np.random.default_rng(seed)
    for case in range(25):
        n_mat = int(rng.integers(2, 5))
        fmts = [DENSE[rng.integers(len(DENSE))] for _ in range(n_mat)]
        superblocks = any(f not in (rein.Q4_0, rein.Q8_0) for f in fmts) or rng.random() < 0.5
        in_dim = int(rng.integers(1, 9)) * 256 if superblocks else int(rng.integers(1, 40)) * 32
        out_dims = [int(rng.choice([int(rng.integers(1, 40)), int(rng.integers(40, 700)), int(rng.integers(700, 4000))]))
                    for _ in range(n_mat)]
        n_rows = int(rng.choice([1, 1, 2, 3, 4]))
        check(fmts, in_dim, out_dims, seed=100 * seed + case, n_rows=n_rows, options=options)


def test_multi_matvec_in_a_captured_graph():
    """the argument table travels by value with the launch: a captured call replays with the tables of the capture,
    whatever the host arrays hold afterwards"""
    fmts, in_dim, out_dims = [rein.Q4_K, rein.Q6_K, rein.Q8_0], 1536, [300, 77, 129]
    packed = [quant.repack_for_matvec(f, random_raw_weights(f, in_dim, n, seed=40 + i), in_dim, n)
              for i, (f, n) in enumerate(zip(fmts, out_dims))]
    xq = orc.quantize_q8(np.random.default_rng(40).standard_normal((1, in_dim)).astype(np.float32))
    dq, dws = dev(xq), [dev(p) for p in packed]
    dys = [dev(np.full(n, np.nan, np.float32)) for n in out_dims]
    stream = hip.Stream()
    stream.begin_capture()
    runtime.matvec_multi_xq8(fmts, dws, dys, out_dims, dq, in_dim, 1, stream)
    exe = stream.end_capture().instantiate()
    for replay in range(3):
        for dy, n in zip(dys, out_dims):
            dy.copy_from_host(np.zeros(n, np.float32))
        hip.synchronize()
        exe.launch(stream)
        stream.synchronize()
        for i, (f, n) in enumerate(zip(fmts, out_dims)):
            d1 = dev(np.full(n, np.nan, np.float32))
            runtime.matvec_xq8(f, dws[i], dq, d1, in_dim, n)
            hip.synchronize()
            assert np.array_equal(bits(dys[i].to_host(np.float32)), bits(d1.to_host(np.float32))), f"replay {replay} matrix {i}"
