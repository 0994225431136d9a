"""The two batched decode kernels that stage the activation rows in LDS -- the dot4 form (rein_mvl_*,
2..4 rows) and the 4x4x4 matrix-instruction form (rein_mvql_*, 3..8 rows) -- against the oracle and,
bit for bit, against the family whose arithmetic each repeats: every dense format, output row
counts that do not divide into workgroups, ragged contractions, each launch geometry (one row group
per wavefront, and persistent wavefronts that stride over row groups), forced rows per wavefront
and workgroup sizes, and the shapes the library sends there by itself.  REIN_MV_LDS and
REIN_QUAD_LDS force the kernels on (1) or off (0)."""
import numpy as np
import pytest

import reinstinct_amd as rein
from reinstinct_amd import hip, quant, runtime
from reinstinct_amd._lib import init
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


def run(fmt, packed, xq, in_dim, out_dim, n_rows):
    dw, dq = dev(packed), dev(xq)
    dy = dev(np.full(n_rows * out_dim, np.nan, np.float32))
    if n_rows <= 8:
        runtime.matvec_batched_xq8(fmt, dw, dq, dy, in_dim, out_dim, n_rows)
    else:
        runtime.mmq_xq8(fmt, dw, dq, dy, in_dim, out_dim, n_rows)           # 9..16 rows arrive through this entry point
    hip.synchronize()
    return dy.to_host(np.float32).reshape(n_rows, out_dim)


def run_lds(options, fmt, packed, xq, in_dim, out_dim, n_rows):
    options.set("REIN_MV_LDS", "1")
    got = run(fmt, packed, xq, in_dim, out_dim, n_rows)
    options.unset("REIN_MV_LDS")
    return got


def run_dot4(options, fmt, packed, xq, in_dim, out_dim, n_rows):
    for name, value in (("REIN_MV_LDS", "0"), ("REIN_SKINNY_FROM", "99"), ("REIN_QUAD_FROM", "99")):
        options.set(name, value)
    got = run(fmt, packed, xq, in_dim, out_dim, n_rows)
    for name in ("REIN_MV_LDS", "REIN_SKINNY_FROM", "REIN_QUAD_FROM"):
        options.unset(name)
    return got


def check(options, fmt, in_dim, out_dim, rows=(2, 3, 4), seed=0):
    raw = random_raw_weights(fmt, in_dim, out_dim, seed=fmt + in_dim + seed)
    packed = quant.repack_for_matvec(fmt, raw, in_dim, out_dim)
    for n_rows in rows:
        print("lds matvec", fmt, in_dim, out_dim, n_rows, flush=True)
        xq = orc.quantize_q8(np.random.default_rng(n_rows + seed).standard_normal((n_rows, in_dim)).astype(np.float32))
        got = run_lds(options, fmt, packed, xq, in_dim, out_dim, n_rows)
        want = orc.matvec_q8(fmt, packed, in_dim, out_dim, xq, n_rows)
        assert_close_f32(got, want, what=f"lds fmt {fmt} {in_dim}->{out_dim} rows {n_rows}")
        same = run_dot4(options, fmt, packed, xq, in_dim, out_dim, n_rows)
        assert np.array_equal(bits(got), bits(same)), f"not the dot4 family's bits: fmt {fmt} {in_dim}->{out_dim} rows {n_rows}"


@pytest.mark.parametrize("fmt", DENSE)
@pytest.mark.parametrize("in_dim,out_dim", [(2048, 389), (512, 3), (256, 64), (5120, 130), (4096, 33), (2304, 4099)])
def test_lds_matvec_parity(fmt, in_dim, out_dim, options):
    check(options, fmt, in_dim, out_dim)


@pytest.mark.parametrize("fmt", [rein.Q4_0, rein.Q8_0])       # 32-weight blocks: any multiple of 32
@pytest.mark.parametrize("in_dim", [32, 96, 352, 544, 1056, 2080, 4128])
def test_lds_matvec_ragged_contraction(fmt, in_dim, options):
    check(options, fmt, in_dim, 37)


@pytest.mark.parametrize("fmt", [rein.Q4_K, rein.Q6_K, rein.Q8_0])
@pytest.mark.parametrize("in_dim,out_dim", [(512, 9001), (256, 40003), (768, 16500)])
def test_lds_matvec_persistent_wavefronts_stride_over_row_groups(fmt, in_dim, out_dim, options):
    # more than 8192 rows: at most four workgroups per CU, each wavefront takes several row groups in turn
    check(options, fmt, in_dim, out_dim)


@pytest.mark.parametrize("rows_per_wave", [1, 2, 4])
@pytest.mark.parametrize("waves", [1, 5, 16])
def test_lds_matvec_forced_geometry(rows_per_wave, waves, options):
    options.set("REIN_MV_ROWS", str(rows_per_wave))
    options.set("REIN_MV_WPB", str(waves))
    fmt, in_dim, out_dim = rein.Q4_K, 1280, 1031
    raw = random_raw_weights(fmt, in_dim, out_dim, seed=waves)
    packed = quant.repack_for_matvec(fmt, raw, in_dim, out_dim)
    for n_rows in (2, 4):
        xq = orc.quantize_q8(np.random.default_rng(n_rows).standard_normal((n_rows, in_dim)).astype(np.float32))
        got = run_lds(options, fmt, packed, xq, in_dim, out_dim, n_rows)
        assert_close_f32(got, orc.matvec_q8(fmt, packed, in_dim, out_dim, xq, n_rows), what=f"R {rows_per_wave} W {waves}")


def test_lds_matvec_largest_contraction_and_fallback_beyond_it(options):
    # four rows x 32768 values fill the CU's 160 KB of LDS exactly; one superblock more and the forced option
    # steps aside for the other families
    fmt, out_dim = rein.Q4_K, 70
    for in_dim in (32768, 33024):
        raw = random_raw_weights(fmt, in_dim, out_dim, seed=in_dim)
        packed = quant.repack_for_matvec(fmt, raw, in_dim, out_dim)
        xq = orc.quantize_q8(np.random.default_rng(1).standard_normal((4, in_dim)).astype(np.float32))
        got = run_lds(options, fmt, packed, xq, in_dim, out_dim, 4)
        assert_close_f32(got, orc.matvec_q8(fmt, packed, in_dim, out_dim, xq, 4), what=f"K {in_dim}")


@pytest.mark.parametrize("fmt,in_dim,out_dim,n_rows", [(rein.Q4_K, 4096, 4100, 3), (rein.Q6_K, 4096, 4100, 4), (rein.Q8_0, 5120, 4100, 3),
                                                      (rein.Q8_0, 5120, 4100, 4), (rein.IQ4_XS, 4096, 4100, 4), (rein.Q5_K, 8192, 8200, 2)])
def test_default_dispatch_takes_the_lds_kernel(fmt, in_dim, out_dim, n_rows, options):
    # 3-4 rows, at most 6144 output rows, from 2^24 weights (Q8_0 at any size, the others up to 20 * 2^20 weights, beyond
    # which the sliced 4x4x4 kernel takes over); 2 rows at contractions of 8192 and more: the same bits as forced
    raw = random_raw_weights(fmt, in_dim, out_dim, seed=n_rows)
    packed = quant.repack_for_matvec(fmt, raw, in_dim, out_dim)
    xq = orc.quantize_q8(np.random.default_rng(fmt).standard_normal((n_rows, in_dim)).astype(np.float32))
    got = run(fmt, packed, xq, in_dim, out_dim, n_rows)
    assert_close_f32(got, orc.matvec_q8(fmt, packed, in_dim, out_dim, xq, n_rows), what="default dispatch")
    assert np.array_equal(bits(got), bits(run_lds(options, fmt, packed, xq, in_dim, out_dim, n_rows)))


# ---- the 4x4x4 matrix-instruction form --------------------------------------------------------------

def run_opts(options, pairs, fmt, packed, xq, in_dim, out_dim, n_rows):
    for name, value in pairs:
        options.set(name, value)
    got = run(fmt, packed, xq, in_dim, out_dim, n_rows)
    for name, _ in pairs:
        options.unset(name)
    return got


def check_quad_lds(options, fmt, in_dim, out_dim, rows=range(3, 9), seed=0, slices="1", depth="1"):
    """slices: wavefronts that share a row group, each taking every slices-th trip of the contraction (None: the
    library's own number).  One slice repeats the 4x4x4 family's arithmetic in its order; several add their partial
    sums in slice order, which is another -- fixed -- order of the same terms."""
    raw = random_raw_weights(fmt, in_dim, out_dim, seed=fmt + in_dim + seed)
    packed = quant.repack_for_matvec(fmt, raw, in_dim, out_dim)
    forced = [("REIN_QUAD_LDS", "1"), ("REIN_MV_LDS", "0")] + ([("REIN_QUAD_SLICES", slices)] if slices else [])
    forced += [("REIN_QUAD_DEPTH", depth)] if depth else []          # None: the library's own number of register sets
    for n_rows in rows:
        print("lds quad", fmt, in_dim, out_dim, n_rows, "slices", slices, flush=True)
        xq = orc.quantize_q8(np.random.default_rng(n_rows + seed).standard_normal((n_rows, in_dim)).astype(np.float32))
        got = run_opts(options, forced, fmt, packed, xq, in_dim, out_dim, n_rows)
        want = orc.matvec_q8(fmt, packed, in_dim, out_dim, xq, n_rows)
        assert_close_f32(got, want, what=f"lds quad fmt {fmt} {in_dim}->{out_dim} rows {n_rows} slices {slices}")
        again = run_opts(options, forced, fmt, packed, xq, in_dim, out_dim, n_rows)
        assert np.array_equal(bits(got), bits(again)), "two runs of the same launch differ"
        same = run_opts(options, [("REIN_QUAD_FROM", "1"), ("REIN_QUAD_LDS", "0"), ("REIN_MV_LDS", "0")], fmt, packed, xq,
                        in_dim, out_dim, n_rows)
        # the other family's kernel (the 4x4x4 kernel without LDS staging up to 8 rows, the skinny MMQ beyond): the same
        # terms; with one slice in the same order, up to how the compiler contracts a format's multiply-adds in each kernel
        assert np.allclose(got, same, rtol=0.0, atol=4e-6 * float(np.abs(same).max())), f"fmt {fmt} {in_dim}->{out_dim} rows {n_rows}"


@pytest.mark.parametrize("fmt", DENSE)
@pytest.mark.parametrize("in_dim,out_dim", [(2048, 389), (512, 3), (256, 64), (5120, 130), (4096, 33), (2304, 4099)])
def test_lds_quad_parity(fmt, in_dim, out_dim, options):
    check_quad_lds(options, fmt, in_dim, out_dim)


@pytest.mark.parametrize("fmt", DENSE)
@pytest.mark.parametrize("in_dim,out_dim", [(2048, 389), (512, 3), (5120, 130), (2304, 4099), (7168, 1030)])
@pytest.mark.parametrize("slices", [None, "2", "3", "8"])
def test_lds_quad_contraction_sliced_over_wavefronts(fmt, in_dim, out_dim, slices, options):
    check_quad_lds(options, fmt, in_dim, out_dim, rows=(3, 4, 5, 8), slices=slices, depth=None if slices is None else "1")


@pytest.mark.parametrize("fmt", [rein.Q4_0, rein.Q8_0])
@pytest.mark.parametrize("in_dim", [32, 96, 352, 544, 1056, 2080])
def test_lds_quad_ragged_contraction(fmt, in_dim, options):
    check_quad_lds(options, fmt, in_dim, 37, rows=(3, 4, 7))


@pytest.mark.parametrize("fmt", [rein.Q4_K, rein.Q6_K, rein.Q8_0])
@pytest.mark.parametrize("in_dim,out_dim", [(256, 70003), (512, 16500)])
def test_lds_quad_persistent_and_widest_workgroups(fmt, in_dim, out_dim, options):
    # 70003 rows: 512 workgroups of eight wavefronts stride over 17501 row groups; 16500: sixteen wavefronts per workgroup
    check_quad_lds(options, fmt, in_dim, out_dim, rows=(3, 8))


@pytest.mark.parametrize("fmt", DENSE)
@pytest.mark.parametrize("in_dim,out_dim", [(2048, 389), (512, 3), (5120, 130), (2304, 4099), (17408, 70)])
@pytest.mark.parametrize("slices", ["1", None])
def test_lds_quad_nine_to_sixteen_rows(fmt, in_dim, out_dim, slices, options):
    # rein_mvql_<fmt>_t16 behind rein_mmq_xq8 (the skinny MMQ otherwise); 16 rows x 17408 values take four phases
    check_quad_lds(options, fmt, in_dim, out_dim, rows=(9, 12, 16), slices=slices)


@pytest.mark.parametrize("fmt", DENSE)
@pytest.mark.parametrize("in_dim,out_dim", [(2048, 389), (512, 3), (5120, 130), (2304, 4099), (17408, 70)])
@pytest.mark.parametrize("slices", ["1", None])
@pytest.mark.parametrize("wide", ["0", "1"])
def test_lds_quad_seventeen_to_thirty_two_rows(fmt, in_dim, out_dim, slices, wide, options):
    # rein_mvql_<fmt>_t32 / _t32w (the builds for eight and for sixteen wavefronts per workgroup) behind rein_mmq_xq8
    # (the 32-token tile launch otherwise); 32 rows x 5120 values take two phases
    options.set("REIN_QUAD_WIDE32", wide)
    check_quad_lds(options, fmt, in_dim, out_dim, rows=(17, 24, 32), slices=slices)
    options.unset("REIN_QUAD_WIDE32")


@pytest.mark.parametrize("fmt", DENSE)
@pytest.mark.parametrize("depth", ["2", None])
def test_lds_quad_two_trips_in_flight(fmt, depth, options):
    # two register sets taking turns (REIN_QUAD_DEPTH=2; None: where the library takes them by itself): persistent wavefronts
    # over an odd and an even number of trips per row group, one row group per wavefront, fewer row groups than wavefronts
    for in_dim, out_dim in ((256, 70003), (512, 16500), (2304, 4099), (1056 if fmt in (rein.Q4_0, rein.Q8_0) else 1280, 37), (512, 3)):
        check_quad_lds(options, fmt, in_dim, out_dim, rows=(3, 4, 8), depth=depth)
    # and with the contraction sliced over wavefronts and staged in phases (an odd and an even number of trips per slice)
    for slices in ("2", "3"):
        check_quad_lds(options, fmt, 17408, 70, rows=(8,), seed=3, slices=slices, depth=depth)
        check_quad_lds(options, fmt, 2304, 1030, rows=(4, 12), seed=3, slices=slices, depth=depth)


@pytest.mark.parametrize("waves", [1, 3, 16])
def test_lds_quad_forced_workgroup_size(waves, options):
    options.set("REIN_MV_WPB", str(waves))
    check_quad_lds(options, rein.Q5_K, 1280, 1031, rows=(4, 5))


@pytest.mark.parametrize("fmt", DENSE)
def test_lds_quad_long_contractions_are_staged_in_phases(fmt, options):
    # eight rows x 17408 values do not fit 160 KB of LDS: two phases of 272 sub-blocks, the partial sums stay in
    # registers in between; 32768 values: three phases; a ragged count of row groups leaves wavefronts without one
    for in_dim, out_dim, rows in ((17408, 70, (5, 8)), (32768, 21, (8,)), (16384, 130, (4, 7))):
        check_quad_lds(options, fmt, in_dim, out_dim, rows=rows, seed=1)
    # phases and slices together: a phase is a whole number of rounds of the slices' trips
    for slices in (None, "3", "5"):
        check_quad_lds(options, fmt, 17408, 70, rows=(8,), seed=2, slices=slices)


@pytest.mark.parametrize("fmt,in_dim,out_dim,n_rows", [(rein.Q6_K, 5120, 4100, 8), (rein.IQ4_XS, 5120, 4100, 6),
                                                      (rein.Q4_K, 2048, 8200, 5), (rein.Q8_0, 1024, 16388, 8),
                                                      (rein.Q5_K, 1280, 14340, 3), (rein.Q4_K, 5120, 4100, 4),
                                                      (rein.Q4_0, 5120, 1030, 7), (rein.IQ3_S, 17408, 1300, 8),
                                                      (rein.Q6_K, 2048, 2100, 12), (rein.Q5_K, 4096, 9000, 16),
                                                      (rein.Q4_K, 14336, 1030, 9), (rein.Q8_0, 2048, 2100, 17),
                                                      (rein.Q4_K, 5120, 1030, 32)])
def test_default_dispatch_takes_the_lds_quad_kernel(fmt, in_dim, out_dim, n_rows, options):
    # 5-8 rows: Q6_K / Q5_K / IQ4_XS everywhere, the other formats up to 20480 rows (from 5 * 2^20 weights); 3-4 rows:
    # every format but Q8_0 up to 8192 rows from 20 * 2^20 weights, and Q5_K, Q8_0, IQ3_S, Q4_K against 14336 rows and more;
    # 9-16 rows: Q6_K / Q5_K on narrow and short-and-mid matrices, the others against few rows with a long contraction;
    # 17-32 rows: every format up to 8192 rows
    raw = random_raw_weights(fmt, in_dim, out_dim, seed=n_rows)
    packed = quant.repack_for_matvec(fmt, raw, in_dim, out_dim)
    xq = orc.quantize_q8(np.random.default_rng(fmt).standard_normal((n_rows, in_dim)).astype(np.float32))
    got = run(fmt, packed, xq, in_dim, out_dim, n_rows)
    assert_close_f32(got, orc.matvec_q8(fmt, packed, in_dim, out_dim, xq, n_rows), what="default dispatch")
    forced = run_opts(options, [("REIN_QUAD_LDS", "1"), ("REIN_MV_LDS", "0")], fmt, packed, xq, in_dim, out_dim, n_rows)
    assert np.array_equal(bits(got), bits(forced)), "the default launch is not the LDS-staged 4x4x4 kernel"
