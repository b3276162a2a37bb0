"""GPU parity of t(X) %*% X on blocks of a few stream columns next to run-length columns: the Gram kernel on the
vector unit that follows the run-length columns by run (k_tsmm_direct) against the CPU oracle and the exact
product, through the C ABI. Every case also checks which kernel ran."""
import numpy as np
import pytest

from parity import assert_fp64_close, assert_matches_truth

pytestmark = pytest.mark.gpu


def rle_group(rng, n_rows, cols, n_vals, mean_run, uncovered=False, bursts=False):
    """RLE group over `cols` (one tuple per run): geometric run lengths; `uncovered` leaves some runs without a tuple,
    `bursts` puts stretches of one-row runs between the long ones."""
    from systemds_amd import synth
    n_runs = int(n_rows / mean_run * 1.5) + 8
    lens = rng.geometric(1.0 / mean_run, size=n_runs)
    if bursts:
        lens[::7] = 1
        lens[1::7] = 1
        lens[2::7] = 2
    lo = -1 if uncovered else 0
    run_codes = rng.integers(lo, n_vals, size=n_runs)
    codes = np.repeat(run_codes, lens)[:n_rows]
    if codes.size < n_rows:
        codes = np.concatenate([codes, np.full(n_rows - codes.size, run_codes[-1])])
    ptr, data = synth.encode_rle(codes, n_vals)
    cols = np.asarray(cols, np.int32)
    return synth.GroupSpec("rle", cols, rng.standard_normal((n_vals, cols.size)), ptr=ptr, rle=data)


def stream_block(seed, n_rows, n_rle=3, n_u16=4, n_u8=2, n_sdc=2, n_dense=2, mean_run=200, cocoded=False, bursts=False,
                 rle_cols=1):
    """RLE columns, then DDC columns of two-byte and of one-byte codes, SDC columns, one uncompressed group."""
    from systemds_amd import synth
    rng = np.random.default_rng(seed)
    specs, c = [], 0

    def cols(n):
        nonlocal c
        r = np.arange(c, c + n, dtype=np.int32)
        c += n
        return r
    for k in range(n_rle):
        burst = bursts and k == 0  # (its long runs three times as long: the group still counts as one of long runs)
        specs.append(rle_group(rng, n_rows, cols(rle_cols), 5 + k, mean_run * (3 if burst else 1), uncovered=k == 1, bursts=burst))
    w = 2 if cocoded else 1
    for k in range(n_u16):
        nv = 300 + 50 * k
        specs.append(synth.GroupSpec("ddc", cols(w), rng.standard_normal((nv, w)), rng.integers(0, nv, n_rows).astype(np.uint16)))
    for k in range(n_u8):
        nv = 3 + 40 * k
        specs.append(synth.GroupSpec("ddc", cols(1), rng.standard_normal((nv, 1)), rng.integers(0, nv, n_rows).astype(np.uint8)))
    for k in range(n_sdc):
        specs.append(synth.sdc_group(rng, n_rows, cols(1), 6 + k, 0.1, 1.5 if k == 0 else None))
    if n_dense:
        specs.append(synth.GroupSpec("unc", cols(n_dense), dense=rng.standard_normal((n_rows, n_dense))))
    return specs, c


def check(cla, ora, specs, n_rows, n_cols, what, expect_direct=True, options=None):
    blk = cla.build_block(n_rows, n_cols, specs)
    for key, value in (options or {}).items():
        blk.set_option(key, value)
    out, nnz = blk.tsmm()
    names = {k["name"] for k in blk.stats()["kernels"]}
    blk.close()
    if expect_direct is not None:
        assert ("k_tsmm_direct" in names) == expect_direct, (what, names)
    ref, rnnz = ora.tsmm(ora.Groups(specs, n_rows, n_cols), 4)
    D = ora.np_decompress(specs, n_rows, n_cols)
    assert np.array_equal(out, out.T)
    assert_matches_truth(out, D.T, D, what=what)
    assert_fp64_close(out, ref, ora.abs_matmul(D.T, D), what=what, n_terms=n_rows)
    assert nnz == rnnz
    return out


@pytest.mark.parametrize("n_rows", [1, 63, 64, 65, 127, 128, 129, 1000, 20011, 150001])
def test_row_counts_around_the_slices(cla, ora, n_rows):
    """Slices of 64 rows, chunks of 128: full, ragged and single-row blocks (a run-length group of a block of a few rows
    counts as one of short runs and is read from its one-code-per-row copy: twelve stream columns then)."""
    specs, n_cols = stream_block(10 + n_rows % 7, n_rows, n_u16=3)
    # (a single row: an offset list may be empty, and a column without row data is not this kernel's)
    check(cla, ora, specs, n_rows, n_cols, f"{n_rows} rows", expect_direct=True if n_rows > 1 else None)


@pytest.mark.parametrize("shape", [dict(n_u16=8, n_u8=0, n_sdc=2, n_dense=2),   # the widths known at compile time
                                   dict(n_u16=8, n_u8=0, n_sdc=2, n_dense=2, n_rle=0),
                                   dict(n_u16=3, n_u8=2, n_sdc=0, n_dense=0),   # odd number of code columns: a filler
                                   dict(n_u16=0, n_u8=5, n_sdc=1, n_dense=1),
                                   dict(n_u16=2, n_u8=2, n_sdc=2, n_dense=4),
                                   dict(n_u16=6, n_u8=4, n_sdc=2, n_dense=0),   # twelve code columns
                                   dict(n_u16=1, n_u8=0, n_sdc=0, n_dense=0, n_rle=8),
                                   dict(n_u16=2, n_u8=1, n_sdc=1, n_dense=2, n_rle=0)])
def test_column_mixes(cla, ora, shape):
    n_rows = 70001
    specs, n_cols = stream_block(3, n_rows, **{**dict(n_rle=3), **shape})
    check(cla, ora, specs, n_rows, n_cols, f"mix {shape}")


def test_short_runs_and_bursts(cla, ora):
    """Runs barely longer than a slice, with stretches of one-row runs: several run ends per slice, window refills."""
    n_rows = 60000
    specs, n_cols = stream_block(5, n_rows, n_rle=4, mean_run=80, bursts=True)
    check(cla, ora, specs, n_rows, n_cols, "short runs")


def test_cocoded_groups(cla, ora):
    """Two columns per DDC group (one stream, two columns) and two columns per RLE group (one run table, two columns)."""
    n_rows = 50021
    specs, n_cols = stream_block(6, n_rows, n_rle=2, n_u16=2, n_u8=1, n_sdc=1, n_dense=2, cocoded=True, rle_cols=2)
    check(cla, ora, specs, n_rows, n_cols, "co-coded")


def test_blocks_outside_the_kernels_shape(cla, ora):
    """More run-length or stream columns than the kernel holds, or the option off: the tile kernel serves the block."""
    n_rows = 30011
    specs, n_cols = stream_block(7, n_rows, n_rle=9, n_u16=2, n_u8=0, n_sdc=0, n_dense=0)
    check(cla, ora, specs, n_rows, n_cols, "nine run-length columns", expect_direct=False)
    specs, n_cols = stream_block(8, n_rows, n_rle=1, n_u16=8, n_u8=3, n_sdc=2, n_dense=0)
    check(cla, ora, specs, n_rows, n_cols, "thirteen stream columns", expect_direct=False)
    specs, n_cols = stream_block(9, n_rows)
    a = check(cla, ora, specs, n_rows, n_cols, "direct")
    b = check(cla, ora, specs, n_rows, n_cols, "tiles", expect_direct=False, options={"tsmm_direct": 0})
    D = ora.np_decompress(specs, n_rows, n_cols)
    assert_fp64_close(a, b, ora.abs_matmul(D.T, D), what="direct vs tiles")


def test_non_finite_run_length_values_take_the_tile_kernel(cla, ora):
    """The run-following kernel handles run-length columns by summation by parts (sums of earlier rows times the step
    of a run-length value), which is the rows' own products only for finite values: a block with an infinite or NaN
    dictionary value next to run-length columns takes the tile kernel, whose cells are the per-row products
    (infinite and NaN cells where the decompressed product has them)."""
    n_rows = 20011
    specs, n_cols = stream_block(31, n_rows)
    rle = next(s for s in specs if s.type == "rle")
    rle.dict[1, 0] = np.inf
    blk = cla.build_block(n_rows, n_cols, specs)
    out, nnz = blk.tsmm()
    names = {k["name"] for k in blk.stats()["kernels"]}
    blk.close()
    assert "k_tsmm_direct" not in names and "k_tsmm_decode" in names, names
    D = ora.np_decompress(specs, n_rows, n_cols)
    with np.errstate(invalid="ignore", over="ignore"):
        truth = D.T @ D
    fin = np.isfinite(truth)
    assert np.array_equal(np.isnan(out), np.isnan(truth))
    assert np.array_equal(np.isinf(out), np.isinf(truth)) and np.array_equal(out[np.isinf(truth)], truth[np.isinf(truth)])
    scale = ora.abs_matmul(np.where(np.isfinite(D), D, 0.0).T, np.where(np.isfinite(D), D, 0.0))
    with np.errstate(invalid="ignore"):
        err = np.abs(out - truth)
    assert np.all(err[fin] <= 1e-12 * scale[fin] + 1e-300)
    assert nnz == np.count_nonzero(out)


def test_long_runs_keep_no_expanded_copy(cla):
    """A run-length group whose runs are long gets no one-code-per-row copy: the block's derived bytes stay far below
    one byte per row and group."""
    n_rows = 400000
    specs, n_cols = stream_block(11, n_rows, n_rle=4, n_u16=2, n_u8=0, n_sdc=0, n_dense=0, mean_run=1000)
    blk = cla.build_block(n_rows, n_cols, specs)
    blk.tsmm()
    derived = blk.derived_bytes()
    blk.close()
    assert derived < n_rows, derived


def crafted_rle(rng, n_rows, col, lens, n_vals=6):
    """RLE column with the given run lengths (cycled to n_rows rows), random tuples."""
    from systemds_amd import synth
    lens = np.resize(np.asarray(lens), int(n_rows // max(int(np.mean(lens)), 1)) + len(lens))
    codes = np.repeat(rng.integers(0, n_vals, size=lens.size), lens)[:n_rows]
    ptr, data = synth.encode_rle(codes, n_vals)
    return synth.GroupSpec("rle", np.array([col], np.int32), rng.standard_normal((n_vals, 1)), ptr=ptr, rle=data)


@pytest.mark.parametrize("q", [1, 2, 7, 10, 16, 23])
def test_right_multiply_follows_the_runs(cla, ora, q):
    """X %*% B on a block with run-length columns of long runs: their part of a row comes from the merged run table
    (k_run_sums), also where more run starts fall into one slice of 128 rows than a slice's record holds."""
    from systemds_amd import synth
    n_rows = 90001
    rng = np.random.default_rng(40 + q)
    specs = [crafted_rle(rng, n_rows, 0, [3000] * 6 + [3] * 150 + [5000]),       # stretches of three-row runs
             crafted_rle(rng, n_rows, 1, [700, 90, 1300, 2, 2, 2, 2500]),
             crafted_rle(rng, n_rows, 2, [128] * 50 + [4096])]                     # run ends on slice borders
    specs.append(synth.GroupSpec("ddc", np.array([3], np.int32), rng.standard_normal((500, 1)), rng.integers(0, 500, n_rows).astype(np.uint16)))
    specs.append(synth.GroupSpec("ddc", np.array([4], np.int32), rng.standard_normal((9, 1)), rng.integers(0, 9, n_rows).astype(np.uint8)))
    specs.append(synth.sdc_group(rng, n_rows, [5], 4, 0.2, -0.5))
    specs.append(synth.GroupSpec("unc", np.array([6, 7], np.int32), dense=rng.standard_normal((n_rows, 2))))
    n_cols = 8
    B = rng.standard_normal((n_cols, q))
    blk = cla.build_block(n_rows, n_cols, specs)
    out, nnz = blk.rmm(B)
    names = {k["name"] for k in blk.stats()["kernels"]}
    blk.close()
    if q != 16:  # (exactly sixteen columns go to the tile kernel first)
        assert {"k_rmm_direct", "k_run_sums"} <= names, names
    ref, rnnz = ora.rmm(ora.Groups(specs, n_rows, n_cols), B, 4)
    D = ora.np_decompress(specs, n_rows, n_cols)
    assert_matches_truth(out, D, B, what=f"X%*%B q={q}")
    assert_fp64_close(out, ref, ora.abs_matmul(D, B), what=f"X%*%B q={q}", n_terms=n_cols)
    assert nnz == rnnz
