"""GPU parity of the unary aggregates on compressed blocks (cla_aggregate), against the
aggregate of the decompressed matrix (also where the library itself aggregates decompressed row chunks: row
minima / maxima, row sums of squares next to an uncompressed group, everything but sums on overlapping groups,
CLALibCompAgg.java:220-232, 419-452): sum / sumSq by long-double accumulation at the 1e-12
bar of the multiply path (scale = sum of |terms|), min / max up to the rounding of the SDC
default morph ((dict - default) + default), which the reference's decompression has as well.
Mirrors the aggregate cases of the reference's CompressedTestBase (T/CompressedTestBase.java
unaryAggregate tests: the compressed result against the uncompressed operator)."""
import numpy as np
import pytest

from conftest import host_groups, mixed_block
from parity import assert_fp64_close

pytestmark = pytest.mark.gpu

OPS = ["sum", "sumsq", "min", "max"]
DIRS = ["all", "row", "col"]


def truth(D, op, direction):
    L = D.astype(np.longdouble)
    axis = {"all": None, "row": 1, "col": 0}[direction]
    if op == "sum":
        return np.asarray(L.sum(axis=axis), np.longdouble).astype(np.float64).reshape(-1), np.abs(D).sum(axis=axis).reshape(-1)
    if op == "sumsq":
        return np.asarray((L * L).sum(axis=axis), np.longdouble).astype(np.float64).reshape(-1), (D * D).sum(axis=axis).reshape(-1)
    f = np.min if op == "min" else np.max
    return np.asarray(f(D, axis=axis)).reshape(-1), np.asarray(np.abs(D).max(axis=axis)).reshape(-1) + 2.0


def check(cla, specs, D, n_rows, n_cols, op, direction, what):
    blk = cla.build_block(n_rows, n_cols, specs)
    try:
        out, nnz = blk.aggregate(op, direction)
    finally:
        blk.close()
    ref, scale = truth(D, op, direction)
    assert_fp64_close(out, ref, scale, what=f"{what} {op}/{direction}")
    assert nnz == np.count_nonzero(out)


@pytest.mark.parametrize("op", OPS)
@pytest.mark.parametrize("direction", DIRS)
@pytest.mark.parametrize("seed,n_rows,with_unc", [(1, 37, False), (2, 3000, True), (3, 150001, False), (4, 70000, True)])
def test_mixed_groups(cla, ora, op, direction, seed, n_rows, with_unc):
    specs, n_cols = mixed_block(seed, n_rows, with_unc=with_unc)
    D = ora.np_decompress(specs, n_rows, n_cols)
    check(cla, specs, D, n_rows, n_cols, op, direction, "mixed")


@pytest.mark.parametrize("op", OPS)
@pytest.mark.parametrize("direction", DIRS)
@pytest.mark.parametrize("n_rows,with_unc", [(5000, False), (9001, True)])
def test_overlapping_groups(cla, ora, op, direction, n_rows, with_unc):
    """Sums are linear in the groups; everything else on an overlapping block is the aggregate of the sum of the
    groups' cells (CLALibCompAgg.requireDecompression, CLALibCompAgg.java:220-232)."""
    specs, n_cols = mixed_block(5, n_rows, with_unc=with_unc, overlap=True)
    D = ora.np_decompress(specs, n_rows, n_cols)
    check(cla, specs, D, n_rows, n_cols, op, direction, "overlap")


def test_decompressed_chunks_of_many_rows_and_wide_blocks(cla, ora):
    """More rows than one decompressed chunk holds and more than 256 columns (several column passes); lists with
    2-byte offsets, whose blocks of entries are skipped where they lie outside the chunk."""
    from systemds_amd import synth
    rng = np.random.default_rng(8)
    n_rows = 140001   # 300 columns: 111848 rows per 256 MiB chunk
    specs = []
    for g in range(100):
        specs.append(synth.sdc_group(np.random.default_rng((8, g)), n_rows, np.array([3 * g], np.int32), 5, [0.05, 0.0008][g % 2], [None, 0.5][g % 3 == 0]))
        specs.append(synth.GroupSpec("ddc", np.array([3 * g + 1, 3 * g + 2], np.int32), rng.standard_normal((7, 2)), rng.integers(0, 7, n_rows).astype(np.uint8)))
    D = ora.np_decompress(specs, n_rows, 300)
    for op, direction in (("min", "row"), ("max", "row")):
        check(cla, specs, D, n_rows, 300, op, direction, "wide")
    # the same cells under a second set of groups: column and overall aggregates of the summed cells
    more = [synth.GroupSpec("ddc", np.arange(300, dtype=np.int32)[i::3].copy(), rng.standard_normal((4, 100)), rng.integers(0, 4, n_rows).astype(np.uint8)) for i in range(3)]
    D2 = ora.np_decompress(specs + more, n_rows, 300)
    for op, direction in (("max", "col"), ("min", "all"), ("sumsq", "col"), ("sumsq", "row")):
        check(cla, specs + more, D2, n_rows, 300, op, direction, "wide overlap")


@pytest.mark.parametrize("cfg,scale", [("config2", 200), ("config3", 200), ("config4", 200), ("config5", 500)])
def test_baseline_configs_scaled(cla, ora, cfg, scale):
    from systemds_amd import synth
    c = getattr(synth, cfg)(scale=scale)
    n_rows, n_cols = c["n_rows"], c["n_cols"]
    D = ora.np_decompress(c["groups"], n_rows, n_cols)
    for op in OPS:
        for direction in DIRS:
            check(cla, c["groups"], D, n_rows, n_cols, op, direction, cfg)


def test_host_layer_driver(H, ora, cla):
    """CLALibCompAgg.aggregateUnary with the reference's direction names (ReduceCol = one value per row)."""
    n_rows = 20000
    specs, n_cols = mixed_block(6, n_rows, with_unc=True)
    D = ora.np_decompress(specs, n_rows, n_cols)
    cmb = H.CompressedMatrixBlock(n_rows, n_cols)
    cmb.allocateColGroupList(host_groups(H, ora, specs, n_rows))
    agg = H.CLALibCompAgg.aggregateUnary
    r = agg(cmb, H.AggOp.SUM, H.AggDir.ReduceCol, 4)
    assert (r.getNumRows(), r.getNumColumns()) == (n_rows, 1)
    ref, scale = truth(D, "sum", "row")
    assert_fp64_close(r.toArray().reshape(-1), ref, scale, what="rowSums")
    c = agg(cmb, H.AggOp.MAX, H.AggDir.ReduceRow, 4)
    assert (c.getNumRows(), c.getNumColumns()) == (1, n_cols)
    ref, scale = truth(D, "max", "col")
    assert_fp64_close(c.toArray().reshape(-1), ref, scale, what="colMaxs")
    a = agg(cmb, H.AggOp.SUMSQ, H.AggDir.ReduceAll, 4)
    ref, scale = truth(D, "sumsq", "all")
    assert_fp64_close(a.toArray().reshape(-1), ref, scale, what="sumSq")
    m = agg(cmb, H.AggOp.MIN, H.AggDir.ReduceCol, 4)
    assert (m.getNumRows(), m.getNumColumns()) == (n_rows, 1)
    ref, scale = truth(D, "min", "row")
    assert_fp64_close(m.toArray().reshape(-1), ref, scale, what="rowMins")


@pytest.mark.parametrize("direction", ["all", "col"])
def test_sum_of_squares_of_a_dense_column_under_a_constant(cla, ora, direction):
    """A const group on the columns of an uncompressed group (an overlapping block as the overlapping right
    multiply returns it): sum((v + c)^2) needs the cross term 2 c sum(v), not sum(v^2) + n c^2."""
    from systemds_amd import synth
    rng = np.random.default_rng(12)
    n_rows = 30000
    specs = [synth.GroupSpec("unc", np.array([0, 1], np.int32), dense=rng.standard_normal((n_rows, 2)) + 0.5),
             synth.GroupSpec("const", np.array([1, 2], np.int32), np.array([[3.0, -2.0]])),
             synth.GroupSpec("ddc", np.array([3], np.int32), rng.standard_normal((9, 1)), rng.integers(0, 9, n_rows).astype(np.uint8))]
    D = ora.np_decompress(specs, n_rows, 4)
    check(cla, specs, D, n_rows, 4, "sumsq", direction, "dense + const")
    check(cla, specs, D, n_rows, 4, "sum", direction, "dense + const")


@pytest.mark.parametrize("n_rows", [1023, 2049, 70001])
def test_row_sums_of_squares_on_a_block_with_few_offset_lists(cla, ora, n_rows):
    """One SDC group next to DDC, RLE and constant groups, no uncompressed group: the single-column right multiply of
    such a block decodes rows (value x 1), which the row sums of squares must not take (their squares sit in the
    per-tuple tables)."""
    from systemds_amd import synth
    rng = np.random.default_rng(n_rows)
    specs = [synth.sdc_group(rng, n_rows, np.array([0], np.int32), 17, 0.3, None),
             synth.GroupSpec("ddc", np.array([1, 2], np.int32), rng.standard_normal((300, 2)), rng.integers(0, 300, n_rows).astype(np.uint16)),
             synth.GroupSpec("const", np.array([3], np.int32), np.array([[-0.75]]))]
    run_codes = rng.integers(-1, 4, size=n_rows // 20 + 2)
    codes = np.repeat(run_codes, rng.integers(1, 60, size=run_codes.size))[:n_rows]
    if codes.size < n_rows:
        codes = np.concatenate([codes, np.full(n_rows - codes.size, -1)])
    ptr, data = synth.encode_rle(codes, 4)
    specs.append(synth.GroupSpec("rle", np.array([4], np.int32), rng.standard_normal((4, 1)), ptr=ptr, rle=data))
    D = ora.np_decompress(specs, n_rows, 5)
    for op in OPS:
        for direction in DIRS:
            check(cla, specs, D, n_rows, 5, op, direction, "few lists")


@pytest.mark.parametrize("direction", DIRS)
@pytest.mark.parametrize("op", ["min", "max"])
def test_nan_cells_propagate_like_math_min_max(cla, ora, op, direction):
    """The reference's Builtin MIN / MAX are Math.min / Math.max (functionobjects/Builtin.java:259-264, 308-312): a NaN
    cell makes the aggregate over it NaN. One NaN tuple in a dictionary (it occurs in some rows) and one NaN cell of an
    uncompressed group."""
    from systemds_amd import synth
    n_rows = 5000
    rng = np.random.default_rng(77)
    d = rng.standard_normal((9, 1))
    d[4, 0] = np.nan
    codes = rng.integers(0, 9, n_rows).astype(np.uint8)
    dense = rng.standard_normal((n_rows, 2))
    dense[1234, 1] = np.nan
    specs = [synth.GroupSpec("ddc", np.array([0], np.int32), d, codes),
             synth.GroupSpec("ddc", np.array([1], np.int32), rng.standard_normal((5, 1)), rng.integers(0, 5, n_rows).astype(np.uint8)),
             synth.GroupSpec("unc", np.array([2, 3], np.int32), dense=dense)]
    D = ora.np_decompress(specs, n_rows, 4)
    blk = cla.build_block(n_rows, 4, specs)
    try:
        out, nnz = blk.aggregate(op, direction)
    finally:
        blk.close()
    axis = {"all": None, "row": 1, "col": 0}[direction]
    with np.errstate(invalid="ignore"):
        ref = np.asarray((np.min if op == "min" else np.max)(D, axis=axis)).reshape(-1)
    assert np.array_equal(np.isnan(out), np.isnan(ref)), (op, direction)
    fin = ~np.isnan(ref)
    assert np.allclose(out[fin], ref[fin], rtol=1e-15, atol=0)
    assert nnz == np.count_nonzero(out)
