"""GPU parity of the SDCZeros mat-vec kernels behind cla_lmm / cla_rmm / cla_mmchain: the lane-per-group
kernel on lane-major lists (t(v) %*% X), the lane-per-row kernel on row lists (X %*% u), and the kernels they
replace, each selected through cla_block_set_option and each against the exactly accumulated (long double)
product of the decompressed block at 1e-12. The cases cover what the conversions have to get right, as the
reference's offset tests do for its iterators (OffsetTests.java: first/last row, skip entries of OffsetByte and
OffsetChar, empty stretches): gaps of more than 255 rows, 2-byte offsets, lists of very different lengths in one
block, rows listed by many groups, windows without entries, a last window of one row, dictionaries with a
non-finite value, non-finite values in the vector, groups of several columns, other group types next to the
lists (the output then starts from what they wrote), a default row (SDC with a non-zero default)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

MODES = {"rows+lanes": (1, 1, 1), "lanes": (0, 1, 1), "packed": (0, 0, 1), "tiles": (0, 0, 0)}


def set_mode(blk, mode):
    rows, lanes, packed = MODES[mode]
    blk.set_option("sdc_rows", rows)
    blk.set_option("sdc_lanes", lanes)
    blk.set_option("sdc_packed", packed)


def kernels_of(blk, fn):
    blk.profile(True)
    fn()
    names = [k["name"] for k in blk.stats()["kernels"]]
    blk.profile(False)
    return names


def truth(A, B):
    with np.errstate(invalid="ignore", over="ignore"):
        t = (np.asarray(A, np.float64).astype(np.longdouble) @ np.asarray(B, np.float64).astype(np.longdouble)).astype(np.float64)
        s = np.abs(A) @ np.abs(B)
    return t, s


def assert_close(got, A, B, what):
    t, s = truth(A, B)
    fin = np.isfinite(t)
    assert np.array_equal(np.isfinite(got), fin), f"{what}: finite cells differ"
    assert np.array_equal(got[~fin], t[~fin], equal_nan=True), f"{what}: non-finite cells differ"
    err = np.abs(got[fin] - t[fin])
    assert np.all(err <= 1e-12 * np.maximum(s[fin], np.finfo(float).tiny)), f"{what}: max err/scale {np.max(err / np.maximum(s[fin], 1e-300)):.3e}"


def sdc_block(seed, n_rows, n_groups, density, n_vals, default=None, n_cols_g=1):
    from systemds_amd import synth
    specs, c = [], 0
    for g in range(n_groups):
        d = density[g % len(density)] if isinstance(density, (list, tuple)) else density
        specs.append(synth.sdc_group(np.random.default_rng((seed, g)), n_rows, np.arange(c, c + n_cols_g, dtype=np.int32), n_vals, d, default))
        c += n_cols_g
    return specs, c


CASES = [
    # n_rows, groups, density, tuples
    (1, 3, 0.9, 4),
    (1023, 5, 0.3, 7),
    (1025, 70, 0.05, 64),          # last window of one row, more groups than lanes
    (70001, 130, 0.05, 64),        # dictionaries beyond one slab's share of LDS: two slabs
    (20000, 300, 0.05, 8),         # more groups than a chunk's tag numbers: two slabs
    (200000, 40, 0.0015, 5),       # gaps beyond 255 rows: skip entries, windows without entries
    (300007, 70, 0.001, 3),        # 2-byte offsets
    (50000, 9, 0.0002, 200),
    (123457, 10, [0.3, 0.002, 0.05], 64),  # lists of very different lengths in one slab
    (40000, 66, 0.7, 255),         # dense lists: many chunk rows per window, rows listed by most groups
    (40000, 20, 0.5, 256),         # 256 tuples: no spare code, the older kernels serve
]


@pytest.mark.parametrize("n_rows,n_groups,density,n_vals", CASES)
def test_every_kernel_choice_against_the_decompressed_product(cla, ora, n_rows, n_groups, density, n_vals):
    rng = np.random.default_rng(n_rows + n_groups)
    specs, n = sdc_block(n_rows, n_rows, n_groups, density, n_vals)
    D = ora.np_decompress(specs, n_rows, n)
    blk = cla.build_block(n_rows, n, specs)
    try:
        u = rng.standard_normal((n, 1))
        Y = rng.standard_normal((3, n_rows))
        seen = set()
        for mode in MODES:
            set_mode(blk, mode)
            out, nnz = blk.rmm(u)
            assert_close(out, D, u, f"{mode}: X %*% u")
            assert nnz == np.count_nonzero(out)
            for p in (1, 3):
                out, nnz = blk.lmm(Y[:p])
                assert_close(out, Y[:p], D, f"{mode}: t(v) %*% X, {p} rows")
                assert nnz == np.count_nonzero(out), f"{mode}: non-zeros of t(v) %*% X, {p} rows"
            w = rng.standard_normal((n_rows, 1))
            out, _ = blk.mmchain(u, w, 1)
            Xu, _ = truth(D, u)
            assert_close(out.reshape(-1, 1), D.T, Xu * w, f"{mode}: chain")
            seen |= set(kernels_of(blk, lambda: blk.rmm(u))) | set(kernels_of(blk, lambda: blk.lmm(Y[:1])))
        if n_vals <= 255 and n_rows > 1:
            assert "k_lmm_sdc_lanes" in seen and ("k_rmm_sdc_rows" in seen or "k_rmm_sdc_lanes" in seen), seen
    finally:
        blk.close()


def test_lists_with_more_entries_per_row_than_the_row_lists_hold(cla, ora):
    """90 groups at 60%: rows with more than 40 entries; the row lists are dropped and the lane-major kernel serves."""
    n_rows = 30000
    specs, n = sdc_block(5, n_rows, 90, 0.6, 16)
    D = ora.np_decompress(specs, n_rows, n)
    blk = cla.build_block(n_rows, n, specs)
    try:
        u = np.random.default_rng(1).standard_normal((n, 1))
        out, nnz = blk.rmm(u)
        assert_close(out, D, u, "X %*% u")
        assert nnz == np.count_nonzero(out)
        assert "k_rmm_sdc_rows" not in kernels_of(blk, lambda: blk.rmm(u))
    finally:
        blk.close()


def assert_like_the_oracle(out, ref, Y, D, n_rows, what):
    """Cells the oracle's walk leaves non-finite are equal (also which infinity), the others within 1e-12."""
    fin = np.isfinite(ref)
    assert not fin.all() and fin.any()
    assert np.array_equal(np.isfinite(out), fin), f"{what}: finite cells differ"
    assert np.array_equal(out[~fin], ref[~fin], equal_nan=True), f"{what}: non-finite cells differ"
    clean = lambda a: np.nan_to_num(a, nan=0.0, posinf=0.0, neginf=0.0)
    scale = np.abs(clean(Y)) @ np.abs(clean(D))
    assert np.all(np.abs(out - ref)[fin] <= (1e-12 + n_rows * 2.0 ** -53) * scale[fin]), what


def test_non_finite_values(cla, ora):
    """Non-finite dictionary values and non-finite values of the vector end up where the reference puts them. The
    left multiply sums Y per tuple before it multiplies with the dictionary (ColGroupSDCZeros.leftMultByMatrixNoPreAgg
    / ADictionary pre-aggregation): an infinite dictionary value times values of Y of both signs is one infinity,
    not a NaN, and a row that a group does not list does not enter its sum (no inf * 0). The expected cells
    therefore come from the oracle's walk; padding entries of the lane-major and row lists must not add any."""
    n_rows = 20011
    specs, n = sdc_block(9, n_rows, 12, 0.03, 9)
    rng = np.random.default_rng(2)
    u = rng.standard_normal((n, 1))
    Y = rng.standard_normal((2, n_rows))
    Ybad = Y.copy()
    Ybad[0, 5] = np.inf      # a row that some groups list and others do not
    Ybad[1, 1500] = np.nan
    Ybad[1, n_rows - 1] = -np.inf
    # finite dictionaries: the lane-major kernel runs, the vector holds the non-finite values
    D = ora.np_decompress(specs, n_rows, n)
    G = ora.Groups(specs, n_rows, n)
    blk = cla.build_block(n_rows, n, specs)
    try:
        for mode in ("rows+lanes", "packed", "tiles"):
            set_mode(blk, mode)
            out, _ = blk.lmm(Ybad)
            assert_like_the_oracle(out, ora.lmm(G, Ybad)[0], Ybad, D, n_rows, f"{mode}: t(v) %*% X, non-finite vector")
        set_mode(blk, "rows+lanes")
        assert "k_lmm_sdc_lanes" in kernels_of(blk, lambda: blk.lmm(Ybad))
    finally:
        blk.close()
    # non-finite dictionary values
    specs[1].dict[2, 0] = np.inf
    specs[7].dict[0, 0] = np.nan
    D = ora.np_decompress(specs, n_rows, n)
    G = ora.Groups(specs, n_rows, n)
    blk = cla.build_block(n_rows, n, specs)
    try:
        for mode in ("rows+lanes", "lanes", "packed", "tiles"):
            set_mode(blk, mode)
            out, _ = blk.rmm(u)
            assert_close(out, D, u, f"{mode}: X %*% u, non-finite dictionary")
            for Yt in (Y, Ybad):
                out, _ = blk.lmm(Yt)
                assert_like_the_oracle(out, ora.lmm(G, Yt)[0], Yt, D, n_rows, f"{mode}: t(v) %*% X, non-finite dictionary")
    finally:
        blk.close()


@pytest.mark.parametrize("default", [None, 0.75])
def test_next_to_other_group_types(cla, ora, default):
    """DDC, RLE, uncompressed and constant groups next to the lists (the lists then add to what the other groups
    wrote), groups of two columns (right multiply only: the left multiply falls back), a non-zero default."""
    from systemds_amd import synth
    n_rows = 50021
    rng = np.random.default_rng(11)
    specs, c = sdc_block(3, n_rows, 30, 0.04, 12, default)
    more, c2 = sdc_block(4, n_rows, 3, 0.1, 5, default, n_cols_g=2)
    for s in more:
        s.cols = s.cols + c
    specs += more
    c += c2
    codes = rng.integers(0, 20, n_rows).astype(np.uint8)
    specs.append(synth.GroupSpec("ddc", np.array([c], np.int32), rng.standard_normal((20, 1)), codes))
    specs.append(synth.GroupSpec("const", np.array([c + 1], np.int32), rng.standard_normal((1, 1))))
    specs.append(synth.GroupSpec("unc", np.array([c + 2], np.int32), dense=rng.standard_normal((n_rows, 1))))
    c += 3
    D = ora.np_decompress(specs, n_rows, c)
    blk = cla.build_block(n_rows, c, specs)
    try:
        for mode in MODES:
            set_mode(blk, mode)
            u = rng.standard_normal((c, 1))
            out, nnz = blk.rmm(u)
            assert_close(out, D, u, f"{mode}: X %*% u")
            assert nnz == np.count_nonzero(out)
            Y = rng.standard_normal((2, n_rows))
            out, _ = blk.lmm(Y)
            assert_close(out, Y, D, f"{mode}: t(v) %*% X")
    finally:
        blk.close()


def test_repeated_calls_are_bit_identical(cla, ora):
    """The row lists hold every row's entries in a fixed order: X %*% u does not depend on how the conversion's
    or the kernel's waves were scheduled."""
    n_rows = 100003
    specs, n = sdc_block(21, n_rows, 100, 0.05, 64)
    u = np.random.default_rng(3).standard_normal((n, 1))
    outs = []
    for _ in range(2):
        blk = cla.build_block(n_rows, n, specs)
        out, _ = blk.rmm(u)
        out2, _ = blk.rmm(u)
        assert np.array_equal(out, out2)
        outs.append(out)
        blk.close()
    assert np.array_equal(outs[0], outs[1])
