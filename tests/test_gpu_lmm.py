"""GPU parity of the left multiply (cla_lmm), pre-aggregation (cla_preagg) and the
mm-chain (cla_mmchain) against the CPU oracle, through the C ABI."""
import numpy as np
import pytest

from conftest import mixed_block
from parity import assert_fp64_close, assert_matches_truth

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed,n_rows", [(0, 1), (1, 37), (2, 3000), (3, 20011), (4, 200003)])
@pytest.mark.parametrize("p", [1, 3])
def test_mixed_groups_lmm(cla, ora, seed, n_rows, p):
    specs, n_cols = mixed_block(seed, n_rows)
    Y = np.random.default_rng(seed + 70).standard_normal((p, n_rows))
    blk = cla.build_block(n_rows, n_cols, specs)
    out, nnz = blk.lmm(Y)
    blk.close()
    ref, rnnz = ora.lmm(ora.Groups(specs, n_rows, n_cols), Y, 4)
    D = ora.np_decompress(specs, n_rows, n_cols)
    assert_matches_truth(out, Y, D, what=f"lmm p={p}")
    assert_fp64_close(out, ref, ora.abs_matmul(Y, D), what=f"lmm p={p}", n_terms=n_rows)
    assert nnz == rnnz


def test_c4_scaled_both_products(cla, ora):
    """BASELINE config 4 at 1/50 scale (200,000 x 200 SDCZeros): t(v) %*% X and X %*% u."""
    from systemds_amd import synth
    c = synth.config4(scale=50)
    n_rows, n_cols = c["n_rows"], c["n_cols"]
    blk = cla.build_block(n_rows, n_cols, c["groups"])
    G = ora.Groups(c["groups"], n_rows, n_cols)
    D = ora.np_decompress(c["groups"], n_rows, n_cols)
    out, nnz = blk.lmm(c["v"])
    ref, rnnz = ora.lmm(G, c["v"], 4)
    assert_matches_truth(out, c["v"], D, what="C4 t(v)%*%X")
    assert_fp64_close(out, ref, ora.abs_matmul(c["v"], D), what="C4 t(v)%*%X", n_terms=n_rows)
    assert nnz == rnnz
    out, nnz = blk.rmm(c["u"])
    ref, rnnz = ora.rmm(G, c["u"], 4)
    assert_matches_truth(out, D, c["u"], what="C4 X%*%u")
    assert_fp64_close(out, ref, ora.abs_matmul(D, c["u"]), what="C4 X%*%u", n_terms=n_cols)
    assert nnz == rnnz
    blk.close()


def test_c2_scaled_left_vector(cla, ora):
    from systemds_amd import synth
    c = synth.config2(scale=100, n_cols=40)
    n_rows, n_cols = c["n_rows"], c["n_cols"]
    y = np.random.default_rng(5).standard_normal((1, n_rows))
    blk = cla.build_block(n_rows, n_cols, c["groups"])
    out, nnz = blk.lmm(y)
    blk.close()
    ref, rnnz = ora.lmm(ora.Groups(c["groups"], n_rows, n_cols), y, 4)
    D = ora.np_decompress(c["groups"], n_rows, n_cols)
    assert_matches_truth(out, y, D, what="C2 t(y)%*%X")
    assert_fp64_close(out, ref, ora.abs_matmul(y, D), what="C2 t(y)%*%X", n_terms=n_rows)
    assert nnz == rnnz


def test_preagg_per_group(cla, ora):
    specs, n_cols = mixed_block(11, 30011, with_unc=False)
    Y = np.random.default_rng(12).standard_normal((2, 30011))
    blk = cla.build_block(30011, n_cols, specs)
    G = ora.Groups(specs, 30011, n_cols)
    gi = 0
    for i, s in enumerate(specs):
        if s.type in ("ddc", "sdc", "rle"):
            pre = blk.preagg(gi, Y)
            ref = ora.preaggregate_dense(G, i, Y)
            scale = np.zeros_like(ref)
            refabs = ora.preaggregate_dense(G, i, np.abs(Y))
            assert_fp64_close(pre, ref, refabs + scale, what=f"preagg {s.type}", n_terms=30011)
            # sum over bins = sum of Y over the rows the group covers
            assert np.allclose(pre.sum(axis=1), ref.sum(axis=1), rtol=0, atol=1e-9)
        if s.type not in ("const", "empty"):
            gi += 1
    blk.close()


@pytest.mark.parametrize("ctype", [0, 1])
def test_mmchain(cla, ora, ctype):
    specs, n_cols = mixed_block(21, 40009)
    rng = np.random.default_rng(22)
    v, w = rng.standard_normal(n_cols), rng.standard_normal(40009)
    blk = cla.build_block(40009, n_cols, specs)
    out, nnz = blk.mmchain(v, w if ctype else None, ctype)
    blk.close()
    ref, rnnz = ora.mmchain(ora.Groups(specs, 40009, n_cols), v, w if ctype else None, ctype, 4)
    D = ora.np_decompress(specs, 40009, n_cols)
    inner = np.abs(D) @ np.abs(v)
    if ctype:
        inner = inner * np.abs(w)
    scale = np.abs(D).T @ inner
    assert_fp64_close(out, ref, scale, what="mmchain", n_terms=40009)
    assert nnz == rnnz


@pytest.mark.parametrize("n_rows", [1, 15, 16, 1023, 1024, 1025, 40000, 131072 + 17])
@pytest.mark.parametrize("n_col_g", [1, 2])
@pytest.mark.parametrize("p", [1, 3])
def test_byte_code_blocks_left_multiply(cla, ora, n_rows, n_col_g, p):
    """All groups DDC with byte codes (one code arena): single-column groups take the
    dot-product kernel, co-coded groups the LDS-bin kernel; group counts that do not fill a
    slab, ragged row counts, several rows of Y, a constant group on top."""
    from systemds_amd import synth
    rng = np.random.default_rng(1000 * n_col_g + n_rows % 977 + p)
    n_groups = 23
    specs = []
    for g in range(n_groups):
        n_vals = [2, 17, 256, 100][g % 4]
        cols = np.arange(g * n_col_g, (g + 1) * n_col_g, dtype=np.int32)
        specs.append(synth.GroupSpec("ddc", cols, rng.standard_normal((n_vals, n_col_g)),
                                     rng.integers(0, n_vals, n_rows).astype(np.uint8)))
    n_cols = n_groups * n_col_g + 1
    specs.append(synth.GroupSpec("const", np.array([n_cols - 1], np.int32), np.array([[1.25]])))
    Y = rng.standard_normal((p, n_rows))
    blk = cla.build_block(n_rows, n_cols, specs)
    out, nnz = blk.lmm(Y)
    blk.close()
    D = ora.np_decompress(specs, n_rows, n_cols)
    assert_matches_truth(out, Y, D, what=f"byte-code lmm nColG={n_col_g} p={p}")
    ref, rnnz = ora.lmm(ora.Groups(specs, n_rows, n_cols), Y, 4)
    assert_fp64_close(out, ref, ora.abs_matmul(Y, D), what="byte-code lmm vs oracle", n_terms=n_rows)
    assert nnz == rnnz


def test_mmchain_minus_y(cla, ora):
    """Chain type XtXvy, t(X) %*% ((X %*% v) - y) (CLALibMMChain.java:52), against the exactly accumulated product
    of the decompressed matrix and against the composition of the two multiplies."""
    from parity import assert_matches_truth
    specs, n_cols = mixed_block(23, 40009)
    rng = np.random.default_rng(24)
    v, y = rng.standard_normal(n_cols), rng.standard_normal(40009)
    blk = cla.build_block(40009, n_cols, specs)
    try:
        out, nnz = blk.mmchain(v, y, 2)
        Xv, _ = blk.rmm(v.reshape(-1, 1))
        D = ora.np_decompress(specs, 40009, n_cols)
        assert_matches_truth(out.reshape(-1, 1), D.T, Xv - y.reshape(-1, 1), what="mmchain XtXvy")
        assert nnz == np.count_nonzero(out)
        with pytest.raises(cla.ClaError):
            blk.mmchain(v, None, 2)
        with pytest.raises(cla.ClaError):
            blk.mmchain(v, y, 3)
    finally:
        blk.close()


def test_byte_code_block_with_non_finite_dictionary_values(cla, ora):
    """All groups DDC with byte codes and one column (the dot-form kernel's case): the reference sums Y per tuple
    first and multiplies once (APreAgg.leftMultByMatrix, ADictionary pre-aggregation), so an infinite dictionary
    value under rows of Y of both signs gives one infinity, where Y[r] * dict[code] summed over the rows would give
    NaN. Blocks with such a dictionary take the bin kernels; the cells are the oracle's."""
    from systemds_amd import synth
    c = synth.config2(scale=200, n_cols=24)
    n_rows, n_cols = c["n_rows"], c["n_cols"]
    c["groups"][3].dict[5, 0] = np.inf
    c["groups"][8].dict[0, 0] = -np.inf
    c["groups"][11].dict[2, 0] = np.nan
    Y = np.random.default_rng(6).standard_normal((2, n_rows))
    blk = cla.build_block(n_rows, n_cols, c["groups"])
    try:
        out, nnz = blk.lmm(Y)
        blk.profile(True)
        blk.lmm(Y)
        names = [k["name"] for k in blk.stats()["kernels"]]
        blk.profile(False)
    finally:
        blk.close()
    assert "k_lmm_u8_dot" not in names, names
    ref, rnnz = ora.lmm(ora.Groups(c["groups"], n_rows, n_cols), Y, 4)
    fin = np.isfinite(ref)
    assert not fin.all() and np.array_equal(np.isfinite(out), fin)
    assert np.array_equal(out[~fin], ref[~fin], equal_nan=True)
    D = np.nan_to_num(ora.np_decompress(c["groups"], n_rows, n_cols), nan=0.0, posinf=0.0, neginf=0.0)
    assert_fp64_close(out[fin], ref[fin], ora.abs_matmul(Y, D)[fin], what="t(Y)%*%X, non-finite dictionary", n_terms=n_rows)
    assert nnz == rnnz


@pytest.mark.parametrize("p", [1, 2, 5, 8, 16, 17, 40])
def test_mixed_block_takes_one_decoded_pass(cla, ora, p):
    """C5's shape (RLE, two-byte DDC, offset lists with a default, dense columns): Y %*% X in one pass over the decoded
    rows on the matrix cores, Y as the other operand (`k_lmm_decode`); with the option off the bin kernels give the
    same cells."""
    from systemds_amd import synth
    c = synth.config5(scale=400)
    n_rows, n_cols = c["n_rows"], c["n_cols"]
    Y = np.random.default_rng(p).standard_normal((p, n_rows))
    D = ora.np_decompress(c["groups"], n_rows, n_cols)
    blk = cla.build_block(n_rows, n_cols, c["groups"])
    try:
        out, nnz = blk.lmm(Y)
        blk.profile(True)
        out2, _ = blk.lmm(Y)
        names = [k["name"] for k in blk.stats()["kernels"]]
        blk.profile(False)
        blk.set_option("lmm_joint", 0)
        bins, nnz_b = blk.lmm(Y)
    finally:
        blk.close()
    assert "k_lmm_decode" in names and "k_lmm_preagg_rows" not in names, names
    assert_matches_truth(out, Y, D, what=f"Y %*% X, {p} rows")
    assert_matches_truth(bins, Y, D, what=f"Y %*% X, {p} rows, bin kernels")
    assert_matches_truth(out2, Y, D, what=f"Y %*% X, {p} rows, second call")  # (sums of block partials by atomic adds: the order varies)
    assert nnz == np.count_nonzero(out) and nnz_b == np.count_nonzero(bins)


def test_mixed_block_with_non_finite_values_in_y(cla, ora):
    """An infinite Y at a row that an RLE group's runs or an offset list do not cover stays out of that group's sums
    (the reference aggregates listed rows only): such a Y takes the bin kernels; the cells are the oracle's."""
    n_rows = 40001
    specs, n_cols = mixed_block(13, n_rows, with_unc=True)
    Y = np.random.default_rng(8).standard_normal((2, n_rows))
    Y[0, 7] = np.inf
    Y[1, n_rows - 3] = -np.inf
    Y[1, 12345] = np.nan
    blk = cla.build_block(n_rows, n_cols, specs)
    try:
        out, nnz = blk.lmm(Y)
    finally:
        blk.close()
    ref, rnnz = ora.lmm(ora.Groups(specs, n_rows, n_cols), Y, 4)
    fin = np.isfinite(ref)
    assert np.array_equal(np.isfinite(out), fin)
    assert np.array_equal(out[~fin], ref[~fin], equal_nan=True)
    D = ora.np_decompress(specs, n_rows, n_cols)
    Yc = np.nan_to_num(Y, nan=0.0, posinf=0.0, neginf=0.0)
    assert_fp64_close(out[fin], ref[fin], ora.abs_matmul(Yc, D)[fin], what="Y %*% X, non-finite Y", n_terms=n_rows)


@pytest.mark.parametrize("p", [1, 16, 17, 33])
def test_wide_dense_groups_on_the_matrix_cores(cla, ora, p):
    """Uncompressed groups of 70 and 5 columns (more than one set of four 16-column blocks, a ragged last block) beside
    a DDC group, 20,011 rows (a ragged last row tile per wave): `k_lmm_unc` takes 16 rows of Y per pass."""
    from systemds_amd import synth
    rng = np.random.default_rng(40 + p)
    n_rows, n_cols = 20011, 77
    perm = rng.permutation(n_cols).astype(np.int32)
    dense_a = rng.standard_normal((n_rows, 70))
    dense_a[rng.random((n_rows, 70)) < 0.3] = 0.0
    specs = [synth.GroupSpec("unc", np.sort(perm[:70]), dense=dense_a),
             synth.GroupSpec("unc", np.sort(perm[70:75]), dense=rng.standard_normal((n_rows, 5))),
             synth.GroupSpec("ddc", np.sort(perm[75:]), rng.standard_normal((9, 2)), rng.integers(0, 9, n_rows).astype(np.uint8))]
    Y = rng.standard_normal((p, n_rows))
    D = ora.np_decompress(specs, n_rows, n_cols)
    blk = cla.build_block(n_rows, n_cols, specs)
    try:
        blk.profile(True)
        out, nnz = blk.lmm(Y)
        names = [k["name"] for k in blk.stats()["kernels"]]
    finally:
        blk.close()
    assert "k_lmm_unc" in names, names
    ref, rnnz = ora.lmm(ora.Groups(specs, n_rows, n_cols), Y, 4)
    assert_matches_truth(out, Y, D, what=f"Y %*% X, dense groups, {p} rows")
    assert_fp64_close(out, ref, ora.abs_matmul(Y, D), what=f"Y %*% X, dense groups, {p} rows", n_terms=n_rows)
    assert nnz == rnnz


@pytest.mark.parametrize("shape", ["bytes100", "words60", "mixed"])
@pytest.mark.parametrize("p", [14, 40])
def test_many_rows_of_y_in_chunks_of_columns(cla, ora, shape, p):
    """Blocks that the decode kernel does not take whole go chunk of columns by chunk: 100 single-column byte-code
    groups (the dot kernel serves few rows of Y), 60 columns of two-byte codes (their code tiles exceed LDS
    together), about 100 columns of mixed groups with constant-only columns between them."""
    from systemds_amd import synth
    rng = np.random.default_rng(len(shape) + p)
    n_rows = 30011
    if shape == "bytes100":
        n_cols = 100
        specs = [synth.GroupSpec("ddc", np.array([c], np.int32), rng.standard_normal((50, 1)), rng.integers(0, 50, n_rows).astype(np.uint8))
                 for c in range(n_cols)]
    elif shape == "words60":
        n_cols = 60
        specs = [synth.GroupSpec("ddc", np.array([c], np.int32), rng.standard_normal((700, 1)), rng.integers(0, 700, n_rows).astype(np.uint16))
                 for c in range(n_cols)]
    else:
        specs, n_cols = [], 0
        for k in range(7):
            part, m = mixed_block(50 + k, n_rows, with_unc=True, big_dict=False)
            for g in part:
                g.cols = (np.asarray(g.cols) + n_cols).astype(np.int32)
            specs += part
            n_cols += m + 2  # two columns that no group covers
        specs.append(synth.GroupSpec("const", np.array([n_cols - 1], np.int32), np.array([[0.75]])))
    Y = rng.standard_normal((p, n_rows))
    D = ora.np_decompress(specs, n_rows, n_cols)
    blk = cla.build_block(n_rows, n_cols, specs)
    try:
        out, nnz = blk.lmm(Y)
        blk.profile(True)
        out2, nnz2 = blk.lmm(Y)
        names = [k["name"] for k in blk.stats()["kernels"]]
        blk.profile(False)
        blk.set_option("lmm_joint", 0)
        bins, nnz_b = blk.lmm(Y)
    finally:
        blk.close()
    assert "k_lmm_decode" in names and "k_scatter_cols" in names, (n_cols, names)
    assert_matches_truth(out, Y, D, what=f"Y %*% X in column chunks, {shape}, {p} rows")
    assert_matches_truth(out2, Y, D, what=f"Y %*% X in column chunks, {shape}, {p} rows, second call")
    assert_matches_truth(bins, Y, D, what=f"Y %*% X, {shape}, {p} rows, bin kernels")
    assert nnz == np.count_nonzero(out) and nnz2 == np.count_nonzero(out2) and nnz_b == np.count_nonzero(bins)


def test_repeated_calls_count_their_own_non_zeros(cla, ora):
    """The kernels that serve a whole block count the result's non-zeros themselves (the last workgroup to finish
    does and leaves its ticket counter at zero): calls in a row with different numbers of rows of Y, also queued
    without a wait between them, each report their own count."""
    from devmem import DevBuf
    from systemds_amd import synth
    n_rows, n_cols = 60000, 24
    rng = np.random.default_rng(77)
    specs = [synth.GroupSpec("ddc", np.array([c], np.int32), np.where(rng.random((40, 1)) < 0.3, 0.0, rng.standard_normal((40, 1))),
                             rng.integers(0, 40, n_rows).astype(np.uint8)) for c in range(n_cols)]
    blk = cla.build_block(n_rows, n_cols, specs)
    Ys = [rng.standard_normal((p, n_rows)) * (rng.random((p, 1)) < 0.7) for p in (1, 3, 2, 5, 1)]
    names = set()
    for rep in range(4):
        for Y in Ys:
            out, nnz = blk.lmm(Y)
            assert nnz == np.count_nonzero(out)
            names |= {k["name"] for k in blk.stats()["kernels"]}
    assert "k_lmm_u8_dot" in names and "k_lmm_finish" not in names, names
    # queued back to back on the block's stream: the last call's count is the one reported
    dY = [DevBuf.from_numpy(Y) for Y in Ys]
    dO = [DevBuf(Y.shape[0] * n_cols * 8) for Y in Ys]
    for Y, y, o in zip(Ys, dY, dO):
        blk.lmm_dev_async(y.ptr, Y.shape[0], o.ptr)
    last = blk.nnz()
    outs = [o.to_numpy((Y.shape[0], n_cols)) for o, Y in zip(dO, Ys)]
    assert last == np.count_nonzero(outs[-1])
    for got, Y in zip(outs, Ys):
        assert np.array_equal(got != 0, blk.lmm(Y)[0] != 0)
    blk.close()
