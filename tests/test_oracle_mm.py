"""Pins the oracle's multiply drivers against what the mathematics fixes:
closed-form decompression (numpy, independent of the C code) followed by a
long-double / fsum matrix product. The reference's own tests are differential
in the same way (CompressedTestBase.java:609-626, 666-685, 865-884)."""
import numpy as np
import pytest

from conftest import mixed_block

# fp64 bar: |oracle - truth| <= 1e-12 * (|A| @ |B|), i.e. relative to the magnitude
# of the terms of each dot product (plain per-cell relative error is meaningless
# for cells that cancel to ~0), and max-norm relative error <= 1e-12.
TOL = 1e-12


def assert_close(got, truth, scale, tol=TOL):
    got, truth, scale = np.asarray(got), np.asarray(truth), np.asarray(scale)
    err = np.abs(got - truth)
    bound = tol * np.maximum(scale, np.finfo(float).tiny)
    assert np.all(err <= bound), f"max err/scale {np.max(err / np.maximum(scale, 1e-300)):.3e}"
    assert err.max() <= tol * max(np.abs(truth).max(), 1e-300)


@pytest.mark.parametrize("seed,n_rows", [(0, 1), (1, 37), (2, 3000), (3, 20011)])
@pytest.mark.parametrize("k", [1, 4])
def test_rmm_equals_decompressed_product(ora, seed, n_rows, k):
    specs, n_cols = mixed_block(seed, n_rows)
    G = ora.Groups(specs, n_rows, n_cols)
    D = ora.np_decompress(specs, n_rows, n_cols)
    assert np.abs(ora.decompress(G) - D).max() <= 4e-16 * max(np.abs(D).max(), 1)
    rng = np.random.default_rng(seed + 100)
    for q in (1, 5):
        B = rng.standard_normal((n_cols, q))
        out, nnz = ora.rmm(G, B, k)
        assert_close(out, ora.longdouble_matmul(D, B), ora.abs_matmul(D, B))
        assert nnz == np.count_nonzero(out)


def test_rmm_tiny_fsum_truth(ora):
    specs, n_cols = mixed_block(7, 50)
    G = ora.Groups(specs, 50, n_cols)
    D = ora.np_decompress(specs, 50, n_cols)
    B = np.random.default_rng(8).standard_normal((n_cols, 3))
    out, _ = ora.rmm(G, B, 1)
    assert_close(out, ora.fsum_matmul(D, B), ora.abs_matmul(D, B))


def test_rmm_single_ddc_is_table_lookup(ora):
    # one single-column DDC group: out[r] = dict[code[r]] * v exactly (one product, no sum)
    from systemds_amd import synth
    rng = np.random.default_rng(3)
    d = rng.standard_normal((16, 1))
    codes = rng.integers(0, 16, 1000).astype(np.uint8)
    G = ora.Groups([synth.GroupSpec("ddc", np.array([0], np.int32), d, codes)], 1000, 1)
    out, _ = ora.rmm(G, np.array([[3.25]]), 1)
    assert np.array_equal(out[:, 0], d[codes, 0] * 3.25)


def test_preagg_values_skip_zero_and_order(ora):
    # zero dictionary cells are skipped (Dictionary.java:898-905): an inf in B must not
    # turn a zero tuple into NaN
    d = np.array([[0.0, 2.0], [1.0, 0.0]])
    B = np.array([[np.inf, 1.0], [3.0, 4.0]])
    T = ora.preagg_values_from_dense(d, np.array([0, 1], np.int32), B)
    assert np.array_equal(T, np.array([[6.0, 8.0], [np.inf, 1.0]]))


@pytest.mark.parametrize("seed,n_rows", [(0, 1), (1, 37), (2, 3000), (3, 20011)])
@pytest.mark.parametrize("k", [1, 4])
def test_lmm_equals_product_with_decompressed(ora, seed, n_rows, k):
    specs, n_cols = mixed_block(seed, n_rows)
    G = ora.Groups(specs, n_rows, n_cols)
    D = ora.np_decompress(specs, n_rows, n_cols)
    rng = np.random.default_rng(seed + 200)
    for p in (1, 6):
        Y = rng.standard_normal((p, n_rows))
        out, nnz = ora.lmm(G, Y, k)
        assert_close(out, ora.longdouble_matmul(Y, D), ora.abs_matmul(Y, D))
        assert nnz == np.count_nonzero(out)


def test_preaggregate_row_sum_identity(ora):
    # sum_k pre[i,k] = sum of Y[i, rows covered by the group]
    specs, n_cols = mixed_block(5, 4000)
    G = ora.Groups(specs, 4000, n_cols)
    Y = np.random.default_rng(6).standard_normal((3, 4000))
    for gi, s in enumerate(specs):
        if s.type not in ("ddc", "sdc", "rle"):
            continue
        pre = ora.preaggregate_dense(G, gi, Y)
        if s.type == "ddc":
            covered = np.ones(4000, bool)
        elif s.type == "sdc":
            covered = np.zeros(4000, bool)
            covered[ora.py_offset_decode(s.deltas, s.first)] = s.n_offsets > 0
        else:
            covered = np.zeros(4000, bool)
            for k in range(s.n_vals):
                covered[ora.py_rle_rows(s.ptr, s.rle, k)] = True
        assert np.allclose(pre.sum(axis=1), (Y * covered).sum(axis=1), rtol=0, atol=1e-11)


@pytest.mark.parametrize("seed,n_rows", [(0, 1), (1, 37), (2, 3000), (3, 20011)])
@pytest.mark.parametrize("k", [1, 4])
def test_tsmm_equals_gram_matrix(ora, seed, n_rows, k):
    for with_unc in (False, True):
        specs, n_cols = mixed_block(seed, n_rows, with_unc=with_unc)
        G = ora.Groups(specs, n_rows, n_cols)
        D = ora.np_decompress(specs, n_rows, n_cols)
        out, nnz = ora.tsmm(G, k)
        truth = ora.longdouble_matmul(D.T, D)
        assert_close(out, truth, ora.abs_matmul(D.T, D), tol=TOL)
        assert np.array_equal(out, out.T)
        assert nnz == np.count_nonzero(out)
        # every pair of DDC groups against the closed form t(dictA) %*% N %*% dictB with the integer co-occurrence
        # counts N = bincount(codeA * nB + codeB) (what preAggregateDDC_DDC + the dictionary product compute), in long double
        ddc = [s for s in specs if s.type == "ddc"]
        for i, a in enumerate(ddc):
            for b in ddc[i + 1:]:
                nA, nB = a.dict.shape[0], b.dict.shape[0]
                N = np.bincount(a.codes.astype(np.int64) * nB + b.codes.astype(np.int64), minlength=nA * nB).reshape(nA, nB)
                want = (a.dict.astype(np.longdouble).T @ N.astype(np.longdouble) @ b.dict.astype(np.longdouble)).astype(np.float64)
                scale = np.abs(a.dict).T @ N.astype(np.float64) @ np.abs(b.dict)
                assert_close(out[np.ix_(a.cols, b.cols)], want, scale, tol=TOL)


def test_tsmm_diagonal_closed_form(ora):
    # diag = sum_k counts[k] * dict[k]^2 for a lone DDC column (AColGroupCompressed.tsmmDense)
    from systemds_amd import synth
    rng = np.random.default_rng(9)
    d = rng.standard_normal((5, 1))
    codes = rng.integers(0, 5, 777).astype(np.uint8)
    G = ora.Groups([synth.GroupSpec("ddc", np.array([0], np.int32), d, codes),
                    synth.GroupSpec("ddc", np.array([1], np.int32), d, codes)], 777, 2)
    out, _ = ora.tsmm(G, 1)
    cnt = np.bincount(codes, minlength=5)
    assert np.array_equal(ora.counts(G, 0), cnt)
    assert abs(out[0, 0] - float((cnt * d[:, 0] ** 2).sum())) <= 1e-12 * out[0, 0]
    assert abs(out[0, 1] - out[0, 0]) <= 1e-12 * out[0, 0]


def test_counts_and_cooc_bit_exact(ora):
    specs, n_cols = mixed_block(4, 9000)
    G = ora.Groups(specs, 9000, n_cols)

    def row_codes(s):
        rc = np.full(9000, -1, np.int64)
        if s.type == "ddc":
            rc[:] = s.codes
        elif s.type == "sdc" and s.n_offsets:
            rc[ora.py_offset_decode(s.deltas, s.first)] = s.codes
        elif s.type == "rle":
            for k in range(s.n_vals):
                rc[ora.py_rle_rows(s.ptr, s.rle, k)] = k
        return rc
    coded = [i for i, s in enumerate(specs) if s.type in ("ddc", "sdc", "rle")]
    for i in coded:
        rc = row_codes(specs[i])
        assert np.array_equal(ora.counts(G, i), np.bincount(rc[rc >= 0], minlength=specs[i].n_vals))
    for i in coded:
        for j in coded:
            if specs[i].n_vals * specs[j].n_vals > 200000:
                continue
            a, b = row_codes(specs[i]), row_codes(specs[j])
            m = (a >= 0) & (b >= 0)
            truth = np.zeros((specs[i].n_vals, specs[j].n_vals), np.int64)
            np.add.at(truth, (a[m], b[m]), 1)
            N = ora.cooc(G, i, j)
            assert np.array_equal(N, truth)
            assert np.array_equal(N.sum(axis=1), np.bincount(a[m], minlength=specs[i].n_vals))


def test_mmchain(ora):
    """XtXv and XtwXv against the chain accumulated in long double, at the 1e-12 bar of the path: relative to
    the magnitude of the terms summed into each cell, |D|' (|w| * (|D| |v|))."""
    specs, n_cols = mixed_block(12, 2500)
    G = ora.Groups(specs, 2500, n_cols)
    D = ora.np_decompress(specs, 2500, n_cols)
    L = D.astype(np.longdouble)
    rng = np.random.default_rng(13)
    v, w = rng.standard_normal(n_cols), rng.standard_normal(2500)
    inner_scale = np.abs(D) @ np.abs(v)
    out, _ = ora.mmchain(G, v, None, 0)
    truth = (L.T @ (L @ v.astype(np.longdouble))).astype(np.float64)
    assert_close(out.reshape(-1), truth, np.abs(D).T @ inner_scale)
    out, _ = ora.mmchain(G, v, w, 1)
    truth = (L.T @ (w.astype(np.longdouble) * (L @ v.astype(np.longdouble)))).astype(np.float64)
    assert_close(out.reshape(-1), truth, np.abs(D).T @ (np.abs(w) * inner_scale))


def test_edge_sdc_lists(ora):
    from systemds_amd import synth
    n_rows = 70000
    rng = np.random.default_rng(1)
    for rows in ([], [0], [n_rows - 1], [3, 69999], [0, 255, 510, 66000], list(range(0, n_rows, 1))):
        rows = np.array(rows, np.int64)
        d = rng.standard_normal((3, 1))
        codes = rng.integers(0, 3, rows.size).astype(np.uint8)
        deltas, first, last, n = synth.encode_offsets(rows)
        for default in (None, np.array([0.5])):
            s = synth.GroupSpec("sdc", np.array([0], np.int32), d, codes, default, deltas, first, last, n)
            G = ora.Groups([s], n_rows, 1)
            D = ora.np_decompress([s], n_rows, 1)
            out, _ = ora.rmm(G, np.array([[2.0]]), 1)
            assert np.allclose(out, D * 2.0, rtol=1e-15, atol=0)
            Y = rng.standard_normal((2, n_rows))
            out, _ = ora.lmm(G, Y, 1)
            assert np.allclose(out, Y @ D, rtol=1e-12, atol=1e-11)


# ---------------------------------------------------------------------------
# compressed x compressed: t(left) %*% right (CLALibLeftMultBy.java:100-112, 249-284)
# ---------------------------------------------------------------------------
def _cc_truth(ora, specsL, nL, specsR, nR, n_rows):
    DL = ora.np_decompress(specsL, n_rows, nL)
    DR = ora.np_decompress(specsR, n_rows, nR)
    return DL, DR


@pytest.mark.parametrize("seed,n_rows", [(0, 1), (1, 37), (2, 3000), (3, 20011)])
@pytest.mark.parametrize("unc_l,unc_r", [(False, False), (True, False), (False, True), (True, True)])
def test_lmm_compressed_equals_decompressed_product(ora, seed, n_rows, unc_l, unc_r):
    specsL, nL = mixed_block(seed, n_rows, with_unc=unc_l)
    specsR, nR = mixed_block(seed + 50, n_rows, with_unc=unc_r, with_const=seed % 2 == 0)
    DL, DR = _cc_truth(ora, specsL, nL, specsR, nR, n_rows)
    out, nnz = ora.lmm_compressed(ora.Groups(specsR, n_rows, nR), ora.Groups(specsL, n_rows, nL))
    assert out.shape == (nL, nR)
    assert_close(out, ora.longdouble_matmul(DL.T, DR), ora.abs_matmul(DL.T, DR))
    assert nnz == np.count_nonzero(out)


def test_lmm_compressed_tiny_fsum_truth(ora):
    specsL, nL = mixed_block(11, 50)
    specsR, nR = mixed_block(12, 50)
    DL, DR = _cc_truth(ora, specsL, nL, specsR, nR, 50)
    out, _ = ora.lmm_compressed(ora.Groups(specsR, 50, nR), ora.Groups(specsL, 50, nL))
    assert_close(out, ora.fsum_matmul(DL.T, DR), ora.abs_matmul(DL.T, DR))


def test_lmm_compressed_is_not_its_transpose(ora):
    # a transposed operand (t(right) %*% left) or swapped output strides must fail: nL != nR and asymmetric data
    specsL, nL = mixed_block(21, 400, with_unc=False, with_const=False)
    specsR, nR = mixed_block(22, 400, with_unc=True)
    assert nL != nR
    DL, DR = _cc_truth(ora, specsL, nL, specsR, nR, 400)
    out, _ = ora.lmm_compressed(ora.Groups(specsR, 400, nR), ora.Groups(specsL, 400, nL))
    assert_close(out, ora.longdouble_matmul(DL.T, DR), ora.abs_matmul(DL.T, DR))
    other, _ = ora.lmm_compressed(ora.Groups(specsL, 400, nL), ora.Groups(specsR, 400, nR))
    assert_close(other, out.T, ora.abs_matmul(DR.T, DL))


def test_lmm_compressed_same_block_is_tsmm(ora):
    # left is right (same index structures, the dictionaries meet scaled by the counts): equals the TSMM
    specs, n = mixed_block(31, 5000, with_unc=False)
    G = ora.Groups(specs, 5000, n)
    out, _ = ora.lmm_compressed(G, G)
    D = ora.np_decompress(specs, 5000, n)
    assert_close(out, ora.longdouble_matmul(D.T, D), ora.abs_matmul(D.T, D))
    ts, _ = ora.tsmm(G)
    assert_close(out, ts, 2 * ora.abs_matmul(D.T, D))


def test_lmm_compressed_constants_only(ora):
    # const x const: n * cL (x) cR exactly; const x DDC: cL (x) colSums(right)
    from systemds_amd import synth
    n = 1000
    cl = synth.GroupSpec("const", np.array([0, 1], np.int32), np.array([[2.0, -3.0]]))
    cr = synth.GroupSpec("const", np.array([0], np.int32), np.array([[0.5]]))
    out, _ = ora.lmm_compressed(ora.Groups([cr], n, 1), ora.Groups([cl], n, 2))
    assert np.array_equal(out, np.array([[1000.0], [-1500.0]]))
    codes = (np.arange(n) % 4).astype(np.uint8)
    dd = synth.GroupSpec("ddc", np.array([0], np.int32), np.array([[1.0], [2.0], [4.0], [8.0]]), codes)
    out, _ = ora.lmm_compressed(ora.Groups([dd], n, 1), ora.Groups([cl], n, 2))
    assert np.array_equal(out, np.array([[2.0 * 250 * 15], [-3.0 * 250 * 15]]))
