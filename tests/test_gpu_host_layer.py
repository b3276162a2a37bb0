"""The CLALib* drivers of the C++ host layer on the GPU, against the dense product.

Written the way the reference's component tests are (CompressedTestBase.java: build a
CompressedMatrixBlock, run the operation compressed and on the decompressed MatrixBlock,
compare), over every logical-transpose combination CLALibMatrixMult accepts.
"""
import numpy as np
import pytest

from conftest import host_groups, mixed_block
from parity import assert_fp64_close

pytestmark = pytest.mark.gpu


def build(H, ora, seed, n_rows, **kw):
    specs, n_cols = mixed_block(seed, n_rows, **kw)
    cmb = H.CompressedMatrixBlock(n_rows, n_cols)
    cmb.allocateColGroupList(host_groups(H, ora, specs, n_rows))
    return cmb, ora.np_decompress(specs, n_rows, n_cols), specs


def close(got, A, B, what, ora):
    truth = ora.longdouble_matmul(A, B)
    assert_fp64_close(got, truth, np.abs(A) @ np.abs(B), what=what)


@pytest.mark.parametrize("seed,n_rows", [(0, 1), (1, 513), (2, 20000)])
def test_decompress(H, ora, cla, seed, n_rows):
    """Exact up to the SDC default-tuple morph (dict - default) + default, which the
    reference's decompression performs as well (CLALibDecompress.java:310-357)."""
    cmb, D, _ = build(H, ora, seed, n_rows)
    out = cmb.decompress(4)
    assert_fp64_close(out.toArray(), D, np.abs(D) + 2.0, what="decompress")
    sdc_cols = [5, 6]   # the SDC group with a default tuple
    keep = np.setdiff1d(np.arange(D.shape[1]), sdc_cols)
    assert np.array_equal(out.toArray()[:, keep], D[:, keep])
    assert out.getNonZeros() == np.count_nonzero(out.toArray())
    assert np.array_equal(H.CLALibDecompress.decompress(cmb, 1).toArray(), out.toArray())


@pytest.mark.parametrize("seed,n_rows", [(3, 77), (4, 30000)])
def test_matrix_multiply_all_transpose_combinations(H, ora, cla, seed, n_rows):
    cmb, D, _ = build(H, ora, seed, n_rows)
    n_cols = D.shape[1]
    rng = np.random.default_rng(seed)
    mm = H.CLALibMatrixMult.matrixMultiply
    B = rng.standard_normal((n_cols, 3))
    Y = rng.standard_normal((2, n_rows))
    # compressed on the left
    close(mm(cmb, H.MatrixBlock(B), 4).toArray(), D, B, "X %*% B", ora)
    close(mm(cmb, H.MatrixBlock(B.T.copy()), 4, False, True).toArray(), D, B, "X %*% t(Bt)", ora)
    close(mm(cmb, H.MatrixBlock(Y.T.copy()), 4, True, False).toArray(), D.T, Y.T, "t(X) %*% Yt", ora)
    close(mm(cmb, H.MatrixBlock(Y), 4, True, True).toArray(), D.T, Y.T, "t(X) %*% t(Y)", ora)
    # compressed on the right
    close(mm(H.MatrixBlock(Y), cmb, 4).toArray(), Y, D, "Y %*% X", ora)
    close(mm(H.MatrixBlock(Y.T.copy()), cmb, 4, True, False).toArray(), Y, D, "t(Yt) %*% X", ora)
    close(mm(H.MatrixBlock(B.T.copy()), cmb, 4, False, True).toArray(), B.T, D.T, "Bt %*% t(X)", ora)
    close(mm(H.MatrixBlock(B), cmb, 4, True, True).toArray(), B.T, D.T, "t(B) %*% t(X)", ora)
    # the member entry point checks dimensions like checkAggregateBinaryOperations
    ret = cmb.aggregateBinaryOperations(cmb, H.MatrixBlock(B), 4)
    close(ret.toArray(), D, B, "aggregateBinaryOperations", ora)
    assert ret.getNonZeros() == np.count_nonzero(ret.toArray())
    with pytest.raises(H.DMLRuntimeException):
        cmb.aggregateBinaryOperations(cmb, H.MatrixBlock(Y), 4)


def test_left_mult_drivers(H, ora, cla):
    cmb, D, _ = build(H, ora, 6, 9000)
    rng = np.random.default_rng(6)
    Y = rng.standard_normal((3, 9000))
    close(H.CLALibLeftMultBy.leftMultByMatrix(cmb, H.MatrixBlock(Y), 2).toArray(), Y, D, "leftMultByMatrix", ora)
    close(H.CLALibLeftMultBy.leftMultByMatrixTransposed(cmb, H.MatrixBlock(Y.T.copy()), 2).toArray(), Y, D,
          "leftMultByMatrixTransposed", ora)


def test_both_sides_compressed(H, ora, cla):
    a, DA, _ = build(H, ora, 7, 300)
    b, DB, _ = build(H, ora, 8, 300)
    mm = H.CLALibMatrixMult.matrixMultiply
    close(mm(a, b, 1, True, False).toArray(), DA.T, DB, "t(A) %*% B compressed-compressed", ora)
    # the wider block takes the right-hand role and the result is transposed back (CLALibMatrixMult.java:104-111)
    w, DW, _ = build(H, ora, 9, 300, with_unc=False)
    assert DW.shape[1] != DA.shape[1]
    close(mm(a, w, 1, True, False).toArray(), DA.T, DW, "t(A) %*% W", ora)
    close(mm(w, a, 1, True, False).toArray(), DW.T, DA, "t(W) %*% A", ora)
    close(H.CLALibLeftMultBy.leftMultByMatrixTransposed(w, a, 2).toArray(), DA.T, DW, "leftMultByMatrixTransposed(cmb, cmb)", ora)
    short, _, _ = build(H, ora, 10, 200)
    with pytest.raises(H.DMLCompressionException):
        H.CLALibLeftMultBy.leftMultByMatrixTransposed(a, short, 1)
    c = H.CompressedMatrixBlock(DA.shape[1], 2)
    c.allocateColGroupList([H.ColGroupUncompressed.create(H.MatrixBlock(np.random.default_rng(1).standard_normal((DA.shape[1], 2))))])
    close(mm(a, c, 1).toArray(), DA, c.decompress().toArray(), "A %*% C compressed-compressed", ora)


@pytest.mark.parametrize("with_unc", [False, True])
def test_tsmm(H, ora, cla, with_unc):
    cmb, D, _ = build(H, ora, 9, 12000, with_unc=with_unc)
    for ret in (H.CLALibTSMM.leftMultByTransposeSelf(cmb, 4), cmb.transposeSelfMatrixMultOperations(H.MMTSJType.LEFT, 4)):
        T = ret.toArray()
        close(T, D.T, D, "t(X) %*% X", ora)
        assert np.array_equal(T, T.T)
        assert ret.getNonZeros() == np.count_nonzero(T)


def test_mmchain_all_types(H, ora, cla):
    cmb, D, _ = build(H, ora, 10, 15000)
    rng = np.random.default_rng(10)
    n_cols = D.shape[1]
    v = rng.standard_normal((n_cols, 1))
    w = rng.standard_normal((15000, 1))
    Dl, vl, wl = D.astype(np.longdouble), v.astype(np.longdouble), w.astype(np.longdouble)
    scale = np.abs(D).T @ (np.abs(D) @ np.abs(v))
    for ct, want, sc in ((H.ChainType.XtXv, Dl.T @ (Dl @ vl), scale),
                         (H.ChainType.XtwXv, Dl.T @ (wl * (Dl @ vl)), np.abs(D).T @ (np.abs(w) * (np.abs(D) @ np.abs(v)))),
                         (H.ChainType.XtXvy, Dl.T @ ((Dl @ vl) - wl), scale + np.abs(D).T @ np.abs(w))):
        got = cmb.chainMatrixMultOperations(H.MatrixBlock(v), None if ct == H.ChainType.XtXv else H.MatrixBlock(w), ct, 4)
        assert (got.getNumRows(), got.getNumColumns()) == (n_cols, 1)
        assert_fp64_close(got.toArray(), want.astype(np.float64), sc, what=f"mmchain {ct}")


def test_overlapping_groups(H, ora, cla):
    """Groups that share columns (the result of a compressed right multiply) add up."""
    cmb, D, _ = build(H, ora, 11, 4000, overlap=True)
    cmb.setOverlapping(True)
    assert cmb.isOverlapping()
    assert_fp64_close(cmb.decompress().toArray(), D, np.abs(D) + 1.0, what="overlapping decompress", n_terms=4)
    B = np.random.default_rng(11).standard_normal((D.shape[1], 2))
    got = H.CLALibRightMultBy.rightMultByMatrix(cmb, H.MatrixBlock(B), 2).toArray()
    assert_fp64_close(got, ora.longdouble_matmul(D, B), np.abs(D) @ np.abs(B) + 1.0, what="overlapping X %*% B")
    with pytest.raises(H.NotImplementedException):
        H.CLALibRightMultBy.rightMultByMatrix(cmb, H.MatrixBlock(B), 2, True)


def test_group_list_can_be_replaced(H, ora, cla):
    """allocateColGroupList drops the device copy of the previous groups."""
    cmb, D, specs = build(H, ora, 12, 1000)
    B = np.ones((D.shape[1], 1))
    first = H.CLALibRightMultBy.rightMultByMatrix(cmb, H.MatrixBlock(B)).toArray()
    specs2, _ = mixed_block(13, 1000)
    cmb.allocateColGroupList(host_groups(H, ora, specs2, 1000))
    D2 = ora.np_decompress(specs2, 1000, D.shape[1])
    second = H.CLALibRightMultBy.rightMultByMatrix(cmb, H.MatrixBlock(B)).toArray()
    close(first, D, B, "before", ora)
    close(second, D2, B, "after", ora)


@pytest.mark.parametrize("seed,n_rows", [(5, 300), (6, 40000)])
def test_serialised_block_goes_straight_to_the_device(H, ora, cla, seed, n_rows):
    """Bytes in the layout of CompressedMatrixBlock.write (C/CompressedMatrixBlock.java:493-523), written by the
    Python restatement in the type variants the reference's factories pick from, are read into column groups and
    multiplied on the GPU without a JVM in between."""
    from oracle import cla_wire
    specs, n_cols = mixed_block(seed, n_rows, with_unc=True)
    D = ora.np_decompress(specs, n_rows, n_cols)
    variants = []
    for i, s in enumerate(specs):
        v = {}
        if s.type == "ddc" and i % 2 == 0:
            v["dict"] = "MATRIX_BLOCK_DICT"
            v["block"] = "SPARSE_BLOCK"
        if s.type == "unc":
            v["block"] = "SPARSE_BLOCK"
        if len(s.cols) > 2:
            v["index"] = "ARRAY"
        variants.append(v)
    cmb = H.readCompressedMatrixBlock(cla_wire.compressed_block(n_rows, n_cols, specs, variants=variants))
    rng = np.random.default_rng(seed)
    B = rng.standard_normal((n_cols, 5))
    Y = rng.standard_normal((2, n_rows))
    mm = H.CLALibMatrixMult.matrixMultiply
    close(mm(cmb, H.MatrixBlock(B), 4).toArray(), D, B, "X %*% B from bytes", ora)
    close(mm(H.MatrixBlock(Y), cmb, 4).toArray(), Y, D, "Y %*% X from bytes", ora)
    close(cmb.transposeSelfMatrixMultOperations(H.MMTSJType.LEFT, 4).toArray(), D.T, D, "t(X) %*% X from bytes", ora)


def test_overlapping_right_multiply_stays_compressed(H, ora, cla):
    """rightMultByMatrix with allowOverlap (RMMOverlapping, CLALibRightMultBy.java:157-201): the product is a
    compressed block again and feeds the next multiplies without ever being decompressed."""
    n_rows = 30000
    cmb, D, _ = build(H, ora, 8, n_rows, with_unc=False)
    rng = np.random.default_rng(8)
    B = rng.standard_normal((D.shape[1], 4))
    xb = H.rightMultByMatrixOverlapping(cmb, H.MatrixBlock(B), 4)
    assert xb.isCompressed() and xb.isOverlapping() and xb.isDeviceOnly()
    assert (xb.getNumRows(), xb.getNumColumns()) == (n_rows, 4)
    P = ora.longdouble_matmul(D, B)
    absP = np.abs(D) @ np.abs(B)
    assert_fp64_close(xb.decompress(4).toArray(), P, absP, what="decompress(XB)")
    C = rng.standard_normal((4, 3))
    mm = H.CLALibMatrixMult.matrixMultiply
    assert_fp64_close(mm(xb, H.MatrixBlock(C), 4).toArray(), ora.longdouble_matmul(P, C), absP @ np.abs(C), what="(XB) %*% C")
    Y = rng.standard_normal((2, n_rows))
    assert_fp64_close(mm(H.MatrixBlock(Y), xb, 4).toArray(), ora.longdouble_matmul(Y, P), np.abs(Y) @ absP, what="Y %*% (XB)")
    # t(XB) %*% (XB) is not linear in the groups: the library decompresses the block and multiplies on the matrix
    # cores, as the reference does for overlapping blocks (CLALibTSMM.java:73-77)
    tsmm = xb.transposeSelfMatrixMultOperations(H.MMTSJType.LEFT, 4).toArray()
    assert_fp64_close(tsmm, ora.longdouble_matmul(P.T, P), absP.T @ absP, what="t(XB) %*% (XB)")  # (absP: the rounding of P = X B enters too)
    with pytest.raises(H.NotImplementedException):
        H.writeCompressedMatrixBlock(xb)
    with pytest.raises(H.NotImplementedException):   # by-value result cannot be compressed
        H.CLALibRightMultBy.rightMultByMatrix(cmb, H.MatrixBlock(B), 4, True)
