"""Full-size runs of the benchmark configurations through the C ABI.

At these sizes a dense copy of X does not fit comfortably, so the checks are
  * the CPU oracle on the same compressed input where it finishes in seconds, and
  * size-independent properties that tie the entry points to each other and to
    closed forms computed with numpy from the codes alone:
      adjoint      y (X v)          == (y X) v
      gram         v' (X'X) v       == |X v|^2
      linearity    X (a u + b w)    == a X u + b X w
      columns      (X B)[:, j]      == X B[:, j]
      counts       cla_counts       == bincount(codes)             (integers, exact)
      co-occurrence cla_cooc        == bincount(codesA * nB + codesB) (integers, exact)
      gram cells   (X'X)[a, b]      == sum_k counts[k] d[k, a] d[k, b]
fp64 tolerance: 1e-12 relative to the magnitude of the summed terms (parity.py);
scalar identities that sum over all rows use 1e-10 of the absolute sum, which one
dropped or doubled row out of 10^7 still violates by three orders of magnitude.
"""
import numpy as np
import pytest

from parity import assert_fp64_close

pytestmark = pytest.mark.gpu

CPU_THREADS = 16


def col_max(specs, n_cols):
    """max |X[:, c]| per column, from the dictionaries / dense values."""
    m = np.zeros(n_cols)
    for s in specs:
        if s.type == "unc":
            v = np.abs(s.dense).max(axis=0)
        elif s.type == "empty":
            continue
        else:
            v = np.abs(s.dict).max(axis=0)
            if s.default is not None:
                v = np.maximum(v, np.abs(s.default))
        np.maximum.at(m, s.cols, v)
    return m


def rmm_scale(specs, n_rows, n_cols, B):
    """Upper bound of |X| @ |B|, the same for every row."""
    return np.broadcast_to(col_max(specs, n_cols) @ np.abs(B), (n_rows, B.shape[1]))


def ld_dot(a, b):
    return float(np.dot(np.asarray(a, np.longdouble).ravel(), np.asarray(b, np.longdouble).ravel()))


def assert_scalar_close(a, b, scale, what, tol=1e-10):
    assert abs(a - b) <= tol * scale, f"{what}: {a!r} vs {b!r} (scale {scale:.3e})"


# --------------------------------------------------------------------------- C2
@pytest.fixture(scope="module")
def c2(cla, ora):
    from systemds_amd import synth
    c = synth.config2()
    blk = cla.build_block(c["n_rows"], c["n_cols"], c["groups"])
    yield c, blk, ora.Groups(c["groups"], c["n_rows"], c["n_cols"])
    blk.close()


def test_c2_matvec_bit_exact_against_oracle(c2, ora):
    c, blk, G = c2
    out, nnz = blk.rmm(c["v"])
    ref, rnnz = ora.rmm(G, c["v"], CPU_THREADS)
    assert np.array_equal(out, ref)
    assert nnz == rnnz == np.count_nonzero(out)


def test_c2_matmat_columns_equal_matvecs(c2):
    """The wide multiply (matrix-core path) against the mat-vec gather, which is
    bit-exact against the oracle."""
    c, blk, _ = c2
    B = c["B"]
    out, nnz = blk.rmm(B)
    assert out.shape == (c["n_rows"], 64)
    assert nnz == np.count_nonzero(out)
    scale = rmm_scale(c["groups"], c["n_rows"], c["n_cols"], B)
    for j in (0, 31, 63):
        col, _ = blk.rmm(np.ascontiguousarray(B[:, j:j + 1]))
        assert_fp64_close(out[:, j:j + 1], col, scale[:, j:j + 1], what=f"C2 X%*%B column {j}")


def test_c2_linearity_and_adjoint(c2):
    c, blk, _ = c2
    rng = np.random.default_rng(7)
    n, m = c["n_rows"], c["n_cols"]
    u, w = rng.standard_normal((m, 1)), rng.standard_normal((m, 1))
    Xu, _ = blk.rmm(u)
    Xw, _ = blk.rmm(w)
    Xc, _ = blk.rmm(2.0 * u - 3.0 * w)
    scale = rmm_scale(c["groups"], n, m, 2.0 * np.abs(u) + 3.0 * np.abs(w))
    assert_fp64_close(Xc, 2.0 * Xu - 3.0 * Xw, scale, what="C2 linearity", n_terms=4)
    y = rng.standard_normal((1, n))
    yX, _ = blk.lmm(y)
    assert yX.shape == (1, m)
    assert_scalar_close(ld_dot(y, Xu), ld_dot(yX, u), ld_dot(np.abs(y), np.abs(Xu)) + ld_dot(np.abs(yX), np.abs(u)),
                        "C2 adjoint y(Xu) == (yX)u")


def test_c2_lmm_and_mmchain_against_oracle(c2, ora):
    c, blk, G = c2
    rng = np.random.default_rng(8)
    n, m = c["n_rows"], c["n_cols"]
    Y = rng.standard_normal((2, n))
    out, nnz = blk.lmm(Y)
    ref, rnnz = ora.lmm(G, Y, CPU_THREADS)
    cm = col_max(c["groups"], m)
    scale = np.abs(Y).sum(axis=1, keepdims=True) * cm[None, :]
    # both sides sum 10^7 terms per cell in different orders: allow the a-priori bound sqrt(n) u
    assert_fp64_close(out, ref, scale, what="C2 lmm", n_terms=int(np.sqrt(n)))
    assert nnz == rnnz
    v = c["v"]
    w = rng.standard_normal((n, 1))
    for ctype, ww in ((0, None), (1, w)):
        got, _ = blk.mmchain(v, ww, ctype)
        Xv, _ = blk.rmm(v)
        t = Xv if ww is None else Xv * ww
        want, _ = blk.lmm(np.ascontiguousarray(t.T))
        sc = np.abs(t).sum() * cm[:, None]
        assert_fp64_close(got.reshape(-1, 1), want.T, sc, what=f"C2 mmchain ctype={ctype}", n_terms=int(np.sqrt(n)))


def test_c2_counts_exact(c2):
    c, blk, _ = c2
    for g in (0, 17, 99):
        got = blk.counts(g)
        want = np.bincount(c["groups"][g].codes, minlength=256)
        assert np.array_equal(got, want)
        assert int(got.sum()) == c["n_rows"]


def test_c2_gram_of_100_single_column_groups(c2):
    """t(X) %*% X of the 100-column block (column chunks, decoded Gram matrix per pair of chunks): the gram
    identity on all cells, diagonal cells from the counts and cells of two pairs of groups (inside one chunk
    and across chunks) from the integer co-occurrence table."""
    c, blk, _ = c2
    n, m = c["n_rows"], c["n_cols"]
    T, nnz = blk.tsmm()
    assert T.shape == (m, m)
    assert np.array_equal(T, T.T)
    assert nnz == np.count_nonzero(T)
    v = np.random.default_rng(10).standard_normal((m, 1))
    Xv, _ = blk.rmm(v)
    lhs = float((v.T.astype(np.longdouble) @ T.astype(np.longdouble) @ v.astype(np.longdouble))[0, 0])
    assert_scalar_close(lhs, ld_dot(Xv, Xv), float((np.abs(v).T @ np.abs(T) @ np.abs(v))[0, 0]), "C2 v'(X'X)v == |Xv|^2")
    for g in (0, 31, 32, 64, 99):
        s = c["groups"][g]
        cl = np.bincount(s.codes, minlength=s.n_vals).astype(np.longdouble)
        d = s.dict[:, 0].astype(np.longdouble)
        a = int(s.cols[0])
        assert abs(T[a, a] - float(np.sum(cl * d * d))) <= 1e-12 * float(np.sum(cl * d * d)), (g, T[a, a])
    for ga, gb in ((3, 20), (5, 70), (40, 99)):
        sa, sb = c["groups"][ga], c["groups"][gb]
        co = np.bincount(sa.codes.astype(np.int64) * sb.n_vals + sb.codes, minlength=sa.n_vals * sb.n_vals)
        co = co.reshape(sa.n_vals, sb.n_vals)
        assert np.array_equal(blk.cooc(ga, gb), co)
        da, db = sa.dict[:, 0].astype(np.longdouble), sb.dict[:, 0].astype(np.longdouble)
        want = float(da @ co.astype(np.longdouble) @ db)
        sc = float(np.abs(da) @ co.astype(np.longdouble) @ np.abs(db))
        i, j = int(sa.cols[0]), int(sb.cols[0])
        assert abs(T[i, j] - want) <= 1e-12 * sc, (ga, gb, T[i, j], want)


# --------------------------------------------------------------------------- C3
@pytest.fixture(scope="module")
def c3(cla):
    from systemds_amd import synth
    c = synth.config3()
    blk = cla.build_block(c["n_rows"], c["n_cols"], c["groups"])
    yield c, blk
    blk.close()


def test_c3_tsmm_properties(c3):
    c, blk = c3
    n, m = c["n_rows"], c["n_cols"]
    T, nnz = blk.tsmm()
    assert T.shape == (m, m)
    assert np.array_equal(T, T.T)
    assert nnz == np.count_nonzero(T)
    # gram identity
    v = np.random.default_rng(9).standard_normal((m, 1))
    Xv, _ = blk.rmm(v)
    lhs = float((v.T.astype(np.longdouble) @ T.astype(np.longdouble) @ v.astype(np.longdouble))[0, 0])
    rhs = ld_dot(Xv, Xv)
    assert_scalar_close(lhs, rhs, float((np.abs(v).T @ np.abs(T) @ np.abs(v))[0, 0]), "C3 v'(X'X)v == |Xv|^2")
    # cells inside a group from the counts, cells across two groups from the co-occurrence table
    for g in (0, 11, 24):
        s = c["groups"][g]
        cnt = np.bincount(s.codes, minlength=s.n_vals)
        assert np.array_equal(blk.counts(g), cnt)
        a, b = int(s.cols[0]), int(s.cols[1])
        d = s.dict.astype(np.longdouble)
        cl = cnt.astype(np.longdouble)
        for (i, j, p, q) in ((a, a, 0, 0), (a, b, 0, 1), (b, b, 1, 1)):
            want = float(np.sum(cl * d[:, p] * d[:, q]))
            sc = float(np.sum(cl * np.abs(d[:, p] * d[:, q])))
            assert abs(T[i, j] - want) <= 1e-12 * sc, (g, i, j, T[i, j], want)
    for ga, gb in ((0, 1), (7, 23)):
        sa, sb = c["groups"][ga], c["groups"][gb]
        co = np.bincount(sa.codes.astype(np.int64) * sb.n_vals + sb.codes, minlength=sa.n_vals * sb.n_vals)
        co = co.reshape(sa.n_vals, sb.n_vals)
        assert np.array_equal(blk.cooc(ga, gb), co)
        col = co.astype(np.longdouble)
        for p in (0, 1):
            for q in (0, 1):
                da, db = sa.dict[:, p].astype(np.longdouble), sb.dict[:, q].astype(np.longdouble)
                want = float(da @ col @ db)
                sc = float(np.abs(da) @ col @ np.abs(db))
                i, j = int(sa.cols[p]), int(sb.cols[q])
                assert abs(T[i, j] - want) <= 1e-12 * sc, (ga, gb, i, j, T[i, j], want)


def test_c3_with_itself_as_two_compressed_operands(c3, cla):
    """t(L) %*% R with a second, separately built copy of the block on the left (100 joint columns: column
    chunks) equals the block's own Gram matrix."""
    c, blk = c3
    n, m = c["n_rows"], c["n_cols"]
    T, nnz = blk.tsmm()
    left = cla.build_block(n, m, c["groups"])
    try:
        out, onnz = blk.lmm_compressed(left)
    finally:
        left.close()
    assert out.shape == (m, m)
    cm = col_max(c["groups"], m)
    assert_fp64_close(out, T, n * np.outer(cm, cm), what="C3 t(X)%*%X as compressed x compressed", n_terms=int(np.sqrt(n)))
    assert onnz == np.count_nonzero(out)


# --------------------------------------------------------------------------- C4
@pytest.fixture(scope="module")
def c4(cla, ora):
    from systemds_amd import synth
    c = synth.config4()
    blk = cla.build_block(c["n_rows"], c["n_cols"], c["groups"])
    yield c, blk, ora.Groups(c["groups"], c["n_rows"], c["n_cols"])
    blk.close()


def test_c4_left_and_right_multiply(c4, ora):
    c, blk, G = c4
    n, m = c["n_rows"], c["n_cols"]
    cm = col_max(c["groups"], m)
    vX, nnz = blk.lmm(c["v"])
    ref, rnnz = ora.lmm(G, c["v"], CPU_THREADS)
    # 5% of the rows contribute to a cell
    assert_fp64_close(vX, ref, np.abs(c["v"]).sum() * 0.06 * cm[None, :], what="C4 t(v)%*%X", n_terms=int(np.sqrt(n)))
    assert nnz == rnnz
    Xu, nnz = blk.rmm(c["u"])
    ref, rnnz = ora.rmm(G, c["u"], CPU_THREADS)
    assert_fp64_close(Xu, ref, rmm_scale(c["groups"], n, m, c["u"]), what="C4 X%*%u", n_terms=m)
    assert nnz == rnnz == np.count_nonzero(Xu)
    assert_scalar_close(ld_dot(c["v"], Xu), ld_dot(vX, c["u"]),
                        ld_dot(np.abs(c["v"]), np.abs(Xu)) + ld_dot(np.abs(vX), np.abs(c["u"])), "C4 adjoint")
    for g in (0, 150):
        s = c["groups"][g]
        got = blk.counts(g)
        assert np.array_equal(got, np.bincount(s.codes, minlength=s.n_vals))
        assert int(got.sum()) == s.n_offsets


# --------------------------------------------------------------------------- C5
@pytest.fixture(scope="module")
def c5(cla, ora):
    from systemds_amd import synth
    c = synth.config5()
    blk = cla.build_block(c["n_rows"], c["n_cols"], c["groups"])
    yield c, blk, ora.Groups(c["groups"], c["n_rows"], c["n_cols"])
    blk.close()


def test_c5_mixed_right_multiply_and_gram(c5, ora):
    c, blk, G = c5
    n, m = c["n_rows"], c["n_cols"]
    B = c["B"]
    out, nnz = blk.rmm(B)
    ref, rnnz = ora.rmm(G, B, CPU_THREADS)
    assert_fp64_close(out, ref, rmm_scale(c["groups"], n, m, B), what="C5 X%*%B", n_terms=m)
    assert nnz == rnnz
    del ref
    T, tnnz = blk.tsmm()
    assert np.array_equal(T, T.T)
    assert tnnz == np.count_nonzero(T)
    v = np.ascontiguousarray(B[:, :1])
    Xv = out[:, 0]
    lhs = float((v.T.astype(np.longdouble) @ T.astype(np.longdouble) @ v.astype(np.longdouble))[0, 0])
    assert_scalar_close(lhs, ld_dot(Xv, Xv), float((np.abs(v).T @ np.abs(T) @ np.abs(v))[0, 0]), "C5 v'(X'X)v == |Xv|^2")
    dense = c["groups"][-1].dense
    for p in (0, 1):
        for q in (0, 1):
            want = ld_dot(dense[:, p], dense[:, q])
            sc = ld_dot(np.abs(dense[:, p]), np.abs(dense[:, q]))
            assert abs(T[18 + p, 18 + q] - want) <= 1e-10 * sc
