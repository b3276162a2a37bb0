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


# worst observed error / scale of the strict 1e-12 checks against long-double truths, per config
WORST = {}


def note(config, err_over_scale):
    WORST[config] = max(WORST.get(config, 0.0), float(err_over_scale))


def assert_cell(got, want, scale, what, config, tol=1e-12):
    """One cell of a result against its closed form accumulated in long double."""
    err = abs(float(got) - float(want)) / max(float(scale), 1e-300)
    note(config, err)
    assert err <= tol, f"{what}: {got!r} vs {want!r}, err/scale {err:.3e}"


def row_codes(spec, n_rows):
    """(codes[n_rows], values[nCodes] long double) of a single-column group: X[r, col] = values[codes[r]].
    Vectorised twins of AIterator / the RLE run walk (numpy only; the oracle's C code is not involved):
    SDC rows from the cumulated delta entries (a 0 entry adds 255 or 65535 and lists no row), the default as
    one more code; RLE runs marked with +-(k + 1) at their ends and cumulated, zero rows as one more code."""
    d = np.asarray(spec.dict, np.float64)[:, 0]
    nv = d.size
    if spec.type == "ddc":
        return spec.codes, d.astype(np.longdouble)
    if spec.type == "sdc":
        default = 0.0 if spec.default is None else float(spec.default[0])
        codes = np.full(n_rows, nv, np.int32)
        if spec.n_offsets > 0:
            dl = np.asarray(spec.deltas)
            max_v = 65535 if dl.dtype == np.uint16 else 255
            inc = np.where(dl == 0, max_v, dl).astype(np.int64)
            rows = np.concatenate(([spec.first], spec.first + np.cumsum(inc)[dl != 0]))
            assert rows.size == spec.n_offsets and rows[-1] == spec.last
            codes[rows] = spec.codes
        return codes, np.concatenate((d, [default])).astype(np.longdouble)
    assert spec.type == "rle"
    mark = np.zeros(n_rows + 1, np.int32)
    for k in range(nv):
        pairs = np.asarray(spec.rle[spec.ptr[k]:spec.ptr[k + 1]], np.int64).reshape(-1, 2)
        ends = np.cumsum(pairs.sum(axis=1))
        starts = ends - pairs[:, 1]
        keep = pairs[:, 1] > 0
        np.add.at(mark, starts[keep], k + 1)
        np.add.at(mark, ends[keep], -(k + 1))
    codes = np.cumsum(mark[:-1], dtype=np.int32) - 1
    codes[codes < 0] = nv
    return codes, np.concatenate((d, [0.0])).astype(np.longdouble)


def coded_cell(ca, va, cb, vb):
    """sum_r va[ca[r]] * vb[cb[r]] and sum_r |.| from the exact integer co-occurrence table."""
    N = np.bincount(ca.astype(np.int64) * vb.size + cb, minlength=va.size * vb.size).reshape(va.size, vb.size)
    NL = N.astype(np.longdouble)
    return float(va @ NL @ vb), float(np.abs(va) @ NL @ np.abs(vb))


def dense_coded_cell(x, cb, vb):
    """sum_r x[r] * vb[cb[r]]: per-code sums of x in chunks of 2^20 rows (each chunk summed in fp64 by bincount,
    2^20 * 2^-53 = 1.2e-10 of a chunk's |sum| at the very worst, 1e-13 in practice; chunks and codes cumulated
    in long double)."""
    S = np.zeros(vb.size, np.longdouble)
    A = np.zeros(vb.size, np.longdouble)
    for i in range(0, x.size, 1 << 20):
        xs, cs = x[i:i + (1 << 20)], cb[i:i + (1 << 20)]
        S += np.bincount(cs, weights=xs, minlength=vb.size)
        A += np.bincount(cs, weights=np.abs(xs), minlength=vb.size)
    return float(S @ vb), float(A @ np.abs(vb))


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
    """The wide multiply (matrix-core path): three columns against the mat-vec gather (which is bit-exact against
    the oracle), and all 64 columns of 120,000 sampled rows against the long-double product of the rows decoded
    from the codes in numpy, at the strict 1e-12 bar."""
    from parity import assert_matches_truth
    c, blk, _ = c2
    B = c["B"]
    out, nnz = blk.rmm(B)
    assert out.shape == (c["n_rows"], 64)
    assert nnz == np.count_nonzero(out)
    scale = rmm_scale(c["groups"], c["n_rows"], c["n_cols"], B)
    for j in (0, 31, 63):
        col, _ = blk.rmm(np.ascontiguousarray(B[:, j:j + 1]))
        assert_fp64_close(out[:, j:j + 1], col, scale[:, j:j + 1], what=f"C2 X%*%B column {j}")
    rows = np.sort(np.random.default_rng(21).choice(c["n_rows"], 120_000, replace=False))
    rows[:3] = (0, 1, c["n_rows"] - 1)  # the first and the last row are always among them
    rows.sort()
    D = np.stack([g.dict[g.codes[rows], 0] for g in c["groups"]], axis=1)
    note("C2 X%*%B", assert_matches_truth(out[rows], D, B, what="C2 X%*%B, 120000 sampled rows x 64 columns"))


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
    # all 25 blocks inside a group from the counts; cells across 20 pairs of groups from the co-occurrence table
    # (numpy bincount of the code pairs; for two of the pairs also cla_cooc, bit for bit)
    for g in range(len(c["groups"])):
        s = c["groups"][g]
        cnt = np.bincount(s.codes, minlength=s.n_vals)
        if g in (0, 11, 24):
            assert np.array_equal(blk.counts(g), cnt)
        a, b = int(s.cols[0]), int(s.cols[1])
        d = s.dict.astype(np.longdouble)
        cl = cnt.astype(np.longdouble)
        for (i, j, p, q) in ((a, a, 0, 0), (a, b, 0, 1), (b, b, 1, 1)):
            want = float(np.sum(cl * d[:, p] * d[:, q]))
            sc = float(np.sum(cl * np.abs(d[:, p] * d[:, q])))
            assert_cell(T[i, j], want, sc, f"C3 group {g} cell ({i},{j})", "C3 t(X)%*%X")
    rng = np.random.default_rng(33)
    pairs = {(0, 1), (7, 23), (0, 24), (11, 12)}
    while len(pairs) < 20:
        ga, gb = sorted(rng.choice(len(c["groups"]), 2, replace=False).tolist())
        pairs.add((ga, gb))
    for ga, gb in sorted(pairs):
        sa, sb = c["groups"][ga], c["groups"][gb]
        co = np.bincount(sa.codes.astype(np.int64) * sb.n_vals + sb.codes, minlength=sa.n_vals * sb.n_vals)
        co = co.reshape(sa.n_vals, sb.n_vals)
        if (ga, gb) in ((0, 1), (7, 23)):
            assert np.array_equal(blk.cooc(ga, gb), co)
        col = co.astype(np.longdouble)
        db = sb.dict.astype(np.longdouble)
        P, PA = col @ db, col @ np.abs(db)   # 4096 x 2 each
        for p in (0, 1):
            da = sa.dict[:, p].astype(np.longdouble)
            for q in (0, 1):
                i, j = int(sa.cols[p]), int(sb.cols[q])
                assert_cell(T[i, j], float(da @ P[:, q]), float(np.abs(da) @ PA[:, q]), f"C3 groups {ga},{gb} cell ({i},{j})",
                            "C3 t(X)%*%X")


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
    # strict bar against long-double closed forms: every cell of t(v) %*% X from the per-code sums of v over the
    # group's listed rows, and X %*% u on 50,000 sampled rows decoded from the offset lists
    from parity import assert_matches_truth
    v = c["v"].reshape(-1)
    sample = np.sort(np.random.default_rng(23).choice(n, 50_000, replace=False))
    D = np.zeros((sample.size, m))
    for g, s in enumerate(c["groups"]):
        dl = np.asarray(s.deltas)
        inc = np.where(dl == 0, 255 if dl.dtype == np.uint8 else 65535, dl).astype(np.int64)
        rows = np.concatenate(([s.first], s.first + np.cumsum(inc)[dl != 0]))
        assert rows.size == s.n_offsets
        want, sc = dense_coded_cell(v[rows], s.codes, s.dict[:, 0].astype(np.longdouble))
        assert_cell(vX[0, g], want, sc, f"C4 t(v)%*%X column {g}", "C4 t(v)%*%X")
        pos = np.searchsorted(rows, sample)
        hit = (pos < rows.size) & (rows[np.minimum(pos, rows.size - 1)] == sample)
        D[hit, g] = s.dict[s.codes[pos[hit]], 0]
    note("C4 X%*%u", assert_matches_truth(Xu[sample], D, c["u"], what="C4 X%*%u, 50000 sampled rows"))


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
    # Cells of every class at the strict bar, from closed forms that need no dense copy of X: every column as
    # one code per row plus a value table (RLE by run expansion of that column, SDC from its offset rows), cells
    # of two coded columns from the integer co-occurrence of their codes, dense x coded from per-code sums of the
    # dense column, dense x dense by a long-double dot product.
    specs = c["groups"]
    col = {}
    for s in specs:
        if s.type != "unc":
            col[int(s.cols[0])] = row_codes(s, n)
    dense = specs[-1].dense
    kinds = {"rle": range(0, 8), "ddc": range(8, 16), "sdc": range(16, 18), "dense": range(18, 20)}
    cells = [(a, a) for a in range(m)]                                   # the whole diagonal
    cells += [(0, 1), (2, 7), (8, 9), (10, 15), (16, 17), (18, 19)]      # inside a class
    cells += [(0, 8), (3, 12), (7, 15), (1, 16), (6, 17), (9, 16), (14, 17), (2, 18), (5, 19), (11, 18), (13, 19),
              (16, 18), (17, 19)]                                        # every pair of classes
    for a, b in cells:
        if a in col and b in col:
            want, sc = coded_cell(*col[a], *col[b])
        elif a in col or b in col:
            k, x = (a, dense[:, b - 18]) if a in col else (b, dense[:, a - 18])
            want, sc = dense_coded_cell(x, *col[k])
        else:
            want, sc = ld_dot(dense[:, a - 18], dense[:, b - 18]), ld_dot(np.abs(dense[:, a - 18]), np.abs(dense[:, b - 18]))
        ka = next(k for k, r in kinds.items() if a in r)
        kb = next(k for k, r in kinds.items() if b in r)
        assert_cell(T[a, b], want, sc, f"C5 t(X)%*%X cell ({a},{b}) {ka} x {kb}", "C5 t(X)%*%X")
    # X %*% B on 100,000 sampled rows decoded from the same per-column codes, against the long-double product
    from parity import assert_matches_truth
    rows = np.sort(np.random.default_rng(22).choice(n, 100_000, replace=False))
    D = np.empty((rows.size, m))
    for a in range(m):
        D[:, a] = np.asarray(col[a][1][col[a][0][rows]], np.float64) if a in col else dense[rows, a - 18]
    note("C5 X%*%B", assert_matches_truth(out[rows], D, B, what="C5 X%*%B, 100000 sampled rows"))


def test_zz_report_worst_errors():
    """Writes the worst err/scale seen by the strict checks of this module (for the design notes); runs last."""
    import json
    import os
    print("worst err/scale against long-double truths:", json.dumps(WORST))
    out_dir = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "gpurun_out")
    if os.path.isdir(out_dir):
        with open(os.path.join(out_dir, "full_size_parity.json"), "w") as f:
            json.dump(WORST, f, indent=1)
    assert all(v <= 1e-12 for v in WORST.values())
