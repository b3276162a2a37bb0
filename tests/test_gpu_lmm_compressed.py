"""GPU parity of the compressed x compressed left multiply (cla_lmm_compressed): t(left) %*% right
for two compressed blocks, as CLALibLeftMultBy.leftMultByMatrixTransposed does
(C/lib/CLALibLeftMultBy.java:100-112, 170-284), against the CPU oracle and the decompressed truth."""
import numpy as np
import pytest

from conftest import mixed_block
from parity import assert_fp64_close, assert_matches_truth

pytestmark = pytest.mark.gpu


def check(cla, ora, specsL, nL, specsR, nR, n_rows, what, keep=False, route=0):
    left = cla.build_block(n_rows, nL, specsL)
    right = cla.build_block(n_rows, nR, specsR).set_option("tsmm_route", route)
    out, nnz = right.lmm_compressed(left)
    ref, rnnz = ora.lmm_compressed(ora.Groups(specsR, n_rows, nR), ora.Groups(specsL, n_rows, nL))
    DL = ora.np_decompress(specsL, n_rows, nL)
    DR = ora.np_decompress(specsR, n_rows, nR)
    assert out.shape == (nL, nR)
    assert_matches_truth(out, DL.T, DR, what=what)
    assert_fp64_close(out, ref, ora.abs_matmul(DL.T, DR), what=what, n_terms=n_rows)
    assert nnz == rnnz
    if keep:
        return left, right, out
    left.close()
    right.close()


@pytest.mark.parametrize("path", [0, 1, 2], ids=["auto", "pairs", "decode"])
@pytest.mark.parametrize("seed,n_rows", [(0, 1), (1, 37), (2, 3000), (4, 150001)])
def test_mixed_groups(cla, ora, path, seed, n_rows):
    """Every pairing of DDC / SDC / SDCZeros / RLE / const / empty groups, on the per-pair path and on the
    decoded path (the library picks by cost; the option tsmm_route of the right block forces one)."""
    specsL, nL = mixed_block(seed, n_rows, with_unc=False)
    # two 70000-tuple dictionaries cannot meet on the per-pair path (the accumulator of either side exceeds LDS):
    # the library then decodes; the forced per-pair run keeps one of them small
    specsR, nR = mixed_block(seed + 50, n_rows, with_unc=False, with_const=seed % 2 == 0,
                             big_dict=path != 1)
    check(cla, ora, specsL, nL, specsR, nR, n_rows, f"t(L) %*% R route {path}", route=path)


@pytest.mark.parametrize("unc_l,unc_r", [(True, False), (False, True), (True, True)])
def test_uncompressed_groups(cla, ora, unc_l, unc_r):
    specsL, nL = mixed_block(5, 20011, with_unc=unc_l)
    specsR, nR = mixed_block(6, 20011, with_unc=unc_r)
    check(cla, ora, specsL, nL, specsR, nR, 20011, f"t(L) %*% R unc={unc_l},{unc_r}")


def test_not_transposed_and_cached(cla, ora):
    """Different column counts on the two sides; a second call reuses the joint descriptor, another left block
    replaces it, and swapping the operands gives the transpose."""
    n_rows = 70001
    specsL, nL = mixed_block(7, n_rows, with_unc=False, with_const=False)
    specsR, nR = mixed_block(8, n_rows, with_unc=False)
    assert nL != nR
    left, right, out = check(cla, ora, specsL, nL, specsR, nR, n_rows, "first", keep=True)
    again, _ = right.lmm_compressed(left)
    DL = ora.np_decompress(specsL, n_rows, nL)
    DR = ora.np_decompress(specsR, n_rows, nR)
    # (floating-point atomics: the order of the partial sums differs from call to call)
    assert_fp64_close(again, out, ora.abs_matmul(DL.T, DR), what="second call", n_terms=n_rows)
    swapped, _ = left.lmm_compressed(right)
    assert_fp64_close(swapped, out.T, ora.abs_matmul(DR.T, DL), what="swapped", n_terms=n_rows)
    specsO, nO = mixed_block(9, n_rows, with_unc=False)
    other = cla.build_block(n_rows, nO, specsO)
    left.close()   # the cached joint descriptor of (left, right) is stale now and must not be used
    out2, _ = right.lmm_compressed(other)
    assert_matches_truth(out2, ora.np_decompress(specsO, n_rows, nO).T, DR, what="other left")
    # the blocks still serve their own entry points
    ts, _ = right.tsmm()
    assert_matches_truth(ts, DR.T, DR, what="right tsmm after")
    other.close()
    right.close()


def test_same_block_is_tsmm(cla, ora):
    specs, n = mixed_block(10, 30000, with_unc=False)
    blk = cla.build_block(30000, n, specs)
    out, _ = blk.lmm_compressed(blk)
    ts, _ = blk.tsmm()
    D = ora.np_decompress(specs, 30000, n)
    assert_matches_truth(out, D.T, D, what="t(X) %*% X as compressed x compressed")
    assert_matches_truth(ts, D.T, D, what="t(X) %*% X")
    assert_fp64_close(out, ts, 2 * ora.abs_matmul(D.T, D), what="the two against each other")
    blk.close()


def test_wide_blocks_take_the_pair_path(cla, ora):
    """More than 64 columns over both blocks: only the per-pair path applies (C2- and C3-shaped blocks)."""
    from systemds_amd import synth
    a = synth.config2(scale=500, n_cols=60)
    b = synth.config3(scale=500)
    assert a["n_rows"] == b["n_rows"]
    check(cla, ora, a["groups"], a["n_cols"], b["groups"], b["n_cols"], a["n_rows"], "C2 x C3")


def test_errors(cla):
    specsL, nL = mixed_block(1, 100, with_unc=False)
    specsR, nR = mixed_block(2, 101, with_unc=False)
    left = cla.build_block(100, nL, specsL)
    right = cla.build_block(101, nR, specsR)
    with pytest.raises(cla.ClaError) as e:
        right.lmm_compressed(left)
    assert e.value.code == cla.ERR_INVALID
    left.close()
    right.close()


def test_uncompressed_groups_on_wide_blocks(cla, ora):
    """More than 64 columns over both blocks and an uncompressed group: chunks of the left side meet chunks of the
    right side as decoded blocks of at most 64 columns."""
    from systemds_amd import synth
    a = synth.config2(scale=1000, n_cols=70)
    specsU, nU = mixed_block(3, a["n_rows"], with_unc=True)
    check(cla, ora, specsU, nU, a["groups"], a["n_cols"], a["n_rows"], "t(unc) %*% wide")
    check(cla, ora, a["groups"], a["n_cols"], specsU, nU, a["n_rows"], "t(wide) %*% unc")


def test_overlapping_operand(cla, ora):
    """An overlapping block (the result of cla_rmm_overlapping) on either side: no per-cell-pair form exists, the
    joint rows are decompressed and multiplied on the matrix cores."""
    n_rows = 5000
    specs, n = mixed_block(11, n_rows, with_unc=False)
    D = ora.np_decompress(specs, n_rows, n)
    B = np.random.default_rng(1).standard_normal((n, 3))
    P = ora.longdouble_matmul(D, B)
    blk = cla.build_block(n_rows, n, specs)
    child = blk.rmm_overlapping(B)
    out, _ = blk.lmm_compressed(child)      # t(XB) %*% X
    absP = np.abs(D) @ np.abs(B)            # (bounds P's own rounding as well as its cells)
    assert_fp64_close(out, ora.longdouble_matmul(P.T, D), absP.T @ np.abs(D), what="t(XB) %*% X")
    out, _ = child.lmm_compressed(blk)      # t(X) %*% XB
    assert_fp64_close(out, ora.longdouble_matmul(D.T, P), np.abs(D).T @ absP, what="t(X) %*% XB")
    out, _ = blk.lmm_compressed(blk)
    assert_matches_truth(out, D.T, D, what="t(X) %*% X afterwards")
    child.close()
    blk.close()


def test_constants_only_on_one_side(cla, ora):
    """A block of const / empty groups only against a mixed block: the outer products with the column sums."""
    from systemds_amd import synth
    n_rows = 3000
    consts = [synth.GroupSpec("const", np.array([0, 2], np.int32), np.array([[1.5, -2.0]])),
              synth.GroupSpec("empty", np.array([1], np.int32))]
    specs, n = mixed_block(12, n_rows, with_unc=False)
    check(cla, ora, consts, 3, specs, n, n_rows, "const %*% mixed")
    check(cla, ora, specs, n, consts, 3, n_rows, "mixed %*% const")


@pytest.mark.parametrize("with_unc", [False, True])
def test_constant_columns_at_the_seam_of_wide_blocks(cla, ora, with_unc):
    """More than 64 columns over both blocks (column chunks), the right block starting and the left block ending
    with columns that only carry a constant: those belong to their own side, whichever group comes next."""
    from systemds_amd import synth
    n_rows = 1025
    rng = np.random.default_rng(77)

    def block(lead_const, trail_const, n_ddc):
        specs, c = [], 0
        if lead_const:
            specs.append(synth.GroupSpec("const", np.arange(c, c + 2, dtype=np.int32), rng.standard_normal((1, 2))))
            c += 2
        for _ in range(n_ddc):
            nv = int(rng.choice([3, 40, 300]))
            codes = rng.integers(0, nv, n_rows).astype(np.uint8 if nv <= 256 else np.uint16)
            specs.append(synth.GroupSpec("ddc", np.arange(c, c + 2, dtype=np.int32), rng.standard_normal((nv, 2)), codes))
            c += 2
        if with_unc:
            specs.append(synth.GroupSpec("unc", np.arange(c, c + 3, dtype=np.int32), dense=rng.standard_normal((n_rows, 3))))
            c += 3
        if trail_const:
            specs.append(synth.GroupSpec("const", np.arange(c, c + 3, dtype=np.int32), rng.standard_normal((1, 3))))
            c += 3
        return specs, c

    specsL, nL = block(True, True, 9)
    specsR, nR = block(True, True, 30)
    assert nL + nR > 64
    check(cla, ora, specsL, nL, specsR, nR, n_rows, "constants at the seam")
    check(cla, ora, specsR, nR, specsL, nL, n_rows, "constants at the seam, roles swapped")


def test_one_tuple_dictionary_against_many_rows(cla, ora):
    """A group with a single tuple (an SDC group of one value, 17 columns) against a DDC group of three tuples over
    100003 rows on the per-pair path: nearly every row adds one of three values into the same accumulator cells.
    Such a sum drifts with its length, so the row range per accumulator is kept short; the result stays within
    the 1e-12 bar of the exact product."""
    from systemds_amd import synth
    n_rows = 100003
    rng = np.random.default_rng(201)
    left = [synth.sdc_group(rng, n_rows, np.arange(0, 17, dtype=np.int32), 1, 0.6, 0.75)]
    right = [synth.GroupSpec("ddc", np.arange(0, 33, dtype=np.int32), rng.standard_normal((3, 33)),
                             rng.integers(0, 3, n_rows).astype(np.uint8)),
             synth.sdc_group(rng, n_rows, np.arange(33, 38, dtype=np.int32), 300, 0.1, 0.75),
             synth.GroupSpec("const", np.arange(38, 70, dtype=np.int32), rng.standard_normal((1, 32)))]
    L = cla.build_block(n_rows, 17, left)
    R = cla.build_block(n_rows, 70, right)
    try:
        out, _ = R.lmm_compressed(L)
        DL, DR = ora.np_decompress(left, n_rows, 17), ora.np_decompress(right, n_rows, 70)
        assert_matches_truth(out, DL.T, DR, what="one tuple x three tuples")
        out, _ = R.tsmm()
        assert_matches_truth(out, DR.T, DR, what="tsmm with a three-tuple dictionary")
    finally:
        L.close()
        R.close()
