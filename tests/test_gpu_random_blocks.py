"""Randomised differential test through the C ABI: blocks of random group mixes (every group type, one to three
columns per group, dictionaries from 1 to 5000 tuples, row counts around the tile sizes, narrow blocks and blocks of
more than 64 columns) through every multiply, the chain, the sums and the compressed x compressed product, each
against the exactly accumulated (long double) product of the decompressed matrix, as the reference's own tests
compare every compressed operation with the uncompressed one (CompressedTestBase.java:507-522, 609-626, 666-685)."""
import numpy as np
import pytest

from parity import assert_matches_truth

pytestmark = pytest.mark.gpu

ROWS = [1, 63, 1023, 1024, 1025, 4096, 4097, 30000, 100003]


def rand_block(rng, n_rows, max_groups, allow_unc=True):
    from systemds_amd import synth
    specs, c = [], 0

    def cols(n):
        nonlocal c
        r = np.arange(c, c + n, dtype=np.int32)
        c += n
        return r

    for _ in range(int(rng.integers(1, max_groups + 1))):
        kind = rng.choice(["ddc", "ddc", "sdc", "sdcz", "rle", "unc", "const", "empty"])
        if kind == "unc" and not allow_unc:
            kind = "ddc"
        nc = int(rng.choice([1, 1, 2, 3]))
        if kind == "ddc":
            nv = int(rng.choice([1, 3, 16, 256, 300, 5000]))
            codes = rng.integers(0, nv, n_rows).astype(np.uint8 if nv <= 256 else np.uint16)
            specs.append(synth.GroupSpec("ddc", cols(nc), rng.standard_normal((nv, nc)), codes))
        elif kind in ("sdc", "sdcz"):
            dens = float(rng.choice([0.0005, 0.01, 0.1, 0.6]))
            specs.append(synth.sdc_group(rng, n_rows, cols(nc), int(rng.choice([1, 5, 64, 300])), dens,
                                         None if kind == "sdcz" else 0.75))
        elif kind == "rle":
            nv = int(rng.choice([1, 4, 32]))
            run_codes = rng.integers(-1, nv, size=n_rows // int(rng.choice([3, 50, 1000])) + 2)
            run_lens = rng.integers(1, int(rng.choice([4, 100, 3000])), size=run_codes.size)
            codes = np.repeat(run_codes, run_lens)[:n_rows]
            if codes.size < n_rows:
                codes = np.concatenate([codes, np.full(n_rows - codes.size, -1)])
            ptr, data = synth.encode_rle(codes, nv)
            specs.append(synth.GroupSpec("rle", cols(1), rng.standard_normal((nv, 1)), ptr=ptr, rle=data))
        elif kind == "unc":
            specs.append(synth.GroupSpec("unc", cols(nc), dense=rng.standard_normal((n_rows, nc))))
        elif kind == "const":
            specs.append(synth.GroupSpec("const", cols(nc), rng.standard_normal((1, nc))))
        else:
            specs.append(synth.GroupSpec("empty", cols(nc)))
    return specs, c


@pytest.mark.parametrize("seed,max_groups", [(7, 12), (11, 12), (59, 12), (23, 45), (31, 45), (47, 60)])
def test_random_blocks_against_the_decompressed_product(cla, ora, seed, max_groups):
    rng = np.random.default_rng(seed)
    for case in range(5):
        n_rows = int(rng.choice(ROWS))
        specs, n = rand_block(rng, n_rows, max_groups)
        what = f"seed {seed} case {case}: {n_rows} x {n} {[s.type for s in specs]}"
        D = ora.np_decompress(specs, n_rows, n)
        blk = cla.build_block(n_rows, n, specs)
        try:
            for q in (1, int(rng.choice([2, 5, 10, 16])), int(rng.choice([17, 40, 64]))):
                B = rng.standard_normal((n, q))
                out, nnz = blk.rmm(B)
                assert_matches_truth(out, D, B, what=f"{what} rmm q={q}")
                assert nnz == np.count_nonzero(out)
            for p in (1, 3):
                Y = rng.standard_normal((p, n_rows))
                out, _ = blk.lmm(Y)
                assert_matches_truth(out, Y, D, what=f"{what} lmm p={p}")
            out, _ = blk.tsmm()
            assert_matches_truth(out, D.T, D, what=f"{what} tsmm")
            v, w = rng.standard_normal((n, 1)), rng.standard_normal((n_rows, 1))
            out, _ = blk.mmchain(v, w, 1)
            Xv, _ = blk.rmm(v)
            assert_matches_truth(out.reshape(-1, 1), D.T, Xv * w, what=f"{what} mmchain")
            out, _ = blk.aggregate("sum", "col")
            assert_matches_truth(out.reshape(1, -1), np.ones((1, n_rows)), D, what=f"{what} colSums")
            out, _ = blk.aggregate("sum", "row")
            assert_matches_truth(out.reshape(-1, 1), D, np.ones((n, 1)), what=f"{what} rowSums")
            out, nnz = blk.decompress()
            assert np.array_equal(out, ora.decompress(ora.Groups(specs, n_rows, n)))
            # t(left) %*% block with a second random block on the left
            specs2, n2 = rand_block(rng, n_rows, max(3, max_groups // 2))
            D2 = ora.np_decompress(specs2, n_rows, n2)
            left = cla.build_block(n_rows, n2, specs2)
            try:
                out, _ = blk.lmm_compressed(left)
                assert_matches_truth(out, D2.T, D, what=f"{what} t(L)%*%R with {[s.type for s in specs2]}")
            finally:
                left.close()
        finally:
            blk.close()


@pytest.mark.parametrize("seed,n_rows,n_dense,n_ddc", [(3, 4097, 40, 80), (4, 30000, 70, 50), (5, 1025, 33, 140)])
def test_wide_blocks_with_wide_uncompressed_groups(cla, ora, seed, n_rows, n_dense, n_ddc):
    """More than 110 columns holding an uncompressed group of more than 32 columns (no column chunk takes it), for
    t(X) %*% X and as either side of the compressed x compressed product: the block is decompressed and multiplied
    on the matrix cores, as the reference does whenever a block holds an uncompressed group (CLALibTSMM.java:73-77);
    then the overlapping result of a right multiply through t(X B) %*% (X B)
    (CompressedTestBase.java:507-522 testTransposeSelfLeftMultOverload)."""
    from systemds_amd import synth
    rng = np.random.default_rng(seed)
    specs = [synth.GroupSpec("unc", np.arange(0, n_dense, dtype=np.int32), dense=rng.standard_normal((n_rows, n_dense)))]
    c = n_dense
    for _ in range(n_ddc // 2):
        nv = int(rng.choice([3, 40, 300]))
        codes = rng.integers(0, nv, n_rows).astype(np.uint8 if nv <= 256 else np.uint16)
        specs.append(synth.GroupSpec("ddc", np.arange(c, c + 2, dtype=np.int32), rng.standard_normal((nv, 2)), codes))
        c += 2
    specs.append(synth.sdc_group(rng, n_rows, np.arange(c, c + 1, dtype=np.int32), 5, 0.05, 0.5))
    c += 1
    assert c > 110
    D = ora.np_decompress(specs, n_rows, c)
    blk = cla.build_block(n_rows, c, specs)
    specs2, n2 = rand_block(rng, n_rows, 6)
    D2 = ora.np_decompress(specs2, n_rows, n2)
    other = cla.build_block(n_rows, n2, specs2)
    try:
        out, nnz = blk.tsmm()
        assert np.array_equal(out, out.T) and nnz == np.count_nonzero(out)
        assert_matches_truth(out, D.T, D, what="tsmm, wide dense group")
        out, _ = blk.lmm_compressed(other)
        assert_matches_truth(out, D2.T, D, what="t(L) %*% wide")
        out, _ = other.lmm_compressed(blk)
        assert_matches_truth(out, D.T, D2, what="t(wide) %*% R")
        B = rng.standard_normal((c, 9))
        child = blk.rmm_overlapping(B)
        P = (D.astype(np.longdouble) @ B.astype(np.longdouble)).astype(np.float64)
        out, _ = child.tsmm()
        child.close()
        scale = np.abs(D) @ np.abs(B)
        assert np.all(np.abs(out - (P.T.astype(np.longdouble) @ P.astype(np.longdouble)).astype(np.float64)) <= 2e-12 * (scale.T @ scale))
    finally:
        blk.close()
        other.close()
