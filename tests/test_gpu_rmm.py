"""GPU parity of the right multiply (cla_rmm) against the CPU oracle, through the C ABI."""
import numpy as np
import pytest

from conftest import mixed_block
from parity import assert_fp64_close, assert_matches_truth

pytestmark = pytest.mark.gpu


def run_both(cla, ora, specs, n_rows, n_cols, B):
    blk = cla.build_block(n_rows, n_cols, specs)
    G = ora.Groups(specs, n_rows, n_cols)
    out, nnz = blk.rmm(B)
    ref, rnnz = ora.rmm(G, B, 4)
    blk.close()
    return out, nnz, ref, rnnz


def abs_scale(ora, specs, n_rows, n_cols, B):
    return ora.abs_matmul(ora.np_decompress(specs, n_rows, n_cols), B)


def test_c1_matvec_full_size_bit_exact(cla, ora):
    """BASELINE config 1: 100,000 x 20 DDC-16 u8, X %*% v. The mat-vec gather sums
    the groups in list order with unfused arithmetic, so it must equal the oracle
    bit for bit."""
    from systemds_amd import synth
    c = synth.config1()
    out, nnz, ref, rnnz = run_both(cla, ora, c["groups"], c["n_rows"], c["n_cols"], c["v"])
    assert np.array_equal(out, ref)
    assert nnz == rnnz == np.count_nonzero(ref)


@pytest.mark.parametrize("n_rows", [1, 15, 16, 17, 4095, 4096, 4097, 100003])
@pytest.mark.parametrize("dtype", [np.uint8, np.uint16, np.int32])
def test_ddc_matvec_ragged_sizes(cla, ora, n_rows, dtype):
    from systemds_amd import synth
    rng = np.random.default_rng(n_rows)
    n_vals = {np.uint8: 200, np.uint16: 3000, np.int32: 5000}[dtype]
    n_cols = 13
    specs = [synth.GroupSpec("ddc", np.array([c], np.int32), rng.standard_normal((n_vals, 1)),
                             rng.integers(0, n_vals, n_rows).astype(dtype)) for c in range(n_cols)]
    v = rng.standard_normal((n_cols, 1))
    out, nnz, ref, rnnz = run_both(cla, ora, specs, n_rows, n_cols, v)
    assert np.array_equal(out, ref)
    assert nnz == rnnz


def test_c2_scaled_matvec_and_matmat(cla, ora):
    """BASELINE config 2 at 1/100 scale (100,000 rows): X %*% v and X %*% B(100x64)."""
    from systemds_amd import synth
    c = synth.config2(scale=100)
    scale_v = abs_scale(ora, c["groups"], c["n_rows"], c["n_cols"], c["v"])
    out, nnz, ref, rnnz = run_both(cla, ora, c["groups"], c["n_rows"], c["n_cols"], c["v"])
    assert np.array_equal(out, ref)
    assert_fp64_close(out, ref, scale_v, what="C2 X%*%v")
    assert nnz == rnnz
    scale_B = abs_scale(ora, c["groups"], c["n_rows"], c["n_cols"], c["B"])
    out, nnz, ref, rnnz = run_both(cla, ora, c["groups"], c["n_rows"], c["n_cols"], c["B"])
    assert_fp64_close(out, ref, scale_B, what="C2 X%*%B", n_terms=c["n_cols"])
    D = ora.np_decompress(c["groups"], c["n_rows"], c["n_cols"])
    assert_matches_truth(out[:4000], D[:4000], c["B"], what="C2 X%*%B (first 4000 rows)")
    assert nnz == rnnz


@pytest.mark.parametrize("seed,n_rows", [(0, 1), (1, 37), (2, 3000), (3, 20011), (4, 70001)])
@pytest.mark.parametrize("q", [1, 5, 64])
def test_mixed_groups(cla, ora, seed, n_rows, q):
    """Every group type in one block (DDC u8/u16/int, SDCZeros, SDC with default, RLE,
    uncompressed, const, empty)."""
    specs, n_cols = mixed_block(seed, n_rows)
    B = np.random.default_rng(seed + 50).standard_normal((n_cols, q))
    out, nnz, ref, rnnz = run_both(cla, ora, specs, n_rows, n_cols, B)
    assert_fp64_close(out, ref, abs_scale(ora, specs, n_rows, n_cols, B), what=f"mixed q={q}", n_terms=n_cols)
    D = ora.np_decompress(specs, n_rows, n_cols)
    assert_matches_truth(out[:3000], D[:3000], B, what=f"mixed q={q}")
    assert nnz == rnnz


def test_co_coded_ddc(cla, ora):
    """C3-shaped groups (two columns per group, u16 codes) in a right multiply."""
    from systemds_amd import synth
    c = synth.config3(scale=200, n_pairs=5)
    rng = np.random.default_rng(77)
    for q in (1, 3):
        B = rng.standard_normal((c["n_cols"], q))
        out, nnz, ref, rnnz = run_both(cla, ora, c["groups"], c["n_rows"], c["n_cols"], B)
        assert_fp64_close(out, ref, abs_scale(ora, c["groups"], c["n_rows"], c["n_cols"], B), what="co-coded")
        assert nnz == rnnz


def test_zero_results_are_counted_as_zero(cla, ora):
    from systemds_amd import synth
    d = np.array([[0.0], [1.0], [-1.0]])
    codes = np.array([0, 1, 2, 0, 0, 1] * 100, np.uint8)
    codes2 = codes.copy()
    codes2[500:] = (codes2[500:] + 1) % 3
    specs = [synth.GroupSpec("ddc", np.array([0], np.int32), d, codes),
             synth.GroupSpec("ddc", np.array([1], np.int32), -d, codes2)]
    v = np.array([[2.0], [2.0]])
    out, nnz, ref, rnnz = run_both(cla, ora, specs, codes.size, 2, v)
    assert np.array_equal(out, ref)
    assert nnz == rnnz == np.count_nonzero(ref)
    assert 0 < nnz < codes.size


def test_counts_bit_exact(cla, ora):
    specs, n_cols = mixed_block(9, 50000, with_unc=False)
    blk = cla.build_block(50000, n_cols, specs)
    G = ora.Groups(specs, 50000, n_cols)
    gi = 0
    for i, s in enumerate(specs):
        if s.type in ("ddc", "sdc", "rle"):
            assert np.array_equal(blk.counts(gi), ora.counts(G, i)), s.type
        if s.type not in ("const", "empty"):
            gi += 1
    blk.close()


def test_error_behaviour(cla):
    """Errors are negative codes + message, never exceptions from native code
    (the caller falls back to its own kernels, LibMatrixNative.java:123-135)."""
    blk = cla.ClaBlock(100, 2)
    with pytest.raises(cla.ClaError, match="code >="):
        blk.add_ddc([0], np.zeros((2, 1)), np.full(100, 5, np.uint8))
        blk.finalize()
    blk.close()
    blk = cla.ClaBlock(100, 2)
    with pytest.raises(cla.ClaError, match="column index"):
        blk.add_ddc([2], np.zeros((2, 1)), np.zeros(100, np.uint8))
    with pytest.raises(cla.ClaError, match="not finalized"):
        blk.rmm(np.zeros((2, 1)))
    blk.close()
    blk = cla.ClaBlock(1000, 1)
    with pytest.raises(cla.ClaError, match="inconsistent"):
        blk.add_sdc([0], np.ones((1, 1)), None, np.zeros(3, np.uint8), np.array([5, 7], np.uint8), 1, 99, 3)
        blk.finalize()
    blk.close()


@pytest.mark.parametrize("seed", range(8))
def test_wide_right_multiply_on_uneven_ddc_blocks(cla, ora, seed):
    """All-DDC blocks with dictionaries of very different sizes, tuple widths 1-3, both code widths and wide B:
    the matrix-core right multiply cuts them into LDS slabs. Seed 1 (512 rows, 38 groups, 55 columns) has its
    largest dictionary range and its largest column count in different slabs."""
    from systemds_amd import synth
    rng = np.random.default_rng(2024)
    for _ in range(seed + 1):   # the seed-th block of one random sequence
        n_rows = int(rng.choice([1, 15, 511, 512, 513, 1000, 4097, 20000, 70001]))
        specs, c = [], 0
        for _g in range(int(rng.integers(1, 40))):
            nc = int(rng.choice([1, 1, 1, 2, 3]))
            nv = int(rng.choice([2, 16, 200, 256, 300, 1000, 3000]))
            codes = rng.integers(0, nv, n_rows).astype(np.uint8 if nv <= 256 else np.uint16)
            specs.append(synth.GroupSpec("ddc", np.arange(c, c + nc, dtype=np.int32), rng.standard_normal((nv, nc)), codes))
            c += nc
        if rng.random() < 0.3:
            specs.append(synth.GroupSpec("const", np.array([c], np.int32), np.array([[1.25]])))
            c += 1
        q = int(rng.choice([8, 9, 16, 33, 64, 65, 100]))
        B = rng.standard_normal((c, q))
    out, nnz, ref, rnnz = run_both(cla, ora, specs, n_rows, c, B)
    D = ora.np_decompress(specs, n_rows, c)
    assert_matches_truth(out, D, B, what=f"uneven DDC block {seed}")
    assert_fp64_close(out, ref, abs_scale(ora, specs, n_rows, c, B), what=f"uneven DDC block {seed}", n_terms=c)
    assert nnz == rnnz
