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


def _u8_block(rng, n_rows, n_cols, n_vals=200, zero_cells=False):
    from systemds_amd import synth
    specs = []
    for c in range(n_cols):
        d = rng.standard_normal((n_vals, 1))
        if zero_cells:
            d[rng.integers(0, n_vals, 5)] = 0.0
        specs.append(synth.GroupSpec("ddc", np.array([c], np.int32), d, rng.integers(0, n_vals, n_rows).astype(np.uint8)))
    return specs


@pytest.mark.parametrize("n_rows,n_cols", [(1, 3), (2047, 20), (70001, 37), (300000, 100)])
@pytest.mark.parametrize("with_const", [False, True])
def test_matvec_fused_tables_equal_preaggregated_tables(cla, ora, n_rows, n_cols, with_const):
    """Byte-code blocks with one column per group: the gather kernel that makes its tables on the way into
    LDS (the default) against the one that reads tables pre-aggregated by a kernel of their own
    (rmm_disable bit 1) and against the oracle, bit for bit; non-zero counts through the rotating counters
    over several calls."""
    from systemds_amd import synth
    rng = np.random.default_rng(n_rows + n_cols)
    specs = _u8_block(rng, n_rows, n_cols, zero_cells=True)
    nc = n_cols
    if with_const:
        specs.append(synth.GroupSpec("const", np.array([nc], np.int32), np.array([[0.75]])))
        nc += 1
    blk = cla.build_block(n_rows, nc, specs)
    G = ora.Groups(specs, n_rows, nc)
    for rep in range(5):
        v = rng.standard_normal((nc, 1))
        if rep == 3:
            v[:] = 0.0  # every result cell is the constants' term (or zero): the count must follow
        ref, rnnz = ora.rmm(G, v, 4)
        out, nnz = blk.rmm(v)
        assert np.array_equal(out, ref) and nnz == rnnz
        blk.set_option("rmm_disable", 2)
        out2, nnz2 = blk.rmm(v)
        blk.set_option("rmm_disable", 0)
        assert np.array_equal(out2, ref) and nnz2 == rnnz
    blk.close()


def test_matvec_fused_tables_non_finite_vector(cla, ora):
    """Dictionary.preaggValuesFromDense skips zero dictionary cells (Dictionary.java:893-908), so an infinite
    entry of v must not turn a zero cell into NaN; infinite and NaN entries meet non-zero cells as usual."""
    rng = np.random.default_rng(5)
    n_rows, n_cols = 50000, 24
    specs = _u8_block(rng, n_rows, n_cols, zero_cells=True)
    blk = cla.build_block(n_rows, n_cols, specs)
    G = ora.Groups(specs, n_rows, n_cols)
    v = rng.standard_normal((n_cols, 1))
    v[3] = np.inf
    v[7] = -np.inf
    ref, rnnz = ora.rmm(G, v, 4)
    out, nnz = blk.rmm(v)
    assert np.array_equal(out, ref, equal_nan=True) and nnz == rnnz
    assert np.isfinite(out).any() and not np.isfinite(out).all()
    v[11] = np.nan
    ref, rnnz = ora.rmm(G, v, 4)
    out, nnz = blk.rmm(v)
    assert np.array_equal(out, ref, equal_nan=True) and nnz == rnnz
    blk.close()


def test_async_calls_leave_the_count_on_the_device(cla, ora):
    """cla_*_dev_async queue the kernels and return; cla_block_nnz reads the count of the last call."""
    from devmem import DevBuf
    from systemds_amd import synth
    c = synth.config2(scale=200)
    n, m = c["n_rows"], c["n_cols"]
    blk = cla.build_block(n, m, c["groups"])
    G = ora.Groups(c["groups"], n, m)
    dv = DevBuf.from_numpy(c["v"])
    dz = DevBuf.from_numpy(np.zeros_like(c["v"]))
    dout = DevBuf(n * 8)
    ref, rnnz = ora.rmm(G, c["v"], 4)
    for _ in range(7):  # more calls than counters in the rotation
        assert blk.rmm_dev_async(dv.ptr, 1, dout.ptr) == 0
    assert blk.nnz() == rnnz
    assert np.array_equal(dout.to_numpy(n), ref[:, 0])
    assert blk.rmm_dev_async(dz.ptr, 1, dout.ptr) == 0
    assert blk.nnz() == 0
    assert blk.rmm_dev(dv.ptr, 1, dout.ptr) == rnnz
    # the other drivers: same results as their synchronous forms
    dB = DevBuf.from_numpy(c["B"])
    doB = DevBuf(n * 64 * 8)
    want = blk.rmm_dev(dB.ptr, 64, doB.ptr)
    keep = doB.to_numpy((n, 64))
    doB.zero()
    assert blk.rmm_dev_async(dB.ptr, 64, doB.ptr) == 0 and blk.nnz() == want
    assert np.array_equal(keep, doB.to_numpy((n, 64)))
    dy = DevBuf.from_numpy(np.random.default_rng(1).standard_normal((1, n)))
    do1 = DevBuf(m * 8)
    want = blk.lmm_dev(dy.ptr, 1, do1.ptr)
    keep = do1.to_numpy(m)
    assert blk.lmm_dev_async(dy.ptr, 1, do1.ptr) == 0 and blk.nnz() == want
    np.testing.assert_allclose(do1.to_numpy(m), keep, rtol=1e-12)
    do2 = DevBuf(m * 8)
    want = blk.mmchain_dev(dv.ptr, None, 0, do2.ptr)
    assert blk.mmchain_dev_async(dv.ptr, None, 0, do2.ptr) == 0 and blk.nnz() == want
    blk.close()
    c3 = synth.config3(scale=500)
    blk = cla.build_block(c3["n_rows"], c3["n_cols"], c3["groups"])
    do3 = DevBuf(c3["n_cols"] ** 2 * 8)
    want = blk.tsmm_dev(do3.ptr)
    assert blk.tsmm_dev_async(do3.ptr) == 0 and blk.nnz() == want
    blk.close()


def test_options_and_failed_finalize(cla):
    blk = cla.ClaBlock(100, 2)
    with pytest.raises(cla.ClaError, match="unknown option"):
        blk.set_option("no_such_switch", 1)
    with pytest.raises(cla.ClaError, match="takes 0..2"):
        blk.set_option("tsmm_route", 3)
    # a failed finalize leaves the block unusable: every further add or finalize is refused
    blk.add_ddc([0], np.zeros((2, 1)), np.full(100, 5, np.uint8))
    with pytest.raises(cla.ClaError, match="code >="):
        blk.finalize()
    with pytest.raises(cla.ClaError, match="earlier cla_block_finalize"):
        blk.finalize()
    with pytest.raises(cla.ClaError, match="earlier cla_block_finalize"):
        blk.add_const([1], np.ones((1, 1)))
    blk.close()


def kernels_of(blk, fn):
    blk.profile(True)
    fn()
    names = [k["name"] for k in blk.stats()["kernels"]]
    blk.profile(False)
    return names


@pytest.mark.parametrize("q", [21, 24, 40])
@pytest.mark.parametrize("with_other_groups", [False, True])
def test_wide_right_multiply_on_offset_lists(cla, ora, q, with_other_groups):
    """B wider than what a 1024-row output tile of all columns takes in LDS: the tile kernel of the offset lists runs
    per chunk of columns (21 = 11 + 10, 40 = 4 x 10) instead of one atomic add per entry and column in global memory."""
    from systemds_amd import synth
    rng = np.random.default_rng(q)
    n_rows = 30011
    specs, c = [], 0
    for g in range(12):
        specs.append(synth.sdc_group(np.random.default_rng((q, g)), n_rows, np.array([c], np.int32), 20, [0.1, 0.004][g % 2], [None, 0.25][g % 3 == 0]))
        c += 1
    if with_other_groups:
        specs.append(synth.GroupSpec("ddc", np.array([c, c + 1], np.int32), rng.standard_normal((9, 2)), rng.integers(0, 9, n_rows).astype(np.uint8)))
        specs.append(synth.GroupSpec("unc", np.array([c + 2], np.int32), dense=rng.standard_normal((n_rows, 1))))
        c += 3
    B = rng.standard_normal((c, q))
    D = ora.np_decompress(specs, n_rows, c)
    blk = cla.build_block(n_rows, c, specs)
    try:
        out, nnz = blk.rmm(B)
        names = kernels_of(blk, lambda: blk.rmm(B))
    finally:
        blk.close()
    assert_matches_truth(out, D, B, what=f"X %*% B, {q} columns")
    assert nnz == np.count_nonzero(out)
    assert "k_rmm_sdc_scatter" not in names and names.count("k_rmm_sdc_tiles") >= 2, names


@pytest.mark.parametrize("q", [2, 3, 5, 7])
def test_narrow_right_multiply_on_a_wide_ddc_block(cla, ora, q):
    """80 single-column groups of 256 tuples: more dictionary than the narrow-B kernels hold in LDS; B of 2 to 7
    columns then goes to the matrix-core kernel, zero padded."""
    from systemds_amd import synth
    c = synth.config2(scale=250, n_cols=80)
    n_rows, n_cols = c["n_rows"], c["n_cols"]
    B = np.random.default_rng(q).standard_normal((n_cols, q))
    D = ora.np_decompress(c["groups"], n_rows, n_cols)
    blk = cla.build_block(n_rows, n_cols, c["groups"])
    try:
        out, nnz = blk.rmm(B)
        names = kernels_of(blk, lambda: blk.rmm(B))
    finally:
        blk.close()
    assert_matches_truth(out, D, B, what=f"X %*% B, {q} columns")
    assert nnz == np.count_nonzero(out)
    assert "k_rmm_mfma" in names, names


def test_single_column_on_a_mixed_block_takes_the_decode_kernel(cla, ora):
    """X %*% v on a block of RLE, DDC, dense and a few offset-list groups (C5's shape)."""
    from systemds_amd import synth
    c = synth.config5(scale=500)
    n_rows, n_cols = c["n_rows"], c["n_cols"]
    v = np.random.default_rng(4).standard_normal((n_cols, 1))
    D = ora.np_decompress(c["groups"], n_rows, n_cols)
    blk = cla.build_block(n_rows, n_cols, c["groups"])
    try:
        out, nnz = blk.rmm(v)
        names = kernels_of(blk, lambda: blk.rmm(v))
        w = np.random.default_rng(5).standard_normal((n_rows, 1))
        chain, _ = blk.mmchain(v, w, 1)
    finally:
        blk.close()
    assert_matches_truth(out, D, v, what="C5 X %*% v")
    assert nnz == np.count_nonzero(out)
    assert "k_rmm_direct" in names, names
    assert_matches_truth(chain.reshape(-1, 1), D.T, (D @ v) * w, what="C5 chain")


def _plain_stream_block(seed, n_rows, odd_dense=False, overlap=False):
    """Groups that are plain streams on the device: DDC with one- and two-byte codes (single and co-coded columns),
    small RLE and SDC groups (which get one code per row), dense columns, a constant and an empty group. Odd numbers
    of columns per class, so that the filler columns of the kernel take part."""
    from systemds_amd import synth
    rng = np.random.default_rng(seed)
    specs, c = [], 0

    def cols(n):
        nonlocal c
        r = np.arange(c, c + n, dtype=np.int32)
        c += n
        return r
    specs.append(synth.GroupSpec("ddc", cols(1), rng.standard_normal((7, 1)), rng.integers(0, 7, n_rows).astype(np.uint8)))
    specs.append(synth.GroupSpec("ddc", cols(2), rng.standard_normal((200, 2)), rng.integers(0, 200, n_rows).astype(np.uint8)))
    specs.append(synth.GroupSpec("ddc", cols(2), rng.standard_normal((300, 2)), rng.integers(0, 300, n_rows).astype(np.uint16)))
    specs.append(synth.GroupSpec("ddc", cols(1), rng.standard_normal((1500, 1)), rng.integers(0, 1500, n_rows).astype(np.uint16)))
    specs.append(synth.sdc_group(rng, n_rows, cols(1), 5, 0.1, None))
    specs.append(synth.sdc_group(rng, n_rows, cols(2), 6, 0.3, 1.5))
    run_codes = rng.integers(-1, 4, size=n_rows // 20 + 2)
    codes = np.repeat(run_codes, rng.integers(1, 60, size=run_codes.size))[:n_rows]
    if codes.size < n_rows:
        codes = np.concatenate([codes, np.full(n_rows - codes.size, -1)])
    ptr, data = synth.encode_rle(codes, 4)
    specs.append(synth.GroupSpec("rle", cols(1), rng.standard_normal((4, 1)), ptr=ptr, rle=data))
    specs.append(synth.GroupSpec("unc", cols(1 if odd_dense else 2), dense=rng.standard_normal((n_rows, 1 if odd_dense else 2))))
    specs.append(synth.GroupSpec("const", cols(1), np.array([[2.5]])))
    specs.append(synth.GroupSpec("empty", cols(1)))
    if overlap:
        specs.append(synth.GroupSpec("ddc", np.array([0, 3], np.int32), rng.standard_normal((9, 2)), rng.integers(0, 9, n_rows).astype(np.uint8)))
    return specs, c


@pytest.mark.parametrize("n_rows", [1, 2, 127, 128, 129, 255, 4097, 70001])
@pytest.mark.parametrize("q", [1, 2, 3, 7, 10, 16])
def test_narrow_right_multiply_straight_from_the_streams(cla, ora, n_rows, q):
    """X %*% B for at most 16 columns of B on a block of plain streams: codes read straight from global memory
    (`k_rmm_direct`), against the oracle, the long-double truth and the tile kernel (`rmm_direct` 0)."""
    specs, n_cols = _plain_stream_block(n_rows + q, n_rows, overlap=q == 3)
    B = np.random.default_rng(q).standard_normal((n_cols, q))
    D = ora.np_decompress(specs, n_rows, n_cols)
    ref, rnnz = ora.rmm(ora.Groups(specs, n_rows, n_cols), B, 4)
    blk = cla.build_block(n_rows, n_cols, specs)
    try:
        out, nnz = blk.rmm(B)
        names = kernels_of(blk, lambda: blk.rmm(B))
        blk.set_option("rmm_direct", 0)
        out0, nnz0 = blk.rmm(B)
        names0 = kernels_of(blk, lambda: blk.rmm(B))
    finally:
        blk.close()
    # (16 columns of B: the tile kernel first, it has no padding of B to lose there)
    assert ("k_rmm_direct" in names or q == 16) and "k_rmm_direct" not in names0, (names, names0)
    assert_fp64_close(out, ref, ora.abs_matmul(D, B), what=f"direct q={q}", n_terms=n_cols)
    assert_matches_truth(out[:5000], D[:5000], B, what=f"direct q={q}")
    assert_matches_truth(out[-300:], D[-300:], B, what=f"direct q={q}, last rows")
    assert_matches_truth(out0[:5000], D[:5000], B, what=f"tiles q={q}")
    assert nnz == rnnz == np.count_nonzero(out) and nnz0 == rnnz


@pytest.mark.parametrize("q", [4, 5, 6, 8, 9, 11, 12, 13, 14, 15, 17, 32, 37, 64])
def test_narrow_right_multiply_straight_from_the_streams_other_widths(cla, ora, q):
    n_rows = 3000 + q
    specs, n_cols = _plain_stream_block(q, n_rows)
    B = np.random.default_rng(q).standard_normal((n_cols, q))
    D = ora.np_decompress(specs, n_rows, n_cols)
    blk = cla.build_block(n_rows, n_cols, specs)
    try:
        out, nnz = blk.rmm(B)
        names = kernels_of(blk, lambda: blk.rmm(B))
    finally:
        blk.close()
    assert "k_rmm_direct" in names, names  # (37 and 64 columns: 16 per pass)
    assert_matches_truth(out, D, B, what=f"direct q={q}")
    assert nnz == np.count_nonzero(out)


def test_blocks_the_stream_kernel_does_not_take(cla, ora):
    """An odd number of dense columns, four-byte codes: the tile kernel as before."""
    from systemds_amd import synth
    n_rows = 5000
    B = None
    for variant in ("odd_dense", "int_codes"):
        specs, n_cols = _plain_stream_block(11, n_rows, odd_dense=variant == "odd_dense")
        if variant == "int_codes":
            rng = np.random.default_rng(3)
            specs.append(synth.GroupSpec("ddc", np.array([n_cols], np.int32), rng.standard_normal((70000, 1)),
                                         rng.integers(0, 70000, n_rows).astype(np.int32)))
            n_cols += 1
        B = np.random.default_rng(1).standard_normal((n_cols, 5))
        D = ora.np_decompress(specs, n_rows, n_cols)
        blk = cla.build_block(n_rows, n_cols, specs)
        try:
            out, nnz = blk.rmm(B)
            names = kernels_of(blk, lambda: blk.rmm(B))
        finally:
            blk.close()
        assert "k_rmm_direct" not in names, (variant, names)
        assert_matches_truth(out, D, B, what=f"{variant}")
        assert nnz == np.count_nonzero(out)


@pytest.mark.parametrize("q", [17, 40, 64])
def test_wide_right_multiply_in_passes_of_the_tile_kernel(cla, ora, q):
    """Long runs (no one-code-per-row copy: it would dwarf the group), two-byte DDC codes and three dense columns: the
    tile kernel takes B 16 columns per pass."""
    from systemds_amd import synth
    n_rows = 150001
    rng = np.random.default_rng(q)
    specs, c = [], 0
    for _ in range(3):
        lens = rng.geometric(1.0 / 3000.0, size=n_rows // 2000 + 16)
        codes = np.repeat(rng.integers(-1, 8, size=lens.size), lens)[:n_rows]
        if codes.size < n_rows:
            codes = np.concatenate([codes, np.full(n_rows - codes.size, -1)])
        ptr, data = synth.encode_rle(codes, 8)
        specs.append(synth.GroupSpec("rle", np.array([c], np.int32), rng.standard_normal((8, 1)), ptr=ptr, rle=data))
        c += 1
    specs.append(synth.GroupSpec("ddc", np.array([c, c + 1], np.int32), rng.standard_normal((700, 2)), rng.integers(0, 700, n_rows).astype(np.uint16)))
    c += 2
    specs.append(synth.GroupSpec("unc", np.arange(c, c + 3, dtype=np.int32), dense=rng.standard_normal((n_rows, 3))))
    c += 3
    B = rng.standard_normal((c, q))
    D = ora.np_decompress(specs, n_rows, c)
    blk = cla.build_block(n_rows, c, specs)
    try:
        out, nnz = blk.rmm(B)
        names = kernels_of(blk, lambda: blk.rmm(B))
    finally:
        blk.close()
    assert names.count("k_rmm_decode") == (q + 15) // 16, names
    assert_matches_truth(out, D, B, what=f"tile passes q={q}")
    assert nnz == np.count_nonzero(out)


@pytest.mark.parametrize("n_vals,n_groups", [(1000, 20), (1900, 11)])
def test_mat_vec_on_two_byte_codes_with_large_dictionaries(cla, ora, n_vals, n_groups):
    """Single-column DDC groups with two-byte codes whose tables fit a slab of 8 only in blocks of 512 threads (1000
    values) or 1024 threads (1900 values): X %*% v stays on the slab kernel with its tables in LDS."""
    from systemds_amd import synth
    rng = np.random.default_rng(n_vals)
    n_rows = 70003
    specs = [synth.GroupSpec("ddc", np.array([c], np.int32), rng.standard_normal((n_vals, 1)), rng.integers(0, n_vals, n_rows).astype(np.uint16))
             for c in range(n_groups)]
    v = rng.standard_normal((n_groups, 1))
    D = ora.np_decompress(specs, n_rows, n_groups)
    blk = cla.build_block(n_rows, n_groups, specs)
    try:
        blk.profile(True)
        out, nnz = blk.rmm(v)
        names = [k["name"] for k in blk.stats()["kernels"]]
    finally:
        blk.close()
    assert "k_rmm_q1_ddc" in names, names
    assert_matches_truth(out, D, v, what=f"X %*% v, {n_vals} values per column")
    assert nnz == np.count_nonzero(out)


@pytest.mark.parametrize("q", [56, 64, 70])
def test_wide_right_multiply_through_decompressed_rows(cla, ora, q):
    """A block that is mostly offset lists (12 lists beside 4 DDC columns; the tile kernel does not take it) with a
    wide B: decompressed chunks of rows times B on the matrix cores (`k_dense_rmm`; 200,003 rows: a ragged last tile of
    16 rows, 70 columns of B: a second pass of 6 columns); with the decoding kernels off the gather kernels give the
    same cells."""
    from systemds_amd import synth
    rng = np.random.default_rng(q)
    n_rows, n_cols = 200003, 16
    specs = [synth.sdc_group(rng, n_rows, np.array([c], np.int32), 9, 0.1, 0.5 if c % 2 else None) for c in range(12)]
    specs += [synth.GroupSpec("ddc", np.array([12 + c], np.int32), rng.standard_normal((40, 1)), rng.integers(0, 40, n_rows).astype(np.uint8))
              for c in range(4)]
    B = rng.standard_normal((n_cols, q))
    D = ora.np_decompress(specs, n_rows, n_cols)
    blk = cla.build_block(n_rows, n_cols, specs)
    try:
        blk.profile(True)
        out, nnz = blk.rmm(B)
        names = [k["name"] for k in blk.stats()["kernels"]]
        blk.profile(False)
        blk.set_option("rmm_disable", 12)
        gather, nnz_g = blk.rmm(B)
    finally:
        blk.close()
    assert "k_dense_rmm" in names and "k_rmm_rows" not in names, names
    assert_matches_truth(out, D, B, what=f"X %*% B through decompressed rows, {q} columns")
    assert_matches_truth(gather, D, B, what=f"X %*% B, gather kernels, {q} columns")
    assert nnz == np.count_nonzero(out) and nnz_g == np.count_nonzero(gather)
