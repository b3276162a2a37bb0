"""GPU parity of t(X) %*% X (cla_tsmm), integer co-occurrence (cla_cooc) and
decompression (cla_decompress) against the CPU oracle, through the C ABI."""
import numpy as np
import pytest

from conftest import mixed_block
from parity import assert_fp64_close, assert_matches_truth

pytestmark = pytest.mark.gpu


# option values of cla_block_set_option that force one of the interchangeable t(X) %*% X forms
PAIRS, DECODE, NO_CHUNKS = {"tsmm_route": 1}, {"tsmm_route": 2}, {"tsmm_chunks": 0}


def check_tsmm(cla, ora, specs, n_rows, n_cols, what, options=None):
    blk = cla.build_block(n_rows, n_cols, specs)
    for key, value in (options or {}).items():
        blk.set_option(key, value)
    out, nnz = blk.tsmm()
    blk.close()
    ref, rnnz = ora.tsmm(ora.Groups(specs, n_rows, n_cols), 4)
    D = ora.np_decompress(specs, n_rows, n_cols)
    assert np.array_equal(out, out.T)
    assert_matches_truth(out, D.T, D, what=what)
    assert_fp64_close(out, ref, ora.abs_matmul(D.T, D), what=what, n_terms=n_rows)
    assert nnz == rnnz


@pytest.mark.parametrize("seed,n_rows", [(0, 1), (1, 37), (2, 3000), (3, 20011), (4, 150001)])
@pytest.mark.parametrize("with_unc", [False, True])
def test_mixed_groups_tsmm(cla, ora, seed, n_rows, with_unc):
    """Compressed pair path (no uncompressed group) and the decompressing fallback."""
    specs, n_cols = mixed_block(seed, n_rows, with_unc=with_unc)
    check_tsmm(cla, ora, specs, n_rows, n_cols, f"tsmm unc={with_unc}")


@pytest.mark.parametrize("path", [PAIRS, DECODE], ids=["pairs", "decode"])
@pytest.mark.parametrize("seed,n_rows", [(1, 37), (2, 3000), (4, 150001)])
def test_mixed_groups_tsmm_both_paths(cla, ora, path, seed, n_rows):
    """The per-pair path and the decoded Gram matrix on the matrix cores are interchangeable:
    the library picks by cost, the block option tsmm_route forces one."""
    specs, n_cols = mixed_block(seed, n_rows, with_unc=False)
    check_tsmm(cla, ora, specs, n_rows, n_cols, f"tsmm {path}", path)


@pytest.mark.parametrize("path", [None, PAIRS, DECODE], ids=["auto", "pairs", "decode"])
def test_c3_scaled(cla, ora, path):
    """BASELINE config 3 at 1/100 scale: 25 co-coded pairs, 4096 tuples, uint16 codes. The
    dictionaries do not fit LDS together: the decoded path looks them up in global memory. The
    row count is no multiple of the tile, so the last tile is ragged."""
    from systemds_amd import synth
    c = synth.config3(scale=100)
    check_tsmm(cla, ora, c["groups"], c["n_rows"], c["n_cols"], f"C3 {path}", path)


@pytest.mark.parametrize("expand", [True, False])
def test_c5_scaled(cla, ora, expand):
    """BASELINE config 5 at 1/500 scale (mixed RLE + DDC + SDC + dense): both products, with the RLE / SDC
    groups' codes expanded to byte streams for the decode kernels (the default when that is cheap) and with the
    per-tile run and offset-list decoding."""
    from systemds_amd import synth
    opts = {"expand_streams": 1 if expand else 0}
    c = synth.config5(scale=500)
    n_rows, n_cols = c["n_rows"], c["n_cols"]
    check_tsmm(cla, ora, c["groups"], n_rows, n_cols, "C5 tsmm", opts)
    blk = cla.build_block(n_rows, n_cols, c["groups"]).set_option("expand_streams", opts["expand_streams"])
    out, nnz = blk.rmm(c["B"])
    blk.close()
    ref, rnnz = ora.rmm(ora.Groups(c["groups"], n_rows, n_cols), c["B"], 4)
    D = ora.np_decompress(c["groups"], n_rows, n_cols)
    assert_matches_truth(out, D, c["B"], what="C5 X%*%B")
    assert_fp64_close(out, ref, ora.abs_matmul(D, c["B"]), what="C5 X%*%B", n_terms=n_cols)
    assert nnz == rnnz


def test_single_column_groups_use_dense_path(cla, ora):
    """As many groups as columns: the reference decompresses (CLALibTSMM.java:73-77)."""
    from systemds_amd import synth
    c = synth.config4(scale=200, n_cols=12)
    check_tsmm(cla, ora, c["groups"], c["n_rows"], c["n_cols"], "C4-like")
    c = synth.config2(scale=500, n_cols=30)
    check_tsmm(cla, ora, c["groups"], c["n_rows"], c["n_cols"], "C2-like")


@pytest.mark.parametrize("path", [None, PAIRS, NO_CHUNKS], ids=["auto", "pairs", "no_chunks"])
def test_wide_blocks_of_single_column_groups(cla, ora, path):
    """More than 64 columns, as many groups as columns: the decoded Gram matrices of pairs of 32-column chunks
    (the default with that many pairs of groups), or one pass per pair of groups (forced, or chunks switched off)."""
    from systemds_amd import synth
    c = synth.config2(scale=500, n_cols=100)
    check_tsmm(cla, ora, c["groups"], c["n_rows"], c["n_cols"], f"C2 100 columns {path}", path)
    c = synth.config4(scale=500, n_cols=130)
    check_tsmm(cla, ora, c["groups"], c["n_rows"], c["n_cols"], f"C4-like 130 columns {path}", path)


def wide_mixed_block(seed, n_rows, extra_cols=70):
    """mixed_block (every group type, uncompressed and constant columns included) plus single- and two-column
    DDC groups up to more than 64 columns."""
    from systemds_amd import synth
    specs, c = mixed_block(seed, n_rows, with_unc=True)
    rng = np.random.default_rng(seed + 900)
    while c < 11 + extra_cols:
        nc = int(rng.choice([1, 2]))
        nv = int(rng.choice([5, 200, 700]))
        codes = rng.integers(0, nv, n_rows).astype(np.uint8 if nv <= 256 else np.uint16)
        specs.append(synth.GroupSpec("ddc", np.arange(c, c + nc, dtype=np.int32), rng.standard_normal((nv, nc)), codes))
        c += nc
    return specs, c


@pytest.mark.parametrize("seed,n_rows", [(1, 37), (2, 3000), (3, 70001)])
def test_wide_block_with_uncompressed_group(cla, ora, seed, n_rows):
    """More than 64 columns with an uncompressed group: no per-pair form exists, the block is cut into column
    chunks whose pairwise decoded Gram matrices are scattered into the result."""
    specs, n_cols = wide_mixed_block(seed, n_rows)
    assert n_cols > 64
    check_tsmm(cla, ora, specs, n_rows, n_cols, "wide block with an uncompressed group")


def test_cooc_bit_exact(cla, ora):
    specs, n_cols = mixed_block(31, 60007, with_unc=False)
    blk = cla.build_block(60007, n_cols, specs)
    G = ora.Groups(specs, 60007, n_cols)
    idx = [i for i, s in enumerate(specs) if s.type in ("ddc", "sdc", "rle")]
    for a, i in enumerate(idx):
        for b_, j in enumerate(idx):
            if specs[i].n_vals * specs[j].n_vals > 400000:
                continue
            N = blk.cooc(a, b_)
            assert np.array_equal(N, ora.cooc(G, i, j)), (specs[i].type, specs[j].type)
    # large code space (70000 x 300 bins -> HBM atomics): marginals must equal the counts
    N = blk.cooc(2, 1)
    assert np.array_equal(N.sum(axis=1), blk.counts(2))
    assert np.array_equal(N.sum(axis=0), blk.counts(1))
    assert N.sum() == 60007
    blk.close()


@pytest.mark.parametrize("seed,n_rows", [(0, 1), (2, 3000), (4, 70001)])
def test_decompress(cla, ora, seed, n_rows):
    specs, n_cols = mixed_block(seed, n_rows)
    blk = cla.build_block(n_rows, n_cols, specs)
    out, nnz = blk.decompress()
    blk.close()
    ref = ora.decompress(ora.Groups(specs, n_rows, n_cols))
    assert np.array_equal(out, ref)
    assert nnz == np.count_nonzero(ref)
