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


@pytest.mark.parametrize("narrow", [1, 0])
@pytest.mark.parametrize("n_cols,big_dict", [(17, False), (18, True), (20, False), (35, False), (36, True), (50, False), (52, True), (21, False)])
def test_decoded_gram_with_a_narrow_last_column_block(cla, ora, n_cols, big_dict, narrow):
    """Column counts whose last block of 16 holds at most 4 columns: its rows of the Gram matrix come from the
    4 x 4 x 4 matrix instruction (`tsmm_narrow`, the default) instead of 16 x 16 tiles; with at most 32 columns the
    last block's lookups of four steps are packed into one. Mixed group types, one- and two-byte codes,
    dictionaries in LDS and (big_dict) in global memory, a ragged last tile; 21 columns (5 in the last block) take
    the tiles either way."""
    from systemds_amd import synth
    n_rows = 70001
    rng = np.random.default_rng(n_cols)
    specs, c = [], 0
    while c < n_cols:
        left = n_cols - c
        kind = ["ddc", "ddc2", "sdc", "rle", "unc"][len(specs) % 5]
        if kind == "ddc2" and left >= 2:
            nv = 5000 if big_dict else 300
            codes = rng.integers(0, nv, n_rows).astype(np.uint16)
            specs.append(synth.GroupSpec("ddc", np.arange(c, c + 2, dtype=np.int32), rng.standard_normal((nv, 2)), codes))
            c += 2
        elif kind == "sdc":
            specs.append(synth.sdc_group(rng, n_rows, np.array([c], np.int32), 7, 0.1, 0.5))
            c += 1
        elif kind == "rle":
            run_codes = rng.integers(-1, 4, size=n_rows // 40 + 2)
            codes = np.repeat(run_codes, rng.integers(1, 90, size=run_codes.size))[:n_rows]
            codes = np.concatenate([codes, np.full(n_rows - codes.size, -1)]) if codes.size < n_rows else codes
            ptr, data = synth.encode_rle(codes, 4)
            specs.append(synth.GroupSpec("rle", np.array([c], np.int32), rng.standard_normal((4, 1)), ptr=ptr, rle=data))
            c += 1
        elif kind == "unc":
            specs.append(synth.GroupSpec("unc", np.array([c], np.int32), dense=rng.standard_normal((n_rows, 1))))
            c += 1
        else:
            codes = rng.integers(0, 16, n_rows).astype(np.uint8)
            specs.append(synth.GroupSpec("ddc", np.array([c], np.int32), rng.standard_normal((16, 1)), codes))
            c += 1
    check_tsmm(cla, ora, specs, n_rows, n_cols, f"{n_cols} columns, narrow {narrow}", {"tsmm_route": 2, "tsmm_narrow": narrow})


@pytest.mark.parametrize("shape", ["decode", "direct"])
def test_decoded_gram_is_one_kernel_per_call(cla, ora, shape):
    """A block of at most 64 columns that the decoded Gram kernels take runs as one kernel per call: the blocks add
    into an accumulator kept with the block and the last one writes the output, mirrored, counts its non-zeros and
    clears the accumulator (no fill of the output in front, no k_tsmm_finish behind). Repeated and queued calls
    into outputs that hold garbage must all give the first call's result and count, also with other products
    between them."""
    import devmem
    from systemds_amd import synth
    if shape == "decode":
        c = synth.config3(scale=100)
        specs, n_rows, n_cols = c["groups"], c["n_rows"], c["n_cols"]
        kernel = "k_tsmm_decode"
    else:
        from test_gpu_gram_direct import stream_block
        n_rows = 70003
        specs, n_cols = stream_block(21, n_rows)
        kernel = "k_tsmm_direct"
    D = ora.np_decompress(specs, n_rows, n_cols)
    scale = np.abs(D).T @ np.abs(D)
    blk = cla.build_block(n_rows, n_cols, specs)
    try:
        first, nnz = blk.tsmm()
        blk.profile(True)
        blk.tsmm()
        names = [k["name"] for k in blk.stats()["kernels"]]
        blk.profile(False)
        assert names == [kernel], names
        # the same kernel between a fill of the output and k_tsmm_finish (option tsmm_one_kernel 0): the same matrix
        blk.set_option("tsmm_one_kernel", 0)
        blk.profile(True)
        plain, pnnz = blk.tsmm()
        names = [k["name"] for k in blk.stats()["kernels"]]
        blk.profile(False)
        blk.set_option("tsmm_one_kernel", 1)
        assert names == [kernel, "k_tsmm_finish"], names
        assert pnnz == nnz
        assert_fp64_close(plain, first, scale, what=f"{shape}: with and without the tail")
        outs = [devmem.DevBuf.from_numpy(np.full((n_cols, n_cols), np.nan)) for _ in range(3)]
        rng = np.random.default_rng(3)
        blk.tsmm_dev_async(outs[0].ptr)
        blk.tsmm_dev_async(outs[1].ptr)
        blk.rmm(rng.standard_normal((n_cols, 2)))
        blk.lmm(rng.standard_normal((1, n_rows)))
        assert blk.tsmm_dev(outs[2].ptr) == nnz
        for o in outs:
            again = o.to_numpy((n_cols, n_cols))
            assert np.array_equal(again, again.T)
            assert_fp64_close(again, first, scale, what=f"{shape}: repeated call")
            assert np.count_nonzero(again) == nnz
            o.free()
    finally:
        blk.close()
    assert_matches_truth(first, D.T, D, what=f"{shape}: one kernel per call")
    assert nnz == np.count_nonzero(first)
