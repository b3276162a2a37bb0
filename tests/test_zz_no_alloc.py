"""cla_rmm_dev_noalloc (X %*% B with the pre-aggregated tables and the non-zero counter in the library's
static device workspace, no allocation) against cla_rmm_dev on the same inputs, through the C ABI."""
import numpy as np
import pytest

from conftest import mixed_block
from devmem import DevBuf

pytestmark = pytest.mark.gpu


def both(blk, B):
    """(result, nnz) of cla_rmm_dev and of cla_rmm_dev_noalloc for the same device operands."""
    q = B.shape[1]
    dB = DevBuf.from_numpy(B)
    d1, d2 = DevBuf(blk.n_rows * q * 8), DevBuf(blk.n_rows * q * 8)
    d1.zero()
    d2.zero()
    nnz1 = blk.rmm_dev(dB.ptr, q, d1.ptr)
    nnz2 = blk.rmm_dev_noalloc(dB.ptr, q, d2.ptr)
    return d1.to_numpy((blk.n_rows, q)), nnz1, d2.to_numpy((blk.n_rows, q)), nnz2


def test_two_calls_in_a_row_the_second_smaller(cla, ora):
    from systemds_amd import synth
    big = synth.config2(scale=100)                    # 100,000 x 100, byte codes: the mat-vec gather kernel
    small = synth.config2(scale=2000, n_cols=7)       # 5,000 x 7
    for c in (big, small):
        n, m = c["n_rows"], c["n_cols"]
        blk = cla.build_block(n, m, c["groups"])
        ref, rnnz = ora.rmm(ora.Groups(c["groups"], n, m), c["v"][:m], 4)
        want, nnz1, got, nnz2 = both(blk, c["v"][:m])
        blk.close()
        assert np.array_equal(want, ref) and nnz1 == rnnz       # the existing entry point, bit-exact vs the oracle
        assert np.array_equal(got, want) and nnz2 == nnz1       # and the new one equals it bit for bit


def test_wide_right_hand_side_then_a_vector(cla, ora):
    """DDC (all code widths), RLE, uncompressed and constant groups with B of 5 columns: the table-reading
    row kernel. Bit-identical to cla_rmm_dev with its matrix-core and decode kernels switched off (the same
    kernels then run with the block's own table buffer), within the 1e-12 bar of the default dispatch."""
    from parity import assert_matches_truth
    n_rows = 30011
    specs, n_cols = mixed_block(3, n_rows, big_dict=False)
    specs = [s for s in specs if s.type != "sdc"]
    blk = cla.build_block(n_rows, n_cols, specs)
    D = ora.np_decompress(specs, n_rows, n_cols)
    rng = np.random.default_rng(8)
    for q in (5, 1):   # the second call needs a fifth of the workspace of the first
        B = rng.standard_normal((n_cols, q))
        default, nnz0, got, nnz2 = both(blk, B)
        blk.set_option("rmm_disable", 4 | 8)
        same, nnz1, got2, nnz3 = both(blk, B)
        blk.set_option("rmm_disable", 0)
        assert np.array_equal(got, same) and np.array_equal(got2, same) and nnz2 == nnz1 == nnz3 == nnz0
        assert_matches_truth(got, D, B, what=f"no-alloc q={q}")
        assert_matches_truth(default, D, B, what=f"default q={q}")
    blk.close()


def test_refusals(cla):
    n_rows = 2000
    specs, n_cols = mixed_block(4, n_rows)           # holds SDC groups with entries and a 70,000-tuple dictionary
    blk = cla.build_block(n_rows, n_cols, specs)
    dB = DevBuf.from_numpy(np.ones((n_cols, 64)))
    dOut = DevBuf(n_rows * 64 * 8)
    with pytest.raises(cla.ClaError, match="static workspace holds") as e:
        blk.rmm_dev_noalloc(dB.ptr, 64, dOut.ptr)    # 70,000 x 64 doubles of tables
    assert e.value.code == cla.ERR_UNSUPPORTED
    with pytest.raises(cla.ClaError, match="SDC groups") as e:
        blk.rmm_dev_noalloc(dB.ptr, 1, dOut.ptr)
    assert e.value.code == cla.ERR_UNSUPPORTED
    blk.close()
