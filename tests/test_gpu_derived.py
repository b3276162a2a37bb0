"""GPU tests of the two entry points that manage the formats the library derives from a block:
cla_block_drop_derived (frees them; the next call builds them again, with the same results) and
cla_block_prepare (builds at once what the first call of a product would build). Both have no counterpart in the
reference; the products they bracket are checked against each other bit for bit (the same kernels on the same
forms; sums that go through atomic adds may differ in the last bits from run to run and are compared at 1e-12 of the
products' scale) and against the decompressed block."""
import numpy as np
import pytest

from systemds_amd import capi
from test_gpu_gram_direct import stream_block
from test_gpu_sdc_matvec import sdc_block, assert_close

pytestmark = pytest.mark.gpu


def products(blk, B, Y):
    return blk.rmm(B)[0], blk.lmm(Y)[0], blk.tsmm()[0]


def same(first, again):
    """X %*% B bit for bit; Y %*% X and t(X) %*% X (atomic adds across workgroups) to the last bits."""
    assert np.array_equal(first[0], again[0])
    for a, b in zip(first[1:], again[1:]):
        assert np.all(np.abs(a - b) <= 1e-12 * np.maximum(np.abs(a), 1.0) * max(1.0, np.sqrt(a.size))), np.max(np.abs(a - b))


def kernel_names(blk, fn):
    blk.profile(True)
    fn()
    names = {k["name"] for k in blk.stats()["kernels"]}
    blk.profile(False)
    return names


def test_drop_then_the_same_results_sdc(cla, ora):
    n_rows = 70001
    specs, n_cols = sdc_block(3, n_rows, 70, [0.05, 0.02], 40)
    rng = np.random.default_rng(1)
    u, v = rng.standard_normal((n_cols, 1)), rng.standard_normal((1, n_rows))
    blk = cla.build_block(n_rows, n_cols, specs)
    base = blk.derived_bytes()
    first = products(blk, u, v)
    held = blk.derived_bytes()
    assert held > base + n_rows  # lane-major lists and row lists
    blk.drop_derived()
    assert blk.derived_bytes() == base
    again = products(blk, u, v)
    assert blk.derived_bytes() == held
    same(first, again)
    D = ora.np_decompress(specs, n_rows, n_cols)
    assert_close(again[0], D, u, "X%*%u after drop")
    assert_close(again[1], v, D, "t(v)%*%X after drop")
    blk.drop_derived()
    blk.drop_derived()  # nothing held: no-op
    assert blk.derived_bytes() == base
    blk.close()


def test_prepare_builds_what_the_first_call_builds(cla):
    n_rows = 90000
    specs, n_cols = sdc_block(5, n_rows, 64, 0.05, 30)
    rng = np.random.default_rng(2)
    u, v = rng.standard_normal((n_cols, 1)), rng.standard_normal((1, n_rows))
    a = cla.build_block(n_rows, n_cols, specs)
    b = cla.build_block(n_rows, n_cols, specs)
    base = a.derived_bytes()
    # one product at a time: only its form is built
    a.prepare(lmm_rows=1)
    lmm_only = a.derived_bytes()
    out_b = b.lmm(v)[0]
    assert b.derived_bytes() == lmm_only > base
    assert "k_lmm_sdc_lanes" in kernel_names(a, lambda: a.lmm(v))
    assert a.derived_bytes() == lmm_only  # the call after prepare builds nothing
    same((0, out_b), (0, a.lmm(v)[0]))
    a.drop_derived()
    a.prepare(rmm_cols=1)
    rmm_only = a.derived_bytes()
    assert "k_rmm_sdc_rows" in kernel_names(a, lambda: a.rmm(u))
    assert a.derived_bytes() == rmm_only > base
    b.drop_derived()
    assert np.array_equal(b.rmm(u)[0], a.rmm(u)[0])
    assert b.derived_bytes() == rmm_only
    # both: the sum
    a.prepare(lmm_rows=1)
    assert a.derived_bytes() == lmm_only + rmm_only - base
    a.close()
    b.close()


def test_stream_block_drop_and_prepare(cla, ora):
    """Expanded streams, the merged run table, the decode and direct plans of a block of mixed groups."""
    n_rows = 80011
    specs, n_cols = stream_block(4, n_rows, mean_run=300)
    rng = np.random.default_rng(3)
    B, Y = rng.standard_normal((n_cols, 10)), rng.standard_normal((3, n_rows))
    blk = cla.build_block(n_rows, n_cols, specs)
    base = blk.derived_bytes()
    blk.prepare(rmm_cols=10, lmm_rows=3, tsmm=True)
    held = blk.derived_bytes()
    first = products(blk, B, Y)
    assert blk.derived_bytes() == held > base
    assert {"k_rmm_direct", "k_run_sums"} <= kernel_names(blk, lambda: blk.rmm(B))
    assert "k_tsmm_direct" in kernel_names(blk, lambda: blk.tsmm())
    blk.drop_derived()
    assert blk.derived_bytes() == base
    again = products(blk, B, Y)
    assert blk.derived_bytes() == held
    same(first, again)
    D = ora.np_decompress(specs, n_rows, n_cols)
    assert_close(again[0], D, B, "X%*%B after drop")
    assert_close(again[1], Y, D, "Y%*%X after drop")
    assert_close(again[2], D.T, D, "t(X)%*%X after drop")
    blk.close()


def test_byte_code_block_keeps_its_dictionary_image(cla):
    """The padded dictionary image is made at finalize: drop_derived leaves it, the mat-vec stays on the fused kernel."""
    from systemds_amd import synth
    n_rows, n_cols = 50000, 30
    rng = np.random.default_rng(6)
    specs = [synth.GroupSpec("ddc", np.array([c], np.int32), rng.standard_normal((200, 1)), rng.integers(0, 200, n_rows).astype(np.uint8))
             for c in range(n_cols)]
    v = rng.standard_normal((n_cols, 1))
    blk = cla.build_block(n_rows, n_cols, specs)
    base = blk.derived_bytes()
    assert base > 0
    before = kernel_names(blk, lambda: blk.rmm(v))
    out = blk.rmm(v)[0]
    blk.tsmm()
    blk.rmm(rng.standard_normal((n_cols, 64)))  # matrix-core plan
    assert blk.derived_bytes() > base
    blk.drop_derived()
    assert blk.derived_bytes() == base
    assert kernel_names(blk, lambda: blk.rmm(v)) == before
    assert np.array_equal(blk.rmm(v)[0], out)
    blk.close()


def test_wide_block_and_joint_block_go_too(cla, ora):
    """Blocks the library made for its own use (pairs of column chunks of a wide t(X) %*% X, the joint block of a
    compressed left operand) are derived forms as well."""
    from conftest import mixed_block
    n_rows = 20011
    specs, n_cols = stream_block(8, n_rows, n_rle=2, n_u16=30, n_u8=30, n_sdc=4, n_dense=4, cocoded=False)
    assert n_cols > 64
    blk = cla.build_block(n_rows, n_cols, specs)
    base = blk.derived_bytes()
    g1 = blk.tsmm()[0]
    assert blk.derived_bytes() > base
    blk.drop_derived()
    assert blk.derived_bytes() == base
    same((0, g1), (0, blk.tsmm()[0]))
    blk.close()
    sl, cl = mixed_block(11, n_rows)
    sr, cr = mixed_block(12, n_rows)
    left, right = cla.build_block(n_rows, cl, sl), cla.build_block(n_rows, cr, sr)
    p1 = right.lmm_compressed(left)[0]
    right.drop_derived()
    left.drop_derived()
    same((0, p1), (0, right.lmm_compressed(left)[0]))
    left.close()
    right.close()


def test_prepare_rejects_what_it_does_not_know(cla):
    specs, n_cols = sdc_block(7, 5000, 4, 0.1, 5)
    blk = cla.build_block(5000, n_cols, specs)
    lib = capi.load_library()
    assert lib.cla_block_prepare(blk.h, 8, 1, 1) == capi.ERR_INVALID
    assert lib.cla_block_prepare(blk.h, capi.PRODUCT_RMM, 0, 1) == capi.ERR_INVALID
    assert lib.cla_block_prepare(blk.h, capi.PRODUCT_LMM, 1, 0) == capi.ERR_INVALID
    assert lib.cla_block_prepare(blk.h, 0, 0, 0) == 0
    assert lib.cla_block_drop_derived(None) == capi.ERR_INVALID
    blk.close()
