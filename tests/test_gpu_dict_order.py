"""GPU tests of the numbering of DDC tuples by count: finalize renumbers the block's copy of a group with two- or
four-byte codes and a large dictionary (option ddc_reorder, systemds_amd/csrc/k_aux.hip: reorder_ddc_by_count), which
the reference does not do (it numbers by first appearance, ColGroupFactory.java:682-703). Nothing a caller sees may
depend on it: the products are compared with those of a block that keeps the caller's numbering (X %*% B bit for bit,
the products that add across workgroups at 1e-12 of their scale) and with the decompressed block; counts,
co-occurrence and pre-aggregates, which are indexed by code, are compared in the caller's numbering with numpy on the
uploaded codes (integers bit-exact)."""
import numpy as np
import pytest

from systemds_amd import synth
from systemds_amd.capi import ClaBlock

pytestmark = pytest.mark.gpu


def skewed_specs(seed, n_rows):
    """Four DDC groups: two co-coded pairs with 4096 tuples (two-byte codes), one column with 3000 values in four-byte
    codes, one byte-code column (never renumbered). Codes are Zipf-distributed under a random numbering."""
    rng = np.random.default_rng(seed)
    specs = []
    c = 0
    for n_vals, width, dt, s in ((4096, 2, np.uint16, 1.0), (4096, 2, np.uint16, 1.3), (3000, 1, np.int32, 1.1), (200, 1, np.uint8, 1.1)):
        d = rng.uniform(-1, 1, size=(n_vals, width))
        codes = synth._zipf_codes(rng, n_rows, n_vals, s, dt)
        specs.append(synth.GroupSpec("ddc", np.arange(c, c + width, dtype=np.int32), d, codes))
        c += width
    return specs, c


def build(n_rows, n_cols, specs, reorder, profile=False):
    b = ClaBlock(n_rows, n_cols)
    b.set_option("ddc_reorder", reorder)
    if profile:
        b.profile(True)
    for s in specs:
        b.add(s)
    b.finalize()
    names = []
    if profile:
        names = [k["name"] for k in b.stats()["kernels"]]
        b.profile(False)
    return b, names


def close(a, b, scale):
    assert a.shape == b.shape
    assert np.all(np.abs(a - b) <= 1e-12 * scale), float(np.max(np.abs(a - b) / scale))


@pytest.mark.parametrize("n_rows", [70001, 262144])
def test_products_do_not_depend_on_the_numbering(cla, ora, n_rows):
    specs, n_cols = skewed_specs(11, n_rows)
    kept, names0 = build(n_rows, n_cols, specs, 0, profile=True)
    byc, names1 = build(n_rows, n_cols, specs, 1, profile=True)
    assert "k_recode" not in names0
    assert names1.count("k_recode") == 3  # the byte-code group keeps its numbering
    rng = np.random.default_rng(5)
    B, v = rng.standard_normal((n_cols, 7)), rng.standard_normal((n_cols, 1))
    Y = rng.standard_normal((3, n_rows))
    D = ora.np_decompress(specs, n_rows, n_cols)
    for M in (B, v):
        a, b = kept.rmm(M)[0], byc.rmm(M)[0]
        assert np.array_equal(a, b)
        close(b, D @ M, np.abs(D) @ np.abs(M) + 1e-300)
    a, b = kept.lmm(Y)[0], byc.lmm(Y)[0]
    close(a, b, np.abs(Y) @ np.abs(D))
    close(b, (Y.astype(np.longdouble) @ D.astype(np.longdouble)).astype(np.float64), np.abs(Y) @ np.abs(D))
    a, b = kept.tsmm()[0], byc.tsmm()[0]
    close(a, b, np.abs(D).T @ np.abs(D))
    Dl = D.astype(np.longdouble)
    close(b, (Dl.T @ Dl).astype(np.float64), np.abs(D).T @ np.abs(D))
    a, b = kept.mmchain(v)[0], byc.mmchain(v)[0]
    close(a, b, np.abs(D).T @ (np.abs(D) @ np.abs(v)).reshape(-1))
    kept.close()
    byc.close()


def test_code_indexed_results_keep_the_callers_numbering(cla):
    n_rows = 131077
    specs, n_cols = skewed_specs(12, n_rows)
    blk, names = build(n_rows, n_cols, specs, 1, profile=True)
    assert names.count("k_recode") == 3
    rng = np.random.default_rng(6)
    Y = rng.standard_normal((2, n_rows))
    for g, s in enumerate(specs):
        n_vals = s.dict.shape[0]
        codes = s.codes.astype(np.int64)
        assert np.array_equal(blk.counts(g), np.bincount(codes, minlength=n_vals))
        pre = blk.preagg(g, Y)
        for r in range(2):
            ref = np.bincount(codes, weights=Y[r], minlength=n_vals)
            scale = np.bincount(codes, weights=np.abs(Y[r]), minlength=n_vals) + 1e-300
            assert np.all(np.abs(pre[r] - ref) <= 1e-12 * scale)
    for ga, gb in ((0, 1), (2, 0), (1, 3), (3, 2)):
        na, nb = specs[ga].dict.shape[0], specs[gb].dict.shape[0]
        key = specs[ga].codes.astype(np.int64) * nb + specs[gb].codes.astype(np.int64)
        ref = np.bincount(key, minlength=na * nb).reshape(na, nb)
        assert np.array_equal(blk.cooc(ga, gb), ref)
    blk.close()


def test_blocks_that_borrow_the_codes_follow_the_numbering(cla, ora):
    n_rows = 90000
    specs, n_cols = skewed_specs(13, n_rows)
    blk, _ = build(n_rows, n_cols, specs, 1)
    rng = np.random.default_rng(7)
    B = rng.standard_normal((n_cols, 5))
    D = ora.np_decompress(specs, n_rows, n_cols)
    XB = D @ B
    child = blk.rmm_overlapping(B)
    w = rng.standard_normal((5, 2))
    close(child.rmm(w)[0], XB @ w, np.abs(D) @ np.abs(B) @ np.abs(w))
    y = rng.standard_normal((1, n_rows))
    close(child.lmm(y)[0], y @ XB, np.abs(y) @ (np.abs(D) @ np.abs(B)))
    for g in (0, 2):
        assert np.array_equal(child.counts(g), np.bincount(specs[g].codes.astype(np.int64), minlength=specs[g].dict.shape[0]))
    # compressed x compressed: both sides renumbered
    other, _ = build(n_rows, n_cols, skewed_specs(14, n_rows)[0], 1)
    D2 = ora.np_decompress(skewed_specs(14, n_rows)[0], n_rows, n_cols)
    close(blk.lmm_compressed(other)[0], D2.T @ D, np.abs(D2).T @ np.abs(D))
    child.close()
    other.close()
    blk.close()


def test_uniform_codes_and_short_blocks_are_left_alone(cla):
    # fewer than 16 rows per tuple: the pass over the codes would not pay
    n_rows = 40000
    specs, n_cols = skewed_specs(15, n_rows)
    blk, names = build(n_rows, n_cols, specs, 1, profile=True)
    assert names.count("k_recode") == 0
    assert np.array_equal(blk.counts(0), np.bincount(specs[0].codes.astype(np.int64), minlength=4096))
    blk.close()
    # already numbered by descending count: nothing to do
    n_rows = 100000
    codes = np.sort(np.random.default_rng(3).integers(0, 2048, n_rows)).astype(np.uint16)
    order = np.argsort(-np.bincount(codes, minlength=2048), kind="stable")
    lut = np.empty(2048, np.int64)
    lut[order] = np.arange(2048)
    s = synth.GroupSpec("ddc", np.array([0], np.int32), np.random.default_rng(4).standard_normal((2048, 1)), lut[codes].astype(np.uint16))
    blk, names = build(n_rows, 1, [s], 1, profile=True)
    assert names.count("k_recode") == 0
    blk.close()
