"""Edge cases of the row structures through the C ABI, every product against the exactly accumulated product of the
decompressed matrix: RLE groups whose runs and gaps are longer than a 16-bit length holds (the encoder splits them
with zero-length runs and zero gaps, ColGroupRLE.java:1073-1157), and SDC groups whose offset lists are empty,
hold one or two rows, nearly all rows or all rows, at row counts around the byte / char offset widths and the
tile sizes (OffsetFactory.java:105-155, 238-340)."""
import numpy as np
import pytest

from parity import assert_matches_truth

pytestmark = pytest.mark.gpu


def all_products(cla, ora, specs, n_rows, n, rng, what):
    D = ora.np_decompress(specs, n_rows, n)
    blk = cla.build_block(n_rows, n, specs)
    try:
        for q in (1, 4, 24):
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
        out, _ = blk.lmm_compressed(blk)
        assert_matches_truth(out, D.T, D, what=f"{what} with itself")
        v = rng.standard_normal((n, 1))
        out, _ = blk.mmchain(v, None, 0)
        Xv, _ = blk.rmm(v)
        assert_matches_truth(out.reshape(-1, 1), D.T, Xv, what=f"{what} mmchain")
        out, _ = blk.aggregate("sum", "col")
        assert_matches_truth(out.reshape(1, -1), np.ones((1, n_rows)), D, what=f"{what} colSums")
        out, nnz = blk.decompress()
        ref = ora.decompress(ora.Groups(specs, n_rows, n))
        assert np.array_equal(out, ref) and nnz == np.count_nonzero(ref)
    finally:
        blk.close()


@pytest.mark.parametrize("seed", [5, 6])
def test_rle_runs_and_gaps_beyond_16_bits(cla, ora, seed):
    from systemds_amd import synth
    rng = np.random.default_rng(seed)
    for case in range(5):
        n_rows = int(rng.choice([70000, 140001, 300007]))
        specs, c = [], 0
        for _ in range(int(rng.integers(1, 5))):
            nv = int(rng.choice([1, 2, 5]))
            codes = np.full(n_rows, -1)
            pos = int(rng.integers(0, 70000))
            while pos < n_rows:
                ln = int(rng.choice([1, 7, 65535, 65536, 70000, 131070, 131071, 200000]))
                codes[pos:pos + ln] = int(rng.integers(0, nv))
                pos += ln + int(rng.choice([0, 1, 65535, 65536, 90000]))
            ptr, data = synth.encode_rle(codes, nv)
            specs.append(synth.GroupSpec("rle", np.array([c], np.int32), rng.standard_normal((nv, 1)), ptr=ptr, rle=data))
            c += 1
        if rng.random() < 0.5:
            specs.append(synth.GroupSpec("ddc", np.array([c, c + 1], np.int32), rng.standard_normal((7, 2)),
                                         rng.integers(0, 7, n_rows).astype(np.uint8)))
            c += 2
        if rng.random() < 0.5:
            specs.append(synth.sdc_group(rng, n_rows, np.array([c], np.int32), 3, 0.00005, 0.5))
            c += 1
        all_products(cla, ora, specs, n_rows, c, rng, f"rle seed {seed} case {case} ({n_rows} rows)")


@pytest.mark.parametrize("seed", [9, 10])
def test_sdc_offset_lists_from_empty_to_every_row(cla, ora, seed):
    from systemds_amd import synth
    rng = np.random.default_rng(seed)
    for case in range(10):
        n_rows = int(rng.choice([1, 2, 255, 256, 257, 4095, 4096, 4097, 65535, 65536, 65537, 200001]))
        specs, c = [], 0
        for _ in range(int(rng.integers(1, 5))):
            dens = float(rng.choice([0.0, 1.0 / n_rows, 2.0 / n_rows, 0.00002, 0.003, 0.5, 0.999, 1.0]))
            nc = int(rng.choice([1, 2]))
            specs.append(synth.sdc_group(rng, n_rows, np.arange(c, c + nc, dtype=np.int32), int(rng.choice([1, 2, 40, 300])),
                                         dens, None if rng.random() < 0.5 else -1.25))
            c += nc
        if rng.random() < 0.4:
            specs.append(synth.GroupSpec("ddc", np.array([c], np.int32), rng.standard_normal((5, 1)),
                                         rng.integers(0, 5, n_rows).astype(np.uint8)))
            c += 1
        all_products(cla, ora, specs, n_rows, c, rng, f"sdc seed {seed} case {case} ({n_rows} rows)")
