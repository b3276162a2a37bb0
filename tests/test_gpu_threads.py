"""Thread safety of the C ABI as the boundary promises it: calls on different handles may run in parallel (parfor
bodies and Spark tasks multiply different blocks at once, each block on its own stream), calls on one handle
serialise on the handle's lock, and the compressed x compressed product, which takes two handles, may be entered with
the roles swapped by two threads at once."""
import threading

import numpy as np
import pytest

from conftest import mixed_block

pytestmark = pytest.mark.gpu

N_ROWS = 60007


def run_threads(jobs, pick, cross):
    errors = []

    def worker(i):
        blk, B, Y, v, r0, l0, t0, m0 = jobs[pick(i)]
        try:
            for _ in range(25):
                got = (blk.rmm(B)[0], blk.lmm(Y)[0], blk.tsmm()[0], blk.mmchain(v, None, 0)[0])
                for name, a, b in zip(("rmm", "lmm", "tsmm", "mmchain"), got, (r0, l0, t0, m0)):
                    # sums that use atomics differ in their last bits from call to call
                    if not np.allclose(a, b, rtol=1e-11, atol=1e-9):
                        errors.append((i, name, float(np.abs(a - b).max())))
                if cross:
                    other = jobs[(i + 1) % len(jobs)][0]
                    blk.lmm_compressed(other)
        except Exception as e:  # noqa: BLE001 - any failure of a worker fails the test
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    return errors


def test_parallel_calls_on_different_and_on_the_same_handle(cla, ora):
    rng = np.random.default_rng(1)
    jobs = []
    for seed in range(4):
        specs, n = mixed_block(seed + 40, N_ROWS, with_unc=(seed % 2 == 0))
        blk = cla.build_block(N_ROWS, n, specs)
        B, Y, v = rng.standard_normal((n, 8)), rng.standard_normal((2, N_ROWS)), rng.standard_normal((n, 1))
        jobs.append((blk, B, Y, v, blk.rmm(B)[0], blk.lmm(Y)[0], blk.tsmm()[0], blk.mmchain(v, None, 0)[0]))
    try:
        assert run_threads(jobs, lambda i: i, cross=True) == []     # four handles, neighbours also meet as t(L) %*% R
        assert run_threads(jobs, lambda i: 0, cross=False) == []    # one handle from four threads
    finally:
        for j in jobs:
            j[0].close()


def test_parallel_calls_whose_kernels_need_different_amounts_of_lds(cla, ora):
    """Two handles whose products run the same kernels with different dynamic LDS sizes (dictionaries of 16 and of
    3000 tuples; 20 and 90 list groups): the per-kernel LDS allowance is a property of the kernel, not of the call
    that happened to set it last."""
    from systemds_amd import synth
    rng = np.random.default_rng(5)
    n_rows = 40009
    jobs = []
    for n_ddc, n_vals, n_sdc in ((4, 16, 20), (12, 3000, 90)):
        specs, c = [], 0
        for g in range(n_ddc):
            specs.append(synth.GroupSpec("ddc", np.array([c, c + 1], np.int32), rng.standard_normal((n_vals, 2)),
                                         rng.integers(0, n_vals, n_rows).astype(np.uint16 if n_vals > 256 else np.uint8)))
            c += 2
        for g in range(n_sdc):
            specs.append(synth.sdc_group(np.random.default_rng((5, g)), n_rows, np.array([c], np.int32), 30, 0.04, None))
            c += 1
        blk = cla.build_block(n_rows, c, specs)
        B, Y, v = rng.standard_normal((c, 8)), rng.standard_normal((2, n_rows)), rng.standard_normal((c, 1))
        jobs.append((blk, B, Y, v, blk.rmm(B)[0], blk.lmm(Y)[0], blk.tsmm()[0], blk.mmchain(v, None, 0)[0]))
    try:
        assert run_threads(jobs, lambda i: i % 2, cross=False) == []
    finally:
        for j in jobs:
            j[0].close()
