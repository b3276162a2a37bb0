"""Times the products on block shapes beside the benchmark configurations: what the dispatch does off the headline.

    python -m systemds_amd.shapes_bench [--rows N] [--only NAME]

One line per (shape, product): milliseconds per call (operands resident in HBM, three calls queued back to back)
and the three kernels that took most of it (per-kernel times from the library's own events, one profiled call).
Shapes: 60 single-column DDC groups with two-byte codes and 1000 values each; 12 co-coded DDC groups of 4 columns with
byte codes; 30 RLE columns with runs of 200 rows on average; 40 SDC columns (5 % of the rows listed, with a default)
beside 10 byte-code DDC columns; 90 dense columns in 3 uncompressed groups (a quarter of the rows).
"""
import argparse
import time

import numpy as np


def _rle_group(synth, rng, n_rows, col, n_vals, mean_run):
    lens = rng.geometric(1.0 / mean_run, size=int(n_rows / mean_run * 1.3) + 16)
    codes = np.repeat(rng.integers(0, n_vals, size=lens.size), lens)[:n_rows]
    if codes.size < n_rows:
        codes = np.concatenate([codes, np.zeros(n_rows - codes.size, dtype=codes.dtype)])
    ptr, data = synth.encode_rle(codes, n_vals)
    return synth.GroupSpec("rle", np.array([col], np.int32), rng.standard_normal((n_vals, 1)), ptr=ptr, rle=data)


def shapes(synth, rng, n):
    """(name, number of rows, group specs, number of columns) per shape."""
    yield "ddc16x60", n, [synth.GroupSpec("ddc", np.array([c], np.int32), rng.standard_normal((1000, 1)),
                                          rng.integers(0, 1000, n).astype(np.uint16)) for c in range(60)], 60
    yield "cocoded4x12", n, [synth.GroupSpec("ddc", np.arange(4 * g, 4 * g + 4, dtype=np.int32), rng.standard_normal((200, 4)),
                                             rng.integers(0, 200, n).astype(np.uint8)) for g in range(12)], 48
    yield "rle30", n, [_rle_group(synth, rng, n, c, 16, 200) for c in range(30)], 30
    sp = [synth.sdc_group(rng, n, np.array([c], np.int32), 30, 0.05, 1.0) for c in range(40)]
    sp += [synth.GroupSpec("ddc", np.array([40 + c], np.int32), rng.standard_normal((50, 1)), rng.integers(0, 50, n).astype(np.uint8))
           for c in range(10)]
    yield "sdc40+ddc10", n, sp, 50
    yield "dense3x30", n // 4, [synth.GroupSpec("unc", np.arange(30 * g, 30 * g + 30, dtype=np.int32),
                                                dense=rng.standard_normal((n // 4, 30))) for g in range(3)], 90


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--rows", type=int, default=4_000_000)
    ap.add_argument("--only", default=None)
    args = ap.parse_args()
    import torch
    from systemds_amd import capi, synth
    torch.cuda.set_device(0)
    capi.init(0)
    rng = np.random.default_rng(5)
    for name, n, specs, m in shapes(synth, rng, args.rows):
        if args.only and args.only not in name:
            continue
        blk = capi.build_block(n, m, specs)

        def timed(fn, reps=3):
            fn(); fn(); blk.nnz(); torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(reps):
                fn()
            blk.nnz(); torch.cuda.synchronize()
            ms = (time.perf_counter() - t0) / reps * 1e3
            blk.profile(True); fn(); blk.nnz(); ks = blk.stats()["kernels"]; blk.profile(False)
            per = {}
            for k in ks:
                per[k["name"]] = per.get(k["name"], 0.0) + k["ms"]
            top = sorted(per.items(), key=lambda kv: -kv[1])[:3]
            return "%8.2f ms  " % ms + ", ".join("%s %.2f" % (k, v) for k, v in top)

        print("%s: %d x %d" % (name, n, m), flush=True)
        for q in (1, 10, 64):
            B = torch.randn(m, q, dtype=torch.float64, device="cuda")
            out = torch.empty((n, q), dtype=torch.float64, device="cuda")
            print("  X %%*%% B, %2d columns  " % q, timed(lambda: blk.rmm_dev_async(B.data_ptr(), q, out.data_ptr())), flush=True)
            del B, out
        for p in (1, 8, 40):
            Y = torch.randn(p, n, dtype=torch.float64, device="cuda")
            out = torch.empty((p, m), dtype=torch.float64, device="cuda")
            print("  Y %%*%% X, %2d rows     " % p, timed(lambda: blk.lmm_dev_async(Y.data_ptr(), p, out.data_ptr())), flush=True)
            del Y, out
        G = torch.empty((m, m), dtype=torch.float64, device="cuda")
        print("  t(X) %*% X           ", timed(lambda: blk.tsmm_dev_async(G.data_ptr())), flush=True)
        del G
        D = torch.empty((n, m), dtype=torch.float64, device="cuda")
        print("  decompress           ", timed(lambda: blk.decompress_dev(D.data_ptr())), flush=True)
        del D
        blk.close()


if __name__ == "__main__":
    main()
