"""Benchmark of the compressed multiply hot path on one MI355X.

A step = one pass of compressed X %*% v over BASELINE config 2 (10,000,000 x 100,
single-column DDC groups, 256 values per column, Zipf(1.1) uint8 codes), with the
compressed block, v and the output resident in HBM. Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--scale S] [--no-cpu] [--extra]
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth

# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (two runs,
# scaled against a plain 1 GiB copy: 2.0 KiB per FETCH_SIZE unit, 1.0 KiB per WRITE_SIZE
# unit); figures and commands: profiles/k_rmm_q1_u8_C2_matvec.md. Valid for the full-size
# C2 workload only.
MEASURED_TRAFFIC = {"k_rmm_q1_u8": 510678.0 * 2048 + 99626.9 * 1024}


def timed(blk, fn, reps=5, warm=2):
    """Median wall time of fn() (each call returns nnz, i.e. is synchronous) and the
    per-kernel HIP-event times of the last call."""
    import torch
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    ts = []
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    blk.profile(True)
    fn()
    ks = blk.stats()["kernels"]
    blk.profile(False)
    agg = {}
    for k in ks:
        a = agg.setdefault(k["name"], {"ms": 0.0, "launches": 0, "algo_bytes": 0.0})
        a["ms"] += k["ms"]
        a["launches"] += 1
        a["algo_bytes"] += k["algo_bytes"]
    return statistics.median(ts) * 1e3, agg


def other_configs(scale):
    """X %*% v of C1, the other products of C2, t(X) %*% X of C3, both products of C4 and of C5."""
    import numpy as np
    import torch
    from systemds_amd import capi, synth
    out = {}

    def dev(a):
        return torch.from_numpy(np.ascontiguousarray(a)).cuda()

    def run(name, cfg, ops):
        t0 = time.time()
        blk = capi.build_block(cfg["n_rows"], cfg["n_cols"], cfg["groups"])
        up = time.time() - t0
        for op, fn, algo_bytes in ops(blk, cfg):
            ms, ks = timed(blk, fn)
            out[f"{name} {op}"] = {"ms": ms, "rows_per_s": cfg["n_rows"] / (ms * 1e-3), "algo_bytes": algo_bytes,
                                  "algo_GBs": algo_bytes / (ms * 1e-3) / 1e9,
                                  "frac_hbm": algo_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "kernels": ks,
                                  "upload_s": round(up, 2)}
        blk.close()
        torch.cuda.empty_cache()

    def rmm_ops(vname, q):
        def ops(blk, cfg):
            dv = dev(cfg[vname])
            do = torch.empty((cfg["n_rows"], q), dtype=torch.float64, device="cuda")
            bytes_in = blk.device_bytes()
            yield (f"X%*%{vname}", lambda: blk.rmm_dev(dv.data_ptr(), q, do.data_ptr()), bytes_in + cfg["n_rows"] * q * 8.0)
        return ops

    c = synth.config1()
    run("C1", c, rmm_ops("v", 1))
    c = synth.config2(scale=scale)

    def c2_ops(blk, cfg):
        # the left multiply and the chain on the headline block (the adjacent rows of the scope table)
        n, m = cfg["n_rows"], cfg["n_cols"]
        dy = dev(np.random.default_rng(3).standard_normal((1, n)))
        dv = dev(cfg["v"])
        do1 = torch.empty((1, m), dtype=torch.float64, device="cuda")
        do2 = torch.empty((m,), dtype=torch.float64, device="cuda")
        comp = float(blk.device_bytes())
        dB = dev(cfg["B"])
        q = cfg["B"].shape[1]
        do0 = torch.empty((n, q), dtype=torch.float64, device="cuda")
        yield ("X%*%B", lambda: blk.rmm_dev(dB.data_ptr(), q, do0.data_ptr()), comp + n * q * 8.0)
        yield ("t(y)%*%X", lambda: blk.lmm_dev(dy.data_ptr(), 1, do1.data_ptr()), comp + n * 8.0)
        yield ("t(X)%*%(X%*%v)", lambda: blk.mmchain_dev(dv.data_ptr(), None, 0, do2.data_ptr()), 2 * comp + 2 * n * 8.0)
    run("C2", c, c2_ops)
    del c
    c = synth.config3(scale=scale)

    def tsmm_ops(blk, cfg):
        do = torch.empty((cfg["n_cols"], cfg["n_cols"]), dtype=torch.float64, device="cuda")
        yield ("t(X)%*%X", lambda: blk.tsmm_dev(do.data_ptr()), float(blk.device_bytes()))
        # both operands compressed (here the block with itself, 100 columns over the two sides: every group of the
        # left side meets every group of the right side, 625 pairs)
        yield ("t(X)%*%X as compressed x compressed", lambda: blk.lmm_compressed_dev(blk, do.data_ptr()),
               2 * float(blk.device_bytes()))
    run("C3", c, tsmm_ops)
    del c
    c = synth.config4(scale=scale)

    def c4_ops(blk, cfg):
        dv, du = dev(cfg["v"]), dev(cfg["u"])
        do1 = torch.empty((1, cfg["n_cols"]), dtype=torch.float64, device="cuda")
        do2 = torch.empty((cfg["n_rows"], 1), dtype=torch.float64, device="cuda")
        comp = float(sum(g.deltas.nbytes + g.codes.nbytes for g in cfg["groups"]))
        yield ("t(v)%*%X", lambda: blk.lmm_dev(dv.data_ptr(), 1, do1.data_ptr()), comp + cfg["n_rows"] * 8.0)
        yield ("X%*%u", lambda: blk.rmm_dev(du.data_ptr(), 1, do2.data_ptr()), comp + cfg["n_rows"] * 8.0)
    run("C4", c, c4_ops)
    del c
    c = synth.config5(scale=scale)

    def c5_ops(blk, cfg):
        dB = dev(cfg["B"])
        do1 = torch.empty((cfg["n_rows"], 10), dtype=torch.float64, device="cuda")
        do2 = torch.empty((20, 20), dtype=torch.float64, device="cuda")
        comp = float(blk.device_bytes())
        yield ("X%*%B", lambda: blk.rmm_dev(dB.data_ptr(), 10, do1.data_ptr()), comp + cfg["n_rows"] * 80.0)
        yield ("t(X)%*%X", lambda: blk.tsmm_dev(do2.data_ptr()), comp)
        # 40 columns over the two sides: the joint rows are decoded once and multiplied on the matrix cores
        yield ("t(X)%*%X as compressed x compressed", lambda: blk.lmm_compressed_dev(blk, do2.data_ptr()), 2 * comp)
    run("C5", c, c5_ops)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--scale", type=int, default=1, help="divide the number of rows (testing only)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--extra", action="store_true", help="also time X %*% B (100x64) of the same config")
    ap.add_argument("--all", action="store_true", help="also time the other products and BASELINE configs (C1, C2 mat-mat, left multiply and chain, C3, C4, C5)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy (torch) so that a rocprofv3 --pmc run can scale "
                         "FETCH_SIZE / WRITE_SIZE against a kernel of known traffic")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (the path shards by rows, each GPU taking a row range of every group); "
              f"--gpus {args.gpus} is not supported", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from systemds_amd import capi, synth

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)
    capi.init(0)

    t0 = time.time()
    cfg = synth.config2(scale=args.scale)
    n_rows, n_cols = cfg["n_rows"], cfg["n_cols"]
    t_gen = time.time() - t0
    t0 = time.time()
    blk = capi.build_block(n_rows, n_cols, cfg["groups"])
    t_upload = time.time() - t0

    stream = torch.cuda.Stream()
    blk.set_stream(stream.cuda_stream)
    dv = torch.from_numpy(cfg["v"].copy()).cuda()
    dout = torch.empty(n_rows, dtype=torch.float64, device="cuda")
    torch.cuda.synchronize()

    def step():
        return blk.rmm_dev(dv.data_ptr(), 1, dout.data_ptr())

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # whole-job throughput: wall clock over exactly K steps (each step returns nnz,
    # i.e. includes its own stream synchronisation)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        nnz = step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3

    # dominant kernel: HIP events on the stream the kernel is launched on
    blk.profile(True)
    kms, kbytes, kname = [], 0.0, ""
    for _ in range(min(args.steps, 20)):
        step()
        ks = blk.stats()["kernels"]
        dom = max(ks, key=lambda k: k["ms"])
        kms.append(dom["ms"])
        kbytes, kname = dom["algo_bytes"], dom["name"]
    blk.profile(False)
    k_ms = statistics.mean(kms)
    achieved = kbytes / (k_ms * 1e-3) / 1e9

    result = {
        "metric": "compressed X%*%v on DDC 10Mx100: rows/s and achieved HBM GB/s vs peak",
        "value": n_rows / (ms_per_step * 1e-3),
        "unit": "rows/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f64", "data": "synthetic",
        "config": {"workload": f"C2 X%*%v: {n_rows}x{n_cols} fp64 as {n_cols} single-column DDC groups, 256 values, "
                               "Zipf(1.1) uint8 codes, v 100x1; block, v and output resident in HBM",
                   "nnz": int(nnz), "gen_s": round(t_gen, 2), "upload_s": round(t_upload, 2),
                   "block_bytes": int(blk.device_bytes())},
        "roofline": {"bound": "hbm", "kernel": kname, "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "kernel_ms": k_ms, "algo_bytes_per_launch": kbytes,
                     "traffic": MEASURED_TRAFFIC.get(kname) if args.scale == 1 else None},
    }

    if args.calibrate_copy:
        src = torch.empty(1 << 27, dtype=torch.float64, device="cuda").fill_(1.0)  # 1 GiB
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    if args.extra:
        dB = torch.from_numpy(cfg["B"].copy()).cuda()
        doutB = torch.empty((n_rows, 64), dtype=torch.float64, device="cuda")
        for _ in range(2):
            blk.rmm_dev(dB.data_ptr(), 64, doutB.data_ptr())
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        reps = max(args.steps // 5, 3)
        for _ in range(reps):
            blk.rmm_dev(dB.data_ptr(), 64, doutB.data_ptr())
        torch.cuda.synchronize()
        msB = (time.perf_counter() - t0) / reps * 1e3
        bytesB = n_rows * (n_cols + 64 * 8.0)
        result["extra"] = {"C2 X%*%B(100x64)": {"ms": msB, "rows_per_s": n_rows / (msB * 1e-3),
                                                "algo_GBs": bytesB / (msB * 1e-3) / 1e9,
                                                "frac_hbm": bytesB / (msB * 1e-3) / 1e9 / HBM_PEAK_GBS}}
        del doutB

    if args.all:
        blk.close()
        result.setdefault("extra", {}).update(other_configs(args.scale))

    if not args.no_cpu:
        # CPU baseline: the oracle's multithreaded restatement of the reference algorithm
        # (a port, not the SystemDS JVM) on the same full workload, host cores of this box.
        from oracle import cla_oracle as ora
        cores = min(len(os.sched_getaffinity(0)), int(os.environ.get("OMP_NUM_THREADS", "64")))
        G = ora.Groups(cfg["groups"], n_rows, n_cols)
        times = []
        for _ in range(3):
            t0 = time.perf_counter()
            ref, rnnz = ora.rmm(G, cfg["v"], cores)
            times.append(time.perf_counter() - t0)
        cpu_s = statistics.median(times)
        got = dout.cpu().numpy()
        result["cpu_baseline"] = {"value": n_rows / cpu_s, "unit": "rows/s", "cores": cores, "kind": "port",
                                  "sample": f"the full workload ({n_rows} rows x {n_cols} groups), median of 3 passes, "
                                            f"{cpu_s:.3f} s per pass",
                                  "parity_bit_exact": bool(np.array_equal(got, ref[:, 0]) and rnnz == nnz)}

    if not args.all:
        blk.close()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
