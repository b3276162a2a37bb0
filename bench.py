"""Benchmark of the compressed multiply hot path on one MI355X.

A step = one pass of compressed X %*% v over BASELINE config 2 (10,000,000 x 100,
single-column DDC groups, 256 values per column, Zipf(1.1) uint8 codes), with the
compressed block, v and the output resident in HBM. Prints ONE JSON line: the headline
(`value`, `roofline`, `cpu_baseline`) plus, under `extra`, one row per other product of the
BASELINE configs (kernel, kernel time, algorithmic bytes or flops, fraction of the bound, and the CPU
oracle's rate on the same input).

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--scale S] [--no-cpu] [--no-extra]
"""
import argparse
import hashlib
import json
import os
import re
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0     # MI355X published HBM3E bandwidth
MFMA_F64_PEAK_TF = 78.6   # MI355X published dense fp64 matrix rate

# Sources whose text decides what the headline kernel does; a traffic figure measured with rocprofv3 is only
# reported while their hash matches the one recorded next to the figure.
HEADLINE_SOURCES = ["systemds_amd/csrc/k_rmm.hip", "systemds_amd/csrc/cla_device.hpp"]
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "k_rmm_q1_u8_C2_matvec.md")


def headline_source_hash():
    h = hashlib.sha256()
    for rel in HEADLINE_SOURCES:
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def profiled_traffic():
    """HBM bytes per launch of the headline kernel from the committed rocprofv3 --pmc summary (FETCH_SIZE and
    WRITE_SIZE runs scaled against a plain copy), or None when the kernel's sources changed since."""
    try:
        text = open(TRAFFIC_FILE).read()
    except OSError:
        return None, "no profile summary"
    m = re.search(r"traffic_bytes_per_launch:\s*([0-9.eE+]+)\s+source_hash:\s*([0-9a-f]+)", text)
    if not m:
        return None, "profile summary holds no traffic line"
    if m.group(2) != headline_source_hash():
        return None, f"stale: measured at source hash {m.group(2)}, sources now {headline_source_hash()}"
    return float(m.group(1)), f"rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, {os.path.relpath(TRAFFIC_FILE, ROOT)}"


def cpu_row(fn, n_rows, what):
    """CPU baseline of one row: the oracle's multithreaded restatement of the reference algorithm (a port, not the
    SystemDS JVM) on the same compressed input as the GPU row (the whole workload: the longest, C5 t(X)%*%X, takes
    under ten seconds a pass), host cores of this box, median of 3 passes."""
    cores = min(len(os.sched_getaffinity(0)), int(os.environ.get("OMP_NUM_THREADS", "64")))
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        fn(cores)
        times.append(time.perf_counter() - t0)
    sec = statistics.median(times)
    return {"value": n_rows / sec, "unit": "rows/s", "cores": cores, "kind": "port",
            "sample": f"{what}: the full workload ({n_rows} rows), median of 3 passes, {sec:.3f} s per pass"}


DEVICE_WARMUP_MS = 300.0  # set from --device-warmup-ms


def time_async(blk, launch, reps, warm=2):
    """Wall time per call of `launch` (queues the driver's kernels without waiting) over `reps` calls bracketed
    by device synchronisation, and the per-kernel HIP-event times of five more calls. Like the headline, a row is
    timed behind an untimed device warm-up (calls of the same product for --device-warmup-ms: the host work between
    two rows - generating and uploading the next configuration, the CPU legs - leaves the device idle for seconds, and
    its first milliseconds of load run at transient clocks); the figure without it is returned as well."""
    import torch

    def train():
        blk.nnz()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            launch()
        blk.nnz()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / reps * 1e3

    for _ in range(warm):
        launch()
    cold_ms = train()
    t_w = time.perf_counter()
    while time.perf_counter() - t_w < DEVICE_WARMUP_MS * 1e-3:
        for _ in range(max(1, reps // 2)):
            launch()
        blk.nnz()
    ms = train()
    # per-kernel HIP-event times: the median over five profiled calls of each kernel's summed time in a call
    blk.profile(True)
    calls = []
    for _ in range(5):
        launch()
        blk.nnz()
        one = {}
        for k in blk.stats()["kernels"]:
            a = one.setdefault(k["name"], {"ms": 0.0, "launches": 0})
            a["ms"] += k["ms"]
            a["launches"] += 1
        calls.append(one)
    blk.profile(False)
    agg = {name: {"ms": statistics.median(c[name]["ms"] for c in calls if name in c), "launches": calls[-1][name]["launches"]}
           for name in calls[-1]}
    return ms, agg, cold_ms


def extra_row(blk, launch, n_rows, algo_bytes, flops=0.0, reps=10, prepare=None):
    """One row of `extra`: first-call time (includes derived formats built on first use), steady-state wall
    time per call, the dominant kernel with its HIP-event time, and the fraction of the bound that limits the
    call (the larger of the HBM floor and the fp64 matrix floor) over the summed HIP-event times of all its
    kernels. With `prepare` (a call of cla_block_prepare for this product) the row starts from a block without
    derived formats, so that `derived_bytes_built` is this product's alone, and also gives the time of the prepare
    call and of the first product call behind it."""
    import torch
    if prepare:
        blk.drop_derived()
    torch.cuda.synchronize()
    d0 = blk.derived_bytes()
    t0 = time.perf_counter()
    launch()
    blk.nnz()
    first_ms = (time.perf_counter() - t0) * 1e3
    prep = {}
    if prepare:
        blk.drop_derived()
        t0 = time.perf_counter()
        prepare()
        prep["prepare_ms"] = round((time.perf_counter() - t0) * 1e3, 3)
        t0 = time.perf_counter()
        launch()
        blk.nnz()
        prep["first_call_after_prepare_ms"] = round((time.perf_counter() - t0) * 1e3, 3)
    ms, ks, cold_ms = time_async(blk, launch, reps)
    kname = max(ks, key=lambda k: ks[k]["ms"])
    kms = ks[kname]["ms"]
    ksum = sum(v["ms"] for v in ks.values())
    hbm_floor_ms = algo_bytes / (HBM_PEAK_GBS * 1e9) * 1e3
    mfma_floor_ms = flops / (MFMA_F64_PEAK_TF * 1e12) * 1e3
    row = {"ms": round(ms, 5), "cold_ms": round(cold_ms, 5), "first_call_ms": round(first_ms, 3), "rows_per_s": n_rows / (ms * 1e-3),
           "kernel": kname, "kernel_ms": round(kms, 5), "kernels": {k: round(v["ms"], 5) for k, v in ks.items()},
           "kernels_ms": round(ksum, 5), "algo_bytes": algo_bytes, "algo_GBs": algo_bytes / (ksum * 1e-3) / 1e9,
           "frac_hbm": algo_bytes / (ksum * 1e-3) / 1e9 / HBM_PEAK_GBS,
           "derived_bytes_built": int(blk.derived_bytes() - d0), **prep}
    if flops:
        row["flops"] = flops
        row["frac_mfma_f64"] = flops / (ksum * 1e-3) / 1e12 / MFMA_F64_PEAK_TF
    if mfma_floor_ms > hbm_floor_ms:
        row["bound"], row["frac"] = "mfma_f64", row["frac_mfma_f64"]
    else:
        row["bound"], row["frac"] = "hbm", row["frac_hbm"]
    return row


def other_rows(scale, c2, c2_blk, out, cpu=True):
    """The other products of C2 on the headline block, then C3, C4 and C5 (generated, uploaded, measured and
    freed one after the other)."""
    import numpy as np
    import torch
    from systemds_amd import capi, synth

    def dev(a):
        return torch.from_numpy(np.ascontiguousarray(a)).cuda()

    # ---- C2: X %*% B (100 x 64), t(y) %*% X, the chain
    n, m = c2["n_rows"], c2["n_cols"]
    comp = float(c2_blk.device_bytes())
    dB, dv = dev(c2["B"]), dev(c2["v"])
    dy = dev(np.random.default_rng(3).standard_normal((1, n)))
    q = c2["B"].shape[1]
    doB = torch.empty((n, q), dtype=torch.float64, device="cuda")
    do1 = torch.empty((1, m), dtype=torch.float64, device="cuda")
    do2 = torch.empty((m,), dtype=torch.float64, device="cuda")
    out["C2 X%*%B"] = extra_row(c2_blk, lambda: c2_blk.rmm_dev_async(dB.data_ptr(), q, doB.data_ptr()), n,
                                comp + n * q * 8.0, flops=2.0 * n * m * q, reps=5)
    del doB
    out["C2 t(y)%*%X"] = extra_row(c2_blk, lambda: c2_blk.lmm_dev_async(dy.data_ptr(), 1, do1.data_ptr()), n, comp + n * 8.0)
    out["C2 t(X)%*%(X%*%v)"] = extra_row(c2_blk, lambda: c2_blk.mmchain_dev_async(dv.data_ptr(), None, 0, do2.data_ptr()), n,
                                         2 * comp + 2 * n * 8.0)
    c2_blk.close()
    torch.cuda.empty_cache()
    def cpu_rows(cs, legs):
        """CPU legs of one configuration on the GPU rows' own input: legs = [(row name, what, fn(ora, G, cfg, k))]."""
        if not cpu:
            return
        from oracle import cla_oracle as ora
        G = ora.Groups(cs["groups"], cs["n_rows"], cs["n_cols"])
        for name, what, fn in legs:
            if name in out:
                out[name]["cpu_baseline"] = cpu_row(lambda k: fn(ora, G, cs, k), cs["n_rows"], what)
    ys = dy.cpu().numpy()
    cpu_rows(c2, [("C2 X%*%B", "X%*%B", lambda ora, G, c, k: ora.rmm(G, c["B"], k)),
                  ("C2 t(y)%*%X", "t(y)%*%X", lambda ora, G, c, k: ora.lmm(G, ys, k)),
                  ("C2 t(X)%*%(X%*%v)", "t(X)%*%(X%*%v)", lambda ora, G, c, k: ora.mmchain(G, c["v"], None, 0, k))])

    def with_block(cfg, fn, legs=()):
        t0 = time.time()
        blk = capi.build_block(cfg["n_rows"], cfg["n_cols"], cfg["groups"])
        up = round(time.time() - t0, 2)
        try:
            for name, row in fn(blk, cfg):
                row["upload_s"] = up
                row["block_bytes"] = int(blk.device_bytes())
                row["derived_bytes"] = int(blk.derived_bytes())
                out[name] = row
        finally:
            blk.close()
            torch.cuda.empty_cache()
        cpu_rows(cfg, legs)

    # ---- C3: t(X) %*% X (50 x 50); useful flops: the upper triangle once
    def c3_rows(blk, cfg):
        n, m = cfg["n_rows"], cfg["n_cols"]
        do = torch.empty((m, m), dtype=torch.float64, device="cuda")
        yield "C3 t(X)%*%X", extra_row(blk, lambda: blk.tsmm_dev_async(do.data_ptr()), n, float(blk.device_bytes()),
                                       flops=2.0 * n * m * (m + 1) / 2)
    with_block(synth.config3(scale=scale), c3_rows, [("C3 t(X)%*%X", "t(X)%*%X", lambda ora, G, c, k: ora.tsmm(G, k))])

    # ---- C4: t(v) %*% X and X %*% u on SDC lists (compulsory bytes: delta and code bytes once, the vector once)
    def c4_rows(blk, cfg):
        n, m = cfg["n_rows"], cfg["n_cols"]
        dv4, du = dev(cfg["v"]), dev(cfg["u"])
        do1 = torch.empty((1, m), dtype=torch.float64, device="cuda")
        do2 = torch.empty((n, 1), dtype=torch.float64, device="cuda")
        lists = float(sum(g.deltas.nbytes + g.codes.nbytes for g in cfg["groups"]))
        yield "C4 t(v)%*%X", extra_row(blk, lambda: blk.lmm_dev_async(dv4.data_ptr(), 1, do1.data_ptr()), n, lists + n * 8.0,
                                       prepare=lambda: blk.prepare(lmm_rows=1))
        yield "C4 X%*%u", extra_row(blk, lambda: blk.rmm_dev_async(du.data_ptr(), 1, do2.data_ptr()), n, lists + n * 8.0,
                                    prepare=lambda: blk.prepare(rmm_cols=1))
    with_block(synth.config4(scale=scale), c4_rows,
               [("C4 t(v)%*%X", "t(v)%*%X", lambda ora, G, c, k: ora.lmm(G, c["v"].reshape(1, -1), k)),
                ("C4 X%*%u", "X%*%u", lambda ora, G, c, k: ora.rmm(G, c["u"], k))])

    # ---- C5: X %*% B (20 x 10) and t(X) %*% X on the mixed block
    def c5_rows(blk, cfg):
        n, m = cfg["n_rows"], cfg["n_cols"]
        dB5 = dev(cfg["B"])
        do1 = torch.empty((n, 10), dtype=torch.float64, device="cuda")
        do2 = torch.empty((m, m), dtype=torch.float64, device="cuda")
        comp = float(blk.device_bytes())
        yield "C5 X%*%B", extra_row(blk, lambda: blk.rmm_dev_async(dB5.data_ptr(), 10, do1.data_ptr()), n, comp + n * 80.0,
                                    flops=2.0 * n * m * 10, reps=5, prepare=lambda: blk.prepare(rmm_cols=10))
        yield "C5 t(X)%*%X", extra_row(blk, lambda: blk.tsmm_dev_async(do2.data_ptr()), n, comp,
                                       flops=2.0 * n * m * (m + 1) / 2, reps=5, prepare=lambda: blk.prepare(tsmm=True))
    with_block(synth.config5(scale=scale), c5_rows,
               [("C5 X%*%B", "X%*%B", lambda ora, G, c, k: ora.rmm(G, c["B"], k)),
                ("C5 t(X)%*%X", "t(X)%*%X", lambda ora, G, c, k: ora.tsmm(G, k))])


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--scale", type=int, default=1, help="divide the number of rows (testing only)")
    ap.add_argument("--device-warmup-ms", type=float, default=300.0,
                    help="untimed passes of the same step until the device clocks are steady (0 = none)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="headline only: skip the other products and configs")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy (torch) so that a rocprofv3 --pmc run can scale "
                         "FETCH_SIZE / WRITE_SIZE against a kernel of known traffic")
    args = ap.parse_args()
    global DEVICE_WARMUP_MS
    DEVICE_WARMUP_MS = args.device_warmup_ms
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
        # queues the step's kernels on the block's stream; the non-zero count stays on the device
        blk.rmm_dev_async(dv.data_ptr(), 1, dout.data_ptr())

    # Cold figure: the first steps after upload, clocks as the device left them (one untimed call builds what the
    # first call builds; BASELINE's protocol of 3 warm-ups then 20 steps)
    step()
    blk.nnz()
    torch.cuda.synchronize()
    for _ in range(3):
        step()
    blk.nnz()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(20):
        step()
    torch.cuda.synchronize()
    cold_ms_per_step = (time.perf_counter() - t0) / 20 * 1e3
    # Device warm-up (untimed, in front of the W warm-up steps): the first ~10 ms of load after idle run at
    # transient clocks on this device (per-kernel time 0.23 -> 0.28 -> 0.225 ms over the first 60 launches in
    # a rocprofv3 kernel trace), which a 20-step timed region would measure instead of the kernel.
    t_w = time.perf_counter()
    n_dev_warm = 0
    while time.perf_counter() - t_w < args.device_warmup_ms * 1e-3:
        for _ in range(20):
            step()
        blk.nnz()
        n_dev_warm += 20
    for _ in range(args.warmup):
        step()
    blk.nnz()
    torch.cuda.synchronize()
    # whole-job throughput: wall clock over exactly K steps, device idle on both sides; the same K steps are
    # bracketed by one pair of HIP events on the stream the kernels are launched on (the kernel time of a step is
    # that bracket / K: it cannot exceed the wall time, and it carries no per-launch event overhead)
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    with torch.cuda.stream(stream):
        ev0.record(stream)
    for _ in range(args.steps):
        step()
    with torch.cuda.stream(stream):
        ev1.record(stream)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    nnz = blk.nnz()
    ms_per_step = elapsed / args.steps * 1e3
    train_ms = ev0.elapsed_time(ev1) / args.steps

    # dominant kernel: name and algorithmic bytes from the library's own record of one more step; per-launch HIP
    # events (with their bracket overhead) are reported as kernel_ms_events
    blk.profile(True)
    kms, kbytes, kname = [], 0.0, ""
    for _ in range(min(args.steps, 20)):
        step()
        ks = blk.stats()["kernels"]
        dom = max(ks, key=lambda k: k["ms"])
        kms.append(dom["ms"])
        kbytes, kname = dom["algo_bytes"], dom["name"]
    blk.profile(False)
    n_kernels_per_step = len(ks)
    # (a step of this workload is one launch of one kernel: the train's time per step is that kernel's duration plus
    # the gap between two launches)
    k_ms = train_ms if n_kernels_per_step == 1 else statistics.mean(kms)
    achieved = kbytes / (k_ms * 1e-3) / 1e9
    traffic, traffic_note = profiled_traffic() if args.scale == 1 else (None, "scaled-down run")

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
                   "block_bytes": int(blk.device_bytes()), "derived_bytes": int(blk.derived_bytes()),
                   "kernels_per_step": sorted({k["name"] for k in ks}),
                   "device_warmup_steps": n_dev_warm, "cold_ms_per_step": cold_ms_per_step},
        "roofline": {"bound": "hbm", "kernel": kname, "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "kernel_ms": k_ms, "kernel_ms_events": statistics.mean(kms), "kernel_ms_min": min(kms),
                     "algo_bytes_per_launch": kbytes, "traffic": traffic, "traffic_source": traffic_note},
    }

    if args.calibrate_copy:
        src = torch.empty(1 << 27, dtype=torch.float64, device="cuda").fill_(1.0)  # 1 GiB
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

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
        del G, ref, got

    if not args.no_extra:
        extra = {}
        try:
            other_rows(args.scale, cfg, blk, extra, cpu=not args.no_cpu)
        except Exception as e:  # the headline stands on its own: report what was measured and why the rest is missing
            extra["error"] = repr(e)
        result["extra"] = extra
    else:
        blk.close()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
