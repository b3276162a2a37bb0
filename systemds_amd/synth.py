"""Synthetic compressed matrices for the five benchmark configurations.

Column groups are constructed directly (as the reference's own library tests do,
src/test/.../compress/lib/CLALibLMMTest.java:150-182) instead of running the
compression planner. RNG is numpy Generator(PCG64(1000 + config)).

A GroupSpec is a neutral, array-level description of one column group: exactly
the primitive arrays a Java AColGroup holds (byte[]/char[]/int[] codes, double[]
dictionary, AOffset delta bytes, RLE char pairs).
"""
from concurrent.futures import ThreadPoolExecutor
from dataclasses import dataclass
from typing import Optional

import numpy as np


@dataclass
class GroupSpec:
    type: str                              # ddc | sdc | rle | unc | const | empty
    cols: np.ndarray                       # int32 global column ids
    dict: Optional[np.ndarray] = None      # float64 [nVals, nColG]
    codes: Optional[np.ndarray] = None     # uint8 / uint16 / int32
    default: Optional[np.ndarray] = None   # SDC default tuple (None => SDCZeros)
    deltas: Optional[np.ndarray] = None    # uint8 / uint16 AOffset entries
    first: int = 0
    last: int = -1
    n_offsets: int = 0
    ptr: Optional[np.ndarray] = None       # RLE int32 [nVals+1]
    rle: Optional[np.ndarray] = None       # RLE uint16 (gap, len) pairs
    dense: Optional[np.ndarray] = None     # float64 [nRows, nColG]

    @property
    def n_vals(self):
        return 0 if self.dict is None else self.dict.shape[0]


def map_dtype(n_unique):
    """Code width by number of distinct tuples (MapToFactory.java:102-117 collapsed
    to the widths the device path stores: byte, char, int)."""
    if n_unique <= 256:
        return np.uint8
    if n_unique <= 65536:
        return np.uint16
    return np.int32


def encode_offsets(rows, width=None):
    """Sorted unique row list -> (deltas, first, last, n). Vectorised form of
    OffsetFactory.createByte/createChar (OffsetFactory.java:246-335)."""
    rows = np.asarray(rows, dtype=np.int64)
    n = rows.size
    if n == 0:
        return np.zeros(0, np.uint8), 0, -1, 0
    if width is None:
        width = choose_offset_width(rows)
    max_v = 255 if width == 1 else 65535
    dt = np.uint8 if width == 1 else np.uint16
    gaps = np.diff(rows)
    if gaps.size and gaps.min() <= 0:
        raise ValueError("offset rows must be strictly increasing")
    div, mod = gaps // max_v, gaps % max_v
    nz = np.where(mod == 0, div - 1, div)
    val = np.where(mod == 0, max_v, mod)
    end = np.cumsum(nz + 1) - 1
    out = np.zeros(int(end[-1]) + 1 if gaps.size else 0, dt)
    if gaps.size:
        out[end] = val.astype(dt)
    return out, int(rows[0]), int(rows[-1]), int(n)


def choose_offset_width(rows):
    """OffsetFactory.createOffset size comparison (OffsetFactory.java:105-140)."""
    n = len(rows)
    if n < 3:
        return 1
    end_len = n - 1
    rng_ = int(rows[-1]) - int(rows[0])
    corr_b = max(rng_ - end_len * 256, 0) // 256
    corr_c = max(rng_ - end_len * 65535, 0) // 65535

    def byte_cost(ln):
        return 28 + (4 if ln <= 4 else ln + ((8 - (ln - 4) % 8) % 8))

    def char_cost(ln):
        return 28 + (4 if ln <= 2 else ln * 2 + ((8 - (ln * 2 - 4) % 8) % 8))
    byte_size = 16 + 4 + 4 + 4 + 8 + byte_cost(end_len + corr_b)
    char_size = 16 + 4 + 4 + 8 + char_cost(end_len + corr_c)
    return 1 if byte_size < char_size else 2


def encode_rle(codes, n_vals):
    """Per-row code sequence (-1 = zero row) -> (ptr, data) of a ColGroupRLE:
    per value the (gap from previous run end, run length) char pairs of
    genRLEBitmap (ColGroupRLE.java:1073-1157), with (65535, 0) filler runs for
    long gaps and runs cut at length 65535."""
    codes = np.asarray(codes, dtype=np.int64)
    n = codes.size
    CM = 65535
    if n == 0:
        return np.zeros(n_vals + 1, np.int32), np.zeros(0, np.uint16)
    chg = np.flatnonzero(np.diff(codes) != 0) + 1
    starts = np.concatenate(([0], chg))
    ends = np.concatenate((chg, [n]))
    rcodes = codes[starts]
    keep = rcodes >= 0
    starts, ends, rcodes = starts[keep], ends[keep], rcodes[keep]
    # cut runs longer than CM
    lens = ends - starts
    pieces = (lens + CM - 1) // CM
    if pieces.size and pieces.max() > 1:
        idx = np.repeat(np.arange(starts.size), pieces)
        k = np.arange(idx.size) - np.repeat(np.cumsum(pieces) - pieces, pieces)
        s2 = starts[idx] + k * CM
        e2 = np.minimum(s2 + CM, ends[idx])
        starts, ends, rcodes = s2, e2, rcodes[idx]
    order = np.lexsort((starts, rcodes))
    starts, ends, rcodes = starts[order], ends[order], rcodes[order]
    prev_end = np.concatenate(([0], ends[:-1]))
    first_of_val = np.concatenate(([True], rcodes[1:] != rcodes[:-1]))
    prev_end[first_of_val] = 0
    gaps = starts - prev_end
    nfill = np.where(gaps > CM, (gaps - 1) // CM, 0)
    rem = gaps - nfill * CM
    n_pairs = nfill + 1
    total = int(n_pairs.sum())
    data = np.zeros((total, 2), np.uint16)
    pos_last = np.cumsum(n_pairs) - 1
    data[:, 0] = CM
    data[:, 1] = 0
    data[pos_last, 0] = rem.astype(np.uint16)
    data[pos_last, 1] = (ends - starts).astype(np.uint16)
    pairs_per_val = np.bincount(rcodes, weights=n_pairs, minlength=n_vals).astype(np.int64)
    ptr = np.zeros(n_vals + 1, np.int32)
    ptr[1:] = np.cumsum(pairs_per_val) * 2
    return ptr, data.reshape(-1)


def _zipf_codes(rng, n_rows, n_vals, s, dtype):
    p = 1.0 / np.arange(1, n_vals + 1) ** s
    p /= p.sum()
    perm = rng.permutation(n_vals)
    cdf = np.cumsum(p)
    cdf[-1] = 1.0
    u = rng.random(n_rows)
    ranks = np.searchsorted(cdf, u, side="right")
    np.minimum(ranks, n_vals - 1, out=ranks)
    return perm[ranks].astype(dtype)


def sdc_group(rng, n_rows, cols, n_vals, density, default):
    """One SDC group over `cols` with a Bernoulli(density) row mask."""
    cols = np.asarray(cols, np.int32)
    mask = rng.random(n_rows) < density
    rows = np.flatnonzero(mask)
    d = rng.standard_normal((n_vals, cols.size))
    codes = rng.integers(0, n_vals, size=rows.size).astype(map_dtype(n_vals))
    deltas, first, last, n = encode_offsets(rows)
    de = None if default is None else np.full(cols.size, float(default))
    return GroupSpec("sdc", cols, d, codes, de, deltas, first, last, n)


def config1(scale=1):
    """C1: 100,000 x 20, 16 values per column, uniform codes, 20 single-column DDC groups."""
    rng = np.random.default_rng(1001)
    n_rows, n_cols = max(100_000 // scale, 1), 20
    groups = []
    for c in range(n_cols):
        d = rng.standard_normal((16, 1))
        codes = rng.integers(0, 16, size=n_rows).astype(np.uint8)
        groups.append(GroupSpec("ddc", np.array([c], np.int32), d, codes))
    v = rng.standard_normal((n_cols, 1))
    return dict(name="C1", n_rows=n_rows, n_cols=n_cols, groups=groups, v=v)


def _pmap(fn, n, workers=8):
    """Columns are generated from independent per-column RNG streams, so the
    result does not depend on the number of worker threads."""
    if n <= 1:
        return [fn(i) for i in range(n)]
    with ThreadPoolExecutor(max_workers=workers) as ex:
        return list(ex.map(fn, range(n)))


def config2(scale=1, n_cols=100):
    """C2: 10M x 100, 256 values per column, Zipf(1.1) codes, single-column DDC u8."""
    rng = np.random.default_rng(1002)
    n_rows = max(10_000_000 // scale, 1)

    def col(c):
        r = np.random.default_rng((1002, c))
        d = r.standard_normal((256, 1))
        codes = _zipf_codes(r, n_rows, 256, 1.1, np.uint8)
        return GroupSpec("ddc", np.array([c], np.int32), d, codes)
    groups = _pmap(col, n_cols)
    B = rng.standard_normal((n_cols, 64))
    v = rng.standard_normal((n_cols, 1))
    return dict(name="C2", n_rows=n_rows, n_cols=n_cols, groups=groups, B=B, v=v)


def config3(scale=1, n_pairs=25):
    """C3: 10M x 50 as 25 co-coded pairs, 4096 tuples ~U(-1,1), Zipf(1.0), u16 codes."""
    n_rows = max(10_000_000 // scale, 1)

    def grp(g):
        r = np.random.default_rng((1003, g))
        d = r.uniform(-1, 1, size=(4096, 2))
        codes = _zipf_codes(r, n_rows, 4096, 1.0, np.uint16)
        return GroupSpec("ddc", np.array([2 * g, 2 * g + 1], np.int32), d, codes)
    groups = _pmap(grp, n_pairs)
    return dict(name="C3", n_rows=n_rows, n_cols=2 * n_pairs, groups=groups)


def config4(scale=1, n_cols=200):
    """C4: 10M x 200 SDCZeros, 5% non-default rows, 64 values, default 0.0."""
    rng = np.random.default_rng(1004)
    n_rows = max(10_000_000 // scale, 1)
    groups = _pmap(lambda c: sdc_group(np.random.default_rng((1004, c)), n_rows, [c], 64, 0.05, None), n_cols)
    v = rng.standard_normal((1, n_rows))
    u = rng.standard_normal((n_cols, 1))
    return dict(name="C4", n_rows=n_rows, n_cols=n_cols, groups=groups, v=v, u=u)


def config5(scale=1):
    """C5: 50M x 20 = 8 RLE (mean run 1000, 32 values) + 8 DDC (1024 values, u16)
    + 2 SDC (10% non-default, default 1.0, 16 values) + 2 dense columns."""
    rng = np.random.default_rng(1005)
    n_rows = max(50_000_000 // scale, 1)
    groups = []
    for c in range(8):
        n_runs = int(n_rows / 1000 * 1.3) + 16
        lens = rng.geometric(1.0 / 1000.0, size=n_runs)
        ends = np.cumsum(lens)
        n_used = int(np.searchsorted(ends, n_rows, side="left")) + 1
        lens = lens[:n_used]
        run_codes = rng.integers(0, 32, size=n_used)
        # adjacent equal codes merge into one run, which only lengthens it
        codes = np.repeat(run_codes, lens)[:n_rows]
        d = rng.standard_normal((32, 1))
        ptr, data = encode_rle(codes, 32)
        groups.append(GroupSpec("rle", np.array([c], np.int32), d, ptr=ptr, rle=data))
    for c in range(8, 16):
        d = rng.standard_normal((1024, 1))
        codes = rng.integers(0, 1024, size=n_rows).astype(np.uint16)
        groups.append(GroupSpec("ddc", np.array([c], np.int32), d, codes))
    for c in range(16, 18):
        groups.append(sdc_group(rng, n_rows, [c], 16, 0.10, 1.0))
    dense = rng.standard_normal((n_rows, 2))
    groups.append(GroupSpec("unc", np.array([18, 19], np.int32), dense=dense))
    B = rng.standard_normal((20, 10))
    return dict(name="C5", n_rows=n_rows, n_cols=20, groups=groups, B=B)


CONFIGS = {1: config1, 2: config2, 3: config3, 4: config4, 5: config5}
