import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X")


@pytest.fixture(scope="session")
def ora():
    """The CPU oracle (test infrastructure), built on demand."""
    from oracle import cla_oracle
    cla_oracle.build()
    return cla_oracle


@pytest.fixture(scope="session")
def cla():
    """The product library on cuda:0. Fails loudly when the HIP library or the GPU is missing."""
    from systemds_amd import capi
    capi.init(0)
    return capi


def java_random_ints(seed):
    """java.util.Random as a generator factory: returns next_int(bound)."""
    state = [(seed ^ 0x5DEECE66D) & ((1 << 48) - 1)]

    def nxt(bits):
        state[0] = (state[0] * 0x5DEECE66D + 0xB) & ((1 << 48) - 1)
        v = state[0] >> (48 - bits)
        return v - (1 << 32) if v >= (1 << 31) else v

    def next_int(bound):
        if bound & (-bound) == bound:
            return (bound * nxt(31)) >> 31
        while True:
            bits = nxt(31)
            val = bits % bound
            if bits - val + (bound - 1) < (1 << 31):
                return val
    return next_int


def mixed_block(seed, n_rows, with_unc=True, with_const=True, overlap=False, big_dict=True):
    """A small block with every group type, used by several tests."""
    from systemds_amd import synth
    rng = np.random.default_rng(seed)
    specs = []
    c = 0

    def cols(n):
        nonlocal c
        r = np.arange(c, c + n, dtype=np.int32)
        c += n
        return r
    specs.append(synth.GroupSpec("ddc", cols(1), rng.standard_normal((7, 1)), rng.integers(0, 7, n_rows).astype(np.uint8)))
    specs.append(synth.GroupSpec("ddc", cols(2), rng.standard_normal((300, 2)),
                                 rng.integers(0, 300, n_rows).astype(np.uint16)))
    nv = 70000 if big_dict else 700
    specs.append(synth.GroupSpec("ddc", cols(1), rng.standard_normal((nv, 1)),
                                 rng.integers(0, nv, n_rows).astype(np.int32)))
    specs.append(synth.sdc_group(rng, n_rows, cols(1), 5, 0.1, None))
    specs.append(synth.sdc_group(rng, n_rows, cols(2), 6, 0.004, 1.5))
    run_codes = rng.integers(-1, 4, size=n_rows // 20 + 2)
    run_lens = rng.integers(1, 60, size=run_codes.size)
    codes = np.repeat(run_codes, run_lens)[:n_rows]
    if codes.size < n_rows:
        codes = np.concatenate([codes, np.full(n_rows - codes.size, -1)])
    ptr, data = synth.encode_rle(codes, 4)
    specs.append(synth.GroupSpec("rle", cols(1), rng.standard_normal((4, 1)), ptr=ptr, rle=data))
    if with_unc:
        specs.append(synth.GroupSpec("unc", cols(2), dense=rng.standard_normal((n_rows, 2))))
    if with_const:
        specs.append(synth.GroupSpec("const", cols(1), np.array([[2.5]])))
        specs.append(synth.GroupSpec("empty", cols(1)))
    if overlap:  # groups over columns that other groups already cover: the values add up
        specs.append(synth.GroupSpec("ddc", np.array([0, 2], np.int32), rng.standard_normal((9, 2)),
                                     rng.integers(0, 9, n_rows).astype(np.uint8)))
        specs.append(synth.sdc_group(rng, n_rows, [1, 4], 3, 0.2, 0.5))
    return specs, c


@pytest.fixture(scope="session")
def H():
    """The C++ host layer (systemds_amd/host) as a Python module."""
    from systemds_amd import host
    return host.load()


def host_groups(H, ora, specs, n_rows):
    """GroupSpec list -> column groups built with the host layer's factories."""
    out = []
    for s in specs:
        cols = np.asarray(s.cols, np.int32)
        if s.type == "ddc":
            out.append(H.ColGroupDDC.create(cols, H.Dictionary.create(s.dict),
                                            H.MapToFactory.create(s.n_vals, s.codes.astype(np.int32))))
        elif s.type == "sdc":
            rows = ora.py_offset_decode(s.deltas, s.first) if s.n_offsets else np.zeros(0, np.int64)
            width = H.OFF_TYPE.BYTE if s.deltas.dtype == np.uint8 else H.OFF_TYPE.CHAR
            off = H.OffsetFactory.createOffset(rows.astype(np.int32), width)
            mp = H.MapToFactory.create(s.n_vals, s.codes.astype(np.int32))
            d = H.Dictionary.create(s.dict)
            if s.default is None:
                out.append(H.ColGroupSDCZeros.create(cols, n_rows, d, off, mp))
            else:
                out.append(H.ColGroupSDC.create(cols, n_rows, d, s.default, off, mp))
        elif s.type == "rle":
            out.append(H.ColGroupRLE.create(cols, n_rows, H.Dictionary.create(s.dict), s.rle.tolist(), s.ptr))
        elif s.type == "unc":
            out.append(H.ColGroupUncompressed.create(H.MatrixBlock(s.dense), cols))
        elif s.type == "const":
            out.append(H.ColGroupConst.create(cols, s.dict.reshape(-1)))
        else:
            out.append(H.ColGroupEmpty(cols))
    return out
