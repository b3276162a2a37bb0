"""TEST INFRASTRUCTURE ONLY: ctypes wrapper of the CPU oracle (oracle/cla_oracle.c)
plus brute-force numpy truths used to pin the oracle itself.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import this.
"""
import ctypes as C
import math
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libcla_oracle.so")

TYPE_ID = {"ddc": 0, "sdc": 1, "rle": 2, "unc": 3, "const": 4, "empty": 5}


class OraGroup(C.Structure):
    _fields_ = [
        ("type", C.c_int32), ("nColG", C.c_int32), ("nVals", C.c_int32), ("codeWidth", C.c_int32),
        ("cols", C.c_void_p), ("dict", C.c_void_p), ("codes", C.c_void_p), ("def_", C.c_void_p),
        ("deltas", C.c_void_p), ("deltaWidth", C.c_int32), ("first", C.c_int32), ("last", C.c_int32),
        ("pad0", C.c_int32), ("nDeltas", C.c_int64), ("nOffsets", C.c_int64),
        ("ptr", C.c_void_p), ("rle", C.c_void_p), ("nData", C.c_int64), ("dense", C.c_void_p),
    ]


def build(force=False):
    if force or not os.path.exists(LIB_PATH) or \
            os.path.getmtime(LIB_PATH) < os.path.getmtime(os.path.join(HERE, "cla_oracle.c")):
        subprocess.run(["make", "-C", HERE, "-B", "libcla_oracle.so"], check=True, capture_output=True)
    return LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = C.CDLL(LIB_PATH)
        vp, i64, i32 = C.c_void_p, C.c_int64, C.c_int
        L.ora_offset_encoded_size.restype = i64
        L.ora_offset_encoded_size.argtypes = [vp, i64, i32]
        L.ora_offset_encode.restype = i64
        L.ora_offset_encode.argtypes = [vp, i64, i32, vp, i64]
        L.ora_offset_decode.restype = i64
        L.ora_offset_decode.argtypes = [vp, i32, i64, C.c_int32, vp, i64]
        L.ora_offset_choose_width.restype = i32
        L.ora_offset_choose_width.argtypes = [vp, i64]
        L.ora_rle_encode.restype = i64
        L.ora_rle_encode.argtypes = [vp, i64, vp, i64]
        L.ora_rle_decode.restype = i64
        L.ora_rle_decode.argtypes = [vp, i64, vp, i64]
        L.ora_map_width.restype = i32
        L.ora_map_width.argtypes = [i64]
        L.ora_preagg_values_from_dense.restype = None
        L.ora_preagg_values_from_dense.argtypes = [vp, i32, vp, i32, vp, i32, vp]
        L.ora_counts.restype = i32
        L.ora_counts.argtypes = [vp, i64, vp]
        L.ora_cooc.restype = i32
        L.ora_cooc.argtypes = [vp, vp, i64, vp]
        L.ora_decompress.restype = i32
        L.ora_decompress.argtypes = [vp, i32, i64, i32, vp]
        L.ora_preaggregate_dense.restype = i32
        L.ora_preaggregate_dense.argtypes = [vp, i64, vp, i32, vp]
        L.ora_rmm.restype = i64
        L.ora_rmm.argtypes = [vp, i32, i64, i32, vp, i32, vp, i32]
        L.ora_lmm.restype = i64
        L.ora_lmm.argtypes = [vp, i32, i64, i32, vp, i32, vp, i32]
        L.ora_tsmm.restype = i64
        L.ora_tsmm.argtypes = [vp, i32, i64, i32, vp, i32]
        L.ora_lmm_compressed.restype = i64
        L.ora_lmm_compressed.argtypes = [vp, i32, i32, vp, i32, i32, i64, vp]
        L.ora_mmchain.restype = i64
        L.ora_mmchain.argtypes = [vp, i32, i64, i32, vp, vp, i32, vp, i32]
        L.ora_last_error.restype = C.c_char_p
        _lib = L
    return _lib


class OracleError(RuntimeError):
    pass


def _chk(rc):
    if rc < 0:
        raise OracleError((lib().ora_last_error() or b"").decode())
    return rc


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _codes(a):
    a = np.ascontiguousarray(a)
    if a.dtype in (np.uint8, np.int8):
        return a.view(np.uint8), 1
    if a.dtype == np.uint16:
        return a, 2
    return np.ascontiguousarray(a, np.int32), 4


class Groups:
    """ctypes array of ora_group built from GroupSpec-like objects; keeps the
    numpy arrays alive."""

    def __init__(self, specs, n_rows, n_cols):
        self.n_rows, self.n_cols, self.n = int(n_rows), int(n_cols), len(specs)
        self.keep = []
        self.arr = (OraGroup * max(self.n, 1))()
        for i, s in enumerate(specs):
            g = self.arr[i]
            g.type = TYPE_ID[s.type]
            cols = np.ascontiguousarray(s.cols, np.int32)
            self.keep.append(cols)
            g.cols = _p(cols)
            g.nColG = cols.size
            if s.dict is not None:
                d = np.ascontiguousarray(s.dict, np.float64).reshape(-1, cols.size)
                self.keep.append(d)
                g.dict = _p(d)
                g.nVals = d.shape[0]
            if s.codes is not None:
                c, w = _codes(s.codes)
                self.keep.append(c)
                g.codes, g.codeWidth = _p(c), w
            elif s.type == "sdc":
                c = np.zeros(max(int(s.n_offsets), 1), np.uint8)
                self.keep.append(c)
                g.codes, g.codeWidth = _p(c), 1
            if s.type == "sdc":
                if s.default is not None:
                    de = np.ascontiguousarray(s.default, np.float64)
                    self.keep.append(de)
                    g.def_ = _p(de)
                dl = np.ascontiguousarray(s.deltas if s.deltas is not None else np.zeros(0, np.uint8))
                self.keep.append(dl)
                g.deltas = _p(dl)
                g.deltaWidth = 2 if dl.dtype == np.uint16 else 1
                g.nDeltas = dl.size
                g.first, g.last, g.nOffsets = int(s.first), int(s.last), int(s.n_offsets)
            if s.type == "rle":
                ptr = np.ascontiguousarray(s.ptr, np.int32)
                rl = np.ascontiguousarray(s.rle, np.uint16)
                self.keep += [ptr, rl]
                g.ptr, g.rle, g.nData = _p(ptr), _p(rl), rl.size
            if s.type == "unc":
                de = np.ascontiguousarray(s.dense, np.float64)
                self.keep.append(de)
                g.dense = _p(de)

    def group_ptr(self, i):
        return C.cast(C.byref(self.arr[i]), C.c_void_p)

    @property
    def ptr(self):
        return C.cast(self.arr, C.c_void_p)


# ---------------------------------------------------------------------------
# oracle entry points
# ---------------------------------------------------------------------------
def offset_encode(rows, width):
    rows = np.ascontiguousarray(rows, np.int32)
    sz = _chk(lib().ora_offset_encoded_size(_p(rows), rows.size, width)) if rows.size else 0
    out = np.zeros(max(sz, 1), np.uint8 if width == 1 else np.uint16)
    n = _chk(lib().ora_offset_encode(_p(rows), rows.size, width, _p(out), out.size)) if rows.size else 0
    return out[:n]


def offset_decode(deltas, first, cap):
    deltas = np.ascontiguousarray(deltas)
    width = 2 if deltas.dtype == np.uint16 else 1
    rows = np.zeros(max(cap, 1), np.int32)
    n = _chk(lib().ora_offset_decode(_p(deltas), width, deltas.size, int(first), _p(rows), rows.size))
    return rows[:n]


def offset_choose_width(rows):
    rows = np.ascontiguousarray(rows, np.int32)
    return lib().ora_offset_choose_width(_p(rows), rows.size)


def rle_encode(rows):
    rows = np.ascontiguousarray(rows, np.int32)
    out = np.zeros(2 * rows.size + 2 * (int(rows[-1]) // 65535 + 2 if rows.size else 1) + 2, np.uint16)
    n = _chk(lib().ora_rle_encode(_p(rows), rows.size, _p(out), out.size))
    return out[:n]


def rle_decode(data, cap):
    data = np.ascontiguousarray(data, np.uint16)
    rows = np.zeros(max(cap, 1), np.int32)
    n = _chk(lib().ora_rle_decode(_p(data), data.size, _p(rows), rows.size))
    return rows[:n]


def preagg_values_from_dense(dict_, cols, B):
    d = np.ascontiguousarray(dict_, np.float64)
    cols = np.ascontiguousarray(cols, np.int32)
    B = np.ascontiguousarray(B, np.float64)
    out = np.zeros((d.shape[0], B.shape[1]))
    lib().ora_preagg_values_from_dense(_p(d), d.shape[0], _p(cols), cols.size, _p(B), B.shape[1], _p(out))
    return out


def counts(groups, i):
    out = np.zeros(groups.arr[i].nVals, np.int32)
    _chk(lib().ora_counts(groups.group_ptr(i), groups.n_rows, _p(out)))
    return out


def cooc(groups, i, j):
    out = np.zeros((groups.arr[i].nVals, groups.arr[j].nVals), np.int64)
    _chk(lib().ora_cooc(groups.group_ptr(i), groups.group_ptr(j), groups.n_rows, _p(out)))
    return out


def decompress(groups):
    out = np.zeros((groups.n_rows, groups.n_cols))
    _chk(lib().ora_decompress(groups.ptr, groups.n, groups.n_rows, groups.n_cols, _p(out)))
    return out


def preaggregate_dense(groups, i, Y):
    Y = np.ascontiguousarray(Y, np.float64).reshape(-1, groups.n_rows)
    out = np.zeros((Y.shape[0], groups.arr[i].nVals))
    _chk(lib().ora_preaggregate_dense(groups.group_ptr(i), groups.n_rows, _p(Y), Y.shape[0], _p(out)))
    return out


def rmm(groups, B, k=1):
    B = np.ascontiguousarray(B, np.float64).reshape(groups.n_cols, -1)
    out = np.zeros((groups.n_rows, B.shape[1]))
    nnz = _chk(lib().ora_rmm(groups.ptr, groups.n, groups.n_rows, groups.n_cols, _p(B), B.shape[1], _p(out), k))
    return out, nnz


def lmm(groups, Y, k=1):
    Y = np.ascontiguousarray(Y, np.float64).reshape(-1, groups.n_rows)
    out = np.zeros((Y.shape[0], groups.n_cols))
    nnz = _chk(lib().ora_lmm(groups.ptr, groups.n, groups.n_rows, groups.n_cols, _p(Y), Y.shape[0], _p(out), k))
    return out, nnz


def tsmm(groups, k=1):
    out = np.zeros((groups.n_cols, groups.n_cols))
    nnz = _chk(lib().ora_tsmm(groups.ptr, groups.n, groups.n_rows, groups.n_cols, _p(out), k))
    return out, nnz


def lmm_compressed(right, left):
    """t(left) %*% right for two compressed blocks (CLALibLeftMultBy.java:100-112, 249-284)."""
    if left.n_rows != right.n_rows:
        raise OracleError("row counts differ")
    out = np.zeros((left.n_cols, right.n_cols))
    nnz = _chk(lib().ora_lmm_compressed(right.ptr, right.n, right.n_cols, left.ptr, left.n, left.n_cols,
                                        right.n_rows, _p(out)))
    return out, nnz


def mmchain(groups, v, w=None, ctype=0, k=1):
    v = np.ascontiguousarray(v, np.float64).reshape(-1)
    w = None if w is None else np.ascontiguousarray(w, np.float64).reshape(-1)
    out = np.zeros(groups.n_cols)
    nnz = _chk(lib().ora_mmchain(groups.ptr, groups.n, groups.n_rows, groups.n_cols, _p(v), _p(w), ctype, _p(out), k))
    return out, nnz


# ---------------------------------------------------------------------------
# brute force truths (independent of the C restatement)
# ---------------------------------------------------------------------------
def py_offset_decode(deltas, first):
    """Plain-Python restatement of OffsetByte.next (OffsetByte.java:200-212)."""
    deltas = np.asarray(deltas)
    max_v = 65535 if deltas.dtype == np.uint16 else 255
    rows, row = [int(first)], int(first)
    for v in deltas.tolist():
        if v == 0:
            row += max_v
        else:
            row += v
            rows.append(row)
    return np.array(rows, np.int64)


def py_rle_rows(ptr, data, k):
    rows, re = [], 0
    for p in range(int(ptr[k]), int(ptr[k + 1]), 2):
        rs = re + int(data[p])
        re = rs + int(data[p + 1])
        rows.extend(range(rs, re))
    return np.array(rows, np.int64)


def np_decompress(specs, n_rows, n_cols):
    """Closed-form decompression of the group list into a dense matrix."""
    D = np.zeros((n_rows, n_cols))
    for s in specs:
        cols = np.asarray(s.cols)
        if s.type == "ddc":
            D[:, cols] += np.asarray(s.dict).reshape(-1, cols.size)[np.asarray(s.codes).astype(np.int64)]
        elif s.type == "sdc":
            d = np.asarray(s.dict).reshape(-1, cols.size)
            blk = np.zeros((n_rows, cols.size)) if s.default is None else np.tile(np.asarray(s.default, float), (n_rows, 1))
            if s.n_offsets > 0:
                rows = py_offset_decode(s.deltas if s.deltas is not None else np.zeros(0, np.uint8), s.first)
                codes = np.zeros(rows.size, np.int64) if s.codes is None else np.asarray(s.codes).astype(np.int64)
                blk[rows] = d[codes]
            D[:, cols] += blk
        elif s.type == "rle":
            d = np.asarray(s.dict).reshape(-1, cols.size)
            for k in range(d.shape[0]):
                rows = py_rle_rows(s.ptr, s.rle, k)
                if rows.size:
                    D[np.ix_(rows, cols)] += d[k]
        elif s.type == "unc":
            D[:, cols] += np.asarray(s.dense).reshape(n_rows, cols.size)
        elif s.type == "const":
            D[:, cols] += np.asarray(s.dict).reshape(1, -1)
    return D


def fsum_matmul(A, B):
    """Exactly rounded A @ B via math.fsum over exact products split with fma-free
    Dekker arithmetic is overkill here; products are formed in numpy.longdouble
    (64-bit mantissa) and summed with fsum of their double-double parts."""
    A = np.asarray(A, np.float64)
    B = np.asarray(B, np.float64)
    out = np.zeros((A.shape[0], B.shape[1]))
    for i in range(A.shape[0]):
        for j in range(B.shape[1]):
            prod = A[i].astype(np.longdouble) * B[:, j].astype(np.longdouble)
            hi = prod.astype(np.float64)
            lo = (prod - hi.astype(np.longdouble)).astype(np.float64)
            out[i, j] = math.fsum(hi.tolist() + lo.tolist())
    return out


def longdouble_matmul(A, B):
    """A @ B accumulated in numpy.longdouble (x87 80-bit on this platform)."""
    return (np.asarray(A, np.longdouble) @ np.asarray(B, np.longdouble)).astype(np.float64)


def abs_matmul(A, B):
    """|A| @ |B|: the magnitude each output cell's rounding error scales with."""
    return np.abs(np.asarray(A, np.float64)) @ np.abs(np.asarray(B, np.float64))
