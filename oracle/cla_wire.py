"""Serialised CompressedMatrixBlock writer -- TEST INFRASTRUCTURE ONLY (see cla_oracle.py).

Restates the reference's `write` methods with `struct` (java.io.DataOutput is big-endian)
so that the host layer's reader can be fed bytes it did not produce itself. Each function
cites the reference method it follows. The writer can be told to pick any of the type
variants the reference's factories choose between (index, dictionary, map, offset and
matrix-block formats), so every branch of a reader is reachable.

parity unpinned: the reference holds no serialised compressed block (its IO tests write and
read at run time, T/io/IOTest.java), so these bytes are pinned by the cited code only, by
hand-assembled vectors in the tests and by agreement with the independent C++ writer.
"""
import struct

import numpy as np

# ordinals: CG/AColGroup.java:89-92, CG/indexes/IColIndex.java:33-35, CG/dictionary/DictionaryFactory.java:54-56,
# CG/mapping/MapToFactory.java:39-41, CG/offset/OffsetFactory.java:46-52, common/Types.java:440-446
COLGROUP = {k: i for i, k in enumerate(
    "UNCOMPRESSED RLE OLE DDC CONST EMPTY SDC SDCSingle SDCSingleZeros SDCZeros SDCFOR DDCFOR DDCLZW DeltaDDC LinearFunctional".split())}
COLINDEX = {k: i for i, k in enumerate("SINGLE TWO ARRAY RANGE TWORANGE COMBINED".split())}
DICT = {k: i for i, k in enumerate("FP64_DICT MATRIX_BLOCK_DICT INT8_DICT IDENTITY IDENTITY_SLICE PLACE_HOLDER DELTA_DICT".split())}
MAP = {k: i for i, k in enumerate("ZERO BIT UBYTE BYTE CHAR CHAR_BYTE INT".split())}
OFF = {k: i for i, k in enumerate("BYTE CHAR SINGLE_OFFSET TWO_OFFSET EMPTY BYTEUNZ BYTENZ".split())}
BLOCK = {k: i for i, k in enumerate("EMPTY_BLOCK ULTRA_SPARSE_BLOCK SPARSE_BLOCK DENSE_BLOCK DEDUP_BLOCK".split())}


def _i(v):
    return struct.pack(">i", int(v))


def _doubles(a):
    return np.ascontiguousarray(a, dtype=">f8").tobytes()


def col_index(cols, kind=None):
    """CG/indexes/{Single,Two,Array,Range,TwoRanges,Combined}Index.write."""
    cols = [int(c) for c in cols]
    contiguous = all(b == a + 1 for a, b in zip(cols, cols[1:]))
    if kind is None:
        kind = "SINGLE" if len(cols) == 1 else "TWO" if len(cols) == 2 else "RANGE" if contiguous else "ARRAY"
    t = bytes([COLINDEX[kind]])
    if kind == "SINGLE":
        return t + _i(cols[0])
    if kind == "TWO":
        return t + _i(cols[0]) + _i(cols[1])
    if kind == "ARRAY":
        return t + _i(len(cols)) + b"".join(_i(c) for c in cols)
    if kind == "RANGE":
        assert contiguous
        return t + _i(cols[0]) + _i(cols[-1] + 1)
    if kind == "TWORANGE":  # (start, length) twice, TwoRangesIndex.java:59-65
        cut = next(i for i in range(1, len(cols)) if cols[i] != cols[i - 1] + 1)
        a, b = cols[:cut], cols[cut:]
        assert all(y == x + 1 for x, y in zip(b, b[1:]))
        return t + _i(a[0]) + _i(len(a)) + _i(b[0]) + _i(len(b))
    if kind == "COMBINED":  # two indexes back to back, CombinedIndex.java:56-60
        h = len(cols) // 2
        return t + col_index(cols[:h]) + col_index(cols[h:])
    raise ValueError(kind)


def matrix_block(a, fmt=None):
    """R/matrix/data/MatrixBlock.java:2335-2372 and the write* helpers behind it."""
    a = np.asarray(a, np.float64)
    r, c = a.shape
    head = _i(r) + _i(c)
    nnz = int(np.count_nonzero(a))
    if fmt is None:
        fmt = "EMPTY_BLOCK" if nnz == 0 else "DENSE_BLOCK"
    t = bytes([BLOCK[fmt]])
    if fmt == "EMPTY_BLOCK":
        assert nnz == 0
        return head + t
    if fmt == "DENSE_BLOCK":
        return head + t + _doubles(a)
    nnz_info = struct.pack(">q", nnz) if r * c > 2**31 - 1 else _i(nnz)
    if fmt == "SPARSE_BLOCK":  # per row: count, (column, value) pairs
        out = [head, t, nnz_info]
        for i in range(r):
            cols = np.flatnonzero(a[i])
            out.append(_i(len(cols)))
            for j in cols:
                out.append(_i(j) + struct.pack(">d", a[i, j]))
        return b"".join(out)
    if fmt == "ULTRA_SPARSE_BLOCK":  # (row, column, value) triples; (row, value) for a single column
        out = [head, t, _i(nnz)]
        for i, j in zip(*np.nonzero(a)):
            out.append(_i(i) + (_i(j) if c > 1 else b"") + struct.pack(">d", a[i, j]))
        return b"".join(out)
    raise ValueError(fmt)


def dictionary(values, n_col, kind="FP64_DICT", block_fmt=None):
    """CG/dictionary/Dictionary.java:371-376, MatrixBlockDictionary.java:1910-1913, IdentityDictionary.java:382-385."""
    values = np.asarray(values, np.float64).reshape(-1)
    t = bytes([DICT[kind]])
    if kind == "FP64_DICT":
        return t + _i(values.size) + _doubles(values)
    if kind == "MATRIX_BLOCK_DICT":
        return t + matrix_block(values.reshape(-1, n_col), block_fmt)
    if kind == "IDENTITY":
        assert np.array_equal(values.reshape(n_col, n_col), np.eye(n_col))
        return t + _i(n_col)
    raise ValueError(kind)


def map_to_data(codes, unique, kind=None):
    """CG/mapping/MapTo{Zero,Bit,UByte,Byte,Char,CharPByte,Int}.write; the type the factory picks by default
    (MapToFactory.java:102-117)."""
    codes = np.asarray(codes, np.int64)
    n = codes.size
    if kind is None:
        kind = ("ZERO" if unique <= 1 else "BIT" if unique == 2 and n > 32 else "UBYTE" if unique <= 128 else
                "BYTE" if unique <= 256 else "CHAR" if unique <= 65536 else "CHAR_BYTE" if unique <= 16777216 else "INT")
    t = bytes([MAP[kind]])
    if kind == "ZERO":
        return t + _i(n)
    if kind == "BIT":  # bit n of word n >> 6, MapToBit.java:100-103, 173-179
        words = np.zeros((n + 63) // 64, np.uint64)
        for i in np.flatnonzero(codes):
            words[i >> 6] |= np.uint64(1) << np.uint64(i & 63)
        return t + _i(n) + _i(words.size) + words.astype(">u8").tobytes()
    head = t + _i(unique) + _i(n)
    if kind in ("UBYTE", "BYTE"):
        return head + codes.astype(np.uint8).tobytes()
    if kind == "CHAR":
        return head + codes.astype(">u2").tobytes()
    if kind == "CHAR_BYTE":  # all low chars, then all high bytes, MapToCharPByte.java:139-145
        return head + (codes & 0xffff).astype(">u2").tobytes() + (codes >> 16).astype(np.uint8).tobytes()
    if kind == "INT":
        return head + codes.astype(">i4").tobytes()
    raise ValueError(kind)


def offset(rows, kind=None):
    """CG/offset/Offset{Empty,Single,Two,Byte,ByteNZ,ByteUNZ,Char}.write. rows: sorted absolute rows."""
    rows = [int(r) for r in rows]
    n = len(rows)
    if kind is None:
        kind = "EMPTY" if n == 0 else "SINGLE_OFFSET" if n == 1 else "TWO_OFFSET" if n == 2 else "BYTE"
    t = bytes([OFF[kind]])
    if kind == "EMPTY":
        return t
    if kind == "SINGLE_OFFSET":
        return t + _i(rows[0])
    if kind == "TWO_OFFSET":
        return t + _i(rows[0]) + _i(rows[1])
    max_v = 65535 if kind == "CHAR" else 255
    deltas = []
    for a, b in zip(rows, rows[1:]):
        gap = b - a
        while gap > max_v:  # a 0 entry skips max_v rows, OffsetFactory.java:238-340
            deltas.append(0)
            gap -= max_v
        deltas.append(gap)
    head = t + _i(rows[0]) + _i(len(deltas)) + _i(rows[-1])
    if kind == "CHAR":  # no size field: the reader counts the non-zero entries, OffsetChar.java:74-81, 123-134
        return head + np.asarray(deltas, ">u2").tobytes()
    if kind == "BYTE":  # with size, OffsetByte.java:74-83
        return head + _i(n) + bytes(deltas)
    assert 0 not in deltas, "NZ variants hold no skip entries"
    if kind == "BYTEUNZ":
        assert max(deltas, default=0) < 128
    return head + bytes(deltas)  # BYTENZ / BYTEUNZ: no size field, OffsetByteNZ.java:89-98


def _rows(spec):
    """Absolute rows of an SDC spec (first row + delta entries; a 0 entry skips 255 / 65535 rows)."""
    if not spec.n_offsets:
        return []
    d = np.asarray(spec.deltas, np.int64)
    max_v = 255 if spec.deltas.dtype == np.uint8 else 65535
    pos = spec.first + np.cumsum(np.where(d == 0, max_v, d))
    return [int(spec.first)] + pos[d != 0].tolist()


def col_group(spec, n_rows, variant=None):
    """AColGroup.write (type ordinal, column index) followed by the group's own fields:
    CG/ColGroupDDC.java:794-797, ColGroupSDC.java:446-452, ColGroupSDCZeros.java:645-649,
    ColGroupSDCSingle.java:412-417, ColGroupSDCSingleZeros.java:644-647, AColGroupOffset.java:115-127 (RLE),
    ColGroupUncompressed.java:657-660, ADictBasedColGroup.java:225-228 (const), ColGroupEmpty."""
    v = variant or {}
    cols = col_index(spec.cols, v.get("index"))
    n_col = len(spec.cols)

    def head(name):
        return bytes([COLGROUP[name]]) + cols

    def dct():
        return dictionary(spec.dict, n_col, v.get("dict", "FP64_DICT"), v.get("block"))

    if spec.type == "ddc":
        return head("DDC") + dct() + map_to_data(spec.codes, spec.n_vals, v.get("map"))
    if spec.type == "sdc":
        rows = _rows(spec)
        single = v.get("single", False)
        if spec.default is None:
            if single:
                return head("SDCSingleZeros") + dct() + offset(rows, v.get("offset"))
            return head("SDCZeros") + dct() + offset(rows, v.get("offset")) + map_to_data(spec.codes, spec.n_vals, v.get("map"))
        if single:
            return head("SDCSingle") + dct() + offset(rows, v.get("offset")) + _doubles(spec.default)
        return (head("SDC") + dct() + offset(rows, v.get("offset")) + map_to_data(spec.codes, spec.n_vals, v.get("map")) +
                _doubles(spec.default))
    if spec.type == "rle":
        ptr = np.asarray(spec.ptr, np.int64)
        data = np.asarray(spec.rle, np.int64)
        return (head("RLE") + dct() + _i(ptr.size) + ptr.astype(">i4").tobytes() + _i(data.size) +
                data.astype(">u2").tobytes() + b"\x01")
    if spec.type == "unc":
        return head("UNCOMPRESSED") + matrix_block(spec.dense, v.get("block"))
    if spec.type == "const":
        return head("CONST") + dct()
    if spec.type == "empty":
        return head("EMPTY")
    raise ValueError(spec.type)


def compressed_block(n_rows, n_cols, specs, nnz=-1, overlapping=False, variants=None):
    """C/CompressedMatrixBlock.java:493-523: rlen, clen, nonZeros, overlap flag; ColGroupIO.writeGroups: count, groups."""
    variants = variants or [None] * len(specs)
    out = [_i(n_rows), _i(n_cols), struct.pack(">q", nnz), b"\x01" if overlapping else b"\x00", _i(len(specs))]
    for s, v in zip(specs, variants):
        out.append(col_group(s, n_rows, v))
    return b"".join(out)
