"""The C++ host layer above the C ABI: encodings and factory decisions on the CPU.

The factories must take the decisions of the reference's (MapToFactory.java:102-117,
OffsetFactory.java:105-139, 238-282, ColGroupDDC.java:106-113, ColGroupSDC.java:101-117,
ColGroupConst.java:83-102); the encoders are checked against the independent numpy
encoders of systemds_amd.synth and against the C oracle's.
"""
import numpy as np
import pytest

from conftest import host_groups, mixed_block


def test_map_to_factory_types(H):
    T = H.MAP_TYPE
    cases = [((10, 1), T.ZERO, 1), ((10, 2), T.UBYTE, 1), ((33, 2), T.BIT, 1), ((100, 128), T.UBYTE, 1),
             ((100, 129), T.BYTE, 1), ((100, 256), T.BYTE, 1), ((100, 257), T.CHAR, 2), ((100, 65536), T.CHAR, 2),
             ((100, 65537), T.CHAR_BYTE, 4), ((100, 16777216), T.CHAR_BYTE, 4), ((100, 16777217), T.INT, 4)]
    for (size, unique), typ, width in cases:
        assert H.MapToFactory.getType(size, unique) == typ, (size, unique)
        m = H.MapToFactory.create(size, unique)
        assert (m.getType(), m.codeWidth(), m.size(), m.getUnique()) == (typ, width, size, unique)


def test_map_set_get_counts_and_bounds(H):
    rng = np.random.default_rng(0)
    for unique in (3, 200, 300, 70000):
        v = rng.integers(0, unique, 5000).astype(np.int32)
        m = H.MapToFactory.create(unique, v)
        assert [m.getIndex(i) for i in (0, 17, 4999)] == [int(v[0]), int(v[17]), int(v[4999])]
        assert np.array_equal(m.getCounts(), np.bincount(v, minlength=unique))
        with pytest.raises(H.DMLCompressionException):
            m.set(0, unique)


@pytest.mark.parametrize("seed", range(6))
def test_offset_factory_matches_independent_encoders(H, ora, seed):
    from systemds_amd import synth
    rng = np.random.default_rng(seed)
    n_rows = [50, 3000, 200000, 2000000, 700, 400000][seed]
    density = [0.5, 0.01, 0.001, 0.00001, 0.3, 0.05][seed]
    rows = np.flatnonzero(rng.random(n_rows) < density).astype(np.int32)
    if rows.size < 3:
        rows = np.array([1, n_rows // 2, n_rows - 1], np.int32)
    off = H.OffsetFactory.createOffset(rows)
    width = synth.choose_offset_width(rows)
    assert off.getType() == (H.OFF_TYPE.BYTE if width == 1 else H.OFF_TYPE.CHAR)
    assert width == ora.offset_choose_width(rows)
    deltas, first, last, n = synth.encode_offsets(rows, width)
    assert (off.getOffsetToFirst(), off.getOffsetToLast(), off.getSize()) == (first, last, n)
    assert np.array_equal(off.rawDeltas(), deltas)
    assert np.array_equal(off.rawDeltas(), ora.offset_encode(rows, width))
    assert np.array_equal(off.toArray(), rows)
    for t, w in ((H.OFF_TYPE.BYTE, 1), (H.OFF_TYPE.CHAR, 2)):
        o2 = H.OffsetFactory.createOffset(rows, t)
        assert np.array_equal(o2.rawDeltas(), synth.encode_offsets(rows, w)[0])
        assert np.array_equal(o2.toArray(), rows)


def test_offset_gap_multiples_of_max_and_iterator(H):
    # gaps of exactly 255 / 510 end on a full entry (OffsetFactory.java:266-275)
    off = H.OffsetFactory.createOffset(np.array([4, 259, 769, 770, 1026], np.int32), H.OFF_TYPE.BYTE)
    assert off.rawDeltas() == [255, 0, 255, 1, 0, 1]
    it = off.getIterator()
    seen = [(it.value(), it.getDataIndex())]
    while it.value() < off.getOffsetToLast():
        it.next()
        seen.append((it.value(), it.getDataIndex()))
    assert seen == [(4, 0), (259, 1), (769, 2), (770, 3), (1026, 4)]
    it = off.getIterator()
    assert it.skipTo(700) == 769 and it.getDataIndex() == 2
    empty = H.OffsetFactory.createOffset(np.zeros(0, np.int32))
    assert empty.getSize() == 0 and empty.toArray() == []
    one = H.OffsetFactory.createOffset(np.array([9], np.int32))
    assert (one.getSize(), one.getOffsetToFirst(), one.getOffsetToLast(), one.rawDeltas()) == (1, 9, 9, [])
    with pytest.raises(H.DMLCompressionException):
        H.OffsetFactory.createOffset(np.array([5, 5, 6], np.int32))
    with pytest.raises(H.DMLCompressionException):
        H.OffsetFactory.createOffset(np.array([-1, 5, 6], np.int32))


def test_rle_bitmap_matches_independent_encoders(H, ora):
    from systemds_amd import synth
    rng = np.random.default_rng(3)
    n_rows = 300000
    run_codes = rng.integers(-1, 3, size=200)
    run_lens = rng.integers(1, 4000, size=200)
    run_lens[50] = 140000                       # a run longer than 65535 rows
    codes = np.repeat(run_codes, run_lens)[:n_rows]
    codes = np.concatenate([codes, np.full(n_rows - codes.size, -1)]) if codes.size < n_rows else codes
    ptr, data = synth.encode_rle(codes, 3)
    rows = [np.flatnonzero(codes == k).astype(np.int32).tolist() for k in range(3)]
    d2, p2 = H.ColGroupRLE.genRLEBitmap(rows)
    assert np.array_equal(p2, ptr) and np.array_equal(d2, data)
    for k in range(3):
        assert np.array_equal(np.asarray(d2[p2[k]:p2[k + 1]], np.uint16), ora.rle_encode(np.asarray(rows[k], np.int32)))


def test_group_factories_simplify_like_the_reference(H):
    CT = H.CompressionType
    cols = np.array([2, 5], np.int32)
    d = H.Dictionary.create(np.arange(1.0, 7.0))           # 3 tuples of 2
    assert H.Dictionary.create(np.zeros(4)) is None        # all-zero dictionary -> null
    m3 = H.MapToFactory.create(3, np.array([0, 1, 2, 1], np.int32))
    g = H.ColGroupDDC.create(cols, d, m3)
    assert (g.getCompType(), g.getNumValues(), g.getNumCols(), g.getColIndices()) == (CT.DDC, 3, 2, [2, 5])
    assert H.ColGroupDDC.create(cols, None, m3).getCompType() == CT.EMPTY
    one = H.MapToFactory.create(4, 1)
    assert H.ColGroupDDC.create(cols, H.Dictionary.create(np.array([1.0, 2.0])), one).getCompType() == CT.CONST
    with pytest.raises(H.DMLCompressionException):
        H.ColGroupDDC.create(cols, d, H.MapToFactory.create(4, np.array([0, 1, 2, 3], np.int32)))
    off = H.OffsetFactory.createOffset(np.array([1, 4, 6, 7], np.int32))
    assert H.ColGroupSDC.create(cols, 10, d, np.zeros(2), off, m3).getCompType() == CT.SDCZeros
    assert H.ColGroupSDC.create(cols, 10, d, np.array([0.0, 1.0]), off, m3).getCompType() == CT.SDC
    assert H.ColGroupSDC.create(cols, 10, None, np.zeros(2), off, m3).getCompType() == CT.EMPTY
    assert H.ColGroupSDC.create(cols, 10, None, np.array([3.0, 0.0]), off, m3).getCompType() == CT.SDC
    assert H.ColGroupSDCZeros.create(cols, 10, None, off, m3).getCompType() == CT.EMPTY
    with pytest.raises(H.DMLCompressionException):     # list longer than the map
        H.ColGroupSDCZeros.create(cols, 10, d, H.OffsetFactory.createOffset(np.array([1, 2, 3, 4, 5], np.int32)), m3)
    with pytest.raises(H.DMLCompressionException):     # last offset beyond the rows
        H.ColGroupSDCZeros.create(cols, 7, d, off, m3)
    assert H.ColGroupConst.create(cols, np.zeros(2)).getCompType() == CT.EMPTY
    assert H.ColGroupConst.create(cols, 2.5).getCompType() == CT.CONST
    with pytest.raises(H.DMLCompressionException):
        H.ColGroupConst.create(cols, np.array([1.0, 2.0, 3.0]))
    with pytest.raises(H.DMLCompressionException):
        H.ColGroupDDC.create(np.array([5, 2], np.int32), d, m3)      # unsorted column index
    assert H.ColGroupUncompressed.create(H.MatrixBlock(np.zeros((4, 2))), cols).getCompType() == CT.EMPTY
    assert H.ColGroupUncompressed.create(H.MatrixBlock(np.ones((4, 2))), cols).getCompType() == CT.UNCOMPRESSED
    with pytest.raises(H.DMLCompressionException):
        H.ColGroupUncompressed.create(H.MatrixBlock(np.ones((4, 3))), cols)


def test_block_checks_and_empty_results_need_no_device(H, ora):
    specs, n_cols = mixed_block(5, 200)
    groups = host_groups(H, ora, specs, 200)
    assert [g.getCompType() for g in groups].count(H.CompressionType.SDC) == 1
    cmb = H.CompressedMatrixBlock(200, n_cols)
    cmb.allocateColGroupList(groups)
    assert not cmb.isEmpty() and cmb.isCompressed() and not cmb.isOverlapping()
    with pytest.raises(H.DMLCompressionException):
        H.CompressedMatrixBlock(200, 3).allocateColGroupList(groups)      # column index out of range
    # dimension errors come before any device work
    with pytest.raises(H.DMLRuntimeException):
        H.CLALibRightMultBy.rightMultByMatrix(cmb, H.MatrixBlock(np.ones((n_cols + 1, 2))))
    with pytest.raises(H.DMLRuntimeException):
        H.CLALibLeftMultBy.leftMultByMatrix(cmb, H.MatrixBlock(np.ones((2, 199))))
    with pytest.raises(H.DMLRuntimeException):
        cmb.transposeSelfMatrixMultOperations(H.MMTSJType.RIGHT)
    with pytest.raises(H.DMLRuntimeException):
        cmb.chainMatrixMultOperations(H.MatrixBlock(np.ones((n_cols, 2))), None, H.ChainType.XtXv)
    with pytest.raises(H.DMLRuntimeException):
        cmb.chainMatrixMultOperations(H.MatrixBlock(np.ones((n_cols, 1))), None, H.ChainType.XtwXv)
    # empty operands give empty results without touching the device
    ret = H.CLALibRightMultBy.rightMultByMatrix(cmb, H.MatrixBlock(n_cols, 3))
    assert (ret.getNumRows(), ret.getNumColumns(), ret.getNonZeros()) == (200, 3, 0)
    e = H.CompressedMatrixBlock(200, 2)
    e.allocateColGroupList([H.ColGroupEmpty(np.array([0, 1], np.int32))])
    assert e.isEmpty()
    assert H.CLALibTSMM.leftMultByTransposeSelf(e).toArray().shape == (2, 2)
    assert not H.CLALibLeftMultBy.leftMultByMatrix(e, H.MatrixBlock(np.ones((3, 200)))).toArray().any()


def test_product_has_no_cpu_fallback(H, ora):
    """Without a GPU every multiply must raise; it must not compute on the host."""
    from systemds_amd import capi
    try:
        capi.init(0)
    except capi.ClaError:
        pass
    else:
        pytest.skip("a GPU is present")
    specs, n_cols = mixed_block(1, 50)
    cmb = H.CompressedMatrixBlock(50, n_cols)
    cmb.allocateColGroupList(host_groups(H, ora, specs, 50))
    with pytest.raises(H.DMLRuntimeException, match="GPU only"):
        H.CLALibRightMultBy.rightMultByMatrix(cmb, H.MatrixBlock(np.ones((n_cols, 2))))
    with pytest.raises(H.DMLRuntimeException, match="GPU only"):
        cmb.decompress()
