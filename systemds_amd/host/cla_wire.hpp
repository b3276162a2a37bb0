// Serialised CompressedMatrixBlock <-> host-layer objects, byte for byte the layout of
// the reference's Writable implementation (java.io.DataOutput: big-endian, char = 2 bytes,
// boolean = 1 byte):
//   CompressedMatrixBlock.write / readFields     C/CompressedMatrixBlock.java:470-523
//   ColGroupIO.readGroups / readColGroup         CG/ColGroupIO.java:50-137
//   AColGroup.write (type ordinal + col index)   CG/AColGroup.java:207-212
//   IColIndex                                    CG/indexes/ColIndexFactory.java:38-56
//   IDictionary                                  CG/dictionary/DictionaryFactory.java:54-77
//   AMapToData                                   CG/mapping/MapToFactory.java:227-246
//   AOffset                                      CG/offset/OffsetFactory.java:178-197
//   MatrixBlock                                  R/matrix/data/MatrixBlock.java:2111-2372
// Group and dictionary types the multiply path does not cover (frame-of-reference, delta,
// LZW, OLE, linear functional, quantised / place-holder dictionaries, dedup dense blocks)
// raise NotImplementedException; a caller keeps such blocks on the CPU.
#pragma once
#include "cla_host.hpp"
#include <cstring>

namespace sysds {
namespace compress {
namespace io {

// java.io.DataInput over a byte buffer
class DataInput {
public:
	DataInput(const uint8_t* p, size_t n) : cur(p), end(p + n) {}
	size_t remaining() const { return (size_t) (end - cur); }
	uint8_t readByte() { need(1); return *cur++; }
	bool readBoolean() { return readByte() != 0; }
	uint16_t readChar() { need(2); const uint16_t v = (uint16_t) ((cur[0] << 8) | cur[1]); cur += 2; return v; }
	int32_t readInt() {
		need(4);
		const uint32_t v = ((uint32_t) cur[0] << 24) | ((uint32_t) cur[1] << 16) | ((uint32_t) cur[2] << 8) | (uint32_t) cur[3];
		cur += 4;
		return (int32_t) v;
	}
	int64_t readLong() {
		const uint64_t hi = (uint32_t) readInt(), lo = (uint32_t) readInt();
		return (int64_t) ((hi << 32) | lo);
	}
	double readDouble() {
		const int64_t bits = readLong();
		double d;
		std::memcpy(&d, &bits, 8);
		return d;
	}
	void readFully(uint8_t* dst, size_t n) { need(n); std::memcpy(dst, cur, n); cur += n; }

private:
	void need(size_t n) const {
		if((size_t) (end - cur) < n) throw DMLRuntimeException("EOFException: serialised block ends early");
	}
	const uint8_t* cur;
	const uint8_t* end;
};

// java.io.DataOutput into a byte vector
class DataOutput {
public:
	std::vector<uint8_t> bytes;
	void writeByte(int v) { bytes.push_back((uint8_t) v); }
	void writeBoolean(bool v) { bytes.push_back(v ? 1 : 0); }
	void writeChar(int v) { bytes.push_back((uint8_t) (v >> 8)); bytes.push_back((uint8_t) v); }
	void writeInt(int32_t v) { for(int s = 24; s >= 0; s -= 8) bytes.push_back((uint8_t) ((uint32_t) v >> s)); }
	void writeLong(int64_t v) { for(int s = 56; s >= 0; s -= 8) bytes.push_back((uint8_t) ((uint64_t) v >> s)); }
	void writeDouble(double d) { int64_t bits; std::memcpy(&bits, &d, 8); writeLong(bits); }
	void write(const uint8_t* p, size_t n) { bytes.insert(bytes.end(), p, p + n); }
};

// ordinals of the reference's enums as they appear on the wire
enum ColGroupType { UNCOMPRESSED, RLE, OLE, DDC, CONST, EMPTY, SDC, SDCSingle, SDCSingleZeros, SDCZeros, SDCFOR, DDCFOR, DDCLZW, DeltaDDC, LinearFunctional };
enum ColIndexType { SINGLE, TWO, ARRAY, RANGE, TWORANGE, COMBINED };
enum DictType { FP64_DICT, MATRIX_BLOCK_DICT, INT8_DICT, IDENTITY, IDENTITY_SLICE, PLACE_HOLDER, DELTA_DICT };
enum OffType { OFF_BYTE, OFF_CHAR, SINGLE_OFFSET, TWO_OFFSET, OFF_EMPTY, BYTEUNZ, BYTENZ };
enum BlockType { EMPTY_BLOCK, ULTRA_SPARSE_BLOCK, SPARSE_BLOCK, DENSE_BLOCK, DEDUP_BLOCK };

// ------------------------------------------------------------------ MatrixBlock
inline std::shared_ptr<MatrixBlock> readMatrixBlock(DataInput& in) {
	const int rlen = in.readInt(), clen = in.readInt();
	const int fmt = in.readByte();
	if(rlen < 0 || clen < 0) throw DMLRuntimeException("invalid matrix block dimensions");
	if(fmt == DENSE_BLOCK && (uint64_t) rlen * (uint64_t) clen * 8 > in.remaining()) throw DMLRuntimeException("EOFException: dense block ends early");
	auto mb = std::make_shared<MatrixBlock>(rlen, clen);
	double* a = mb->getDenseBlockValues();
	const bool longNnz = (int64_t) rlen * clen > 2147483647LL;
	switch(fmt) {
		case EMPTY_BLOCK: break;
		case DENSE_BLOCK:
			for(int64_t i = 0; i < (int64_t) rlen * clen; i++) a[i] = in.readDouble();
			break;
		case SPARSE_BLOCK: { // nnz, then per row: count and (column, value) pairs
			if(longNnz) in.readLong(); else in.readInt();
			for(int r = 0; r < rlen; r++) {
				const int nr = in.readInt();
				for(int j = 0; j < nr; j++) {
					const int c = in.readInt();
					if(c < 0 || c >= clen) throw DMLRuntimeException("invalid column in sparse block");
					a[(size_t) r * clen + c] = in.readDouble();
				}
			}
			break;
		}
		case ULTRA_SPARSE_BLOCK: { // nnz (always int), then (row, column, value) triples, or (row, value) for one column
			const int64_t nnz = in.readInt();
			for(int64_t i = 0; i < nnz; i++) {
				const int r = in.readInt();
				const int c = clen > 1 ? in.readInt() : 0;
				if(r < 0 || r >= rlen || c < 0 || c >= clen) throw DMLRuntimeException("invalid cell in ultra-sparse block");
				a[(size_t) r * clen + c] = in.readDouble();
			}
			break;
		}
		default: throw NotImplementedException("matrix block format " + std::to_string(fmt));
	}
	mb->recomputeNonZeros();
	return mb;
}

// Dense or empty on the wire (the reference reads either whatever it would have chosen itself).
inline void writeMatrixBlock(const MatrixBlock& mb, DataOutput& out) {
	out.writeInt(mb.getNumRows());
	out.writeInt(mb.getNumColumns());
	const double* a = mb.getDenseBlockValues();
	const int64_t n = (int64_t) mb.getNumRows() * mb.getNumColumns();
	bool any = false;
	for(int64_t i = 0; mb.isAllocated() && i < n && !any; i++) any = a[i] != 0.0;
	if(!any) { out.writeByte(EMPTY_BLOCK); return; }
	out.writeByte(DENSE_BLOCK);
	for(int64_t i = 0; i < n; i++) out.writeDouble(a[i]);
}

// ------------------------------------------------------------------ column indexes
inline IColIndex readColIndex(DataInput& in) {
	const int t = in.readByte();
	IColIndex r;
	switch(t) {
		case SINGLE: r.push_back(in.readInt()); break;
		case TWO: r.push_back(in.readInt()); r.push_back(in.readInt()); break;
		case ARRAY: {
			const int n = in.readInt();
			if(n < 0 || (size_t) n * 4 > in.remaining()) throw DMLRuntimeException("invalid column index length");
			for(int i = 0; i < n; i++) r.push_back(in.readInt());
			break;
		}
		case RANGE: { // [l, u)
			const int l = in.readInt(), u = in.readInt();
			if(u < l || (int64_t) u - l > (1 << 26)) throw DMLRuntimeException("invalid column range");
			for(int i = l; i < u; i++) r.push_back(i);
			break;
		}
		case TWORANGE: { // two ranges as (start, length)
			for(int k = 0; k < 2; k++) {
				const int l = in.readInt(), n = in.readInt();
				if(n < 0 || n > (1 << 26)) throw DMLRuntimeException("invalid column range");
				for(int i = 0; i < n; i++) r.push_back(l + i);
			}
			break;
		}
		case COMBINED: {
			r = readColIndex(in);
			const IColIndex b = readColIndex(in);
			r.insert(r.end(), b.begin(), b.end());
			break;
		}
		default: throw DMLCompressionException("Failed reading column index of type: " + std::to_string(t));
	}
	return r;
}

// The type ColIndexFactory.create would pick: single, two, a range when contiguous, else an array.
inline void writeColIndex(const IColIndex& c, DataOutput& out) {
	if(c.size() == 1) { out.writeByte(SINGLE); out.writeInt(c[0]); return; }
	if(c.size() == 2) { out.writeByte(TWO); out.writeInt(c[0]); out.writeInt(c[1]); return; }
	bool contiguous = true;
	for(size_t i = 1; i < c.size(); i++) contiguous &= c[i] == c[i - 1] + 1;
	if(contiguous) { out.writeByte(RANGE); out.writeInt(c.front()); out.writeInt(c.back() + 1); return; }
	out.writeByte(ARRAY);
	out.writeInt((int32_t) c.size());
	for(int32_t v : c) out.writeInt(v);
}

// ------------------------------------------------------------------ dictionaries
// Dense values; nCol is needed for the identity dictionary only. (Unlike Dictionary::create
// an all-zero array stays a dictionary: the reference's readers construct without that check.)
inline std::shared_ptr<IDictionary> readDictionary(DataInput& in) {
	const int t = in.readByte();
	switch(t) {
		case FP64_DICT: {
			const int n = in.readInt();
			if(n < 0 || (size_t) n * 8 > in.remaining()) throw DMLRuntimeException("invalid dictionary length");
			std::vector<double> v((size_t) n);
			for(int i = 0; i < n; i++) v[i] = in.readDouble();
			return std::make_shared<Dictionary>(std::move(v));
		}
		case MATRIX_BLOCK_DICT: {
			auto mb = readMatrixBlock(in);
			const double* a = mb->getDenseBlockValues();
			return std::make_shared<Dictionary>(std::vector<double>(a, a + (size_t) mb->getNumRows() * mb->getNumColumns()));
		}
		case IDENTITY: {
			const int n = in.readInt();
			if(n <= 0 || n > 46340) throw DMLRuntimeException("invalid identity dictionary size");
			std::vector<double> v((size_t) n * n, 0.0);
			for(int i = 0; i < n; i++) v[(size_t) i * n + i] = 1.0;
			return std::make_shared<Dictionary>(std::move(v));
		}
		default: throw NotImplementedException("dictionary type " + std::to_string(t));
	}
}

inline void writeDictionary(const IDictionary& d, DataOutput& out) {
	out.writeByte(FP64_DICT);
	out.writeInt((int32_t) d.getValues().size());
	for(double v : d.getValues()) out.writeDouble(v);
}

// ------------------------------------------------------------------ maps
inline std::shared_ptr<AMapToData> readMap(DataInput& in) {
	const MAP_TYPE t = (MAP_TYPE) in.readByte();
	auto make = [](MAP_TYPE ty, int unique, int size) {
		const int w = ty == MAP_TYPE::INT || ty == MAP_TYPE::CHAR_BYTE ? 4 : ty == MAP_TYPE::CHAR ? 2 : 1;
		return std::make_shared<AMapToData>(ty, unique, size, w);
	};
	auto checkLen = [&](int n, size_t bytesEach) {
		if(n < 0 || (size_t) n * bytesEach > in.remaining()) throw DMLRuntimeException("invalid map length");
	};
	switch(t) {
		case MAP_TYPE::ZERO: {
			const int size = in.readInt();
			if(size < 0) throw DMLRuntimeException("invalid map length");
			return make(t, 1, size);
		}
		case MAP_TYPE::BIT: { // size, number of longs, longs; bit n of word n / 64
			const int size = in.readInt(), nl = in.readInt();
			checkLen(nl, 8);
			if(size < 0 || (int64_t) nl * 64 < size) throw DMLRuntimeException("invalid bit map length");
			auto m = make(t, 2, size);
			for(int w = 0; w < nl; w++) {
				const uint64_t word = (uint64_t) in.readLong();
				for(int b = 0; b < 64 && w * 64 + b < size; b++) m->set(w * 64 + b, (int) ((word >> b) & 1));
			}
			return m;
		}
		case MAP_TYPE::UBYTE:
		case MAP_TYPE::BYTE: {
			const int unique = in.readInt(), n = in.readInt();
			checkLen(n, 1);
			auto m = make(t, unique, n);
			for(int i = 0; i < n; i++) m->set(i, in.readByte()); // & 0xFF
			return m;
		}
		case MAP_TYPE::CHAR: {
			const int unique = in.readInt(), n = in.readInt();
			checkLen(n, 2);
			auto m = make(t, unique, n);
			for(int i = 0; i < n; i++) m->set(i, in.readChar());
			return m;
		}
		case MAP_TYPE::CHAR_BYTE: { // all chars, then all high bytes
			const int unique = in.readInt(), n = in.readInt();
			checkLen(n, 3);
			auto m = make(t, unique, n);
			std::vector<uint16_t> lo((size_t) n);
			for(int i = 0; i < n; i++) lo[i] = in.readChar();
			for(int i = 0; i < n; i++) m->set(i, lo[i] + ((int) in.readByte() << 16));
			return m;
		}
		case MAP_TYPE::INT: {
			const int unique = in.readInt(), n = in.readInt();
			checkLen(n, 4);
			auto m = make(t, unique, n);
			for(int i = 0; i < n; i++) m->set(i, in.readInt());
			return m;
		}
	}
	throw DMLCompressionException("Failed reading map of type: " + std::to_string((int) t));
}

inline void writeMap(const AMapToData& m, DataOutput& out) {
	const MAP_TYPE t = m.getType();
	const int n = m.size();
	out.writeByte((int) t);
	switch(t) {
		case MAP_TYPE::ZERO: out.writeInt(n); return;
		case MAP_TYPE::BIT: {
			const int nl = (n + 63) / 64;
			out.writeInt(n);
			out.writeInt(nl);
			for(int w = 0; w < nl; w++) {
				uint64_t word = 0;
				for(int b = 0; b < 64 && w * 64 + b < n; b++) word |= (uint64_t) (m.getIndex(w * 64 + b) & 1) << b;
				out.writeLong((int64_t) word);
			}
			return;
		}
		default: break;
	}
	out.writeInt(m.getUnique());
	out.writeInt(n);
	switch(t) {
		case MAP_TYPE::UBYTE:
		case MAP_TYPE::BYTE: for(int i = 0; i < n; i++) out.writeByte(m.getIndex(i)); break;
		case MAP_TYPE::CHAR: for(int i = 0; i < n; i++) out.writeChar(m.getIndex(i)); break;
		case MAP_TYPE::CHAR_BYTE:
			for(int i = 0; i < n; i++) out.writeChar(m.getIndex(i) & 0xffff);
			for(int i = 0; i < n; i++) out.writeByte(m.getIndex(i) >> 16);
			break;
		default: for(int i = 0; i < n; i++) out.writeInt(m.getIndex(i)); break;
	}
}

// ------------------------------------------------------------------ offsets
inline std::shared_ptr<AOffset> readOffset(DataInput& in) {
	const int t = in.readByte();
	auto countRows = [](const std::vector<uint16_t>& d) {
		int n = 1;
		for(uint16_t v : d) n += v != 0;
		return n;
	};
	switch(t) {
		case OFF_EMPTY: return std::make_shared<AOffset>(OFF_TYPE::BYTE, 0, -1, 0, std::vector<uint16_t>());
		case SINGLE_OFFSET: {
			const int off = in.readInt();
			return std::make_shared<AOffset>(OFF_TYPE::BYTE, off, off, 1, std::vector<uint16_t>());
		}
		case TWO_OFFSET: {
			const int first = in.readInt(), last = in.readInt();
			return OffsetFactory::createOffset({first, last});
		}
		case OFF_BYTE:
		case BYTEUNZ:
		case BYTENZ: { // first, length, last (, size), bytes
			const int first = in.readInt(), len = in.readInt(), last = in.readInt();
			const int size = t == OFF_BYTE ? in.readInt() : len + 1;
			if(len < 0 || (size_t) len > in.remaining()) throw DMLRuntimeException("invalid offset length");
			std::vector<uint16_t> d((size_t) len);
			for(int i = 0; i < len; i++) d[i] = in.readByte();
			if(countRows(d) != size) throw DMLCompressionException("Invalid offset: size does not match the entries");
			return std::make_shared<AOffset>(OFF_TYPE::BYTE, first, last, size, std::move(d));
		}
		case OFF_CHAR: { // first, length, last, chars; the size is the number of non-zero entries + 1
			const int first = in.readInt(), len = in.readInt(), last = in.readInt();
			if(len < 0 || (size_t) len * 2 > in.remaining()) throw DMLRuntimeException("invalid offset length");
			std::vector<uint16_t> d((size_t) len);
			for(int i = 0; i < len; i++) d[i] = in.readChar();
			const int size = countRows(d);
			return std::make_shared<AOffset>(OFF_TYPE::CHAR, first, last, size, std::move(d));
		}
		default: throw DMLCompressionException("Failed reading offset of type: " + std::to_string(t));
	}
}

inline void writeOffset(const AOffset& o, DataOutput& out) {
	if(o.getSize() == 0) { out.writeByte(OFF_EMPTY); return; }
	if(o.getSize() == 1) { out.writeByte(SINGLE_OFFSET); out.writeInt(o.getOffsetToFirst()); return; }
	if(o.getSize() == 2) { out.writeByte(TWO_OFFSET); out.writeInt(o.getOffsetToFirst()); out.writeInt(o.getOffsetToLast()); return; }
	const bool byte = o.getType() == OFF_TYPE::BYTE;
	out.writeByte(byte ? OFF_BYTE : OFF_CHAR);
	out.writeInt(o.getOffsetToFirst());
	out.writeInt((int32_t) o.getLength());
	out.writeInt(o.getOffsetToLast());
	if(byte) out.writeInt(o.getSize());
	for(int64_t i = 0; i < o.getLength(); i++)
		if(byte) out.writeByte(o.delta(i)); else out.writeChar(o.delta(i));
}

// ------------------------------------------------------------------ column groups
inline AColGroupPtr readColGroup(DataInput& in, int nRows) {
	const int ctype = in.readByte();
	switch(ctype) {
		case DDC: {
			IColIndex cols = readColIndex(in);
			auto dict = readDictionary(in);
			auto data = readMap(in);
			return ColGroupDDC::create(std::move(cols), std::move(dict), std::move(data));
		}
		case RLE: { // pointers, (gap, run length) chars, zeros flag
			IColIndex cols = readColIndex(in);
			auto dict = readDictionary(in);
			const int np = in.readInt();
			if(np < 1 || (size_t) np * 4 > in.remaining()) throw DMLRuntimeException("invalid RLE pointer length");
			std::vector<int32_t> ptr((size_t) np);
			for(int i = 0; i < np; i++) ptr[i] = in.readInt();
			const int nd = in.readInt();
			if(nd < 0 || (size_t) nd * 2 > in.remaining()) throw DMLRuntimeException("invalid RLE data length");
			std::vector<uint16_t> data((size_t) nd);
			for(int i = 0; i < nd; i++) data[i] = in.readChar();
			in.readBoolean();
			return ColGroupRLE::create(std::move(cols), nRows, std::move(dict), std::move(data), std::move(ptr));
		}
		case CONST: {
			IColIndex cols = readColIndex(in);
			auto dict = readDictionary(in);
			return ColGroupConst::create(std::move(cols), dict->getValues());
		}
		case EMPTY: return std::make_shared<ColGroupEmpty>(readColIndex(in));
		case UNCOMPRESSED: {
			IColIndex cols = readColIndex(in);
			auto mb = readMatrixBlock(in);
			if(mb->getNumRows() != nRows) throw DMLCompressionException("Invalid uncompressed group: number of rows differs from the block");
			return ColGroupUncompressed::create(std::move(mb), std::move(cols));
		}
		case SDC: {
			IColIndex cols = readColIndex(in);
			auto dict = readDictionary(in);
			auto off = readOffset(in);
			auto data = readMap(in);
			std::vector<double> def(cols.size());
			for(double& d : def) d = in.readDouble();
			return ColGroupSDC::create(std::move(cols), nRows, std::move(dict), std::move(def), std::move(off), std::move(data));
		}
		case SDCZeros: {
			IColIndex cols = readColIndex(in);
			auto dict = readDictionary(in);
			auto off = readOffset(in);
			auto data = readMap(in);
			return ColGroupSDCZeros::create(std::move(cols), nRows, std::move(dict), std::move(off), std::move(data));
		}
		case SDCSingle: { // one tuple for every listed row: a map of zeros
			IColIndex cols = readColIndex(in);
			auto dict = readDictionary(in);
			auto off = readOffset(in);
			std::vector<double> def(cols.size());
			for(double& d : def) d = in.readDouble();
			auto data = MapToFactory::create(off->getSize(), 1);
			return ColGroupSDC::create(std::move(cols), nRows, std::move(dict), std::move(def), std::move(off), std::move(data));
		}
		case SDCSingleZeros: {
			IColIndex cols = readColIndex(in);
			auto dict = readDictionary(in);
			auto off = readOffset(in);
			auto data = MapToFactory::create(off->getSize(), 1);
			return ColGroupSDCZeros::create(std::move(cols), nRows, std::move(dict), std::move(off), std::move(data));
		}
		default:
			if(ctype < 0 || ctype > LinearFunctional) throw DMLRuntimeException("Unsupported ColGroup Type used: " + std::to_string(ctype));
			throw NotImplementedException("column group type " + std::to_string(ctype) + " is not on the device path");
	}
}

inline void writeColGroup(const AColGroup& g, DataOutput& out) {
	auto header = [&](int type) { out.writeByte(type); writeColIndex(g.getColIndices(), out); };
	switch(g.getCompType()) {
		case CompressionType::EMPTY: header(EMPTY); return;
		case CompressionType::CONST: header(CONST); writeDictionary(*g.getDictionary(), out); return;
		case CompressionType::DDC: {
			const auto& d = static_cast<const ColGroupDDC&>(g);
			header(DDC);
			writeDictionary(*g.getDictionary(), out);
			writeMap(*d.getMapToData(), out);
			return;
		}
		case CompressionType::SDC:
		case CompressionType::SDCZeros: {
			const auto& s = static_cast<const ColGroupSDCBase&>(g);
			const bool zeros = g.getCompType() == CompressionType::SDCZeros;
			header(zeros ? SDCZeros : SDC);
			writeDictionary(*g.getDictionary(), out);
			writeOffset(*s.getOffsets(), out);
			writeMap(*s.getMapToData(), out);
			if(!zeros)
				for(double v : s.getDefaultTuple()) out.writeDouble(v);
			return;
		}
		case CompressionType::RLE: {
			const auto& r = static_cast<const ColGroupRLE&>(g);
			header(RLE);
			writeDictionary(*g.getDictionary(), out);
			out.writeInt((int32_t) r.getPtr().size());
			for(int32_t p : r.getPtr()) out.writeInt(p);
			out.writeInt((int32_t) r.getData().size());
			for(uint16_t c : r.getData()) out.writeChar(c);
			out.writeBoolean(true); // rows outside all runs are zero
			return;
		}
		case CompressionType::UNCOMPRESSED: {
			const auto& u = static_cast<const ColGroupUncompressed&>(g);
			header(UNCOMPRESSED);
			writeMatrixBlock(*u.getData(), out);
			return;
		}
		default: throw NotImplementedException("column group type cannot be serialised");
	}
}

// CompressedMatrixBlock.read: rlen, clen, nonZeros, overlapping flag, group count, groups
inline std::shared_ptr<CompressedMatrixBlock> readCompressedMatrixBlock(const uint8_t* bytes, size_t n) {
	DataInput in(bytes, n);
	const int rlen = in.readInt(), clen = in.readInt();
	const int64_t nnz = in.readLong();
	const bool overlapping = in.readBoolean();
	if(rlen < 0 || clen < 0) throw DMLRuntimeException("invalid compressed block dimensions");
	const int nGroups = in.readInt();
	if(nGroups < 0 || (size_t) nGroups > in.remaining()) throw DMLRuntimeException("invalid number of column groups");
	std::vector<AColGroupPtr> groups;
	for(int i = 0; i < nGroups; i++) groups.push_back(readColGroup(in, rlen));
	auto cmb = std::make_shared<CompressedMatrixBlock>(rlen, clen);
	cmb->allocateColGroupList(std::move(groups));
	cmb->setOverlapping(overlapping);
	cmb->setNonZeros(nnz);
	return cmb;
}

inline std::vector<uint8_t> writeCompressedMatrixBlock(const CompressedMatrixBlock& cmb) {
	if(cmb.isDeviceOnly()) throw NotImplementedException("a device-only block has no host-side column groups to serialise");
	DataOutput out;
	out.writeInt(cmb.getNumRows());
	out.writeInt(cmb.getNumColumns());
	out.writeLong(cmb.getNonZeros());
	out.writeBoolean(cmb.isOverlapping());
	out.writeInt((int32_t) cmb.getColGroups().size());
	for(const auto& g : cmb.getColGroups()) writeColGroup(*g, out);
	return std::move(out.bytes);
}

} // namespace io
} // namespace compress
} // namespace sysds
