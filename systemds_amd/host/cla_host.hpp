// Host side of the compressed multiply path above the C ABI (cla_hip.h), in C++.
//
// It mirrors the classes a SystemDS caller touches on this path, with the same
// names, argument meaning and error behaviour, so that code written against
// org.apache.sysds.runtime.compress reads the same here:
//
//   MatrixBlock, CompressedMatrixBlock            C/CompressedMatrixBlock.java:119-132, 587-627
//   AMapToData, MapToFactory                      CG/mapping/MapToFactory.java:102-117
//   AOffset, AIterator, OffsetFactory             CG/offset/OffsetFactory.java:105-139, OffsetByte.java, OffsetChar.java
//   Dictionary                                    CG/dictionary/Dictionary.java
//   ColGroupDDC / SDC / SDCZeros / RLE /          CG/ColGroupDDC.java:106-113, ColGroupSDC.java:101-117,
//   Uncompressed / Const / Empty                  ColGroupSDCZeros.java:94-104, ColGroupRLE.java:75-91, ColGroupConst.java:136-158
//   CLALibMatrixMult, CLALibRightMultBy,          C/lib/CLALibMatrixMult.java:42-94, CLALibRightMultBy.java:51-102,
//   CLALibLeftMultBy, CLALibTSMM, CLALibMMChain,  CLALibLeftMultBy.java:73-145, CLALibTSMM.java:46-94, CLALibMMChain.java:92-148,
//   CLALibDecompress                              CLALibDecompress.java:56-66
//
// (C/ = src/main/java/org/apache/sysds/runtime/compress/, CG/ = C/colgroup/.)
//
// All arithmetic of the path runs on the device behind the C ABI; this layer owns
// the encodings on the host, uploads a block once (hipHandle) and maps return codes
// to the reference's exception types. There is no CPU compute fallback: without the
// HIP library or a gfx950 device every multiply throws.
#pragma once
#include "../../include/cla_hip.h"

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace sysds {

struct DMLRuntimeException : std::runtime_error { using std::runtime_error::runtime_error; };
struct DMLCompressionException : DMLRuntimeException { using DMLRuntimeException::DMLRuntimeException; };
struct NotImplementedException : DMLRuntimeException { using DMLRuntimeException::DMLRuntimeException; };

// Maps a negative C ABI return value to the exception the reference would throw.
inline int64_t checkNative(int64_t rc, const char* what) {
	if(rc >= 0) return rc;
	const std::string msg = std::string(what) + ": " + cla_last_error();
	if(rc == -CLA_ERR_UNSUPPORTED) throw NotImplementedException(msg);
	if(rc == -CLA_ERR_INVALID) throw DMLCompressionException(msg);
	throw DMLRuntimeException(msg);
}

enum class CompressionType { DDC, SDC, SDCZeros, RLE, UNCOMPRESSED, CONST, EMPTY };
enum class MMTSJType { NONE, LEFT, RIGHT };
enum class ChainType { XtXv, XtwXv, XtXvy, NONE };

// ------------------------------------------------------------------ MatrixBlock
// Dense row-major fp64 block (the DenseBlockFP64 case of matrix/data/MatrixBlock.java).
class MatrixBlock {
public:
	MatrixBlock() = default;
	MatrixBlock(int rl, int cl, bool allocate = true) : rlen(rl), clen(cl) {
		if(rl < 0 || cl < 0) throw DMLRuntimeException("Invalid negative dimensions");
		if(allocate) allocateDenseBlock();
	}
	MatrixBlock(int rl, int cl, std::vector<double> v) : rlen(rl), clen(cl), values(std::move(v)) {
		if((size_t) rl * cl != values.size()) throw DMLRuntimeException("Invalid dense block length");
		recomputeNonZeros();
	}
	virtual ~MatrixBlock() = default;
	virtual bool isCompressed() const { return false; }

	int getNumRows() const { return rlen; }
	int getNumColumns() const { return clen; }
	int64_t getNonZeros() const { return nonZeros; }
	void setNonZeros(int64_t n) { nonZeros = n; }
	virtual bool isEmpty() const { return rlen == 0 || clen == 0 || nonZeros == 0; }
	bool isAllocated() const { return values.size() == (size_t) rlen * clen && !values.empty(); }
	void allocateDenseBlock() { values.assign((size_t) rlen * clen, 0.0); }
	void reset(int rl, int cl) { rlen = rl; clen = cl; nonZeros = 0; allocateDenseBlock(); }
	double* getDenseBlockValues() { return values.data(); }
	const double* getDenseBlockValues() const { return values.data(); }
	double get(int r, int c) const { return values.empty() ? 0.0 : values[(size_t) r * clen + c]; }
	void set(int r, int c, double v) { values[(size_t) r * clen + c] = v; }
	int64_t recomputeNonZeros() {
		int64_t n = 0;
		for(double v : values) n += v != 0.0;
		return nonZeros = n;
	}
	// LibMatrixReorg.transpose for the dense case.
	MatrixBlock transpose() const {
		MatrixBlock t(clen, rlen);
		if(!values.empty())
			for(int r = 0; r < rlen; r++)
				for(int c = 0; c < clen; c++) t.values[(size_t) c * rlen + r] = values[(size_t) r * clen + c];
		t.nonZeros = nonZeros;
		return t;
	}

protected:
	int rlen = 0, clen = 0;
	int64_t nonZeros = 0;
	std::vector<double> values;
};

namespace compress {

using IColIndex = std::vector<int32_t>;

struct ColIndexFactory {
	static IColIndex create(int l, int u) { // [l, u)
		IColIndex r;
		for(int i = l; i < u; i++) r.push_back(i);
		return r;
	}
	static IColIndex create(std::vector<int32_t> idx) {
		for(size_t i = 1; i < idx.size(); i++)
			if(idx[i] <= idx[i - 1]) throw DMLCompressionException("Invalid column indexes: not sorted or duplicate");
		return idx;
	}
	static IColIndex createI(std::initializer_list<int32_t> idx) { return create(std::vector<int32_t>(idx)); }
};

// ------------------------------------------------------------------ AMapToData
enum class MAP_TYPE { ZERO, BIT, UBYTE, BYTE, CHAR, CHAR_BYTE, INT };

// Row -> tuple index. The device stores three widths (unsigned byte, char, int); the
// narrower reference types (zero, bit, ubyte) are widened to a byte and char+byte to int.
class AMapToData {
public:
	virtual ~AMapToData() = default;
	int getUnique() const { return nUnique; }
	void setUnique(int u) { nUnique = u; }
	int size() const { return n; }
	MAP_TYPE getType() const { return type; }
	int codeWidth() const { return width; }
	const void* raw() const { return width == 1 ? (const void*) b8.data() : width == 2 ? (const void*) b16.data() : (const void*) b32.data(); }
	int getIndex(int i) const { return width == 1 ? b8[i] : width == 2 ? b16[i] : b32[i]; }
	void set(int i, int v) {
		if(v < 0 || v >= std::max(nUnique, 1)) throw DMLCompressionException("Invalid map value " + std::to_string(v));
		if(width == 1) b8[i] = (uint8_t) v; else if(width == 2) b16[i] = (uint16_t) v; else b32[i] = v;
	}
	void fill(int v) { for(int i = 0; i < n; i++) set(i, v); }
	std::vector<int32_t> getCounts() const {
		std::vector<int32_t> c((size_t) std::max(nUnique, 1), 0);
		for(int i = 0; i < n; i++) c[getIndex(i)]++;
		return c;
	}
	// AMapToData.verify: every index below the number of unique values.
	void verify() const {
		for(int i = 0; i < n; i++)
			if(getIndex(i) >= nUnique) throw DMLCompressionException("Invalid construction with too high index in map");
	}
	AMapToData(MAP_TYPE t, int unique, int size, int w) : type(t), nUnique(unique), n(size), width(w) {
		if(w == 1) b8.assign(size, 0); else if(w == 2) b16.assign(size, 0); else b32.assign(size, 0);
	}

private:
	MAP_TYPE type;
	int nUnique, n, width;
	std::vector<uint8_t> b8;
	std::vector<uint16_t> b16;
	std::vector<int32_t> b32;
};

struct MapToFactory {
	// The type the reference picks for a number of unique values (MapToFactory.java:102-117).
	static MAP_TYPE getType(int size, int unique) {
		if(unique <= 1) return MAP_TYPE::ZERO;
		if(unique == 2 && size > 32) return MAP_TYPE::BIT;
		if(unique <= 128) return MAP_TYPE::UBYTE;
		if(unique <= 256) return MAP_TYPE::BYTE;
		if(unique <= 65536) return MAP_TYPE::CHAR;
		if(unique <= 16777216) return MAP_TYPE::CHAR_BYTE;
		return MAP_TYPE::INT;
	}
	static std::shared_ptr<AMapToData> create(int size, int unique) {
		const MAP_TYPE t = getType(size, unique);
		const int w = unique <= 256 ? 1 : unique <= 65536 ? 2 : 4;
		return std::make_shared<AMapToData>(t, unique, size, w);
	}
	static std::shared_ptr<AMapToData> create(int unique, const std::vector<int32_t>& values) {
		auto m = create((int) values.size(), unique);
		for(size_t i = 0; i < values.size(); i++) m->set((int) i, values[i]);
		return m;
	}
};

// ------------------------------------------------------------------ AOffset
class AOffset;

// Walks an offset list like CG/offset/AIterator.java: value() is the current row,
// getDataIndex() the position in the group's map.
class AIterator {
public:
	int value() const { return row; }
	int getDataIndex() const { return dataIdx; }
	int getOffsetsIndex() const { return pos; }
	bool isNotOver(int ub) const { return row < ub; }
	int next();
	int skipTo(int idx) {
		while(row < idx && row < last()) next();
		return row;
	}

private:
	friend class AOffset;
	int last() const;
	const AOffset* off = nullptr;
	int row = 0, dataIdx = 0, pos = 0;
};

enum class OFF_TYPE { BYTE, CHAR };

// Delta encoded sorted row list: first row outside the array, then one entry per
// following row holding the distance; an entry 0 stands for "+255" (byte) or "+65535"
// (char) without a row (OffsetByte.java / OffsetChar.java).
class AOffset {
public:
	AOffset(OFF_TYPE t, int first_, int last_, int size_, std::vector<uint16_t> d)
		: type(t), first(first_), last(last_), n(size_), deltas16(std::move(d)) {
		if(t == OFF_TYPE::BYTE) {
			deltas8.assign(deltas16.begin(), deltas16.end());
			deltas16.clear();
		}
	}
	OFF_TYPE getType() const { return type; }
	int getOffsetToFirst() const { return first; }
	int getOffsetToLast() const { return last; }
	int getSize() const { return n; }
	int64_t getLength() const { return (int64_t) (type == OFF_TYPE::BYTE ? deltas8.size() : deltas16.size()); }
	int deltaWidth() const { return type == OFF_TYPE::BYTE ? 1 : 2; }
	const void* raw() const { return type == OFF_TYPE::BYTE ? (const void*) deltas8.data() : (const void*) deltas16.data(); }
	int delta(int64_t i) const { return type == OFF_TYPE::BYTE ? deltas8[i] : deltas16[i]; }
	int maxV() const { return type == OFF_TYPE::BYTE ? 255 : 65535; }
	AIterator getIterator() const {
		AIterator it;
		it.off = this; it.row = first; it.dataIdx = 0; it.pos = 0;
		return it;
	}
	std::vector<int32_t> toArray() const {
		std::vector<int32_t> r;
		if(n == 0) return r;
		AIterator it = getIterator();
		r.push_back(it.value());
		while(it.value() < last) r.push_back(it.next());
		return r;
	}
	// AOffset.verify: the list decodes to `size` rows and ends at offsetToLast.
	void verify(int size) const {
		if(n != size) throw DMLCompressionException("Invalid offset: size " + std::to_string(n) + " vs " + std::to_string(size));
		if(n > 0 && (int) toArray().size() != size) throw DMLCompressionException("Invalid offset: decoded length differs");
	}

private:
	OFF_TYPE type;
	int first, last, n;
	std::vector<uint8_t> deltas8;
	std::vector<uint16_t> deltas16;
};

inline int AIterator::last() const { return off->getOffsetToLast(); }
inline int AIterator::next() {
	int d = off->delta(pos++);
	while(d == 0) { row += off->maxV(); d = off->delta(pos++); }
	row += d;
	dataIdx++;
	return row;
}

struct OffsetFactory {
	// OffsetFactory.java:230-236
	static int correctionByte(int nRows, int size) { return (int) (std::max<int64_t>((int64_t) nRows - (int64_t) size * 256, 0) / 256); }
	static int correctionChar(int nRows, int size) { return (int) (std::max<int64_t>((int64_t) nRows - (int64_t) size * 65535, 0) / 65535); }
	// JVM array costs used by the size comparison (utils/MemoryEstimates.java byteArrayCost / charArrayCost)
	static int64_t byteArrayCost(int64_t len) { return 28 + (len <= 4 ? 4 : len + ((8 - (len - 4) % 8) % 8)); }
	static int64_t charArrayCost(int64_t len) { return 28 + (len <= 2 ? 4 : len * 2 + ((8 - (len * 2 - 4) % 8) % 8)); }
	// OffsetFactory.java:105-139: the narrower in-memory estimate wins. (OffsetSingle / OffsetTwo /
	// OffsetEmpty are byte lists with 0, 1 or no entries here.)
	static std::shared_ptr<AOffset> createOffset(const std::vector<int32_t>& idx) {
		const int n = (int) idx.size();
		if(n == 0) return std::make_shared<AOffset>(OFF_TYPE::BYTE, 0, -1, 0, std::vector<uint16_t>());
		if(idx[0] < 0) throw DMLCompressionException("Invalid negative offset");
		if(n < 3) return createOffset(idx, OFF_TYPE::BYTE);
		const int endLength = n - 1;
		const int range = idx[n - 1] - idx[0];
		const int64_t byteSize = 16 + 4 + 4 + 4 + 8 + byteArrayCost(endLength + correctionByte(range, endLength));
		const int64_t charSize = 16 + 4 + 4 + 8 + charArrayCost(endLength + correctionChar(range, endLength));
		return createOffset(idx, byteSize < charSize ? OFF_TYPE::BYTE : OFF_TYPE::CHAR);
	}
	static std::shared_ptr<AOffset> createOffset(const std::vector<int32_t>& idx, OFF_TYPE t) {
		const int n = (int) idx.size();
		if(n == 0) return std::make_shared<AOffset>(t, 0, -1, 0, std::vector<uint16_t>());
		if(idx[0] < 0) throw DMLCompressionException("Invalid negative offset");
		const int maxV = t == OFF_TYPE::BYTE ? 255 : 65535;
		std::vector<uint16_t> d;
		d.reserve(n);
		for(int i = 1; i < n; i++) {
			int64_t gap = (int64_t) idx[i] - idx[i - 1];
			if(gap <= 0) throw DMLCompressionException("Invalid input to create offset, all values should be continuously increasing.");
			// a gap that is a multiple of maxV ends on a full entry, not on a skip
			while(gap > maxV) { d.push_back(0); gap -= maxV; }
			d.push_back((uint16_t) gap);
		}
		return std::make_shared<AOffset>(t, idx[0], idx[n - 1], n, std::move(d));
	}
};

// ------------------------------------------------------------------ Dictionary
// Dense tuple values, nVals x nCol row-major (CG/dictionary/Dictionary.java).
class Dictionary {
public:
	static std::shared_ptr<Dictionary> create(std::vector<double> v) {
		if(v.empty()) throw DMLCompressionException("Invalid construction of dictionary with empty array of values");
		bool any = false;
		for(double x : v) any |= x != 0.0;
		return any ? std::make_shared<Dictionary>(std::move(v)) : nullptr; // all zero -> null, as the reference
	}
	explicit Dictionary(std::vector<double> v) : values(std::move(v)) {}
	const std::vector<double>& getValues() const { return values; }
	int getNumberOfValues(int nCol) const { return (int) (values.size() / (size_t) nCol); }
	double getValue(int r, int c, int nCol) const { return values[(size_t) r * nCol + c]; }

private:
	std::vector<double> values;
};
using IDictionary = Dictionary;

// ------------------------------------------------------------------ column groups
class AColGroup {
public:
	virtual ~AColGroup() = default;
	const IColIndex& getColIndices() const { return cols; }
	int getNumCols() const { return (int) cols.size(); }
	virtual CompressionType getCompType() const = 0;
	virtual int getNumValues() const { return dict ? dict->getNumberOfValues(getNumCols()) : 0; }
	const std::shared_ptr<IDictionary>& getDictionary() const { return dict; }
	// Adds this group to a device block under construction.
	virtual void upload(cla_handle h) const = 0;

protected:
	AColGroup(IColIndex c, std::shared_ptr<IDictionary> d) : cols(std::move(c)), dict(std::move(d)) {
		if(cols.empty()) throw DMLCompressionException("Invalid column group without columns");
	}
	IColIndex cols;
	std::shared_ptr<IDictionary> dict;
};
using AColGroupPtr = std::shared_ptr<AColGroup>;

class ColGroupEmpty : public AColGroup {
public:
	explicit ColGroupEmpty(IColIndex c) : AColGroup(std::move(c), nullptr) {}
	CompressionType getCompType() const override { return CompressionType::EMPTY; }
	void upload(cla_handle h) const override { checkNative(cla_block_add_empty(h, cols.data(), getNumCols()), "ColGroupEmpty"); }
};

class ColGroupConst : public AColGroup {
public:
	// ColGroupConst.java:83-102, 136-158: all-zero values collapse to an empty group.
	static AColGroupPtr create(IColIndex c, std::shared_ptr<IDictionary> d) {
		if(d == nullptr) return std::make_shared<ColGroupEmpty>(std::move(c));
		if((size_t) d->getValues().size() != c.size())
			throw DMLCompressionException("Invalid construction of const column group: number of columns and values differ");
		return AColGroupPtr(new ColGroupConst(std::move(c), std::move(d)));
	}
	static AColGroupPtr create(IColIndex c, const std::vector<double>& values) {
		if(values.size() != c.size())
			throw DMLCompressionException("Invalid number of values in vs columns: " + std::to_string(values.size()) + " vs " + std::to_string(c.size()));
		return create(std::move(c), Dictionary::create(values));
	}
	static AColGroupPtr create(IColIndex c, double value) { return create(c, std::vector<double>(c.size(), value)); }
	const std::vector<double>& getValues() const { return dict->getValues(); }
	int getNumValues() const override { return 1; }
	CompressionType getCompType() const override { return CompressionType::CONST; }
	void upload(cla_handle h) const override {
		checkNative(cla_block_add_const(h, cols.data(), getNumCols(), dict->getValues().data()), "ColGroupConst");
	}

private:
	ColGroupConst(IColIndex c, std::shared_ptr<IDictionary> d) : AColGroup(std::move(c), std::move(d)) {}
};

class ColGroupDDC : public AColGroup {
public:
	// ColGroupDDC.java:106-113
	static AColGroupPtr create(IColIndex c, std::shared_ptr<IDictionary> d, std::shared_ptr<AMapToData> data) {
		if(data == nullptr) throw DMLCompressionException("Invalid DDC construction without a map");
		if(data->getUnique() == 1) return ColGroupConst::create(std::move(c), std::move(d));
		if(d == nullptr) return std::make_shared<ColGroupEmpty>(std::move(c));
		if(data->getUnique() != d->getNumberOfValues((int) c.size()))
			throw DMLCompressionException("Invalid map to dict Map has:" + std::to_string(data->getUnique()) + " while dict has " +
				std::to_string(d->getNumberOfValues((int) c.size())));
		data->verify();
		return AColGroupPtr(new ColGroupDDC(std::move(c), std::move(d), std::move(data)));
	}
	const std::shared_ptr<AMapToData>& getMapToData() const { return map; }
	std::vector<int32_t> getCounts() const { return map->getCounts(); }
	CompressionType getCompType() const override { return CompressionType::DDC; }
	void upload(cla_handle h) const override {
		checkNative(cla_block_add_ddc(h, cols.data(), getNumCols(), dict->getValues().data(), getNumValues(), map->raw(), map->codeWidth()),
			"ColGroupDDC");
	}

private:
	ColGroupDDC(IColIndex c, std::shared_ptr<IDictionary> d, std::shared_ptr<AMapToData> m)
		: AColGroup(std::move(c), std::move(d)), map(std::move(m)) {}
	std::shared_ptr<AMapToData> map;
};

// SDC and SDCZeros share the storage; SDCZeros has no default tuple.
class ColGroupSDCBase : public AColGroup {
public:
	const std::shared_ptr<AOffset>& getOffsets() const { return offsets; }
	const std::shared_ptr<AMapToData>& getMapToData() const { return map; }
	const std::vector<double>& getDefaultTuple() const { return defaultTuple; }
	int getNumRows() const { return numRows; }
	void upload(cla_handle h) const override {
		checkNative(cla_block_add_sdc(h, cols.data(), getNumCols(), dict->getValues().data(), getNumValues(),
			defaultTuple.empty() ? nullptr : defaultTuple.data(), map->raw(), map->codeWidth(), offsets->raw(), offsets->deltaWidth(),
			offsets->getLength(), offsets->getOffsetToFirst(), offsets->getOffsetToLast(), offsets->getSize()), "ColGroupSDC");
	}

protected:
	ColGroupSDCBase(IColIndex c, int nRows, std::shared_ptr<IDictionary> d, std::vector<double> def, std::shared_ptr<AOffset> o,
		std::shared_ptr<AMapToData> m)
		: AColGroup(std::move(c), std::move(d)), numRows(nRows), defaultTuple(std::move(def)), offsets(std::move(o)), map(std::move(m)) {
		if(offsets == nullptr || map == nullptr) throw DMLCompressionException("Invalid SDC construction without offsets or map");
		if(map->getUnique() != dict->getNumberOfValues(getNumCols()))
			throw DMLCompressionException("Invalid construction of SDC group: number of dictionary values and unique map values differ");
		if(offsets->getSize() != map->size())
			throw DMLCompressionException("Invalid construction of SDC group: offsets and map have different lengths");
		if(offsets->getSize() > 0 && offsets->getOffsetToLast() >= numRows)
			throw DMLCompressionException("Invalid construction of SDC group: last offset beyond the number of rows");
		map->verify();
	}
	int numRows;
	std::vector<double> defaultTuple;
	std::shared_ptr<AOffset> offsets;
	std::shared_ptr<AMapToData> map;
};

class ColGroupSDCZeros : public ColGroupSDCBase {
public:
	// ColGroupSDCZeros.java:94-104
	static AColGroupPtr create(IColIndex c, int numRows, std::shared_ptr<IDictionary> d, std::shared_ptr<AOffset> o,
		std::shared_ptr<AMapToData> data) {
		if(d == nullptr) return std::make_shared<ColGroupEmpty>(std::move(c));
		return AColGroupPtr(new ColGroupSDCZeros(std::move(c), numRows, std::move(d), std::move(o), std::move(data)));
	}
	CompressionType getCompType() const override { return CompressionType::SDCZeros; }

private:
	ColGroupSDCZeros(IColIndex c, int n, std::shared_ptr<IDictionary> d, std::shared_ptr<AOffset> o, std::shared_ptr<AMapToData> m)
		: ColGroupSDCBase(std::move(c), n, std::move(d), {}, std::move(o), std::move(m)) {}
};

class ColGroupSDC : public ColGroupSDCBase {
public:
	// ColGroupSDC.java:101-117. (The single-value specialisations SDCSingle / SDCSingleZeros
	// are kept as SDC / SDCZeros with a one-entry dictionary: the device treats them alike.)
	static AColGroupPtr create(IColIndex c, int numRows, std::shared_ptr<IDictionary> d, std::vector<double> defaultTuple,
		std::shared_ptr<AOffset> o, std::shared_ptr<AMapToData> data) {
		if(defaultTuple.size() != c.size())
			throw DMLCompressionException("Invalid construction of SDC group: default tuple and columns differ in length");
		bool allZero = true;
		for(double v : defaultTuple) allZero &= v == 0.0;
		if(d == nullptr && allZero) return std::make_shared<ColGroupEmpty>(std::move(c));
		if(d == nullptr) { // only the default is non-zero: rows in the list are zero
			d = std::make_shared<Dictionary>(std::vector<double>(c.size(), 0.0));
			data = MapToFactory::create(o->getSize(), 1);
		}
		if(allZero) return ColGroupSDCZeros::create(std::move(c), numRows, std::move(d), std::move(o), std::move(data));
		return AColGroupPtr(new ColGroupSDC(std::move(c), numRows, std::move(d), std::move(defaultTuple), std::move(o), std::move(data)));
	}
	CompressionType getCompType() const override { return CompressionType::SDC; }

private:
	ColGroupSDC(IColIndex c, int n, std::shared_ptr<IDictionary> d, std::vector<double> def, std::shared_ptr<AOffset> o,
		std::shared_ptr<AMapToData> m)
		: ColGroupSDCBase(std::move(c), n, std::move(d), std::move(def), std::move(o), std::move(m)) {}
};

class ColGroupRLE : public AColGroup {
public:
	// ColGroupRLE.java:75-91: data = (gap, run length) char pairs per value, ptr[nVals + 1].
	static AColGroupPtr create(IColIndex c, int numRows, std::shared_ptr<IDictionary> d, std::vector<uint16_t> data, std::vector<int32_t> ptr) {
		if(d == nullptr) return std::make_shared<ColGroupEmpty>(std::move(c));
		if((int) ptr.size() != d->getNumberOfValues((int) c.size()) + 1 || ptr.front() != 0 || ptr.back() != (int) data.size())
			throw DMLCompressionException("Invalid RLE construction: pointers do not match dictionary and data");
		return AColGroupPtr(new ColGroupRLE(std::move(c), numRows, std::move(d), std::move(data), std::move(ptr)));
	}
	// ColGroupRLE's bitmap encoder (CG/ColGroupRLE.java genRLEBitmap): sorted row lists per value.
	static void genRLEBitmap(const std::vector<std::vector<int32_t>>& rowsPerValue, std::vector<uint16_t>& data, std::vector<int32_t>& ptr) {
		data.clear();
		ptr.assign(1, 0);
		for(const auto& rows : rowsPerValue) {
			int lastEnd = 0; // first row after the previous run
			size_t i = 0;
			while(i < rows.size()) {
				size_t j = i + 1;
				while(j < rows.size() && rows[j] == rows[j - 1] + 1) j++;
				int start = rows[i], len = (int) (j - i);
				int gap = start - lastEnd;
				while(gap > 65535) { data.push_back(65535); data.push_back(0); gap -= 65535; }
				while(len > 65535) { data.push_back((uint16_t) gap); data.push_back(65535); gap = 0; len -= 65535; }
				data.push_back((uint16_t) gap);
				data.push_back((uint16_t) len);
				lastEnd = rows[j - 1] + 1;
				i = j;
			}
			ptr.push_back((int32_t) data.size());
		}
	}
	int getNumRows() const { return numRows; }
	const std::vector<uint16_t>& getData() const { return data; }
	const std::vector<int32_t>& getPtr() const { return ptr; }
	CompressionType getCompType() const override { return CompressionType::RLE; }
	void upload(cla_handle h) const override {
		checkNative(cla_block_add_rle(h, cols.data(), getNumCols(), dict->getValues().data(), getNumValues(), ptr.data(), data.data(),
			(int64_t) data.size()), "ColGroupRLE");
	}

private:
	ColGroupRLE(IColIndex c, int n, std::shared_ptr<IDictionary> d, std::vector<uint16_t> dt, std::vector<int32_t> p)
		: AColGroup(std::move(c), std::move(d)), numRows(n), data(std::move(dt)), ptr(std::move(p)) {}
	int numRows;
	std::vector<uint16_t> data;
	std::vector<int32_t> ptr;
};

class ColGroupUncompressed : public AColGroup {
public:
	// ColGroupUncompressed.java:127-142
	static AColGroupPtr create(std::shared_ptr<MatrixBlock> mb, IColIndex c) {
		if(mb == nullptr || mb->getNumColumns() != (int) c.size())
			throw DMLCompressionException("Invalid construction of uncompressed column group: columns and matrix differ");
		if(mb->isEmpty()) return std::make_shared<ColGroupEmpty>(std::move(c));
		return AColGroupPtr(new ColGroupUncompressed(std::move(c), std::move(mb)));
	}
	static AColGroupPtr create(std::shared_ptr<MatrixBlock> mb) { return create(mb, ColIndexFactory::create(0, mb->getNumColumns())); }
	const std::shared_ptr<MatrixBlock>& getData() const { return data; }
	int getNumValues() const override { return data->getNumRows(); }
	CompressionType getCompType() const override { return CompressionType::UNCOMPRESSED; }
	void upload(cla_handle h) const override {
		checkNative(cla_block_add_uncompressed(h, cols.data(), getNumCols(), data->getDenseBlockValues()), "ColGroupUncompressed");
	}

private:
	ColGroupUncompressed(IColIndex c, std::shared_ptr<MatrixBlock> mb) : AColGroup(std::move(c), nullptr), data(std::move(mb)) {}
	std::shared_ptr<MatrixBlock> data;
};

// Selects HIP device 0 on first use (the library computes on a gfx950 device only).
inline void ensureDevice() {
	static bool ready = false;
	if(ready) return;
	checkNative(cla_init(0), "cla_init");
	ready = true;
}

// ------------------------------------------------------------------ CompressedMatrixBlock
class CompressedMatrixBlock : public MatrixBlock {
public:
	CompressedMatrixBlock(int rl, int cl) : MatrixBlock(rl, cl, false) {}
	~CompressedMatrixBlock() override { releaseDevice(); }
	CompressedMatrixBlock(const CompressedMatrixBlock&) = delete;
	CompressedMatrixBlock& operator=(const CompressedMatrixBlock&) = delete;
	bool isCompressed() const override { return true; }

	// CompressedMatrixBlock.allocateColGroupList / allocateColGroup
	// A block that lives on the device only: the overlapping result of a right multiply. It has
	// no host-side column groups; every linear operation of this class works on it.
	static std::shared_ptr<CompressedMatrixBlock> adoptDevice(int rl, int cl, cla_handle h) {
		auto r = std::make_shared<CompressedMatrixBlock>(rl, cl);
		r->handle = h;
		r->deviceOnly = true;
		r->overlappingColGroups = true;
		return r;
	}
	bool isDeviceOnly() const { return deviceOnly; }
	void allocateColGroupList(std::vector<AColGroupPtr> groups) {
		releaseDevice();
		deviceOnly = false;
		for(const auto& g : groups) {
			if(g == nullptr) throw DMLCompressionException("Invalid null column group");
			for(int c : g->getColIndices())
				if(c < 0 || c >= clen) throw DMLCompressionException("Invalid column index " + std::to_string(c) + " in column group");
		}
		colGroups = std::move(groups);
	}
	void allocateColGroup(AColGroupPtr g) { allocateColGroupList({std::move(g)}); }
	const std::vector<AColGroupPtr>& getColGroups() const { return colGroups; }
	bool isOverlapping() const { return (deviceOnly || colGroups.size() != 1) && overlappingColGroups; }
	void setOverlapping(bool o) { overlappingColGroups = o; }
	bool isEmpty() const override {
		if(deviceOnly) return rlen == 0 || clen == 0;
		if(rlen == 0 || clen == 0 || colGroups.empty()) return true;
		for(const auto& g : colGroups)
			if(g->getCompType() != CompressionType::EMPTY) return false;
		return true;
	}

	// The device copy of the block, uploaded on first use and kept until the block dies
	// or its groups change.
	cla_handle hipHandle() {
		if(handle != nullptr) return handle;
		ensureDevice();
		cla_handle h = cla_block_create(rlen, clen);
		if(h == nullptr) throw DMLRuntimeException(std::string("cla_block_create: ") + cla_last_error());
		try {
			for(const auto& g : colGroups) g->upload(h);
			checkNative(cla_block_finalize(h), "cla_block_finalize");
		}
		catch(...) {
			cla_block_free(h);
			throw;
		}
		return handle = h;
	}
	void releaseDevice() {
		if(handle != nullptr) cla_block_free(handle);
		handle = nullptr;
	}

	MatrixBlock decompress(int k = 1);
	MatrixBlock aggregateBinaryOperations(MatrixBlock& m1, MatrixBlock& m2, int k = 1, bool transposeLeft = false, bool transposeRight = false);
	MatrixBlock transposeSelfMatrixMultOperations(MMTSJType tstype, int k = 1);
	MatrixBlock chainMatrixMultOperations(const MatrixBlock& v, const MatrixBlock* w, ChainType ctype, int k = 1);

private:
	std::vector<AColGroupPtr> colGroups;
	bool overlappingColGroups = false;
	bool deviceOnly = false;
	cla_handle handle = nullptr;
};

// ------------------------------------------------------------------ drivers
namespace lib {

struct CLALibDecompress {
	static MatrixBlock decompress(CompressedMatrixBlock& cmb, int /*k*/) {
		MatrixBlock ret(cmb.getNumRows(), cmb.getNumColumns());
		if(cmb.isEmpty()) return ret;
		ret.setNonZeros(checkNative(cla_decompress(cmb.hipHandle(), ret.getDenseBlockValues()), "decompress"));
		return ret;
	}
};

// CLALibCompAgg.aggregateUnary (C/lib/CLALibCompAgg.java:78-127) for sum, sumSq, min, max in the
// three directions of the reference's index functions (ReduceAll, ReduceCol = per row,
// ReduceRow = per column). Where the reference decompresses and aggregates (overlapping blocks
// for all but sums, :220-232), the library does the same on the device, chunk of rows by chunk of rows.
enum class AggOp { SUM = CLA_AGG_SUM, SUMSQ = CLA_AGG_SUMSQ, MIN = CLA_AGG_MIN, MAX = CLA_AGG_MAX };
enum class AggDir { ReduceAll = CLA_AGG_ALL, ReduceCol = CLA_AGG_ROW, ReduceRow = CLA_AGG_COL };

struct CLALibCompAgg {
	static MatrixBlock aggregateUnary(CompressedMatrixBlock& m, AggOp op, AggDir dir, int /*k*/) {
		const int rr = dir == AggDir::ReduceCol ? m.getNumRows() : 1;
		const int rc = dir == AggDir::ReduceRow ? m.getNumColumns() : 1;
		MatrixBlock ret(rr, rc);
		if(m.getNumRows() == 0 || m.getNumColumns() == 0) return ret;
		const int64_t nnz = cla_aggregate(m.hipHandle(), (int32_t) op, (int32_t) dir, ret.getDenseBlockValues());
		if(nnz == -CLA_ERR_UNSUPPORTED) throw NotImplementedException(std::string("aggregateUnary: ") + cla_last_error());
		ret.setNonZeros(checkNative(nnz, "aggregateUnary"));
		return ret;
	}
};

struct CLALibRightMultBy {
	// ret = m1 %*% m2 (dense result; the overlapping compressed result of the reference's
	// allowOverlap = true branch is not produced here).
	static MatrixBlock rightMultByMatrix(CompressedMatrixBlock& m1, MatrixBlock& m2, int k, bool allowOverlap = false) {
		try {
			const int rr = m1.getNumRows(), rc = m2.getNumColumns();
			if(m1.getNumColumns() != m2.getNumRows())
				throw DMLRuntimeException("Dimensions do not match for matrix multiplication (" + std::to_string(m1.getNumColumns()) +
					"!=" + std::to_string(m2.getNumRows()) + ").");
			if(m1.isEmpty() || m2.isEmpty()) return MatrixBlock(rr, rc);
			if(allowOverlap) throw NotImplementedException("a compressed result cannot be returned by value: use rightMultByMatrixOverlapping");
			MatrixBlock dense2;
			MatrixBlock* rhs = &m2;
			if(m2.isCompressed()) {
				dense2 = CLALibDecompress::decompress(static_cast<CompressedMatrixBlock&>(m2), k);
				rhs = &dense2;
			}
			MatrixBlock ret(rr, rc);
			ret.setNonZeros(checkNative(cla_rmm(m1.hipHandle(), rhs->getDenseBlockValues(), rc, ret.getDenseBlockValues()), "RMM"));
			return ret;
		}
		catch(const NotImplementedException&) { throw; }
		catch(const std::exception& e) {
			throw DMLRuntimeException(std::string("Failed Right MM: ") + e.what());
		}
	}
};

// The allowOverlap = true branch of rightMultByMatrix (RMMOverlapping, CLALibRightMultBy.java:157-201):
// the product stays compressed, its groups share the index structures of m1's groups.
inline std::shared_ptr<CompressedMatrixBlock> rightMultByMatrixOverlapping(CompressedMatrixBlock& m1, MatrixBlock& m2, int k) {
	if(m1.getNumColumns() != m2.getNumRows())
		throw DMLRuntimeException("Dimensions do not match for matrix multiplication (" + std::to_string(m1.getNumColumns()) + "!=" +
			std::to_string(m2.getNumRows()) + ").");
	MatrixBlock dense2;
	MatrixBlock* rhs = &m2;
	if(m2.isCompressed()) {
		dense2 = CLALibDecompress::decompress(static_cast<CompressedMatrixBlock&>(m2), k);
		rhs = &dense2;
	}
	cla_handle h = cla_rmm_overlapping(m1.hipHandle(), rhs->getDenseBlockValues(), m2.getNumColumns());
	if(h == nullptr) throw NotImplementedException(std::string("RMMOverlapping: ") + cla_last_error());
	return CompressedMatrixBlock::adoptDevice(m1.getNumRows(), m2.getNumColumns(), h);
}

struct CLALibLeftMultBy {
	// ret = left %*% right
	static MatrixBlock leftMultByMatrix(CompressedMatrixBlock& right, MatrixBlock& left, int k) {
		try {
			if(left.getNumColumns() != right.getNumRows())
				throw DMLRuntimeException("Dimensions do not match for matrix multiplication (" + std::to_string(left.getNumColumns()) +
					"!=" + std::to_string(right.getNumRows()) + ").");
			if(left.isEmpty() || right.isEmpty()) return MatrixBlock(left.getNumRows(), right.getNumColumns());
			MatrixBlock denseL;
			MatrixBlock* lhs = &left;
			if(left.isCompressed()) {
				denseL = CLALibDecompress::decompress(static_cast<CompressedMatrixBlock&>(left), k);
				lhs = &denseL;
			}
			MatrixBlock ret(left.getNumRows(), right.getNumColumns());
			ret.setNonZeros(checkNative(cla_lmm(right.hipHandle(), lhs->getDenseBlockValues(), left.getNumRows(), ret.getDenseBlockValues()), "LMM"));
			return ret;
		}
		catch(const NotImplementedException&) { throw; }
		catch(const std::exception& e) {
			throw DMLCompressionException(std::string("Failed CLA LMM: ") + e.what());
		}
	}
	// ret = t(left) %*% right
	static MatrixBlock leftMultByMatrixTransposed(CompressedMatrixBlock& right, MatrixBlock& left, int k) {
		if(left.getNumRows() != right.getNumRows())
			throw DMLCompressionException("Failed CLA LMM: dimensions do not match for transposed left multiplication");
		if(left.isEmpty() || right.isEmpty()) return MatrixBlock(left.getNumColumns(), right.getNumColumns());
		MatrixBlock denseL;
		const MatrixBlock* src = &left;
		if(left.isCompressed()) {
			// both sides compressed (CLALibLeftMultBy.java:100-112): every left group meets every right group on
			// the device; shapes that path does not take decompress the left side, as the non-compressed overload does
			CompressedMatrixBlock& cl = static_cast<CompressedMatrixBlock&>(left);
			MatrixBlock ret(left.getNumColumns(), right.getNumColumns());
			const int64_t nnz = cla_lmm_compressed(right.hipHandle(), cl.hipHandle(), ret.getDenseBlockValues());
			if(nnz != -CLA_ERR_UNSUPPORTED) {
				try {
					ret.setNonZeros(checkNative(nnz, "Compressed Transposed LMM"));
				}
				catch(const std::exception& e) {
					throw DMLCompressionException(std::string("Failed CLA Compressed Transposed LMM: ") + e.what());
				}
				return ret;
			}
			denseL = CLALibDecompress::decompress(cl, k);
			src = &denseL;
		}
		MatrixBlock t = src->transpose();
		return leftMultByMatrix(right, t, k);
	}
};

struct CLALibTSMM {
	// ret = t(cmb) %*% cmb
	static MatrixBlock leftMultByTransposeSelf(CompressedMatrixBlock& cmb, int /*k*/) {
		const int n = cmb.getNumColumns();
		MatrixBlock ret(n, n);
		if(cmb.isEmpty()) return ret;
		ret.setNonZeros(checkNative(cla_tsmm(cmb.hipHandle(), ret.getDenseBlockValues()), "TSMM"));
		return ret;
	}
};

struct CLALibMMChain {
	// t(x) %*% (x %*% v), t(x) %*% (w * (x %*% v)) or t(x) %*% ((x %*% v) - w); v and w are column vectors.
	static MatrixBlock mmChain(CompressedMatrixBlock& x, const MatrixBlock& v, const MatrixBlock* w, ChainType ctype, int k) {
		if(ctype == ChainType::NONE) throw DMLRuntimeException("Invalid mmchain type 'NONE'.");
		if(v.getNumColumns() != 1 || v.getNumRows() != x.getNumColumns())
			throw DMLRuntimeException("Dimensions mismatch on mmchain operation (v is not a vector of the number of columns of x)");
		if(ctype != ChainType::XtXv && (w == nullptr || w->getNumColumns() != 1 || w->getNumRows() != x.getNumRows()))
			throw DMLRuntimeException("Dimensions mismatch on mmchain operation (w is not a vector of the number of rows of x)");
		MatrixBlock out(x.getNumColumns(), 1);
		if(x.isEmpty()) return out;
		// all three chain types run on the device: X %*% v, then * w (XtwXv) or - w (XtXvy), then t(.) %*% X
		const double* wp = ctype == ChainType::XtXv ? nullptr : w->getDenseBlockValues();
		const int ct = ctype == ChainType::XtXv ? 0 : ctype == ChainType::XtwXv ? 1 : 2;
		out.setNonZeros(checkNative(cla_mmchain(x.hipHandle(), v.getDenseBlockValues(), wp, ct, out.getDenseBlockValues()), "MMChain"));
		return out;
	}
};

struct CLALibMatrixMult {
	// m1 %*% m2 with optional logical transposes; exactly one side compressed
	// (CLALibMatrixMult.java:42-94: a transposed compressed side swaps the operands,
	// t(t(m2) %*% t(m1)), a transposed dense side is transposed physically).
	static MatrixBlock matrixMultiply(MatrixBlock& m1, MatrixBlock& m2, int k, bool transposeLeft = false, bool transposeRight = false) {
		MatrixBlock* a = &m1;
		MatrixBlock* b = &m2;
		if(a->isCompressed() && b->isCompressed()) {
			// doubleCompressedMatrixMultiply (CLALibMatrixMult.java:95-124): t(m1) %*% m2 stays compressed on both
			// sides (the wider block takes the right-hand role, the result is transposed back); the other
			// combinations decompress the right-hand side
			auto& ca = static_cast<CompressedMatrixBlock&>(*a);
			auto& cb = static_cast<CompressedMatrixBlock&>(*b);
			if(transposeLeft && !transposeRight) { // t(m1) %*% m2
				if(ca.getNumColumns() > cb.getNumColumns())
					return CLALibLeftMultBy::leftMultByMatrixTransposed(ca, cb, k).transpose();
				return CLALibLeftMultBy::leftMultByMatrixTransposed(cb, ca, k);
			}
			MatrixBlock d = CLALibDecompress::decompress(cb, k);
			return matrixMultiply(m1, d, k, transposeLeft, transposeRight);
		}
		bool transposeOutput = false;
		MatrixBlock tmpT;
		if(transposeLeft || transposeRight) {
			if((a->isCompressed() && transposeLeft) || (b->isCompressed() && transposeRight)) {
				transposeOutput = true;
				std::swap(a, b);
				const bool tmpLeft = transposeLeft;
				transposeLeft = !transposeRight;
				transposeRight = !tmpLeft;
			}
			if(!a->isCompressed() && transposeLeft) {
				tmpT = a->transpose();
				a = &tmpT;
				transposeLeft = false;
			}
			else if(!b->isCompressed() && transposeRight) {
				tmpT = b->transpose();
				b = &tmpT;
				transposeRight = false;
			}
		}
		const bool right = a->isCompressed();
		if(!right && !b->isCompressed()) throw DMLRuntimeException("Invalid call to compressed matrix multiply without a compressed side");
		MatrixBlock ret = right ? CLALibRightMultBy::rightMultByMatrix(static_cast<CompressedMatrixBlock&>(*a), *b, k)
		                        : CLALibLeftMultBy::leftMultByMatrix(static_cast<CompressedMatrixBlock&>(*b), *a, k);
		return transposeOutput ? ret.transpose() : ret;
	}
};

} // namespace lib

inline MatrixBlock CompressedMatrixBlock::decompress(int k) { return lib::CLALibDecompress::decompress(*this, k); }
inline MatrixBlock CompressedMatrixBlock::aggregateBinaryOperations(MatrixBlock& m1, MatrixBlock& m2, int k, bool tl, bool tr) {
	const int inner1 = tl ? m1.getNumRows() : m1.getNumColumns();
	const int inner2 = tr ? m2.getNumColumns() : m2.getNumRows();
	if(inner1 != inner2)
		throw DMLRuntimeException("Dimensions do not match for matrix multiplication (" + std::to_string(inner1) + "!=" + std::to_string(inner2) + ").");
	return lib::CLALibMatrixMult::matrixMultiply(m1, m2, k, tl, tr);
}
inline MatrixBlock CompressedMatrixBlock::transposeSelfMatrixMultOperations(MMTSJType tstype, int k) {
	if(tstype == MMTSJType::LEFT) return lib::CLALibTSMM::leftMultByTransposeSelf(*this, k);
	throw DMLRuntimeException(std::string("Invalid MMTSJ type '") + (tstype == MMTSJType::RIGHT ? "RIGHT" : "NONE") + "'.");
}
inline MatrixBlock CompressedMatrixBlock::chainMatrixMultOperations(const MatrixBlock& v, const MatrixBlock* w, ChainType ctype, int k) {
	return lib::CLALibMMChain::mmChain(*this, v, w, ctype, k);
}

} // namespace compress
} // namespace sysds
