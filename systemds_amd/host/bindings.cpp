// Python view of the C++ host layer (cla_host.hpp), used by the tests so that they
// read like the reference's own component tests (src/test/java/org/apache/sysds/test/
// component/compress/): build column groups with the factories, put them into a
// CompressedMatrixBlock, call the CLALib* drivers, compare with the dense product.
#include "cla_host.hpp"
#include "cla_wire.hpp"

#include <pybind11/numpy.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

namespace py = pybind11;
using namespace sysds;
using namespace sysds::compress;
using namespace sysds::compress::lib;

using DArr = py::array_t<double, py::array::c_style | py::array::forcecast>;
using IArr = py::array_t<int32_t, py::array::c_style | py::array::forcecast>;

static std::vector<double> to_vec(const DArr& a) { return std::vector<double>(a.data(), a.data() + a.size()); }
static std::vector<int32_t> to_ivec(const IArr& a) { return std::vector<int32_t>(a.data(), a.data() + a.size()); }

static std::shared_ptr<MatrixBlock> mb_from_array(const DArr& a) {
	if(a.ndim() != 2) throw DMLRuntimeException("MatrixBlock needs a 2-d array");
	return std::make_shared<MatrixBlock>((int) a.shape(0), (int) a.shape(1), to_vec(a));
}

static py::array_t<double> mb_to_array(const MatrixBlock& m) {
	py::array_t<double> out({(py::ssize_t) m.getNumRows(), (py::ssize_t) m.getNumColumns()});
	if(m.isAllocated()) std::copy(m.getDenseBlockValues(), m.getDenseBlockValues() + (size_t) m.getNumRows() * m.getNumColumns(), out.mutable_data());
	else std::fill(out.mutable_data(), out.mutable_data() + out.size(), 0.0);
	return out;
}

PYBIND11_MODULE(_clahost, m) {
	m.doc() = "C++ host layer of the compressed multiply path (mirrors org.apache.sysds.runtime.compress)";

	auto eRt = py::register_exception<DMLRuntimeException>(m, "DMLRuntimeException", PyExc_RuntimeError);
	auto eCo = py::register_exception<DMLCompressionException>(m, "DMLCompressionException", eRt.ptr());
	py::register_exception<NotImplementedException>(m, "NotImplementedException", eRt.ptr());
	(void) eCo;

	py::enum_<CompressionType>(m, "CompressionType")
		.value("DDC", CompressionType::DDC).value("SDC", CompressionType::SDC).value("SDCZeros", CompressionType::SDCZeros)
		.value("RLE", CompressionType::RLE).value("UNCOMPRESSED", CompressionType::UNCOMPRESSED)
		.value("CONST", CompressionType::CONST).value("EMPTY", CompressionType::EMPTY);
	py::enum_<MMTSJType>(m, "MMTSJType").value("NONE", MMTSJType::NONE).value("LEFT", MMTSJType::LEFT).value("RIGHT", MMTSJType::RIGHT);
	py::enum_<ChainType>(m, "ChainType").value("XtXv", ChainType::XtXv).value("XtwXv", ChainType::XtwXv)
		.value("XtXvy", ChainType::XtXvy).value("NONE", ChainType::NONE);
	py::enum_<MAP_TYPE>(m, "MAP_TYPE").value("ZERO", MAP_TYPE::ZERO).value("BIT", MAP_TYPE::BIT).value("UBYTE", MAP_TYPE::UBYTE)
		.value("BYTE", MAP_TYPE::BYTE).value("CHAR", MAP_TYPE::CHAR).value("CHAR_BYTE", MAP_TYPE::CHAR_BYTE).value("INT", MAP_TYPE::INT);
	py::enum_<OFF_TYPE>(m, "OFF_TYPE").value("BYTE", OFF_TYPE::BYTE).value("CHAR", OFF_TYPE::CHAR);

	py::class_<MatrixBlock, std::shared_ptr<MatrixBlock>>(m, "MatrixBlock")
		.def(py::init([](int rl, int cl) { return std::make_shared<MatrixBlock>(rl, cl); }))
		.def(py::init(&mb_from_array))
		.def("getNumRows", &MatrixBlock::getNumRows)
		.def("getNumColumns", &MatrixBlock::getNumColumns)
		.def("getNonZeros", &MatrixBlock::getNonZeros)
		.def("recomputeNonZeros", &MatrixBlock::recomputeNonZeros)
		.def("isEmpty", &MatrixBlock::isEmpty)
		.def("isCompressed", &MatrixBlock::isCompressed)
		.def("get", &MatrixBlock::get)
		.def("transpose", &MatrixBlock::transpose)
		.def("toArray", &mb_to_array);

	py::class_<AMapToData, std::shared_ptr<AMapToData>>(m, "AMapToData")
		.def("getUnique", &AMapToData::getUnique)
		.def("size", &AMapToData::size)
		.def("getType", &AMapToData::getType)
		.def("codeWidth", &AMapToData::codeWidth)
		.def("getIndex", &AMapToData::getIndex)
		.def("set", &AMapToData::set)
		.def("fill", &AMapToData::fill)
		.def("getCounts", &AMapToData::getCounts)
		.def("verify", &AMapToData::verify);
	py::class_<MapToFactory>(m, "MapToFactory")
		.def_static("getType", &MapToFactory::getType)
		.def_static("create", [](int size, int unique) { return MapToFactory::create(size, unique); })
		.def_static("create", [](int unique, const IArr& values) { return MapToFactory::create(unique, to_ivec(values)); });

	py::class_<AIterator>(m, "AIterator")
		.def("value", &AIterator::value)
		.def("next", &AIterator::next)
		.def("getDataIndex", &AIterator::getDataIndex)
		.def("getOffsetsIndex", &AIterator::getOffsetsIndex)
		.def("isNotOver", &AIterator::isNotOver)
		.def("skipTo", &AIterator::skipTo);
	py::class_<AOffset, std::shared_ptr<AOffset>>(m, "AOffset")
		.def("getType", &AOffset::getType)
		.def("getOffsetToFirst", &AOffset::getOffsetToFirst)
		.def("getOffsetToLast", &AOffset::getOffsetToLast)
		.def("getSize", &AOffset::getSize)
		.def("getLength", &AOffset::getLength)
		.def("getIterator", &AOffset::getIterator, py::keep_alive<0, 1>())
		.def("toArray", &AOffset::toArray)
		.def("verify", &AOffset::verify)
		.def("rawDeltas", [](const AOffset& o) {
			std::vector<int> d((size_t) o.getLength());
			for(int64_t i = 0; i < o.getLength(); i++) d[(size_t) i] = o.delta(i);
			return d;
		});
	py::class_<OffsetFactory>(m, "OffsetFactory")
		.def_static("createOffset", [](const IArr& idx) { return OffsetFactory::createOffset(to_ivec(idx)); })
		.def_static("createOffset", [](const IArr& idx, OFF_TYPE t) { return OffsetFactory::createOffset(to_ivec(idx), t); })
		.def_static("correctionByte", &OffsetFactory::correctionByte)
		.def_static("correctionChar", &OffsetFactory::correctionChar);

	py::class_<Dictionary, std::shared_ptr<Dictionary>>(m, "Dictionary")
		.def_static("create", [](const DArr& v) { return Dictionary::create(to_vec(v)); })
		.def("getNumberOfValues", &Dictionary::getNumberOfValues)
		.def("getValues", [](const Dictionary& d) { return py::array_t<double>((py::ssize_t) d.getValues().size(), d.getValues().data()); });

	py::class_<AColGroup, AColGroupPtr>(m, "AColGroup")
		.def("getColIndices", &AColGroup::getColIndices)
		.def("getNumCols", &AColGroup::getNumCols)
		.def("getNumValues", &AColGroup::getNumValues)
		.def("getDictionary", &AColGroup::getDictionary)
		.def("getCompType", &AColGroup::getCompType);
	py::class_<ColGroupEmpty, AColGroup, std::shared_ptr<ColGroupEmpty>>(m, "ColGroupEmpty")
		.def(py::init([](const IArr& c) { return std::make_shared<ColGroupEmpty>(ColIndexFactory::create(to_ivec(c))); }));
	py::class_<ColGroupConst, AColGroup, std::shared_ptr<ColGroupConst>>(m, "ColGroupConst")
		.def_static("create", [](const IArr& c, const DArr& v) { return ColGroupConst::create(ColIndexFactory::create(to_ivec(c)), to_vec(v)); })
		.def_static("create", [](const IArr& c, double v) { return ColGroupConst::create(ColIndexFactory::create(to_ivec(c)), v); });
	py::class_<ColGroupDDC, AColGroup, std::shared_ptr<ColGroupDDC>>(m, "ColGroupDDC")
		.def_static("create", [](const IArr& c, std::shared_ptr<Dictionary> d, std::shared_ptr<AMapToData> map) {
			return ColGroupDDC::create(ColIndexFactory::create(to_ivec(c)), std::move(d), std::move(map));
		})
		.def("getMapToData", &ColGroupDDC::getMapToData)
		.def("getCounts", &ColGroupDDC::getCounts);
	py::class_<ColGroupSDCBase, AColGroup, std::shared_ptr<ColGroupSDCBase>>(m, "ColGroupSDCBase")
		.def("getOffsets", &ColGroupSDCBase::getOffsets)
		.def("getMapToData", &ColGroupSDCBase::getMapToData)
		.def("getDefaultTuple", &ColGroupSDCBase::getDefaultTuple);
	py::class_<ColGroupSDCZeros, ColGroupSDCBase, std::shared_ptr<ColGroupSDCZeros>>(m, "ColGroupSDCZeros")
		.def_static("create", [](const IArr& c, int nRows, std::shared_ptr<Dictionary> d, std::shared_ptr<AOffset> o, std::shared_ptr<AMapToData> map) {
			return ColGroupSDCZeros::create(ColIndexFactory::create(to_ivec(c)), nRows, std::move(d), std::move(o), std::move(map));
		});
	py::class_<ColGroupSDC, ColGroupSDCBase, std::shared_ptr<ColGroupSDC>>(m, "ColGroupSDC")
		.def_static("create", [](const IArr& c, int nRows, std::shared_ptr<Dictionary> d, const DArr& def, std::shared_ptr<AOffset> o,
			std::shared_ptr<AMapToData> map) {
			return ColGroupSDC::create(ColIndexFactory::create(to_ivec(c)), nRows, std::move(d), to_vec(def), std::move(o), std::move(map));
		});
	py::class_<ColGroupRLE, AColGroup, std::shared_ptr<ColGroupRLE>>(m, "ColGroupRLE")
		.def_static("create", [](const IArr& c, int nRows, std::shared_ptr<Dictionary> d, const std::vector<uint16_t>& data, const IArr& ptr) {
			return ColGroupRLE::create(ColIndexFactory::create(to_ivec(c)), nRows, std::move(d), data, to_ivec(ptr));
		})
		.def_static("genRLEBitmap", [](const std::vector<std::vector<int32_t>>& rows) {
			std::vector<uint16_t> data;
			std::vector<int32_t> ptr;
			ColGroupRLE::genRLEBitmap(rows, data, ptr);
			return py::make_tuple(data, ptr);
		})
		.def("getData", &ColGroupRLE::getData)
		.def("getPtr", &ColGroupRLE::getPtr);
	py::class_<ColGroupUncompressed, AColGroup, std::shared_ptr<ColGroupUncompressed>>(m, "ColGroupUncompressed")
		.def_static("create", [](std::shared_ptr<MatrixBlock> mb, const IArr& c) {
			return ColGroupUncompressed::create(std::move(mb), ColIndexFactory::create(to_ivec(c)));
		})
		.def_static("create", [](std::shared_ptr<MatrixBlock> mb) { return ColGroupUncompressed::create(std::move(mb)); })
		.def("getData", &ColGroupUncompressed::getData);

	py::class_<CompressedMatrixBlock, MatrixBlock, std::shared_ptr<CompressedMatrixBlock>>(m, "CompressedMatrixBlock")
		.def(py::init([](int rl, int cl) { return std::make_shared<CompressedMatrixBlock>(rl, cl); }))
		.def("allocateColGroupList", &CompressedMatrixBlock::allocateColGroupList)
		.def("allocateColGroup", &CompressedMatrixBlock::allocateColGroup)
		.def("getColGroups", &CompressedMatrixBlock::getColGroups)
		.def("isOverlapping", &CompressedMatrixBlock::isOverlapping)
		.def("setOverlapping", &CompressedMatrixBlock::setOverlapping)
		.def("releaseDevice", &CompressedMatrixBlock::releaseDevice)
		.def("isDeviceOnly", &CompressedMatrixBlock::isDeviceOnly)
		.def("decompress", &CompressedMatrixBlock::decompress, py::arg("k") = 1)
		.def("aggregateBinaryOperations", &CompressedMatrixBlock::aggregateBinaryOperations, py::arg("m1"), py::arg("m2"), py::arg("k") = 1,
			py::arg("transposeLeft") = false, py::arg("transposeRight") = false)
		.def("transposeSelfMatrixMultOperations", &CompressedMatrixBlock::transposeSelfMatrixMultOperations, py::arg("tstype"), py::arg("k") = 1)
		.def("chainMatrixMultOperations", [](CompressedMatrixBlock& x, const MatrixBlock& v, const MatrixBlock* w, ChainType ct, int k) {
			return x.chainMatrixMultOperations(v, w, ct, k);
		}, py::arg("v"), py::arg("w").none(true), py::arg("ctype"), py::arg("k") = 1);

	py::class_<CLALibRightMultBy>(m, "CLALibRightMultBy")
		.def_static("rightMultByMatrix", &CLALibRightMultBy::rightMultByMatrix, py::arg("m1"), py::arg("m2"), py::arg("k") = 1,
			py::arg("allowOverlap") = false);
	m.def("rightMultByMatrixOverlapping", &rightMultByMatrixOverlapping, py::arg("m1"), py::arg("m2"), py::arg("k") = 1);
	py::class_<CLALibLeftMultBy>(m, "CLALibLeftMultBy")
		.def_static("leftMultByMatrix", &CLALibLeftMultBy::leftMultByMatrix, py::arg("right"), py::arg("left"), py::arg("k") = 1)
		.def_static("leftMultByMatrixTransposed", &CLALibLeftMultBy::leftMultByMatrixTransposed, py::arg("right"), py::arg("left"), py::arg("k") = 1);
	py::class_<CLALibTSMM>(m, "CLALibTSMM")
		.def_static("leftMultByTransposeSelf", &CLALibTSMM::leftMultByTransposeSelf, py::arg("cmb"), py::arg("k") = 1);
	py::enum_<AggOp>(m, "AggOp").value("SUM", AggOp::SUM).value("SUMSQ", AggOp::SUMSQ).value("MIN", AggOp::MIN).value("MAX", AggOp::MAX);
	py::enum_<AggDir>(m, "AggDir").value("ReduceAll", AggDir::ReduceAll).value("ReduceCol", AggDir::ReduceCol).value("ReduceRow", AggDir::ReduceRow);
	py::class_<CLALibCompAgg>(m, "CLALibCompAgg")
		.def_static("aggregateUnary", &CLALibCompAgg::aggregateUnary, py::arg("m"), py::arg("op"), py::arg("dir"), py::arg("k") = 1);
	py::class_<CLALibMMChain>(m, "CLALibMMChain")
		.def_static("mmChain", [](CompressedMatrixBlock& x, const MatrixBlock& v, const MatrixBlock* w, ChainType ct, int k) {
			return CLALibMMChain::mmChain(x, v, w, ct, k);
		}, py::arg("x"), py::arg("v"), py::arg("w").none(true), py::arg("ctype"), py::arg("k") = 1);
	py::class_<CLALibMatrixMult>(m, "CLALibMatrixMult")
		.def_static("matrixMultiply", &CLALibMatrixMult::matrixMultiply, py::arg("m1"), py::arg("m2"), py::arg("k") = 1,
			py::arg("transposeLeft") = false, py::arg("transposeRight") = false);
	// CompressedMatrixBlock.read / write on byte strings
	m.def("readCompressedMatrixBlock", [](const py::bytes& b) {
		const std::string s = b; // copies; the block owns its data afterwards
		return io::readCompressedMatrixBlock((const uint8_t*) s.data(), s.size());
	});
	m.def("writeCompressedMatrixBlock", [](const CompressedMatrixBlock& cmb) {
		const std::vector<uint8_t> v = io::writeCompressedMatrixBlock(cmb);
		return py::bytes((const char*) v.data(), v.size());
	});
	py::class_<CLALibDecompress>(m, "CLALibDecompress")
		.def_static("decompress", &CLALibDecompress::decompress, py::arg("cmb"), py::arg("k") = 1);
}
