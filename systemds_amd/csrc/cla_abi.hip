// C ABI of libclahip.so (see include/cla_hip.h): block construction, finalize,
// host/device entry points of the multiply drivers. Host-side logic only; the
// kernels live in k_*.hip.
#include "../../include/cla_hip.h"
#include "cla_device.hpp"
#include <algorithm>
#include <cstdarg>
#include <cstring>
#include <map>
#include <mutex>
#include <unordered_set>
#include <new>
#include <stdexcept>

// No exception may cross the C ABI (a JNI or FFM caller would abort the JVM instead of falling
// back): every exported function runs its body between these two.
#define CLA_TRY try {
#define CLA_CATCH_BODY(onAlloc, onOther)                                                          \
	}                                                                                             \
	catch(const std::bad_alloc&) { cla::set_error("host memory allocation failed"); onAlloc; }   \
	catch(const std::exception& e) { cla::set_error("unexpected exception: %s", e.what()); onOther; } \
	catch(...) { cla::set_error("unexpected exception"); onOther; }
#define CLA_CATCH_CODE(T) CLA_CATCH_BODY(return (T) -CLA_ERR_DEVICE, return (T) -CLA_ERR_INVALID)
#define CLA_CATCH_NULL CLA_CATCH_BODY(return nullptr, return nullptr)
#define CLA_CATCH_VOID CLA_CATCH_BODY(return, return)

// Workspace of the entry point that allocates nothing (cla_rmm_dev_noalloc): the non-zero counter in the
// first 256 bytes, then the pre-aggregated tables. One copy per GPU, held until the process ends. In host
// code the name is only a handle for hipGetSymbolAddress: kernels get the address looked up at cla_init.
constexpr size_t CLA_SCRATCH_BYTES = (size_t) 4 << 20;
static __device__ __align__(256) unsigned char scratch[CLA_SCRATCH_BYTES];

namespace cla {

constexpr int MAX_DEVICES = 64;
static unsigned char* g_scratchPtr[MAX_DEVICES] = {}; // device address of `scratch` per device (set at cla_init)
static std::mutex g_scratchMu[MAX_DEVICES];           // one call at a time works in a device's copy of `scratch`

static thread_local char t_err[1024] = "";
int g_ldsPerBlock = 65536;
int g_numCU = 256;
static int g_device = -1;
static hipDeviceProp_t g_prop;
static std::mutex g_initMu;

void set_error(const char* fmt, ...) {
	va_list ap;
	va_start(ap, fmt);
	vsnprintf(t_err, sizeof(t_err), fmt, ap);
	va_end(ap);
}

Prof::Prof(cla_block* blk, const char* name, long grid, long block, long lds, double algoBytes) : b(blk) {
	KernelStat k;
	k.name = name; k.grid = grid; k.block = block; k.lds = lds; k.algoBytes = algoBytes;
	if(b->profile && hipEventCreate(&k.e0) == hipSuccess && hipEventCreate(&k.e1) == hipSuccess)
		(void) hipEventRecord(k.e0, b->stream);
	idx = b->lastStats.size();
	b->lastStats.push_back(k);
}

Prof::~Prof() {
	KernelStat& k = b->lastStats[idx];
	if(k.e0 && k.e1) (void) hipEventRecord(k.e1, b->stream);
}

void clear_stats(cla_block* b) {
	for(auto& k : b->lastStats) {
		if(k.e0) (void) hipEventDestroy(k.e0);
		if(k.e1) (void) hipEventDestroy(k.e1);
	}
	b->lastStats.clear();
}

int ensure_tables(cla_block* b, size_t nDoubles) {
	if(nDoubles <= b->tablesCap) return 0;
	if(b->dTables) CLA_HIP(hipFree(b->dTables));
	b->dTables = nullptr; b->tablesCap = 0;
	CLA_HIP(hipMalloc((void**) &b->dTables, nDoubles * sizeof(double)));
	b->tablesCap = nDoubles;
	return 0;
}

hipError_t allow_full_lds(const void* kernel) {
	static std::mutex mu;
	static std::unordered_set<const void*> said;
	std::lock_guard<std::mutex> lk(mu);
	if(said.count(kernel)) return hipSuccess;
	// (the kernel's static shared memory counts against the same limit)
	hipFuncAttributes fa;
	hipError_t e = hipFuncGetAttributes(&fa, kernel);
	if(e != hipSuccess) return e;
	const int room = g_ldsPerBlock - (int) fa.sharedSizeBytes;
	e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, room > 0 ? room : 0);
	if(e == hipSuccess) said.insert(kernel);
	return e;
}

int ensure_scratch(cla_block* b, size_t bytes) {
	if(bytes <= b->scratchCap) return 0;
	if(b->dScratch) CLA_HIP(hipFree(b->dScratch));
	b->dScratch = nullptr; b->scratchCap = 0;
	CLA_HIP(hipMalloc(&b->dScratch, bytes));
	b->scratchCap = bytes;
	return 0;
}

int ensure_gram_acc(cla_block* b) {
	if(b->dGramAcc != nullptr) return 0;
	const size_t bytes = sizeof(double) * std::max<size_t>((size_t) b->nCols * b->nCols, 1);
	CLA_HIP(hipMalloc((void**) &b->dGramAcc, bytes));
	CLA_HIP(hipMemset(b->dGramAcc, 0, bytes));
	return 0;
}

static int ensure_stage(double** p, size_t* cap, size_t nDoubles) {
	if(nDoubles <= *cap) return 0;
	if(*p) CLA_HIP(hipFree(*p));
	*p = nullptr; *cap = 0;
	CLA_HIP(hipMalloc((void**) p, std::max<size_t>(nDoubles, 1) * sizeof(double)));
	*cap = nDoubles;
	return 0;
}

static int upload(HostGroup& g, const void* src, size_t bytes, const void** dst) {
	void* d = nullptr;
	CLA_HIP(hipMalloc(&d, bytes + UPLOAD_SLACK));
	g.owned.push_back(d);
	CLA_HIP(hipMemset((char*) d + bytes, 1, UPLOAD_SLACK));
	if(bytes) CLA_HIP(hipMemcpy(d, src, bytes, hipMemcpyHostToDevice));
	else CLA_HIP(hipStreamSynchronize(nullptr));
	g.bytes += (int64_t) bytes;
	*dst = d;
	return 0;
}

static void free_group(HostGroup& g) {
	for(void* p : g.owned) (void) hipFree(p);
	g.owned.clear();
}

static int check_ready() {
	if(g_device < 0) {
		set_error("cla_init has not been called (or failed): no HIP device selected");
		return -CLA_ERR_STATE;
	}
	hipError_t e = hipSetDevice(g_device);
	if(e != hipSuccess) {
		set_error("hipSetDevice(%d) failed: %s", g_device, hipGetErrorString(e));
		return -CLA_ERR_DEVICE;
	}
	return 0;
}

static int check_cols(cla_block* b, const int32_t* cols, int32_t nColG) {
	if(!cols || nColG <= 0) { set_error("column group without column indexes"); return -CLA_ERR_INVALID; }
	for(int j = 0; j < nColG; j++)
		if(cols[j] < 0 || cols[j] >= b->nCols) {
			set_error("column index %d outside [0,%d)", cols[j], b->nCols);
			return -CLA_ERR_INVALID;
		}
	return 0;
}

static int check_open(cla_block* b) {
	if(!b) { set_error("null block handle"); return -CLA_ERR_INVALID; }
	if(b->poisoned) { set_error("an earlier cla_block_finalize on this block failed; free it"); return -CLA_ERR_STATE; }
	if(b->finalized) { set_error("block already finalized"); return -CLA_ERR_STATE; }
	return check_ready();
}

static int check_final(cla_block* b) {
	if(!b) { set_error("null block handle"); return -CLA_ERR_INVALID; }
	if(!b->finalized) { set_error("block not finalized"); return -CLA_ERR_STATE; }
	return check_ready();
}

static int init_group(cla_block* b, HostGroup& g, int type, const int32_t* cols, int nColG, const double* dict,
	int nVals) {
	memset(&g.d, 0, sizeof(g.d));
	g.d.type = type; g.d.nColG = nColG; g.d.nVals = nVals;
	g.cols.assign(cols, cols + nColG);
	int rc = upload(g, cols, sizeof(int32_t) * (size_t) nColG, (const void**) &g.d.cols);
	if(rc) return rc;
	if(dict) g.dict.assign(dict, dict + (size_t) nVals * nColG);
	(void) b;
	return 0;
}

static int upload_dict(HostGroup& g) {
	return upload(g, g.dict.data(), sizeof(double) * g.dict.size(), (const void**) &g.d.dict);
}

// One pair of column chunks of a block with more than 64 columns (launch_tsmm_chunked): a block of its own
// that borrows the row data.
struct SubBlock {
	cla_block* blk;
	int32_t* dColMap;   // column of `b` per column of blk (-1: padding behind the first chunk)
	int nA, nB;         // columns of the first (padding included) / second chunk
	bool writeA, writeB, crossOnly;
};

// One chunk of columns of Y %*% X on the decode kernel (launch_lmm_chunked), likewise.
struct LmmSub {
	cla_block* blk;   // null: the columns that no group covers (row sums of Y times their constants)
	int32_t* dColMap; // column of the block per column of blk
	int k;
};

int finish_finalize(cla_block* b, cla_block* arenaFrom, bool buildArena = true);
static void free_subs(cla_block* b);
static void free_lmm_subs(cla_block* b);

} // namespace cla

using namespace cla;

extern "C" {

int cla_init(int device) {
	CLA_TRY
	std::lock_guard<std::mutex> lk(g_initMu);
	int n = 0;
	hipError_t e = hipGetDeviceCount(&n);
	if(e != hipSuccess || n <= 0) {
		set_error("no HIP device visible (%s); libclahip computes on the GPU only",
			e != hipSuccess ? hipGetErrorString(e) : "device count 0");
		g_device = -1;
		return -CLA_ERR_DEVICE;
	}
	if(device < 0 || device >= n) { set_error("device %d out of range (have %d)", device, n); return -CLA_ERR_INVALID; }
	CLA_HIP(hipSetDevice(device));
	CLA_HIP(hipGetDeviceProperties(&g_prop, device));
	if(strncmp(g_prop.gcnArchName, "gfx950", 6) != 0) {
		set_error("device %d is %s; this library holds gfx950 (MI355X) code only", device, g_prop.gcnArchName);
		g_device = -1;
		return -CLA_ERR_DEVICE;
	}
	g_numCU = g_prop.multiProcessorCount;
	g_ldsPerBlock = (int) g_prop.sharedMemPerBlock;
	if(g_prop.maxSharedMemoryPerMultiProcessor > (size_t) g_ldsPerBlock)
		g_ldsPerBlock = (int) g_prop.maxSharedMemoryPerMultiProcessor;
	if(device < MAX_DEVICES && g_scratchPtr[device] == nullptr) {
		// this device's copy of the static workspace (every GPU holds its own at its own address)
		unsigned char* p = nullptr;
		CLA_HIP(hipGetSymbolAddress((void**) &p, HIP_SYMBOL(scratch)));
		g_scratchPtr[device] = p;
	}
	g_device = device;
	return 0;
	CLA_CATCH_CODE(int)
}

const char* cla_last_error(void) { return t_err; }

int cla_device_info(char* json, size_t cap) {
	CLA_TRY
	int rc = check_ready();
	if(rc) return rc;
	snprintf(json, cap,
		"{\"name\":\"%s\",\"arch\":\"%s\",\"cus\":%d,\"lds_per_block\":%zu,\"lds_per_cu\":%zu,\"hbm_bytes\":%zu,"
		"\"clock_khz\":%d,\"mem_clock_khz\":%d,\"mem_bus_bits\":%d,\"l2_bytes\":%d}",
		g_prop.name, g_prop.gcnArchName, g_prop.multiProcessorCount, g_prop.sharedMemPerBlock,
		g_prop.maxSharedMemoryPerMultiProcessor, g_prop.totalGlobalMem, g_prop.clockRate, g_prop.memoryClockRate,
		g_prop.memoryBusWidth, g_prop.l2CacheSize);
	return 0;
	CLA_CATCH_CODE(int)
}

cla_handle cla_block_create(int64_t nRows, int32_t nCols) {
	CLA_TRY
	if(check_ready()) return nullptr;
	if(nRows < 0 || nRows > 0x7fffffffLL || nCols <= 0) {
		set_error("invalid block shape %lld x %d", (long long) nRows, nCols);
		return nullptr;
	}
	static std::atomic<uint64_t> nextSerial{1};
	cla_block* b = new cla_block();
	b->serial = nextSerial.fetch_add(1);
	b->nRows = nRows;
	b->nCols = nCols;
	b->constV.assign((size_t) nCols, 0.0);
	if(hipStreamCreate(&b->stream) != hipSuccess) { set_error("hipStreamCreate failed"); delete b; return nullptr; }
	b->ownStream = true;
	if(hipMalloc((void**) &b->dCounters, 8 * sizeof(unsigned long long)) != hipSuccess ||
		hipHostMalloc((void**) &b->hCounters, 8 * sizeof(unsigned long long)) != hipSuccess) {
		set_error("allocating counters failed");
		cla_block_free(b);
		return nullptr;
	}
	if(hipMemset(b->dCounters, 0, 8 * sizeof(unsigned long long)) != hipSuccess) {
		set_error("clearing counters failed");
		cla_block_free(b);
		return nullptr;
	}
	return b;
	CLA_CATCH_NULL
}

void cla_block_free(cla_handle b) {
	CLA_TRY
	if(!b) return;
	if(b->refs.fetch_sub(1) > 1) return; // blocks made from this one still use its streams
	cla_block* parent = b->parent;
	if(b->joint) { cla_block_free(b->joint); b->joint = nullptr; }
	free_subs(b);
	free_lmm_subs(b);
	if(g_device >= 0) (void) hipSetDevice(g_device);
	if(b->stream) (void) hipStreamSynchronize(b->stream);
	clear_stats(b);
	for(auto& g : b->groups) free_group(g);
	if(b->dGroups) (void) hipFree(b->dGroups);
	if(b->dConstV) (void) hipFree(b->dConstV);
	if(b->dAllDict) (void) hipFree(b->dAllDict);
	if(b->dQ1Slabs) (void) hipFree(b->dQ1Slabs);
	if(b->dArena && !b->arenaShared) (void) hipFree(b->dArena);
	if(b->dTblOff) (void) hipFree(b->dTblOff);
	if(b->dTables) (void) hipFree(b->dTables);
	if(b->dStageIn) (void) hipFree(b->dStageIn);
	if(b->dStageOut) (void) hipFree(b->dStageOut);
	if(b->dScratch) (void) hipFree(b->dScratch);
	if(b->dChain) (void) hipFree(b->dChain);
	if(b->dSdcPlan) (void) hipFree(b->dSdcPlan);
	if(b->dSdcDesc) (void) hipFree(b->dSdcDesc);
	if(b->dSdcPacked) (void) hipFree(b->dSdcPacked);
	if(b->dLaneMeta) (void) hipFree(b->dLaneMeta);
	if(b->dLaneData) (void) hipFree(b->dLaneData);
	if(b->dRowsMeta) (void) hipFree(b->dRowsMeta);
	if(b->dMfPlan) (void) hipFree(b->dMfPlan);
	dec_plans_drop(b);
	if(b->dRowsData) (void) hipFree(b->dRowsData);
	if(b->dDictPad) (void) hipFree(b->dDictPad);
	if(b->dCountsAll) (void) hipFree(b->dCountsAll);
	if(b->dOnes) (void) hipFree(b->dOnes);
	for(uint8_t* p : b->expCodes)
		if(p) (void) hipFree(p);
	if(b->dCounters) (void) hipFree(b->dCounters);
	if(b->dGramAcc) (void) hipFree(b->dGramAcc);
	if(b->hCounters) (void) hipHostFree(b->hCounters);
	if(b->ownStream && b->stream) (void) hipStreamDestroy(b->stream);
	delete b;
	if(parent) cla_block_free(parent);
	CLA_CATCH_VOID
}

int cla_block_add_ddc(cla_handle b, const int32_t* cols, int32_t nColG, const double* dict, int32_t nVals,
	const void* codes, int32_t codeWidth) {
	CLA_TRY
	int rc = check_open(b);
	if(rc) return rc;
	if((rc = check_cols(b, cols, nColG))) return rc;
	if(!dict || nVals <= 0) { set_error("DDC group needs a dictionary"); return -CLA_ERR_INVALID; }
	if(codeWidth != 1 && codeWidth != 2 && codeWidth != 4) {
		set_error("unsupported map width %d (MapToByte/UByte=1, MapToChar=2, MapToInt=4)", codeWidth);
		return -CLA_ERR_UNSUPPORTED;
	}
	if(!codes && b->nRows > 0) { set_error("DDC group without codes"); return -CLA_ERR_INVALID; }
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	HostGroup g;
	if((rc = init_group(b, g, G_DDC, cols, nColG, dict, nVals)) || (rc = upload_dict(g)) ||
		(rc = upload(g, codes, (size_t) b->nRows * codeWidth, &g.d.codes))) {
		free_group(g);
		return rc;
	}
	g.d.codeWidth = codeWidth;
	b->groups.push_back(std::move(g));
	return 0;
	CLA_CATCH_CODE(int)
}

int cla_block_add_sdc(cla_handle b, const int32_t* cols, int32_t nColG, const double* dict, int32_t nVals,
	const double* defaultTuple, const void* codes, int32_t codeWidth, const void* deltas, int32_t deltaWidth,
	int64_t nDeltas, int32_t offsetToFirst, int32_t offsetToLast, int64_t nOffsets) {
	CLA_TRY
	int rc = check_open(b);
	if(rc) return rc;
	if((rc = check_cols(b, cols, nColG))) return rc;
	if(!dict || nVals <= 0) { set_error("SDC group needs a dictionary"); return -CLA_ERR_INVALID; }
	if(codeWidth != 1 && codeWidth != 2 && codeWidth != 4) {
		set_error("unsupported map width %d", codeWidth);
		return -CLA_ERR_UNSUPPORTED;
	}
	if(nOffsets < 0 || nOffsets > b->nRows || nDeltas < 0) { set_error("invalid offset list size"); return -CLA_ERR_INVALID; }
	if(nOffsets > 0 && (offsetToFirst < 0 || offsetToLast < offsetToFirst)) {
		set_error("Invalid negative offset / first %d last %d", offsetToFirst, offsetToLast);
		return -CLA_ERR_INVALID;
	}
	if(nDeltas > 0 && deltaWidth != 1 && deltaWidth != 2) {
		set_error("unsupported offset width %d (OffsetByte=1, OffsetChar=2)", deltaWidth);
		return -CLA_ERR_UNSUPPORTED;
	}
	if(nDeltas > 0 && !deltas) { set_error("offset deltas missing"); return -CLA_ERR_INVALID; }
	if(nOffsets > 0 && nDeltas < nOffsets - 1) { set_error("offset list shorter than its size"); return -CLA_ERR_INVALID; }
	if(nOffsets > 1 && !codes && nVals > 1) { set_error("SDC group without codes"); return -CLA_ERR_INVALID; }
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	HostGroup g;
	if((rc = init_group(b, g, G_SDCZ, cols, nColG, dict, nVals))) { free_group(g); return rc; }
	if(defaultTuple) {
		// ColGroupSDC.extractCommon: dictionary minus the default tuple, default into constV
		g.def.assign(defaultTuple, defaultTuple + nColG);
		for(int k = 0; k < nVals; k++)
			for(int j = 0; j < nColG; j++) g.dict[(size_t) k * nColG + j] -= defaultTuple[j];
	}
	std::vector<uint8_t> zeros;
	const void* codeSrc = codes;
	if(!codes) { zeros.assign((size_t) std::max<int64_t>(nOffsets, 1) * codeWidth, 0); codeSrc = zeros.data(); }
	if((rc = upload_dict(g)) || (rc = upload(g, codeSrc, (size_t) nOffsets * codeWidth, &g.d.codes)) ||
		(rc = upload(g, deltas, (size_t) nDeltas * (nDeltas ? deltaWidth : 1), &g.d.deltas))) {
		free_group(g);
		return rc;
	}
	g.d.codeWidth = codeWidth;
	g.d.deltaWidth = nDeltas ? deltaWidth : 1;
	g.d.nDeltas = nDeltas; g.d.nOffsets = nOffsets;
	g.d.first = nOffsets ? offsetToFirst : 0;
	g.d.last = nOffsets ? offsetToLast : -1;
	b->groups.push_back(std::move(g));
	return 0;
	CLA_CATCH_CODE(int)
}

int cla_block_add_rle(cla_handle b, const int32_t* cols, int32_t nColG, const double* dict, int32_t nVals,
	const int32_t* ptr, const uint16_t* data, int64_t nData) {
	CLA_TRY
	int rc = check_open(b);
	if(rc) return rc;
	if((rc = check_cols(b, cols, nColG))) return rc;
	if(!dict || nVals <= 0 || !ptr) { set_error("RLE group needs a dictionary and run pointers"); return -CLA_ERR_INVALID; }
	if(nData < 0 || (nData & 1) || ptr[0] != 0 || ptr[nVals] != nData) {
		set_error("RLE run array malformed (nData %lld, ptr[0] %d, ptr[nVals] %d)", (long long) nData, ptr[0], ptr[nVals]);
		return -CLA_ERR_INVALID;
	}
	// Merge the per-value run lists into one table sorted by run start
	// (rs = re + gap; re = rs + len per value, CG/ColGroupRLE.java:114-117).
	struct Run { int64_t s, e; int32_t k; };
	std::vector<Run> runs;
	runs.reserve((size_t) nData / 2);
	for(int k = 0; k < nVals; k++) {
		if(ptr[k + 1] < ptr[k] || ((ptr[k + 1] - ptr[k]) & 1)) { set_error("RLE ptr not monotone/even at value %d", k); return -CLA_ERR_INVALID; }
		int64_t rs = 0, re = 0;
		for(int p = ptr[k]; p < ptr[k + 1]; p += 2) {
			rs = re + data[p];
			re = rs + data[p + 1];
			if(re > b->nRows) { set_error("RLE run of value %d ends at %lld beyond %lld rows", k, (long long) re, (long long) b->nRows); return -CLA_ERR_INVALID; }
			if(re > rs) runs.push_back({rs, re, k});
		}
	}
	std::sort(runs.begin(), runs.end(), [](const Run& a, const Run& c) { return a.s < c.s; });
	std::vector<int32_t> runStart, runCode;
	int64_t pos = 0;
	for(const Run& r : runs) {
		if(r.s < pos) { set_error("RLE runs overlap at row %lld", (long long) r.s); return -CLA_ERR_INVALID; }
		if(r.s > pos) { runStart.push_back((int32_t) pos); runCode.push_back(-1); }
		runStart.push_back((int32_t) r.s);
		runCode.push_back(r.k);
		pos = r.e;
	}
	if(pos < b->nRows || runStart.empty()) { runStart.push_back((int32_t) pos); runCode.push_back(-1); }
	const int nRuns = (int) runCode.size();
	runStart.push_back((int32_t) b->nRows);
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	HostGroup g;
	if((rc = init_group(b, g, G_RLE, cols, nColG, dict, nVals)) || (rc = upload_dict(g)) ||
		(rc = upload(g, runStart.data(), sizeof(int32_t) * runStart.size(), (const void**) &g.d.runStart)) ||
		(rc = upload(g, runCode.data(), sizeof(int32_t) * runCode.size(), (const void**) &g.d.runCode))) {
		free_group(g);
		return rc;
	}
	g.d.nRuns = nRuns;
	b->groups.push_back(std::move(g));
	return 0;
	CLA_CATCH_CODE(int)
}

int cla_block_add_uncompressed(cla_handle b, const int32_t* cols, int32_t nColG, const double* values) {
	CLA_TRY
	int rc = check_open(b);
	if(rc) return rc;
	if((rc = check_cols(b, cols, nColG))) return rc;
	if(!values && b->nRows > 0) { set_error("uncompressed group without values"); return -CLA_ERR_INVALID; }
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	HostGroup g;
	if((rc = init_group(b, g, G_UNC, cols, nColG, nullptr, 0)) ||
		(rc = upload(g, values, sizeof(double) * (size_t) b->nRows * nColG, (const void**) &g.d.dense))) {
		free_group(g);
		return rc;
	}
	b->groups.push_back(std::move(g));
	return 0;
	CLA_CATCH_CODE(int)
}

int cla_block_add_const(cla_handle b, const int32_t* cols, int32_t nColG, const double* row) {
	CLA_TRY
	int rc = check_open(b);
	if(rc) return rc;
	if((rc = check_cols(b, cols, nColG))) return rc;
	if(!row) { set_error("const group without values"); return -CLA_ERR_INVALID; }
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	// ColGroupConst.addToCommon (CG/ColGroupConst.java:330-362)
	for(int j = 0; j < nColG; j++) b->constV[cols[j]] += row[j];
	b->hasConst = true;
	return 0;
	CLA_CATCH_CODE(int)
}

int cla_block_add_empty(cla_handle b, const int32_t* cols, int32_t nColG) {
	CLA_TRY
	int rc = check_open(b);
	if(rc) return rc;
	if((rc = check_cols(b, cols, nColG))) return rc;
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	b->hasConst = true; // CLALibUtils.shouldPreFilter is true for empty groups as well
	return 0;
	CLA_CATCH_CODE(int)
}

// Finalize changes the block as it goes (SDC defaults into the constants, acceleration structures group by
// group): a failure half way leaves it unusable, so the block is then marked and only cla_block_free takes it.
static int finalize_groups(cla_block* b) {
	int rc;
	int tblOff = 0, colOff = 0, maxVals = 0;
	for(size_t gi = 0; gi < b->groups.size(); gi++) {
		HostGroup& g = b->groups[gi];
		DGroup& G = g.d;
		G.tblOff = tblOff;
		G.colOff = colOff;
		tblOff += G.nVals;
		colOff += G.nColG;
		maxVals = std::max(maxVals, G.nVals);
		if(G.type == G_DDC || G.type == G_SDCZ) {
			int ok = 1;
			const int64_t n = G.type == G_DDC ? b->nRows : G.nOffsets;
			if((rc = launch_validate_codes(b, G.codes, G.codeWidth, n, G.nVals, &ok))) return rc;
			if(!ok) {
				set_error("group %zu holds a code >= its number of dictionary entries (%d)", gi, G.nVals);
				return -CLA_ERR_INVALID;
			}
			if(b->opt.ddcReorder && (rc = reorder_ddc_by_count(b, (int) gi))) return rc;
		}
		if(G.type == G_SDCZ) {
			if(!g.def.empty()) {
				for(int j = 0; j < G.nColG; j++) b->constV[g.cols[j]] += g.def[j];
				b->hasConst = true;
			}
			if((rc = launch_sdc_build(b, g))) return rc;
			b->hasSdc = true;
		}
		if(G.type == G_RLE) b->hasRle = true;
		if(G.type == G_UNC) b->hasUnc = true;
	}
	b->totalVals = tblOff;
	b->totalColsG = colOff;
	b->maxVals = maxVals;
	return finish_finalize(b, nullptr);
}

int cla_block_finalize(cla_handle b) {
	CLA_TRY
	int rc = check_open(b);
	if(rc) return rc;
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	b->poisoned = true; // until every step has succeeded (also when a step throws)
	if((rc = finalize_groups(b))) return rc;
	b->poisoned = false;
	return 0;
	CLA_CATCH_CODE(int)
}

} // extern "C"

namespace cla {

// Block-level part of finalize: dictionaries back to back, descriptor array, constants, table
// offsets, code arena (built, or borrowed from arenaFrom whose groups this block mirrors one to
// one; never built for a block whose code streams are borrowed, buildArena false), mat-vec slabs.
int finish_finalize(cla_block* b, cla_block* arenaFrom, bool buildArena) {
	const int maxVals = b->maxVals;
	const size_t nG = b->groups.size();
	// all dictionaries back to back in one allocation (kernels copy a slab of
	// consecutive groups' dictionaries into LDS as one contiguous range)
	{
		size_t total = 0;
		for(auto& g : b->groups) total += g.dict.size();
		b->dictNonFinite = false;
		for(auto& g : b->groups)
			for(double v : g.dict) b->dictNonFinite |= !std::isfinite(v);
		// (two doubles of padding: 16-byte copies of a dictionary range with an odd number of doubles read 8 bytes more)
		CLA_HIP(hipMalloc((void**) &b->dAllDict, sizeof(double) * (total + 2)));
		size_t off = 0;
		for(auto& g : b->groups) {
			if(g.dict.empty()) continue;
			CLA_HIP(hipMemcpy(b->dAllDict + off, g.dict.data(), sizeof(double) * g.dict.size(), hipMemcpyHostToDevice));
			void* old = const_cast<double*>(g.d.dict);
			g.owned.erase(std::remove(g.owned.begin(), g.owned.end(), old), g.owned.end());
			CLA_HIP(hipFree(old));
			g.d.dict = b->dAllDict + off;
			off += g.dict.size();
		}
	}
	std::vector<DGroup> flat(nG);
	for(size_t i = 0; i < nG; i++) flat[i] = b->groups[i].d;
	CLA_HIP(hipMalloc((void**) &b->dGroups, sizeof(DGroup) * std::max<size_t>(nG, 1)));
	if(nG) CLA_HIP(hipMemcpy(b->dGroups, flat.data(), sizeof(DGroup) * nG, hipMemcpyHostToDevice));
	CLA_HIP(hipMalloc((void**) &b->dConstV, sizeof(double) * (size_t) b->nCols));
	CLA_HIP(hipMemcpy(b->dConstV, b->constV.data(), sizeof(double) * (size_t) b->nCols, hipMemcpyHostToDevice));

	// table offsets (prefix sums of nVals) for kernels that stage tables in LDS
	{
		std::vector<int32_t> off(nG + 1, 0);
		for(size_t i = 0; i < nG; i++) off[i + 1] = off[i] + b->groups[i].d.nVals;
		CLA_HIP(hipMalloc((void**) &b->dTblOff, sizeof(int32_t) * (nG + 1)));
		CLA_HIP(hipMemcpy(b->dTblOff, off.data(), sizeof(int32_t) * (nG + 1), hipMemcpyHostToDevice));
	}

	// code arena: all groups DDC with one code width -> one allocation, uniform stride
	bool allDdc = nG > 0 && b->nRows > 0;
	const int cw = nG ? b->groups[0].d.codeWidth : 0;
	for(auto& g : b->groups)
		if(g.d.type != G_DDC || g.d.codeWidth != cw) allDdc = false;
	if(allDdc && arenaFrom != nullptr && arenaFrom->dArena != nullptr && arenaFrom->groups.size() == nG) {
		b->dArena = arenaFrom->dArena; // the descriptors already point into it
		b->arenaShared = true;
		b->arenaStride = arenaFrom->arenaStride;
		b->arenaWidth = arenaFrom->arenaWidth;
	}
	else if(allDdc && buildArena) {
		const size_t stride = (((size_t) b->nRows * cw) + 255) & ~(size_t) 255;
		CLA_HIP(hipMalloc((void**) &b->dArena, stride * nG));
		for(size_t i = 0; i < nG; i++) {
			HostGroup& g = b->groups[i];
			uint8_t* dst = b->dArena + i * stride;
			CLA_HIP(hipMemcpyAsync(dst, g.d.codes, (size_t) b->nRows * cw, hipMemcpyDeviceToDevice, b->stream));
			CLA_HIP(hipStreamSynchronize(b->stream));
			void* old = const_cast<void*>(g.d.codes);
			g.owned.erase(std::remove(g.owned.begin(), g.owned.end(), old), g.owned.end());
			CLA_HIP(hipFree(old));
			g.d.codes = dst;
			flat[i].codes = dst;
		}
		CLA_HIP(hipMemcpy(b->dGroups, flat.data(), sizeof(DGroup) * nG, hipMemcpyHostToDevice));
		b->arenaStride = stride;
		b->arenaWidth = cw;
	}

	// Slabs of groups whose mat-vec tables fit the LDS budget. Inside a slab every
	// table gets the same LDS stride (the largest nVals of the block) plus one
	// all-zero table, so table addresses are pure arithmetic; every slab but the
	// last holds a multiple of 8 groups (two batches of 4, see k_rmm_q1_ddc).
	{
		int budget = 52 * 1024;
		budget = std::min(budget, g_ldsPerBlock);
		b->q1Slabs.clear();
		b->q1LdsBytes = 0;
		const int mx = std::max(maxVals, 1);
		int per = budget / (mx * 8) - 1;   // groups per slab, one slot kept for the zero table
		// a thread stages at most 16 table values (Q1_TPT) for the next slab; the smallest block has 256 threads
		per = std::min(per, 16 * 256 / mx);
		per = per / 8 * 8;
		b->q1Threads = 256;
		if(per < 8) { // large dictionaries: two blocks of 512 threads per CU with half of its LDS each, else one of 1024 threads
			const int all = std::min(g_ldsPerBlock, 160 * 1024) - 8 * 1024;
			per = std::min(all / 2 / (mx * 8) - 1, 16 * 512 / mx) / 8 * 8;
			if(per >= 8) b->q1Threads = 512;
			else {
				per = std::min(all / (mx * 8) - 1, 16 * 1024 / mx) / 8 * 8;
				if(per >= 8) b->q1Threads = 1024;
			}
		}
		if(nG > 0 && per >= 8) {
			for(size_t i = 0; i < nG; i += per) {
				const size_t j = std::min(nG, i + (size_t) per);
				bool uniform = true;
				for(size_t g = i; g < j; g++) uniform &= b->groups[g].d.nVals == mx;
				b->q1Slabs.push_back(make_int4((int) i, (int) j, mx, uniform ? 1 : 0));
			}
			const size_t most = std::min(nG, (size_t) per);
			b->q1LdsBytes = (int32_t) ((most + 1) * mx * 8);
			CLA_HIP(hipMalloc((void**) &b->dQ1Slabs, sizeof(int4) * b->q1Slabs.size()));
			CLA_HIP(hipMemcpy(b->dQ1Slabs, b->q1Slabs.data(), sizeof(int4) * b->q1Slabs.size(), hipMemcpyHostToDevice));
		}
	}
	b->device_bytes_cached = 0;
	for(auto& g : b->groups) b->device_bytes_cached += g.bytes;
	{
		const int rc = ensure_dict_pad(b);
		if(rc) return rc;
	}
	b->finalized = true;
	return 0;
}

} // namespace cla

extern "C" {

int cla_block_set_stream(cla_handle b, void* hipStream) {
	CLA_TRY
	if(!b) { set_error("null block handle"); return -CLA_ERR_INVALID; }
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	if(b->ownStream && b->stream) { (void) hipStreamSynchronize(b->stream); (void) hipStreamDestroy(b->stream); }
	b->stream = (hipStream_t) hipStream;
	b->ownStream = false;
	return 0;
	CLA_CATCH_CODE(int)
}

int cla_block_set_option(cla_handle b, const char* key, int32_t value) {
	CLA_TRY
	if(!b || !key) { set_error("set_option: null handle or key"); return -CLA_ERR_INVALID; }
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	struct Entry { const char* name; int Options::*field; int lo, hi; };
	static const Entry table[] = {
		{"tsmm_route", &Options::tsmmRoute, 0, 2},         {"tsmm_chunks", &Options::tsmmChunks, 0, 1},
		{"tsmm_wide_dense", &Options::tsmmWideDense, 0, 1}, {"tsmm_mfma", &Options::tsmmMfma, 0, 1},
		{"tsmm_pair_dot", &Options::tsmmPairDot, 0, 1},     {"rmm_direct", &Options::rmmDirect, 0, 1},
		{"tsmm_direct", &Options::tsmmDirect, 0, 1},
		{"tsmm_narrow", &Options::tsmmNarrow, 0, 1},     {"expand_streams", &Options::expandStreams, 0, 1},
		{"rmm_disable", &Options::rmmDisable, 0, 15},       {"lmm_disable", &Options::lmmDisable, 0, 3},
		{"sdc_packed", &Options::sdcPacked, 0, 1},
		{"sdc_lanes", &Options::sdcLanes, 0, 1},
		{"sdc_rows", &Options::sdcRows, 0, 1},
		{"lmm_joint", &Options::lmmJoint, 0, 1},
		{"ddc_reorder", &Options::ddcReorder, 0, 1},
		{"tsmm_one_kernel", &Options::tsmmOneKernel, 0, 1},
	};
	for(const Entry& e : table)
		if(strcmp(e.name, key) == 0) {
			if(value < e.lo || value > e.hi) { set_error("set_option: %s takes %d..%d (got %d)", key, e.lo, e.hi, value); return -CLA_ERR_INVALID; }
			b->opt.*(e.field) = value;
			dec_plans_drop(b); // plans kept with the block were made under the old options
			return 0;
		}
	set_error("set_option: unknown option '%s'", key);
	return -CLA_ERR_INVALID;
	CLA_CATCH_CODE(int)
}

int cla_selftest_exception(int kind) {
	CLA_TRY
	if(kind == 0) throw std::bad_alloc();
	if(kind == 1) throw std::length_error("selftest");
	if(kind == 2) throw 42;
	if(kind == 3) { std::vector<double> v; v.reserve(v.max_size() + 1); } // what an absurd size argument does
	return 0;
	CLA_CATCH_CODE(int)
}

int32_t cla_block_num_groups(cla_handle b) { return b ? (int32_t) b->groups.size() : -CLA_ERR_INVALID; }
int64_t cla_block_num_rows(cla_handle b) { return b ? b->nRows : -CLA_ERR_INVALID; }
int32_t cla_block_num_cols(cla_handle b) { return b ? b->nCols : -CLA_ERR_INVALID; }
int32_t cla_block_group_num_values(cla_handle b, int32_t group) {
	CLA_TRY
	if(!b) return -CLA_ERR_INVALID;
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	if(group < 0 || group >= (int32_t) b->groups.size()) return -CLA_ERR_INVALID;
	return b->groups[group].d.type == G_UNC ? 0 : b->groups[group].d.nVals;
	CLA_CATCH_CODE(int32_t)
}

int64_t cla_block_device_bytes(cla_handle b) {
	CLA_TRY
	if(!b) return -CLA_ERR_INVALID;
	int64_t s = 0;
	for(auto& g : b->groups) s += g.bytes;
	return s;
	CLA_CATCH_CODE(int64_t)
}

int64_t cla_block_derived_bytes(cla_handle b) {
	if(!b) return -CLA_ERR_INVALID;
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	int64_t s = b->derivedBytes;
	if(b->joint) s += b->joint->derivedBytes;
	for(void* p : b->subs) s += ((SubBlock*) p)->blk ? ((SubBlock*) p)->blk->derivedBytes : 0;
	for(void* p : b->lmmSubs) s += ((LmmSub*) p)->blk ? ((LmmSub*) p)->blk->derivedBytes : 0;
	return s;
}

// Everything the library derived from the block's own representation after finalize goes: the next call that wants a form builds it
// again. (Workspaces of the host-pointer entry points are no derived forms and stay.)
static int drop_derived(cla_block* b) {
	if(g_device >= 0) (void) hipSetDevice(g_device);
	if(b->stream) CLA_HIP(hipStreamSynchronize(b->stream));
	if(b->joint) { cla_block_free(b->joint); b->joint = nullptr; b->jointSerial = 0; }
	free_subs(b);
	free_lmm_subs(b);
	b->lmmSubWidth = 0;
	dec_plans_drop(b);
	auto drop = [](auto*& p) { if(p) { (void) hipFree((void*) p); p = nullptr; } };
	drop(b->dSdcPlan); drop(b->dSdcDesc); drop(b->dSdcPacked);
	b->sdcPlanGroup = -2; b->sdcPackFailed = false;
	drop(b->dLaneMeta); drop(b->dLaneData);
	b->laneState = 0; b->laneSlabs = 0; b->laneDictLds = 0; b->laneDictTotal = 0; b->laneLmm = false;
	drop(b->dRowsMeta); drop(b->dRowsData);
	b->rowsState = 0; b->rowsTbl = 0;
	drop(b->dMfPlan);
	b->mfState = 0;
	drop(b->dCountsAll);
	for(uint8_t*& p : b->expCodes) drop(p);
	b->expCodes.clear();
	b->expTried = false;
	b->derivedBytes = b->dDictPad ? b->dictPadBytes : 0; // (the padded dictionary image is made at finalize and stays)
	return 0;
}

int cla_block_drop_derived(cla_handle b) {
	CLA_TRY
	int rc = check_final(b);
	if(rc) return rc;
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	return drop_derived(b);
	CLA_CATCH_CODE(int)
}

static int64_t rmm_dev(cla_handle b, const double* dB, int32_t nColB, double* dOut, bool sync);
static int64_t lmm_dev(cla_handle b, const double* dY, int32_t nRowY, double* dOut, bool sync);
static int64_t tsmm_dev(cla_handle b, double* dOut, bool sync);

int cla_block_prepare(cla_handle b, uint32_t products, int32_t nColB, int32_t nRowY) {
	CLA_TRY
	int rc = check_final(b);
	if(rc) return rc;
	if((products & ~(uint32_t) (CLA_PRODUCT_RMM | CLA_PRODUCT_LMM | CLA_PRODUCT_TSMM)) != 0 ||
		((products & CLA_PRODUCT_RMM) && nColB <= 0) || ((products & CLA_PRODUCT_LMM) && nRowY <= 0)) {
		set_error("prepare: unknown product bit or a product without its operand's width");
		return -CLA_ERR_INVALID;
	}
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	// Each product runs once on operands of zeros in buffers of this call: the drivers build what they would build on
	// their first call (which forms that is depends on the block, the operand's width and the options, nothing else).
	struct Tmp {
		double* p = nullptr;
		~Tmp() { if(p) (void) hipFree(p); }
		int zeros(size_t n, hipStream_t st) {
			CLA_HIP(hipMalloc((void**) &p, std::max<size_t>(n, 1) * sizeof(double)));
			CLA_HIP(hipMemsetAsync(p, 0, std::max<size_t>(n, 1) * sizeof(double), st));
			return 0;
		}
	};
	const bool profile = b->profile;
	b->profile = false;
	int64_t r = 0;
	if(r >= 0 && (products & CLA_PRODUCT_RMM)) {
		Tmp in, out;
		if((rc = in.zeros((size_t) b->nCols * nColB, b->stream)) || (rc = out.zeros((size_t) b->nRows * nColB, b->stream))) r = rc;
		else r = rmm_dev(b, in.p, nColB, out.p, true);
	}
	if(r >= 0 && (products & CLA_PRODUCT_LMM)) {
		Tmp in, out;
		if((rc = in.zeros((size_t) b->nRows * nRowY, b->stream)) || (rc = out.zeros((size_t) b->nCols * nRowY, b->stream))) r = rc;
		else r = lmm_dev(b, in.p, nRowY, out.p, true);
	}
	if(r >= 0 && (products & CLA_PRODUCT_TSMM)) {
		Tmp out;
		if((rc = out.zeros((size_t) b->nCols * b->nCols, b->stream))) r = rc;
		else r = tsmm_dev(b, out.p, true);
	}
	b->profile = profile;
	clear_stats(b);
	return r < 0 ? (int) r : 0;
	CLA_CATCH_CODE(int)
}

// ---- drivers -------------------------------------------------------------

// sync: wait for the driver's kernels and return its non-zero count; otherwise leave the count in the
// device counter (cla_block_nnz reads it on request) and return at once
static int64_t finish_nnz(cla_block* b, bool sync = true) {
	if(!sync) return 0;
	CLA_HIP(hipMemcpyAsync(b->hCounters, b->dCounters + b->nnzSlot, sizeof(unsigned long long), hipMemcpyDeviceToHost, b->stream));
	CLA_HIP(hipStreamSynchronize(b->stream));
	return (int64_t) b->hCounters[0];
}

static int64_t rmm_dev(cla_handle b, const double* dB, int32_t nColB, double* dOut, bool sync) {
	int rc = check_final(b);
	if(rc) return rc;
	if(!dB || !dOut || nColB <= 0) { set_error("rmm: invalid right-hand side"); return -CLA_ERR_INVALID; }
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	b->nnzSlot = 0;
	if((rc = launch_rmm(b, dB, nColB, dOut, b->dCounters))) return rc;
	return finish_nnz(b, sync);
}

int64_t cla_rmm_dev(cla_handle b, const double* dB, int32_t nColB, double* dOut) {
	CLA_TRY
	return rmm_dev(b, dB, nColB, dOut, true);
	CLA_CATCH_CODE(int64_t)
}

int cla_rmm_dev_async(cla_handle b, const double* dB, int32_t nColB, double* dOut) {
	CLA_TRY
	return (int) rmm_dev(b, dB, nColB, dOut, false);
	CLA_CATCH_CODE(int)
}

int64_t cla_rmm_dev_noalloc(cla_handle b, const double* dB, int32_t nColB, double* dOut) {
	CLA_TRY
	int rc = check_final(b);
	if(rc) return rc;
	if(!dB || !dOut || nColB <= 0) { set_error("rmm: invalid right-hand side"); return -CLA_ERR_INVALID; }
	unsigned char* ws = g_device < MAX_DEVICES ? g_scratchPtr[g_device] : nullptr;
	if(!ws) { set_error("rmm without allocation: no static workspace on device %d", g_device); return -CLA_ERR_STATE; }
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	// All calls on a GPU share its copy of the workspace, whatever block and stream they come from: held from the first
	// kernel's launch until the stream has drained (the call waits for that anyway, so the lock costs nothing).
	std::lock_guard<std::mutex> lkScratch(g_scratchMu[g_device]);
	// the counter and the tables live in the static workspace (the pre-aggregation kernel clears the counter
	// and rewrites every table entry that is read); event pairs of the profiling mode would be allocations
	unsigned long long* dNnz = (unsigned long long*) ws;
	const bool profile = b->profile;
	b->profile = false;
	rc = launch_rmm(b, dB, nColB, dOut, dNnz, 0, (double*) (ws + 256), (CLA_SCRATCH_BYTES - 256) / sizeof(double));
	b->profile = profile;
	if(rc) return rc;
	CLA_HIP(hipMemcpyAsync(b->hCounters, dNnz, sizeof(unsigned long long), hipMemcpyDeviceToHost, b->stream));
	CLA_HIP(hipStreamSynchronize(b->stream));
	return (int64_t) b->hCounters[0];
	CLA_CATCH_CODE(int64_t)
}

int64_t cla_block_nnz(cla_handle b) {
	CLA_TRY
	int rc = check_final(b);
	if(rc) return rc;
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	return finish_nnz(b, true);
	CLA_CATCH_CODE(int64_t)
}

int64_t cla_rmm(cla_handle b, const double* B, int32_t nColB, double* out) {
	CLA_TRY
	int rc = check_final(b);
	if(rc) return rc;
	if(!B || !out || nColB <= 0) { set_error("rmm: invalid right-hand side"); return -CLA_ERR_INVALID; }
	const size_t nIn = (size_t) b->nCols * nColB, nOut = (size_t) b->nRows * nColB;
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	if((rc = ensure_stage(&b->dStageIn, &b->stageInCap, nIn)) || (rc = ensure_stage(&b->dStageOut, &b->stageOutCap, nOut)))
		return rc;
	CLA_HIP(hipMemcpyAsync(b->dStageIn, B, nIn * sizeof(double), hipMemcpyHostToDevice, b->stream));
	const int64_t nnz = cla_rmm_dev(b, b->dStageIn, nColB, b->dStageOut);
	if(nnz < 0) return nnz;
	if(nOut) CLA_HIP(hipMemcpy(out, b->dStageOut, nOut * sizeof(double), hipMemcpyDeviceToHost));
	return nnz;
	CLA_CATCH_CODE(int64_t)
}


int64_t cla_decompress_dev(cla_handle b, double* dOut) {
	CLA_TRY
	int rc = check_final(b);
	if(rc) return rc;
	if(!dOut) { set_error("decompress: null output"); return -CLA_ERR_INVALID; }
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	b->nnzSlot = 0;
	if((rc = launch_decompress(b, dOut, b->dCounters))) return rc;
	return finish_nnz(b);
	CLA_CATCH_CODE(int64_t)
}

int64_t cla_decompress(cla_handle b, double* out) {
	CLA_TRY
	int rc = check_final(b);
	if(rc) return rc;
	if(!out) { set_error("decompress: null output"); return -CLA_ERR_INVALID; }
	const size_t nOut = (size_t) b->nRows * b->nCols;
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	if((rc = ensure_stage(&b->dStageOut, &b->stageOutCap, nOut))) return rc;
	const int64_t nnz = cla_decompress_dev(b, b->dStageOut);
	if(nnz < 0) return nnz;
	if(nOut) CLA_HIP(hipMemcpy(out, b->dStageOut, nOut * sizeof(double), hipMemcpyDeviceToHost));
	return nnz;
	CLA_CATCH_CODE(int64_t)
}

static int64_t lmm_dev(cla_handle b, const double* dY, int32_t nRowY, double* dOut, bool sync) {
	int rc = check_final(b);
	if(rc) return rc;
	if(!dY || !dOut || nRowY <= 0) { set_error("lmm: invalid left-hand side"); return -CLA_ERR_INVALID; }
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	b->nnzSlot = 0;
	if((rc = launch_lmm(b, dY, nRowY, dOut, b->dCounters))) return rc;
	return finish_nnz(b, sync);
}

int64_t cla_lmm_dev(cla_handle b, const double* dY, int32_t nRowY, double* dOut) {
	CLA_TRY
	return lmm_dev(b, dY, nRowY, dOut, true);
	CLA_CATCH_CODE(int64_t)
}

int cla_lmm_dev_async(cla_handle b, const double* dY, int32_t nRowY, double* dOut) {
	CLA_TRY
	return (int) lmm_dev(b, dY, nRowY, dOut, false);
	CLA_CATCH_CODE(int)
}

int64_t cla_lmm(cla_handle b, const double* Y, int32_t nRowY, double* out) {
	CLA_TRY
	int rc = check_final(b);
	if(rc) return rc;
	if(!Y || !out || nRowY <= 0) { set_error("lmm: invalid left-hand side"); return -CLA_ERR_INVALID; }
	const size_t nIn = (size_t) nRowY * b->nRows, nOut = (size_t) nRowY * b->nCols;
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	if((rc = ensure_stage(&b->dStageIn, &b->stageInCap, nIn)) || (rc = ensure_stage(&b->dStageOut, &b->stageOutCap, nOut)))
		return rc;
	if(nIn) CLA_HIP(hipMemcpyAsync(b->dStageIn, Y, nIn * sizeof(double), hipMemcpyHostToDevice, b->stream));
	const int64_t nnz = cla_lmm_dev(b, b->dStageIn, nRowY, b->dStageOut);
	if(nnz < 0) return nnz;
	CLA_HIP(hipMemcpy(out, b->dStageOut, nOut * sizeof(double), hipMemcpyDeviceToHost));
	return nnz;
	CLA_CATCH_CODE(int64_t)
}

static int64_t tsmm_dev(cla_handle b, double* dOut, bool sync) {
	int rc = check_final(b);
	if(rc) return rc;
	if(!dOut) { set_error("tsmm: null output"); return -CLA_ERR_INVALID; }
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	b->nnzSlot = 0;
	if((rc = launch_tsmm(b, dOut, b->dCounters))) return rc;
	return finish_nnz(b, sync);
}

int64_t cla_tsmm_dev(cla_handle b, double* dOut) {
	CLA_TRY
	return tsmm_dev(b, dOut, true);
	CLA_CATCH_CODE(int64_t)
}

int cla_tsmm_dev_async(cla_handle b, double* dOut) {
	CLA_TRY
	return (int) tsmm_dev(b, dOut, false);
	CLA_CATCH_CODE(int)
}

int64_t cla_tsmm(cla_handle b, double* out) {
	CLA_TRY
	int rc = check_final(b);
	if(rc) return rc;
	if(!out) { set_error("tsmm: null output"); return -CLA_ERR_INVALID; }
	const size_t nOut = (size_t) b->nCols * b->nCols;
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	if((rc = ensure_stage(&b->dStageOut, &b->stageOutCap, nOut))) return rc;
	const int64_t nnz = cla_tsmm_dev(b, b->dStageOut);
	if(nnz < 0) return nnz;
	CLA_HIP(hipMemcpy(out, b->dStageOut, nOut * sizeof(double), hipMemcpyDeviceToHost));
	return nnz;
	CLA_CATCH_CODE(int64_t)
}

} // extern "C"

namespace cla {

// Uncompressed group times B[cols, :] (ColGroupUncompressed.rightMultByMatrix, CG/ColGroupUncompressed.java:888-927):
// out[r, j] = sum_h U[r, h] * B[cols[h], j]; thread = one output cell.
__global__ __launch_bounds__(256) void k_unc_times_b(const double* __restrict__ U, int64_t nRows, int nC, const int32_t* __restrict__ cols,
	const double* __restrict__ B, int q, double* __restrict__ out) {
	const int64_t idx = (int64_t) blockIdx.x * 256 + threadIdx.x;
	if(idx >= nRows * q) return;
	const int64_t r = idx / q;
	const int j = (int) (idx - r * q);
	double s = 0.0;
	for(int h = 0; h < nC; h++) s += U[(size_t) r * nC + h] * B[(size_t) cols[h] * q + j];
	out[idx] = s;
}

__global__ __launch_bounds__(256) void k_take_block(const double* __restrict__ G, int n, int r0, int c0, int nr, int nc,
	double* __restrict__ out, unsigned long long* __restrict__ nnz) {
	int cnt = 0;
	for(int idx = threadIdx.x + blockIdx.x * 256; idx < nr * nc; idx += 256 * gridDim.x) {
		const int i = idx / nc, j = idx - i * nc;
		const double v = G[(size_t) (r0 + i) * n + c0 + j];
		out[idx] = v;
		cnt += v != 0.0;
	}
	if(cnt) atomicAdd(nnz, (unsigned long long) cnt);
}

// cbind(left, right) as a block of its own: the groups of `left` first, then those of `right` with
// their columns shifted by left->nCols (rounded up to a multiple of 16 with empty columns between while the whole
// stays within 64 columns: the decoded Gram kernel then computes the left x right tiles only). Row data (codes,
// offsets, runs, dense values) is borrowed from the two blocks, which must outlive it; column lists and
// dictionaries are its own copies. The right side's columns are the last right->nCols ones.
static cla_block* make_joint(cla_block* left, cla_block* right) {
	const int padL = (left->nCols + 15) / 16 * 16;
	const bool padded = padL + right->nCols <= 64;
	const int rightStart = padded ? padL : left->nCols;
	cla_block* c = cla_block_create(left->nRows, rightStart + right->nCols);
	if(!c) return nullptr;
	if(padded) c->crossBlocks = padL / 16;
	c->crossCol = rightStart;
	int tblOff = 0, colOff = 0, maxVals = 0;
	for(int side = 0; side < 2; side++) {
		cla_block* src = side ? right : left;
		const int shift = side ? rightStart : 0;
		for(auto& pg : src->groups) {
			c->groups.emplace_back();
			HostGroup& g = c->groups.back();
			g.d = pg.d; // row data: borrowed
			g.cols = pg.cols;
			for(int& col : g.cols) col += shift;
			g.dict = pg.dict;
			g.codeOrder = pg.codeOrder;
			g.bytes = 0;
			if(upload(g, g.cols.data(), sizeof(int32_t) * g.cols.size(), (const void**) &g.d.cols) ||
				(!g.dict.empty() && upload_dict(g))) {
				cla_block_free(c);
				return nullptr;
			}
			g.bytes = pg.bytes;
			g.d.tblOff = tblOff;
			g.d.colOff = colOff;
			tblOff += g.d.nVals;
			colOff += g.d.nColG;
			maxVals = std::max(maxVals, g.d.nVals);
		}
		for(int j = 0; j < src->nCols; j++) c->constV[(size_t) shift + j] = src->constV[j];
		c->hasConst |= src->hasConst;
		c->hasSdc |= src->hasSdc;
		c->hasRle |= src->hasRle;
		c->hasUnc |= src->hasUnc;
	}
	c->crossSplit = (int32_t) left->groups.size();
	c->totalVals = tblOff;
	c->totalColsG = colOff;
	c->maxVals = maxVals;
	if(finish_finalize(c, nullptr, false)) { cla_block_free(c); return nullptr; }
	return c;
}

// ---------------------------------------------------------------------------
// t(X) %*% X of a block with more than 64 columns through the decoded Gram matrix: the columns are cut
// into chunks of at most 32 (groups stay whole; columns that only carry a constant go along), every
// pair of chunks becomes a block of its own of at most 64 columns that borrows the row data of `b`
// (built once, kept with `b`), and its Gram matrix is scattered into the result. For a joint block
// (crossSplit > 0) only chunks of the left side meet chunks of the right side.
// ---------------------------------------------------------------------------

__global__ __launch_bounds__(256) void k_scatter_gram(const double* __restrict__ S, int k, const int32_t* __restrict__ colMap, int nA,
	int writeA, int writeB, int crossOnly, double* __restrict__ out, int n) {
	for(int idx = threadIdx.x + blockIdx.x * 256; idx < k * k; idx += 256 * gridDim.x) {
		const int r = idx / k, c = idx - r * k;
		const bool rA = r < nA, cA = c < nA;
		bool take;
		if(rA && cA) take = writeA && !crossOnly;
		else if(!rA && !cA) take = writeB && !crossOnly;
		else take = crossOnly ? rA : true; // joint block: the (left, right) block only, the caller takes it from the upper half
		if(take && colMap[r] >= 0 && colMap[c] >= 0) out[(size_t) colMap[r] * n + colMap[c]] = S[idx];
	}
}

static void free_subs(cla_block* b) {
	for(void* p : b->subs) {
		SubBlock* sb = (SubBlock*) p;
		if(sb->dColMap) (void) hipFree(sb->dColMap);
		if(sb->blk) cla_block_free(sb->blk);
		delete sb;
	}
	b->subs.clear();
}

// chunk = groups and constant-only columns of b
struct Chunk { std::vector<int> groups, constCols; int nCols = 0; };

// cross: only the product of chunk A with chunk B will be read. A's columns are then padded with empty columns to
// a multiple of 16, so that the decoded Gram kernel can leave out the tiles inside A and inside B, and the
// per-pair form leaves out the pairs of groups of one chunk.
static cla_block* make_sub(cla_block* b, const Chunk& A, const Chunk& B, bool cross, std::vector<int32_t>& colMap) {
	const int padA = cross ? (A.nCols + 15) / 16 * 16 : A.nCols;
	cla_block* c = cla_block_create(b->nRows, padA + B.nCols);
	if(!c) return nullptr;
	colMap.clear();
	int tblOff = 0, colOff = 0, maxVals = 0;
	for(int side = 0; side < 2; side++) {
		const Chunk& ch = side ? B : A;
		for(int gi : ch.groups) {
			const HostGroup& pg = b->groups[gi];
			c->groups.emplace_back();
			HostGroup& g = c->groups.back();
			g.d = pg.d; // row data: borrowed
			g.cols.resize(pg.cols.size());
			for(size_t j = 0; j < pg.cols.size(); j++) {
				g.cols[j] = (int32_t) colMap.size();
				c->constV[colMap.size()] = b->constV[pg.cols[j]];
				colMap.push_back(pg.cols[j]);
			}
			g.dict = pg.dict;
			g.codeOrder = pg.codeOrder;
			g.bytes = 0;
			if(upload(g, g.cols.data(), sizeof(int32_t) * g.cols.size(), (const void**) &g.d.cols) ||
				(!g.dict.empty() && upload_dict(g))) {
				cla_block_free(c);
				return nullptr;
			}
			g.bytes = pg.bytes;
			g.d.tblOff = tblOff;
			g.d.colOff = colOff;
			tblOff += g.d.nVals;
			colOff += g.d.nColG;
			maxVals = std::max(maxVals, g.d.nVals);
			if(g.d.type == G_SDCZ) c->hasSdc = true;
			if(g.d.type == G_RLE) c->hasRle = true;
			if(g.d.type == G_UNC) c->hasUnc = true;
		}
		for(int col : ch.constCols) {
			c->constV[colMap.size()] = b->constV[col];
			colMap.push_back(col);
		}
		if(side == 0 && cross) {
			c->crossSplit = (int32_t) c->groups.size();
			c->crossBlocks = padA / 16;
			while((int) colMap.size() < padA) { c->constV[colMap.size()] = 0.0; colMap.push_back(-1); }
		}
	}
	c->hasConst = b->hasConst;
	c->totalVals = tblOff;
	c->totalColsG = colOff;
	c->maxVals = maxVals;
	if(finish_finalize(c, nullptr, false)) { cla_block_free(c); return nullptr; }
	return c;
}

// Returns 1 when the block cannot be cut that way (a group of more than 32 columns), 0 when dOut (n x n,
// zeroed by the caller) holds the result: full symmetric, or for a joint block its (left, right) part.
int launch_tsmm_chunked(cla_block* b, double* dOut) {
	const int n = b->nCols, nG = (int) b->groups.size(), split = b->crossSplit;
	if(b->subs.empty()) {
		// chunks per side (one side when the block is no joint block); joint blocks: left columns are those of
		// the first `split` groups and, of the constant-only ones, those in front of the right side's first
		// column (which may itself be a constant-only one)
		std::vector<char> covered((size_t) n, 0);
		for(auto& g : b->groups)
			for(int c : g.cols) covered[c] = 1;
		const int firstRight = split > 0 ? b->crossCol : n;
		std::vector<Chunk> chunks[2];
		auto add_item = [&](int side, int group, int col, int width) -> bool {
			if(width > 32) return false;
			auto& v = chunks[side];
			if(v.empty() || v.back().nCols + width > 32) v.emplace_back();
			if(group >= 0) v.back().groups.push_back(group); else v.back().constCols.push_back(col);
			v.back().nCols += width;
			return true;
		};
		for(int g = 0; g < nG; g++)
			if(!add_item(split > 0 && g >= split ? 1 : 0, g, -1, b->groups[g].d.nColG)) return 1;
		for(int c = 0; c < n; c++)
			if(!covered[c] && !add_item(split > 0 && c >= firstRight ? 1 : 0, -1, c, 1)) return 1;
		std::vector<std::pair<int, int>> pairs; // (chunk of side 0, chunk of side 0 or 1)
		const int m0 = (int) chunks[0].size(), m1 = (int) chunks[1].size();
		if(split > 0) {
			for(int i = 0; i < m0; i++)
				for(int j = 0; j < m1; j++) pairs.emplace_back(i, j);
		}
		else {
			if(m0 < 2) return 1;
			for(int i = 0; i < m0; i++)
				for(int j = i + 1; j < m0; j++) pairs.emplace_back(i, j);
		}
		for(auto& pr : pairs) {
			const Chunk& A = chunks[0][pr.first];
			const Chunk& B = split > 0 ? chunks[1][pr.second] : chunks[0][pr.second];
			SubBlock* sb = new SubBlock();
			sb->blk = nullptr; sb->dColMap = nullptr;
			b->subs.push_back(sb);
			// every diagonal block once: chunk i with its successor, the last chunk with its predecessor
			sb->writeA = split == 0 && pr.second == pr.first + 1;
			sb->writeB = split == 0 && pr.first == m0 - 2 && pr.second == m0 - 1;
			sb->crossOnly = split > 0;
			std::vector<int32_t> colMap;
			sb->blk = make_sub(b, A, B, split > 0 || (!sb->writeA && !sb->writeB), colMap);
			if(!sb->blk) { free_subs(b); return -CLA_ERR_DEVICE; }
			sb->nA = (int) colMap.size() - B.nCols; sb->nB = B.nCols;
			if(hipMalloc((void**) &sb->dColMap, sizeof(int32_t) * colMap.size()) != hipSuccess ||
				hipMemcpy(sb->dColMap, colMap.data(), sizeof(int32_t) * colMap.size(), hipMemcpyHostToDevice) != hipSuccess) {
				set_error("tsmm: column map of a chunk pair could not be uploaded");
				free_subs(b);
				return -CLA_ERR_DEVICE;
			}
		}
	}
	for(void* p : b->subs) {
		SubBlock* sb = (SubBlock*) p;
		cla_block* c = sb->blk;
		c->profile = b->profile;
		c->opt = b->opt;
		if(c->stream != b->stream) {
			if(c->ownStream && c->stream) { (void) hipStreamSynchronize(c->stream); (void) hipStreamDestroy(c->stream); }
			c->stream = b->stream;
			c->ownStream = false;
		}
		const int k = c->nCols;
		int rc = ensure_stage(&c->dStageOut, &c->stageOutCap, (size_t) k * k);
		if(rc) return rc;
		if((rc = launch_tsmm(c, c->dStageOut, c->dCounters))) return rc;
		{
			Prof pf(c, "k_scatter_gram", (k * k + 255) / 256, 256, 0, 0);
			hipLaunchKernelGGL(k_scatter_gram, dim3((unsigned) ((k * k + 255) / 256)), dim3(256), 0, b->stream, c->dStageOut, k, sb->dColMap,
				sb->nA, sb->writeA ? 1 : 0, sb->writeB ? 1 : 0, sb->crossOnly ? 1 : 0, dOut, n);
		}
		CLA_HIP(hipGetLastError());
		b->lastStats.insert(b->lastStats.end(), c->lastStats.begin(), c->lastStats.end());
		c->lastStats.clear(); // (the events moved along)
	}
	return 0;
}

// ---- Y %*% X on the decode kernel

static void free_lmm_subs(cla_block* b) {
	for(void* p : b->lmmSubs) {
		LmmSub* sb = (LmmSub*) p;
		if(sb->dColMap) (void) hipFree(sb->dColMap);
		if(sb->blk) cla_block_free(sb->blk);
		delete sb;
	}
	b->lmmSubs.clear();
}

// out[i, colMap[j]] = S[i, j] for the k columns of a chunk; counts the non-zero cells it writes
__global__ __launch_bounds__(256) void k_scatter_cols(const double* __restrict__ S, int k, const int32_t* __restrict__ colMap, int p,
	double* __restrict__ out, int n, unsigned long long* __restrict__ nnz) {
	int cnt = 0;
	for(int idx = threadIdx.x + blockIdx.x * 256; idx < p * k; idx += 256 * gridDim.x) {
		const int i = idx / k, j = idx - i * k;
		const double v = S[idx];
		out[(size_t) i * n + colMap[j]] = v;
		cnt += v != 0.0;
	}
	if(cnt) atomicAdd(nnz, (unsigned long long) cnt);
}

// rs[i] += sum of Y[i, rows of the block]
__global__ __launch_bounds__(256) void k_y_rowsum(const double* __restrict__ Y, int64_t nRows, int64_t rowsPerBlock, double* __restrict__ rs) {
	__shared__ double red[4];
	const double* y = Y + (size_t) blockIdx.y * nRows;
	const int64_t rb = (int64_t) blockIdx.x * rowsPerBlock, re = min(rb + rowsPerBlock, nRows);
	double s = 0.0;
	for(int64_t r = rb + threadIdx.x; r < re; r += 256) s += y[r];
	s = wave_sum_f64(s);
	if((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
	__syncthreads();
	if(threadIdx.x == 0) unsafeAtomicAdd(&rs[blockIdx.y], red[0] + red[1] + red[2] + red[3]);
}

// out[i, cols[j]] = rs[i] * constV[cols[j]] for the k columns that no group covers
__global__ __launch_bounds__(256) void k_const_cols(const double* __restrict__ rs, const double* __restrict__ constV, const int32_t* __restrict__ cols,
	int k, int p, double* __restrict__ out, int n, unsigned long long* __restrict__ nnz) {
	int cnt = 0;
	for(int idx = threadIdx.x + blockIdx.x * 256; idx < p * k; idx += 256 * gridDim.x) {
		const int i = idx / k, c = cols[idx - i * k];
		const double v = rs[i] * constV[c];
		out[(size_t) i * n + c] = v;
		cnt += v != 0.0;
	}
	if(cnt) atomicAdd(nnz, (unsigned long long) cnt);
}

// Cuts the block into chunks of whole groups of at most `width` columns, a block of its own each; the columns that
// no group covers make a list of their own. 1 when a group is wider than that.
static int build_lmm_subs(cla_block* b, int width) {
	const int n = b->nCols, nG = (int) b->groups.size();
	std::vector<char> covered((size_t) n, 0);
	for(auto& g : b->groups)
		for(int c : g.cols) covered[c] = 1;
	std::vector<Chunk> chunks;
	auto add_item = [&](int group, int w) -> bool {
		if(w > width) return false;
		if(chunks.empty() || chunks.back().nCols + w > width) chunks.emplace_back();
		chunks.back().groups.push_back(group);
		chunks.back().nCols += w;
		return true;
	};
	for(int g = 0; g < nG; g++)
		if(!add_item(g, b->groups[g].d.nColG)) return 1;
	std::vector<int32_t> constOnly;
	for(int c = 0; c < n; c++)
		if(!covered[c]) constOnly.push_back(c);
	const Chunk none;
	for(size_t ci = 0; ci < chunks.size() + (constOnly.empty() ? 0 : 1); ci++) {
		LmmSub* sb = new LmmSub();
		sb->blk = nullptr; sb->dColMap = nullptr; sb->k = 0;
		b->lmmSubs.push_back(sb);
		std::vector<int32_t> colMap;
		if(ci < chunks.size()) {
			sb->blk = make_sub(b, chunks[ci], none, false, colMap);
			if(!sb->blk) { free_lmm_subs(b); return -CLA_ERR_DEVICE; }
		}
		else colMap = constOnly;
		sb->k = (int) colMap.size();
		if(hipMalloc((void**) &sb->dColMap, sizeof(int32_t) * colMap.size()) != hipSuccess ||
			hipMemcpy(sb->dColMap, colMap.data(), sizeof(int32_t) * colMap.size(), hipMemcpyHostToDevice) != hipSuccess) {
			set_error("left multiply: column map of a column chunk could not be uploaded");
			free_lmm_subs(b);
			return -CLA_ERR_DEVICE;
		}
	}
	return 0;
}

// Y %*% X chunk of columns by chunk on the decode kernel: blocks of more than 64 columns, or whose code tiles exceed
// LDS together. The widest chunks that the kernel takes (64, 32, 16 columns) are kept with the block. Returns 1 when
// no width fits or Y holds a value that is not finite, 0 when dOut holds the result and *dNnz its non-zero count.
static int launch_lmm_chunked(cla_block* b, const double* dY, int p, double* dOut, unsigned long long* dNnz) {
	if(b->lmmSubWidth < 0) return 1;
	hipStream_t st = b->stream;
	CLA_HIP(hipMemsetAsync(dNnz, 0, sizeof(unsigned long long), st));
	int width = b->lmmSubWidth ? b->lmmSubWidth : 64;
	for(;;) {
		if(b->lmmSubs.empty()) {
			const int rc = build_lmm_subs(b, width);
			if(rc < 0) return rc;
			if(rc == 1) { free_lmm_subs(b); b->lmmSubWidth = -1; return 1; }
		}
		bool fits = true;
		for(void* q : b->lmmSubs) {
			LmmSub* sb = (LmmSub*) q;
			cla_block* c = sb->blk;
			if(!c) { // row sums of Y for the columns that no group covers
				int rc = ensure_tables(b, (size_t) p); // (the caller's dOut may be the block's output staging buffer)
				if(rc) return rc;
				CLA_HIP(hipMemsetAsync(b->dTables, 0, (size_t) p * sizeof(double), st));
				int64_t rpb = 256 * 1024;
				while(rpb > 8192 && (b->nRows + rpb - 1) / rpb * p < (int64_t) g_numCU * 2) rpb /= 2;
				const dim3 grid((unsigned) ((b->nRows + rpb - 1) / rpb), (unsigned) p);
				Prof pf(b, "k_y_rowsum", (long) grid.x * p, 256, 0, (double) b->nRows * p * 8);
				hipLaunchKernelGGL(k_y_rowsum, grid, dim3(256), 0, st, dY, b->nRows, rpb, b->dTables);
				continue;
			}
			c->profile = b->profile;
			c->opt = b->opt;
			if(c->stream != b->stream) {
				if(c->ownStream && c->stream) { (void) hipStreamSynchronize(c->stream); (void) hipStreamDestroy(c->stream); }
				c->stream = b->stream;
				c->ownStream = false;
			}
			const int k = c->nCols;
			const size_t n = (size_t) p * k;
			int rc = ensure_stage(&c->dStageOut, &c->stageOutCap, n);
			if(rc) return rc;
			CLA_HIP(hipMemsetAsync(c->dStageOut, 0, n * sizeof(double), st));
			for(int p0 = 0; p0 < p && fits; p0 += 16) { // 16 rows of Y per pass over the chunk
				rc = launch_lmm_decode(c, dY + (size_t) p0 * b->nRows, std::min(16, p - p0), c->dStageOut + (size_t) p0 * k, dNnz);
				if(rc < 0) return rc;
				if(rc == 1) fits = false; // (the plan is the same for every pass: only the first can say so)
			}
			b->lastStats.insert(b->lastStats.end(), c->lastStats.begin(), c->lastStats.end());
			c->lastStats.clear(); // (the events moved along)
			if(!fits) break;
		}
		if(fits) break;
		// (what the chunks in front of the one that does not fit have queued finishes on the stream before their blocks go)
		CLA_HIP(hipStreamSynchronize(st));
		clear_stats(b);
		free_lmm_subs(b);
		CLA_HIP(hipMemsetAsync(dNnz, 0, sizeof(unsigned long long), st));
		if(width == 16) { b->lmmSubWidth = -1; return 1; }
		width /= 2;
	}
	b->lmmSubWidth = width;
	{
		unsigned long long bad = 0; // (see launch_lmm_joint)
		CLA_HIP(hipMemcpyAsync(&bad, dNnz, sizeof(bad), hipMemcpyDeviceToHost, st));
		CLA_HIP(hipStreamSynchronize(st));
		if(bad) { clear_stats(b); return 1; }
	}
	CLA_HIP(hipMemsetAsync(dNnz, 0, sizeof(unsigned long long), st));
	for(void* q : b->lmmSubs) {
		LmmSub* sb = (LmmSub*) q;
		const int k = sb->k;
		const int n = p * k;
		if(!sb->blk) {
			Prof pf(b, "k_const_cols", (n + 255) / 256, 256, 0, 0);
			hipLaunchKernelGGL(k_const_cols, dim3((unsigned) std::min((n + 255) / 256, 1024)), dim3(256), 0, st, b->dTables, b->dConstV, sb->dColMap,
				k, p, dOut, b->nCols, dNnz);
			continue;
		}
		Prof pf(b, "k_scatter_cols", (n + 255) / 256, 256, 0, 0);
		hipLaunchKernelGGL(k_scatter_cols, dim3((unsigned) std::min((n + 255) / 256, 1024)), dim3(256), 0, st, sb->blk->dStageOut, k, sb->dColMap, p,
			dOut, b->nCols, dNnz);
	}
	CLA_HIP(hipGetLastError());
	return 0;
}

// Y %*% X in passes over the decoded rows on the matrix cores, 16 rows of Y as the other operand of a pass
// (k_lmm_decode), whatever the block's group mix, where the bin kernels take a pass per row of Y and group type
// (C5, 50 M x 20: 2.0 - 2.35 ms for 1 to 16 rows of Y against 2.9 - 88 ms). Taken for blocks that the offset-list
// kernels do not serve better and, for few rows of Y, the byte-code dot form neither; blocks of more than 64 columns
// or with too many code tiles for LDS go chunk of columns by chunk. Returns 1 when the block is not eligible, 0 when
// dOut (p x nCols) holds the result and *dNnz its non-zero count.
int launch_lmm_joint(cla_block* b, const double* dY, int p, double* dOut, unsigned long long* dNnz) {
	if(!b->opt.lmmJoint || !b->opt.tsmmMfma || p < 1 || b->nRows == 0 || b->crossSplit > 0) return 1;
	if(b->dictNonFinite) return 1; // (the reference sums Y per tuple first: an infinite dictionary value times Y of both signs is no NaN)
	int nLists = 0, nOther = 0;
	bool dotForm = b->dArena != nullptr && b->arenaWidth == 1 && b->maxVals <= 256;
	std::vector<char> seen((size_t) b->nCols, 0);
	for(auto& g : b->groups) {
		if(g.d.type == G_SDCZ) nLists += g.d.nOffsets > 0;
		else nOther += g.d.type == G_UNC || g.d.nVals > 0;
		if(g.d.nColG != 1) dotForm = false;
		if(g.d.type == G_UNC || g.d.nVals > 0)
			for(int c : g.cols) {
				if(seen[c]) return 1; // overlapping groups: the decode kernel wants one group per column
				seen[c] = 1;
			}
	}
	if(nOther == 0 || nLists > nOther) return 1;
	// single-column byte codes: the dot kernel takes a pass per row of Y, a twelfth of what a pass of the decode kernel
	// over 16 rows of Y costs (C2: 0.21 against 2.5 ms)
	if(dotForm && (p + 15) / 16 * 12 >= p) return 1;
	if(b->nCols > 64) return launch_lmm_chunked(b, dY, p, dOut, dNnz);
	hipStream_t st = b->stream;
	const size_t n = (size_t) p * b->nCols;
	int rc = ensure_stage(&b->dStageOut, &b->stageOutCap, n);
	if(rc) return rc;
	CLA_HIP(hipMemsetAsync(b->dStageOut, 0, n * sizeof(double), st));
	CLA_HIP(hipMemsetAsync(dNnz, 0, sizeof(unsigned long long), st));
	for(int p0 = 0; p0 < p; p0 += 16) // 16 rows of Y per pass over the block
		if((rc = launch_lmm_decode(b, dY + (size_t) p0 * b->nRows, std::min(16, p - p0), b->dStageOut + (size_t) p0 * b->nCols, dNnz))) {
			if(rc == 1 && p0 == 0) return launch_lmm_chunked(b, dY, p, dOut, dNnz); // (nothing queued yet)
			if(p0 > 0) clear_stats(b);
			return rc;
		}
	{
		// A row that a group does not cover (outside its runs or its offset list) does not enter that group's sums in
		// the reference, whatever Y holds there; as a decoded 0.0 it turns an infinite Y into NaN. The kernel reports a
		// non-finite value of Y, and such a Y takes the bin kernels (the host has to look: one wait for the stream).
		unsigned long long bad = 0;
		CLA_HIP(hipMemcpyAsync(&bad, dNnz, sizeof(bad), hipMemcpyDeviceToHost, st));
		CLA_HIP(hipStreamSynchronize(st));
		if(bad) { clear_stats(b); return 1; }
	}
	CLA_HIP(hipMemsetAsync(dNnz, 0, sizeof(unsigned long long), st));
	{
		Prof pf(b, "k_take_block", ((int) n + 255) / 256, 256, 0, 0);
		hipLaunchKernelGGL(k_take_block, dim3((unsigned) std::min(((int) n + 255) / 256, 1024)), dim3(256), 0, st, b->dStageOut, b->nCols, 0, 0, p,
			b->nCols, dOut, dNnz);
	}
	CLA_HIP(hipGetLastError());
	return 0;
}

} // namespace cla

extern "C" {

int64_t cla_lmm_compressed_dev(cla_handle right, cla_handle left, double* dOut) {
	CLA_TRY
	int rc = check_final(right);
	if(rc || (rc = check_final(left))) return rc;
	if(!dOut) { set_error("compressed left multiply: null output"); return -CLA_ERR_INVALID; }
	if(left->nRows != right->nRows) {
		set_error("compressed left multiply: %lld rows on the left, %lld on the right", (long long) left->nRows, (long long) right->nRows);
		return -CLA_ERR_INVALID;
	}
	// both blocks' locks, in address order (two threads may call with the roles swapped)
	cla_block* const first = left < right ? left : right;
	cla_block* const second = left < right ? right : left;
	std::lock_guard<std::recursive_mutex> lk(first->mu);
	std::unique_lock<std::recursive_mutex> lk2(second->mu, std::defer_lock);
	if(second != first) lk2.lock();
	if(!right->joint || right->jointSerial != left->serial) {
		if(right->joint) { cla_block_free(right->joint); right->joint = nullptr; }
		right->joint = make_joint(left, right);
		if(!right->joint) return -CLA_ERR_DEVICE;
		right->jointSerial = left->serial;
	}
	cla_block* c = right->joint;
	c->profile = right->profile;
	c->opt = right->opt;
	// the joint block works on the right block's stream
	if(c->stream != right->stream) {
		if(c->ownStream && c->stream) { (void) hipStreamSynchronize(c->stream); (void) hipStreamDestroy(c->stream); }
		c->stream = right->stream;
		c->ownStream = false;
	}
	const size_t n = (size_t) c->nCols;
	if((rc = ensure_stage(&c->dStageOut, &c->stageOutCap, n * n))) return rc;
	if((rc = launch_tsmm(c, c->dStageOut, c->dCounters))) return rc;
	right->nnzSlot = 0;
	CLA_HIP(hipMemsetAsync(right->dCounters, 0, sizeof(unsigned long long), right->stream));
	const int nOut = left->nCols * right->nCols;
	{
		Prof pf(c, "k_take_block", (nOut + 255) / 256, 256, 0, 0);
		hipLaunchKernelGGL(k_take_block, dim3((unsigned) std::min((nOut + 255) / 256, 1024)), dim3(256), 0, right->stream,
			c->dStageOut, (int) n, 0, c->nCols - right->nCols, left->nCols, right->nCols, dOut, right->dCounters);
	}
	CLA_HIP(hipGetLastError());
	clear_stats(right);
	right->lastStats.swap(c->lastStats); // what the kernel statistics of `right` report
	return finish_nnz(right);
	CLA_CATCH_CODE(int64_t)
}

int64_t cla_lmm_compressed(cla_handle right, cla_handle left, double* out) {
	CLA_TRY
	int rc = check_final(right);
	if(rc || (rc = check_final(left))) return rc;
	if(!out) { set_error("compressed left multiply: null output"); return -CLA_ERR_INVALID; }
	const size_t nOut = (size_t) left->nCols * right->nCols;
	cla_block* const first = left < right ? left : right;
	cla_block* const second = left < right ? right : left;
	std::lock_guard<std::recursive_mutex> lk(first->mu);
	std::unique_lock<std::recursive_mutex> lk2(second->mu, std::defer_lock);
	if(second != first) lk2.lock();
	if((rc = ensure_stage(&right->dStageOut, &right->stageOutCap, nOut))) return rc;
	const int64_t nnz = cla_lmm_compressed_dev(right, left, right->dStageOut);
	if(nnz < 0) return nnz;
	CLA_HIP(hipMemcpy(out, right->dStageOut, nOut * sizeof(double), hipMemcpyDeviceToHost));
	return nnz;
	CLA_CATCH_CODE(int64_t)
}

cla_handle cla_rmm_overlapping(cla_handle b, const double* B, int32_t nColB) {
	CLA_TRY
	if(check_final(b)) return nullptr;
	if(!B || nColB <= 0) { set_error("rmm: invalid right-hand side"); return nullptr; }
	const int q = nColB;
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	const size_t nIn = (size_t) b->nCols * q, nT = (size_t) (b->totalVals + 1) * q;
	if(ensure_stage(&b->dStageIn, &b->stageInCap, nIn)) return nullptr;
	if(hipMemcpyAsync(b->dStageIn, B, nIn * sizeof(double), hipMemcpyHostToDevice, b->stream) != hipSuccess) {
		set_error("overlapping right multiply: copying B failed");
		return nullptr;
	}
	if(launch_tables(b, b->dStageIn, q)) return nullptr;
	std::vector<double> T(nT);
	if(hipMemcpyAsync(T.data(), b->dTables, nT * sizeof(double), hipMemcpyDeviceToHost, b->stream) != hipSuccess ||
		hipStreamSynchronize(b->stream) != hipSuccess) {
		set_error("overlapping right multiply: reading the tables failed");
		return nullptr;
	}
	cla_block* c = cla_block_create(b->nRows, q);
	if(!c) return nullptr;
	std::vector<int32_t> cols((size_t) q);
	for(int j = 0; j < q; j++) cols[j] = j;
	int tblOff = 0, colOff = 0, maxVals = 0;
	for(auto& pg : b->groups) {
		const DGroup& P = pg.d;
		if(P.type == G_UNC) {
			// an uncompressed group returns an uncompressed group over all output columns that holds U x B[cols, :]
			// (CG/ColGroupUncompressed.java:888-927); the new block owns it
			c->groups.emplace_back();
			HostGroup& g = c->groups.back();
			memset(&g.d, 0, sizeof(g.d));
			g.d.type = G_UNC; g.d.nColG = q;
			g.cols = cols;
			double* dense = nullptr;
			const size_t nOut = (size_t) std::max<int64_t>(b->nRows, 1) * q;
			if(upload(g, cols.data(), sizeof(int32_t) * (size_t) q, (const void**) &g.d.cols) ||
				hipMalloc((void**) &dense, nOut * sizeof(double)) != hipSuccess) {
				set_error("overlapping right multiply: allocating the product of an uncompressed group failed");
				cla_block_free(c);
				return nullptr;
			}
			g.owned.push_back(dense);
			g.d.dense = dense;
			g.bytes = (int64_t) (nOut * sizeof(double));
			if(b->nRows > 0)
				hipLaunchKernelGGL(k_unc_times_b, dim3((unsigned) ((b->nRows * q + 255) / 256)), dim3(256), 0, b->stream, P.dense, b->nRows,
					P.nColG, P.cols, b->dStageIn, q, dense);
			g.d.tblOff = tblOff;
			g.d.colOff = colOff;
			colOff += q;
			c->hasUnc = true;
			continue;
		}
		// groups without row data (const, empty, SDC without entries) live on in the constants only;
		// the group list stays one to one with the source block otherwise, so the arena can be shared
		if(P.type != G_DDC && P.type != G_SDCZ && P.type != G_RLE) {
			if(b->dArena) { set_error("overlapping right multiply: unexpected group in an arena block"); cla_block_free(c); return nullptr; }
			continue;
		}
		c->groups.emplace_back();
		HostGroup& g = c->groups.back();
		g.d = P; // codes, offsets, checkpoints, tile index, run table: borrowed
		g.cols = cols;
		g.d.nColG = q;
		g.dict.assign(T.begin() + (size_t) P.tblOff * q, T.begin() + (size_t) (P.tblOff + P.nVals) * q);
		g.codeOrder = pg.codeOrder;
		g.bytes = 0;
		if(upload(g, cols.data(), sizeof(int32_t) * (size_t) q, (const void**) &g.d.cols) || upload_dict(g)) { cla_block_free(c); return nullptr; }
		g.bytes = pg.bytes; // what a kernel streams for this group
		g.d.tblOff = tblOff;
		g.d.colOff = colOff;
		tblOff += P.nVals;
		colOff += q;
		maxVals = std::max(maxVals, P.nVals);
		if(P.type == G_SDCZ) c->hasSdc = true;
		if(P.type == G_RLE) c->hasRle = true;
	}
	if(b->hasConst) {
		for(int j = 0; j < q; j++) c->constV[j] = T[(size_t) b->totalVals * q + j];
		c->hasConst = true;
	}
	c->totalVals = tblOff;
	c->totalColsG = colOff;
	c->maxVals = maxVals;
	c->parent = b;
	b->refs.fetch_add(1);
	// (products of uncompressed groups were queued on the source block's stream; the new block has its own)
	if(c->hasUnc && hipStreamSynchronize(b->stream) != hipSuccess) { set_error("overlapping right multiply: device failure"); cla_block_free(c); return nullptr; }
	if(finish_finalize(c, b)) { cla_block_free(c); return nullptr; }
	return c;
	CLA_CATCH_NULL
}

int64_t cla_aggregate_dev(cla_handle b, int32_t op, int32_t dir, double* dOut) {
	CLA_TRY
	int rc = check_final(b);
	if(rc) return rc;
	if(!dOut) { set_error("aggregate: null output"); return -CLA_ERR_INVALID; }
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	b->nnzSlot = 0;
	if((rc = launch_aggregate(b, op, dir, dOut, b->dCounters))) return rc;
	return finish_nnz(b);
	CLA_CATCH_CODE(int64_t)
}

int64_t cla_aggregate(cla_handle b, int32_t op, int32_t dir, double* out) {
	CLA_TRY
	int rc = check_final(b);
	if(rc) return rc;
	if(!out) { set_error("aggregate: null output"); return -CLA_ERR_INVALID; }
	if(dir < CLA_AGG_ALL || dir > CLA_AGG_COL) { set_error("aggregate: unknown direction %d", dir); return -CLA_ERR_INVALID; }
	const size_t nOut = dir == CLA_AGG_ALL ? 1 : dir == CLA_AGG_ROW ? (size_t) b->nRows : (size_t) b->nCols;
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	if((rc = ensure_stage(&b->dStageOut, &b->stageOutCap, std::max<size_t>(nOut, 1)))) return rc;
	const int64_t nnz = cla_aggregate_dev(b, op, dir, b->dStageOut);
	if(nnz < 0) return nnz;
	if(nOut) CLA_HIP(hipMemcpy(out, b->dStageOut, nOut * sizeof(double), hipMemcpyDeviceToHost));
	return nnz;
	CLA_CATCH_CODE(int64_t)
}

static int64_t mmchain_dev(cla_handle b, const double* dV, const double* dW, int32_t ctype, double* dOut, bool sync) {
	int rc = check_final(b);
	if(rc) return rc;
	if(!dV || !dOut) { set_error("mmchain: null vector"); return -CLA_ERR_INVALID; }
	if(ctype < 0 || ctype > 2) { set_error("mmchain: chain type %d not supported (XtXv=0, XtwXv=1, XtXvy=2)", ctype); return -CLA_ERR_UNSUPPORTED; }
	if(ctype != 0 && !dW) { set_error("mmchain: XtwXv and XtXvy need w"); return -CLA_ERR_INVALID; }
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	b->nnzSlot = 0;
	if((rc = launch_mmchain(b, dV, dW, ctype, dOut, b->dCounters))) return rc;
	return finish_nnz(b, sync);
}

int64_t cla_mmchain_dev(cla_handle b, const double* dV, const double* dW, int32_t ctype, double* dOut) {
	CLA_TRY
	return mmchain_dev(b, dV, dW, ctype, dOut, true);
	CLA_CATCH_CODE(int64_t)
}

int cla_mmchain_dev_async(cla_handle b, const double* dV, const double* dW, int32_t ctype, double* dOut) {
	CLA_TRY
	return (int) mmchain_dev(b, dV, dW, ctype, dOut, false);
	CLA_CATCH_CODE(int)
}

int64_t cla_mmchain(cla_handle b, const double* v, const double* w, int32_t ctype, double* out) {
	CLA_TRY
	int rc = check_final(b);
	if(rc) return rc;
	if(!v || !out) { set_error("mmchain: null vector"); return -CLA_ERR_INVALID; }
	if((ctype == 1 || ctype == 2) && !w) { set_error("mmchain: XtwXv and XtXvy need w"); return -CLA_ERR_INVALID; }
	const size_t nV = (size_t) b->nCols, nW = ctype == 1 || ctype == 2 ? (size_t) b->nRows : 0;
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	if((rc = ensure_stage(&b->dStageIn, &b->stageInCap, nV + nW)) || (rc = ensure_stage(&b->dStageOut, &b->stageOutCap, nV)))
		return rc;
	CLA_HIP(hipMemcpyAsync(b->dStageIn, v, nV * sizeof(double), hipMemcpyHostToDevice, b->stream));
	if(nW) CLA_HIP(hipMemcpyAsync(b->dStageIn + nV, w, nW * sizeof(double), hipMemcpyHostToDevice, b->stream));
	const int64_t nnz = cla_mmchain_dev(b, b->dStageIn, nW ? b->dStageIn + nV : nullptr, ctype, b->dStageOut);
	if(nnz < 0) return nnz;
	CLA_HIP(hipMemcpy(out, b->dStageOut, nV * sizeof(double), hipMemcpyDeviceToHost));
	return nnz;
	CLA_CATCH_CODE(int64_t)
}

int cla_cooc(cla_handle b, int32_t gA, int32_t gB, int64_t* out) {
	CLA_TRY
	int rc = check_final(b);
	if(rc) return rc;
	const int nG = (int) b->groups.size();
	if(gA < 0 || gA >= nG || gB < 0 || gB >= nG || !out) { set_error("cooc: bad group pair (%d,%d)", gA, gB); return -CLA_ERR_INVALID; }
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	const size_t n = (size_t) b->groups[gA].d.nVals * b->groups[gB].d.nVals;
	if(n == 0) { set_error("cooc: groups without dictionaries"); return -CLA_ERR_UNSUPPORTED; }
	if((rc = ensure_scratch(b, n * sizeof(unsigned long long)))) return rc;
	if((rc = launch_cooc(b, gA, gB, (unsigned long long*) b->dScratch))) return rc;
	CLA_HIP(hipMemcpyAsync(out, b->dScratch, n * sizeof(int64_t), hipMemcpyDeviceToHost, b->stream));
	CLA_HIP(hipStreamSynchronize(b->stream));
	// back to the caller's numbering of the tuples
	const std::vector<int32_t>&oA = b->groups[gA].codeOrder, &oB = b->groups[gB].codeOrder;
	if(!oA.empty() || !oB.empty()) {
		const size_t nA = (size_t) b->groups[gA].d.nVals, nB = (size_t) b->groups[gB].d.nVals;
		std::vector<int64_t> t(out, out + n);
		for(size_t i = 0; i < nA; i++)
			for(size_t j = 0; j < nB; j++)
				out[(oA.empty() ? i : (size_t) oA[i]) * nB + (oB.empty() ? j : (size_t) oB[j])] = t[i * nB + j];
	}
	return 0;
	CLA_CATCH_CODE(int)
}

int cla_preagg(cla_handle b, int32_t group, const double* Y, int32_t nRowY, double* preAgg) {
	CLA_TRY
	int rc = check_final(b);
	if(rc) return rc;
	if(group < 0 || group >= (int) b->groups.size() || !Y || !preAgg || nRowY <= 0) { set_error("preagg: bad arguments"); return -CLA_ERR_INVALID; }
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	const int nVals = b->groups[group].d.nVals;
	if(nVals <= 0) { set_error("preagg: group %d is not pre-aggregable", group); return -CLA_ERR_UNSUPPORTED; }
	const size_t nIn = (size_t) nRowY * b->nRows, nOut = (size_t) nRowY * nVals;
	if((rc = ensure_stage(&b->dStageIn, &b->stageInCap, nIn)) || (rc = ensure_stage(&b->dStageOut, &b->stageOutCap, nOut)))
		return rc;
	if(nIn) CLA_HIP(hipMemcpyAsync(b->dStageIn, Y, nIn * sizeof(double), hipMemcpyHostToDevice, b->stream));
	if((rc = launch_preagg(b, group, b->dStageIn, nRowY, b->dStageOut))) return rc;
	CLA_HIP(hipMemcpyAsync(preAgg, b->dStageOut, nOut * sizeof(double), hipMemcpyDeviceToHost, b->stream));
	CLA_HIP(hipStreamSynchronize(b->stream));
	const std::vector<int32_t>& order = b->groups[group].codeOrder;
	if(!order.empty()) { // back to the caller's numbering of the tuples
		std::vector<double> t((size_t) nVals);
		for(int r = 0; r < nRowY; r++) {
			double* row = preAgg + (size_t) r * nVals;
			std::copy(row, row + nVals, t.begin());
			for(int k = 0; k < nVals; k++) row[order[k]] = t[k];
		}
	}
	return 0;
	CLA_CATCH_CODE(int)
}

int cla_counts(cla_handle b, int32_t group, int32_t* counts) {
	CLA_TRY
	int rc = check_final(b);
	if(rc) return rc;
	if(group < 0 || group >= (int) b->groups.size() || !counts) { set_error("counts: bad group %d", group); return -CLA_ERR_INVALID; }
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	const int nVals = b->groups[group].d.nVals;
	if(nVals <= 0) { set_error("counts: group %d has no dictionary", group); return -CLA_ERR_UNSUPPORTED; }
	if((rc = ensure_scratch(b, sizeof(int32_t) * (size_t) nVals))) return rc;
	if((rc = launch_counts(b, group, (int32_t*) b->dScratch))) return rc;
	CLA_HIP(hipMemcpyAsync(counts, b->dScratch, sizeof(int32_t) * (size_t) nVals, hipMemcpyDeviceToHost, b->stream));
	CLA_HIP(hipStreamSynchronize(b->stream));
	const std::vector<int32_t>& order = b->groups[group].codeOrder;
	if(!order.empty()) { // back to the caller's numbering of the tuples
		std::vector<int32_t> t(counts, counts + nVals);
		for(int k = 0; k < nVals; k++) counts[order[k]] = t[k];
	}
	return 0;
	CLA_CATCH_CODE(int)
}

int cla_block_profile(cla_handle b, int enable) {
	CLA_TRY
	if(!b) { set_error("null block handle"); return -CLA_ERR_INVALID; }
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	b->profile = enable != 0;
	return 0;
	CLA_CATCH_CODE(int)
}

int cla_stats(cla_handle b, char* json, size_t cap) {
	CLA_TRY
	if(!b || !json || cap < 8) return -CLA_ERR_INVALID;
	std::lock_guard<std::recursive_mutex> lk(b->mu);
	if(b->stream) (void) hipStreamSynchronize(b->stream);
	std::string s = "{\"kernels\":[";
	for(size_t i = 0; i < b->lastStats.size(); i++) {
		KernelStat& k = b->lastStats[i];
		if(k.e0 && k.e1 && k.ms < 0) (void) hipEventElapsedTime(&k.ms, k.e0, k.e1);
		char buf[320];
		snprintf(buf, sizeof(buf),
			"%s{\"name\":\"%s\",\"grid\":%ld,\"block\":%ld,\"lds\":%ld,\"algo_bytes\":%.0f,\"ms\":%.6f}", i ? "," : "",
			k.name.c_str(), k.grid, k.block, k.lds, k.algoBytes, (double) k.ms);
		s += buf;
	}
	s += "]}";
	if(s.size() + 1 > cap) return -CLA_ERR_INVALID;
	memcpy(json, s.c_str(), s.size() + 1);
	return 0;
	CLA_CATCH_CODE(int)
}

} // extern "C"
