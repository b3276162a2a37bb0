// Internal declarations shared by the HIP translation units of libclahip.so.
// Nothing here is part of the exported C ABI (see include/cla_hip.h).
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstdio>
#include <mutex>
#include <atomic>
#include <string>
#include <vector>

namespace cla {

enum : int32_t { G_DDC = 0, G_SDCZ = 1, G_RLE = 2, G_UNC = 3 };

// Offset lists are cut into chunks of SDC_CK delta entries; a checkpoint holds
// the iterator state in front of each chunk. Row tiles of SDC_TILE rows have an
// index entry with the iterator state in front of the first entry of the tile.
constexpr int SDC_CK = 1024;
constexpr int SDC_TILE = 1024;
// Bytes allocated (and filled with 0x01) behind every uploaded array: list walkers read whole registers
// from any byte position of an offset or code list without a bounds check.
constexpr int UPLOAD_SLACK = 128;

// Iterator state of an offset list in front of delta entry `idx`:
// `row` = rows accumulated so far (last emitted row plus pending 0-entry skips),
// `emit` = number of rows emitted so far (= data index of the next row).
struct OffState {
	int32_t idx;
	int32_t emit;
	int32_t row;
	int32_t pad;
};

// Device-visible description of one column group (plain data).
struct DGroup {
	const void* codes;        // DDC: nRows codes; SDCZ: nOffsets codes
	const double* dict;       // nVals x nColG, row-major (SDC: dict - default)
	const int32_t* cols;      // nColG global column ids
	const void* deltas;       // SDCZ: delta entries (u8 / u16)
	const OffState* ckpt;     // SDCZ: one per chunk of SDC_CK delta entries
	const OffState* tileIdx;  // SDCZ: one per row tile of SDC_TILE rows
	const int32_t* runStart;  // RLE: nRuns+1 run starts of the merged run table (last = nRows)
	const int32_t* runCode;   // RLE: code per merged run, -1 = uncovered rows
	const double* dense;      // UNC: nRows x nColG row-major
	int64_t nDeltas;
	int64_t nOffsets;
	int32_t type, codeWidth, nVals, nColG;
	int32_t deltaWidth, first, last, nRuns;
	int32_t tblOff;           // first row of this group's table in the concatenated pre-aggregate
	int32_t colOff;           // first column of this group in "decoded column" order
	int32_t nCkpt, nTiles;
};

struct HostGroup {
	DGroup d;                       // host mirror of the device descriptor
	std::vector<int32_t> cols;
	std::vector<double> dict;       // host copy of the (morphed) dictionary
	std::vector<double> def;        // SDC default tuple (empty => none)
	std::vector<int32_t> codeOrder; // renumbered by count at finalize: the caller's code of each code held here (empty => unchanged)
	std::vector<void*> owned;       // device allocations owned by this group
	int64_t bytes = 0;              // HBM bytes of the compressed representation
};

// Per-block switches set through cla_block_set_option. The defaults are the tuned dispatch; the
// other values force one of the alternative kernels of a driver (each is a complete
// implementation of the same product, so forcing one is how the tests cover it).
struct Options {
	int tsmmRoute = 0;      // 0 cost model, 1 one kernel pass per pair of groups, 2 decoded Gram matrix
	int tsmmChunks = 1;     // more than 64 columns: decoded Gram matrices of pairs of column chunks
	int tsmmWideDense = 0;  // more than 64 columns and as many groups as columns: scalar decompressing form
	int tsmmMfma = 1;       // decoded Gram matrix on the matrix cores (0: scalar form)
	int tsmmNarrow = 1;     // decoded Gram matrix: a last column block of at most 4 columns on the 4 x 4 x 4 matrix instruction
	int tsmmPairDot = 1;    // DDC x DDC pairs in dot form (0: pre-aggregate form with LDS bins)
	int expandStreams = 1;  // one code per row for small RLE / SDCZeros groups in the decode kernels
	int tsmmDirect = 1;     // decoded Gram matrix of blocks with few columns besides run-length columns on the vector unit, run-length columns by run (0: the tile kernel on the matrix cores)
	int rmmDirect = 1;      // X %*% B for narrow B on blocks of plain streams: codes straight from global memory, sums on the vector unit (0: the tile kernel on the matrix cores)
	int rmmDisable = 0;     // bit 0 byte-code mat-vec, 1 fused tables of the byte-code mat-vec, 2 matrix-core kernel, 3 decode kernel
	int lmmDisable = 0;     // bit 0 dot form on byte codes, 1 byte-code bin kernel
	int lmmJoint = 1;       // left multiply of blocks that are not mostly offset lists or byte-code DDC groups in one pass over the decoded rows on the matrix cores (k_lmm_decode)
	int sdcPacked = 1;      // packed SDCZeros lists for the mat-vecs
	int sdcLanes = 1;       // SDCZeros mat-vecs on lane-major lists, one lane per group
	int sdcRows = 1;        // SDCZeros right mat-vec on row lists, one lane per row
	int tsmmOneKernel = 1;  // decoded Gram matrix of a whole block as the call's only kernel (0: a fill in front, k_tsmm_finish behind)
	int ddcReorder = 1;     // finalize renumbers the tuples of large DDC dictionaries by descending count (0: the caller's numbering is kept)
};

struct KernelStat {
	std::string name;
	long grid = 0, block = 0, lds = 0;
	double algoBytes = 0;     // compulsory bytes of this launch (0 = not a streaming kernel)
	hipEvent_t e0 = nullptr, e1 = nullptr; // only when profiling is enabled
	float ms = -1.f;
};

struct DecPlanCache;
struct DirPlan;
struct GdrPlan;

} // namespace cla

struct cla_block {
	int64_t nRows = 0;
	int32_t nCols = 0;
	bool finalized = false;
	// A block made by cla_rmm_overlapping borrows the code streams, offset lists, run tables
	// and the code arena of the block it came from: it holds a reference on that block, which
	// is only torn down when the last reference goes.
	cla_block* parent = nullptr;
	std::atomic<int> refs{1};
	bool arenaShared = false;
	// cbind(left, this) made by cla_lmm_compressed for the last `left` it saw (told apart by
	// serial, which is never reused); it borrows both blocks' row data and holds no reference:
	// it is rebuilt when another left block comes and freed with this block.
	uint64_t serial = 0;
	cla_block* joint = nullptr;
	uint64_t jointSerial = 0;
	int32_t crossSplit = 0;          // > 0: joint block, groups [0, crossSplit) are the left side's
	int32_t crossBlocks = 0;         // > 0: the left side's columns fill the first crossBlocks blocks of 16 columns (padded) and only left x right is read
	int32_t crossCol = 0;            // joint block: first column of the right side
	// blocks of pairs of column chunks for t(X) %*% X on more than 64 columns (launch_tsmm_chunked): built on
	// first use, they borrow this block's row data and are freed with it
	std::vector<void*> subs;
	// blocks of column chunks for Y %*% X on the decode kernel (launch_lmm_chunked), likewise; lmmSubWidth: columns
	// per chunk they were cut for, 0 not tried yet, -1 no width fits
	std::vector<void*> lmmSubs;
	int lmmSubWidth = 0;
	std::vector<cla::HostGroup> groups;
	std::vector<double> constV;      // filtered constants (SDC defaults, const groups), nCols
	bool hasConst = false;
	bool hasUnc = false, hasSdc = false, hasRle = false;
	int32_t totalVals = 0;           // sum of nVals over groups (+1 row for constV)
	int32_t totalColsG = 0;          // sum of nColG over groups
	int32_t maxVals = 0;
	int64_t device_bytes_cached = 0; // HBM bytes of the compressed representation (set at finalize)
	int64_t derivedBytes = 0;        // HBM bytes of the formats derived from it so far (packed lists, expanded streams, padded dictionaries, counts)

	hipStream_t stream = nullptr;
	bool ownStream = false;
	std::recursive_mutex mu;

	cla::DGroup* dGroups = nullptr;  // device array of descriptors
	double* dConstV = nullptr;       // device copy of constV (nCols)
	double* dAllDict = nullptr;      // all (morphed) dictionaries back to back in group order

	// All-DDC blocks of one code width keep their code streams in one arena with a
	// uniform stride, so kernels address stream g as arena + g * arenaStride.
	uint8_t* dArena = nullptr;
	size_t arenaStride = 0;
	int32_t arenaWidth = 0;
	int32_t* dTblOff = nullptr;      // nGroups+1 table offsets (prefix sum of nVals)

	// mat-vec gather kernel: groups packed into LDS-sized slabs (g0, g1, table stride, 0)
	std::vector<int4> q1Slabs;
	int4* dQ1Slabs = nullptr;
	int32_t q1LdsBytes = 0;
	int32_t q1Threads = 256;         // threads per block of k_rmm_q1_ddc: 512 or 1024 where only then 8 tables fit a slab

	// reusable workspaces
	double* dTables = nullptr;  size_t tablesCap = 0;
	double* dStageIn = nullptr; size_t stageInCap = 0;
	double* dStageOut = nullptr; size_t stageOutCap = 0;
	void* dScratch = nullptr;   size_t scratchCap = 0;
	double* dChain = nullptr;   size_t chainCap = 0;   // X %*% v inside the multiply chain
	// exact code counts of all dictionary-coded groups (totalVals int32, group g at tblOff[g]),
	// computed on the first TSMM and kept, like the reference's cached counts
	// (CG/AColGroupValue.java getCounts)
	int32_t* dCountsAll = nullptr;
	double* dOnes = nullptr;         // nCols ones: rowSums(X) = X %*% 1
	// one code per row (0xff = row without a value) of RLE / SDCZeros groups with at most 255 tuples,
	// expanded once for the decode kernels when that costs at most half the block's own bytes
	std::vector<uint8_t*> expCodes;
	bool expTried = false;
	// all groups single-column DDC with byte codes: dictionaries at a fixed stride of 256 entries
	// (zero beyond nVals) followed by the groups' column indexes; built on first use
	double* dDictPad = nullptr;
	int64_t dictPadBytes = 0;
	// list of SDCZeros groups + prefix sums of their nVals, as the row-tile kernels read it;
	// built on first use for all groups (sdcPlanGroup -1) or for one group (its index)
	int32_t* dSdcPlan = nullptr;
	void* dSdcDesc = nullptr;        // one compact descriptor per listed group (k_*_sdc_packed)
	void* dLaneMeta = nullptr;       // lane-per-group kernels (k_sdc_lanes.hip): descriptors, slabs, dictionaries, table index, chunk starts
	void* dLaneData = nullptr;       // the listed groups' lists as lane-major windows, built on first use
	int laneState = 0;               // 0 not planned yet, 1 ready, -1 the lists do not fit these kernels
	int laneSlabs = 0, laneDictLds = 0, laneDictTotal = 0; // slabs, dictionary entries of the largest slab / of all
	size_t laneOff[5] = {0, 0, 0, 0, 0};
	bool laneLmm = false;            // every listed group has one column (the left multiply's condition)
	cla::DecPlanCache* decPlans = nullptr; // decode kernels (k_rmm_decode.hip): plans per product shape, dropped by dec_plans_drop
	cla::DirPlan* dirPlan = nullptr;     // plan of k_rmm_direct (dropped with the decode plans)
	cla::GdrPlan* gdrPlan = nullptr;     // plan of k_tsmm_direct (likewise)
	void* dMfPlan = nullptr;         // matrix-core right multiply (k_rmm_mfma.hip): slab descriptors, column info, code streams, B row list
	int mfState = 0;                 // 0 not planned yet, 1 ready, -1 not eligible
	int mfNSlabs = 0, mfNColsAll = 0, mfWidth = 1, mfMaxKc = 0, mfNRowCol = 0, mfMaxDict = 0;
	size_t mfBufBytes = 0, mfOff[4] = {0, 0, 0, 0};
	void* dRowsMeta = nullptr;       // row-list right multiply (k_sdc_rows.hip): table index, group list, headers, row order
	void* dRowsData = nullptr;       // the listed groups' entries as row lists, built on first use
	int rowsState = 0, rowsTbl = 0;  // 0 not planned yet, 1 ready, -1 the lists do not fit; table entries of all listed groups
	size_t rowsOff[2] = {0, 0};
	size_t rowsColOff = 0;           // the table entries' columns inside dRowsMeta
	bool rowsFusable = false;        // the row-list kernel can make its tables itself (single-column lists only, nothing else in the block)
	bool sdcPackFailed = false;
	bool dictNonFinite = false;      // some dictionary holds an infinity or a NaN (set at finalize): the left multiply then sums Y per tuple first, as the reference does
	bool lmmTailWanted = false;      // left multiply: a kernel that serves the whole block may count the result's non-zeros itself (no constants to add)
	bool lmmTailDone = false;        // ... and one has: no finishing kernel behind it
	bool preUsed = false;            // left multiply: some kernel of the call wrote pre-aggregates (k_lmm_post has work)
	uint32_t* dSdcPacked = nullptr;  // all listed groups' entries as (code << 16 | row inside its 4096-row tile), built on first use
	int sdcPlanGroup = -2;
	std::vector<int32_t> sdcList, sdcBinOff;
	unsigned long long* dCounters = nullptr;   // 8 x u64: 0 - 3 non-zero counts, 6 and 7 ticket counters of the left multiply's and the Gram kernels' tails
	double* dGramAcc = nullptr;      // nCols x nCols, zero between calls: where the blocks of a one-kernel t(X) %*% X add (gram_tail)
	unsigned long long* hCounters = nullptr;   // pinned

	std::vector<cla::KernelStat> lastStats;
	bool profile = false;            // bracket every kernel with HIP events on `stream`
	cla::Options opt;
	// Non-zero counter of the last driver call: index into dCounters. Slot 0 is cleared by the first
	// kernel of a driver; the fused mat-vec kernel rotates over slots 1-3 instead (it counts into one
	// and clears the next, so that no separate clearing step runs between two calls).
	int nnzSlot = 0;
	int nnzRot = 1;
	bool poisoned = false;           // a failed finalize left the block half built: only free is allowed
};

namespace cla {

void set_error(const char* fmt, ...);
extern int g_ldsPerBlock;   // usable LDS bytes per workgroup
// Lets a kernel take up to the device's LDS per workgroup as dynamic shared memory; said once per kernel (a value
// per call could be lowered by a caller on another handle between a call's setting and its launch).
hipError_t allow_full_lds(const void* kernel);
extern int g_numCU;

#define CLA_HIP(expr)                                                                              \
	do {                                                                                           \
		hipError_t _e = (expr);                                                                    \
		if(_e != hipSuccess) {                                                                     \
			cla::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), __FILE__, __LINE__); \
			return -CLA_ERR_DEVICE;                                                                \
		}                                                                                          \
	} while(0)

// ---- launchers implemented in the kernel translation units ----
int launch_validate_codes(cla_block* b, const void* codes, int width, int64_t n, int nVals, int* ok);
int launch_counts(cla_block* b, int group, int32_t* dCounts);
int reorder_ddc_by_count(cla_block* b, int group);
int launch_sdc_build(cla_block* b, HostGroup& g);
int launch_rmm(cla_block* b, const double* dB, int q, double* dOut, unsigned long long* dNnz, int squares = 0,
	double* ws = nullptr, size_t wsDoubles = 0);
int launch_tables(cla_block* b, const double* dB, int q); // dict x B of every group (+ constV x B) into b->dTables
int launch_aggregate(cla_block* b, int op, int dir, double* dOut, unsigned long long* dNnz);
int ensure_counts(cla_block* b);
int launch_rmm_mfma(cla_block* b, const double* dB, int q, const double* dConstRow, double* dOut,
	unsigned long long* dNnz);
int launch_lmm_u8(cla_block* b, const double* dY, int p, double* dPre);
int launch_lmm_u8_dot(cla_block* b, const double* dY, int p, double* dOut);
int launch_lmm_sdc_tiles(cla_block* b, const double* dY, int p, double* dPre, int onlyGroup, double* dOut);
int launch_lmm_sdc_lanes(cla_block* b, const double* dY, int p, double* dOut);
int sdc_plan_all(cla_block* b); // the list of the block's SDCZeros groups with entries (b->sdcList)
int launch_rmm_sdc_lanes(cla_block* b, int constRow, int accumulate, double* dOut, unsigned long long* dNnz);
int launch_rmm_sdc_rows(cla_block* b, int constRow, int accumulate, double* dOut, unsigned long long* dNnz, const double* dU = nullptr,
	unsigned long long* nnzNext = nullptr);
bool rows_fusable(cla_block* b);
int launch_rmm_sdc_tiles(cla_block* b, int q, int constRow, int accumulate, double* dOut, unsigned long long* dNnz);
int launch_tsmm_decode(cla_block* b, double* dOut, unsigned long long* dNnz = nullptr);
int launch_tsmm_direct(cla_block* b, double* dOut, unsigned long long* dNnz = nullptr);
int ensure_gram_acc(cla_block* b); // the zeroed nCols x nCols accumulator of the one-kernel t(X) %*% X (a workspace kept with the block)
int ensure_expanded(cla_block* b);
int launch_rmm_decode(cla_block* b, const double* dB, int q, const double* dConstRow, double* dOut,
	unsigned long long* dNnz);
int launch_decompress(cla_block* b, double* dOut, unsigned long long* dNnz);
int launch_decompress_rows(cla_block* b, int64_t r0, int64_t r1, double* dOut);
int launch_rmm_decompressed(cla_block* b, const double* dB, int q, double* dOut, unsigned long long* dNnz);
void dec_plans_drop(cla_block* b);
int tsmm_decode_fits(cla_block* b);
int launch_lmm_decode(cla_block* b, const double* dY, int p, double* dOut, unsigned long long* dBad);
int launch_lmm_joint(cla_block* b, const double* dY, int p, double* dOut, unsigned long long* dNnz);
int launch_lmm(cla_block* b, const double* dY, int p, double* dOut, unsigned long long* dNnz);
int launch_preagg(cla_block* b, int group, const double* dY, int p, double* dPre);
int launch_tsmm(cla_block* b, double* dOut, unsigned long long* dNnz);
int launch_tsmm_chunked(cla_block* b, double* dOut);
int launch_cooc(cla_block* b, int gA, int gB, unsigned long long* dOut);
int launch_mmchain(cla_block* b, const double* dV, const double* dW, int ctype, double* dOut,
	unsigned long long* dNnz);

// Scope around one kernel launch: records launch geometry and, when the block is
// in profiling mode, HIP events on the block's stream in front of and behind it.
struct Prof {
	cla_block* b;
	size_t idx;
	Prof(cla_block* b, const char* name, long grid, long block, long lds, double algoBytes);
	~Prof();
};
void clear_stats(cla_block* b);

int ensure_tables(cla_block* b, size_t nDoubles);
int ensure_dict_pad(cla_block* b); // padded dictionary image of byte-code blocks with one column per group (no-op otherwise)
int ensure_scratch(cla_block* b, size_t bytes);

} // namespace cla
