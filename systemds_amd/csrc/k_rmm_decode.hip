// Decode-and-multiply on blocks of any group mix, on the matrix cores:
//   k_rmm_decode      X %*% B for narrow B (q <= 16; a single column where the block is not mostly offset lists;
//               wider B 16 columns per pass)
//   k_tsmm_decode<NB> upper triangle of t(X) %*% X for blocks of at most 16 * NB <= 64 columns (or, for a pair of
//               column chunks, only the tiles of the first chunk's column blocks with the second's)
//   k_lmm_decode<NB>  Y %*% X for such blocks, 16 rows of Y per pass: the Gram kernel with Y as the other operand
// and, further down, for blocks whose groups are all plain streams, on the vector unit and without code tiles:
//   k_rmm_direct<q>   X %*% B, codes read straight from global memory (wider B 16 columns per pass)
// A block owns a contiguous range of 1024-row tiles. Per tile every dictionary coded
// group gets its codes expanded into an LDS code tile (DDC: straight copy, prefetched one
// tile ahead in registers together with the rows of uncompressed groups; SDCZeros:
// wave-wide offset decode from the tile index; RLE: run expansion with the run cursor
// carried from tile to tile). The waves then look decoded values up (code tile ->
// dictionary copy in LDS, or the dense tile) straight into v_mfma_f64_16x16x4_f64 operands:
//   X %*% B:    A operand = 16 rows x 4 decoded columns, B operand = 4 rows of B (padded to
//               16 outputs); 64 (or 32) output rows per wave and pass, staged per wave in LDS and
//               written with full-line stores.
//   t(X) %*% X: lane l holds column 16 cb + l % 16 of row l / 16, which is both operands; the
//               NB (NB + 1) / 2 upper 16 x 16 tiles of the Gram matrix stay in registers until
//               the block has walked all its row tiles.
// (Wide B on all-DDC blocks uses k_rmm_mfma instead.)
#include "../../include/cla_hip.h"
#include "cla_runs.hpp"
#include <algorithm>
#include <cstring>
#include <type_traits>

namespace cla {

constexpr int DEC_THREADS = 512;
constexpr int DEC_WAVES = DEC_THREADS / 64;
constexpr int DEC_TILE = SDC_TILE;     // rows per tile = granularity of the offset tile index
constexpr int DEC_WROWS = DEC_TILE / DEC_WAVES; // rows of a tile one wave multiplies
constexpr int DEC_QMAX = 16;
constexpr int DEC_PF = 6;              // 16-byte chunks a thread holds for the next tile
constexpr int DEC_WIN = 2048;           // bytes of an offset list / of its codes kept in LDS per SDC group
constexpr int DEC_TWIN = 32;            // tile index entries kept in LDS per SDC group
constexpr int DEC_SLOT_PAD = 80;       // bytes between code tiles: spreads the columns a wave reads together over the LDS banks

struct DecGroup {
	int32_t type;
	int32_t nC;
	int32_t dictOff;   // doubles from the LDS base: dictionary copy, or the dense tile of an uncompressed group
	int32_t slotOff;   // bytes, into the LDS code tiles (-1: no code tile)
	int32_t slotW;     // 1 or 2 bytes per code in the tile; all ones = row has no value
	int32_t kOff;      // first decoded column of the group (row of the LDS copy of B)
	int32_t copyIdx;   // tile filled by the chunk copy list (index), else -1
	int32_t pad;       // bytes from the LDS base: run window (RLE) / list windows (SDCZeros) of a wave task
};

// Chunk copy list: what is a plain copy of consecutive global bytes per tile (DDC codes
// whose width is the tile's, rows of uncompressed groups), in 16-byte chunks.
struct DecCopy {
	const uint8_t* src;   // first byte of row 0
	int32_t chunk0;       // first chunk of this entry in the flattened chunk numbering
	int32_t bpr;          // bytes per row
	int32_t dstOff;       // bytes from the LDS base
	int32_t pad;
};

// One decoded column as the multiply phase sees it (16 bytes, read from LDS per use).
struct DecCol {
	int32_t slotOff;   // dictionary coded: code tile (bytes into the code tiles)
	int32_t valOff;    // doubles from the LDS base: dictionary copy / dense tile
	int32_t meta;      // kind (0 none or constant only, 1 dictionary coded with a no-value code, 2 dense, 3 dictionary coded on every row) | two-byte codes << 2 | dictionary in global memory << 3 | nC << 4 | h << 18
	int32_t pad;       // group
};

struct DecArgs {
	const DGroup* groups;
	const DecGroup* plan;
	const DecCopy* copies;
	const DecCol* cols;
	const int32_t* tasks;              // wave tasks: DEC_WAVES + 1 list offsets, then group ids per wave
	int nTasks;
	const double* colConst;            // t(X) %*% X: constant part per (padded) column
	int nGroups, nCopies, nChunks;     // nChunks: 16-byte chunks per tile over the copy list
	int nColD;                         // entries of cols (multiple of 4 / of 16)
	int valDoubles, bDoubles, stageDoubles, slotBytes; // LDS sizes
	const double* B;
	int q;
	int ld;                            // columns of B and of the output (>= q: wide B goes in passes of 16 columns)
	const double* constRow;
	const double* Y;                   // left multiply: Y (P x nRows, row-major); out is P x nCols
	int P;
	unsigned long long* badY;          // left multiply: set when Y holds a value that is not finite
	double* out;
	int64_t nRows;
	unsigned long long* nnz;
	int nCols;
	double* acc;                       // t(X) %*% X as the call's only kernel: the blocks add here and the last one writes out (gram_tail)
	unsigned* done;                    // its ticket counter (nullptr: the blocks add into out, the caller fills and finishes)
};

typedef double f64x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void dec_store_code(uint8_t* slot, int w, int i, int code) {
	if(w == 1) slot[i] = (uint8_t) code;
	else ((uint16_t*) slot)[i] = (uint16_t) code;
}

// LDS traffic of one wave is ordered; this keeps the compiler from moving accesses across
__device__ __forceinline__ void dec_wave_sync() {
	__builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
	__builtin_amdgcn_wave_barrier();
	__builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// One decoded column, unpacked once per pass; lookups are then branch-free selects.
struct DecLook {
	int base;      // valOff + h
	int nC;
	int sent;      // no-value code of the column's tile; -1 when the column has no code tile
	bool coded, dense, two;
	__device__ __forceinline__ DecLook(const DecCol D) {
		const int kind = D.meta & 3;
		coded = kind == 1 || kind == 3; dense = kind == 2; two = (D.meta & 4) != 0;
		nC = (D.meta >> 4) & 0x3fff;
		base = D.valOff + (int) ((unsigned) D.meta >> 18);
		sent = kind == 1 ? (two ? 0xffff : 0xff) : -1; // (kind 3: every row has a code, all code values are valid)
	}
	// LDS index (doubles) of the value at tile row rt with code c, and whether the row has one.
	// Rows behind the end of the matrix (in == false) hold stale codes: never used as an index.
	__device__ __forceinline__ int addr(int c, int rt, bool in, bool& valid) const {
		valid = in & (dense | (coded & (c != sent)));
		const int a = base + (coded ? c : rt) * nC;
		return valid ? a : 0;
	}
};

// 64 runs from run wb of an RLE group into its LDS window (starts | ends | codes)
__device__ __forceinline__ void dec_load_runs(int32_t* win, const DGroup& G, int wb, int lane) {
	const int jj = wb + lane;
	const bool inTable = jj < G.nRuns;
	win[lane] = inTable ? G.runStart[jj] : 0x7fffffff;
	win[64 + lane] = inTable ? G.runStart[jj + 1] : 0x7fffffff;
	win[128 + lane] = inTable ? G.runCode[jj] : -1;
}

// DEC_WIN bytes of a stream from byte offset off (multiple of 16) into an LDS window; bytes
// at and beyond `total` are not read.
__device__ __forceinline__ void dec_load_window(uint8_t* win, const uint8_t* src, int64_t off, int64_t total, int lane) {
#pragma unroll
	for(int p = 0; p < DEC_WIN / 1024; p++) {
		const int o = (p * 64 + lane) * 16;
		if(off + o + 16 <= total) *(u32x4*) (win + o) = *(const u32x4*) (src + off + o);
		else
			for(int e = 0; e < 16; e++)
				if(off + o + e < total) win[o + e] = src[off + o + e];
	}
}

// FLAT: dictionaries that do not fit LDS stay in global memory; the lookups then go through
// generic pointers (LDS or global per lane).
// Lanes 4 u .. 4 u + 3 of every 16 lanes (bank u) copied into the other three banks of the 16.
// row_shr:4 d moves a bank d banks up, row_shl:4 d moves it d banks down; the bank mask picks the receiving bank.
__device__ __forceinline__ int dec_spread_bank(int o, int u) {
	int a = o;
	switch(u) {
		case 0:
			a = __builtin_amdgcn_update_dpp(a, o, 0x114, 0xf, 0x2, false);
			a = __builtin_amdgcn_update_dpp(a, o, 0x118, 0xf, 0x4, false);
			a = __builtin_amdgcn_update_dpp(a, o, 0x11c, 0xf, 0x8, false);
			break;
		case 1:
			a = __builtin_amdgcn_update_dpp(a, o, 0x104, 0xf, 0x1, false);
			a = __builtin_amdgcn_update_dpp(a, o, 0x114, 0xf, 0x4, false);
			a = __builtin_amdgcn_update_dpp(a, o, 0x118, 0xf, 0x8, false);
			break;
		case 2:
			a = __builtin_amdgcn_update_dpp(a, o, 0x108, 0xf, 0x1, false);
			a = __builtin_amdgcn_update_dpp(a, o, 0x104, 0xf, 0x2, false);
			a = __builtin_amdgcn_update_dpp(a, o, 0x114, 0xf, 0x8, false);
			break;
		default:
			a = __builtin_amdgcn_update_dpp(a, o, 0x10c, 0xf, 0x1, false);
			a = __builtin_amdgcn_update_dpp(a, o, 0x108, 0xf, 0x2, false);
			a = __builtin_amdgcn_update_dpp(a, o, 0x104, 0xf, 0x4, false);
			break;
	}
	return a;
}

// LM (with GRAM): Y %*% X instead of t(X) %*% X. The decoded rows are the B operand as before, the A operand is Y
// (lane l: row l % 16 of Y at matrix row ... + l / 16), read straight from global memory, 16 consecutive values per lane
// and half; one 16 x 16 tile per column block.
template <int GRAM, int NB, int RPL, int FLAT, int XB = 0, int NAR = 0, int LM = 0>
__device__ __forceinline__ void decode_body(const DecArgs& A) {
	extern __shared__ __align__(16) double smem[];
	double* Bs = smem + A.valDoubles;                              // bDoubles: rows of B in decoded column order, 16 outputs each
	double* stage = GRAM ? smem : Bs + A.bDoubles;                 // stageDoubles: output staging per wave; the Gram tile takes the place of the values when the rows are done
	uint8_t* slots = (uint8_t*) (Bs + A.bDoubles + A.stageDoubles); // slotBytes (multiple of 16)
	DecCol* colS = (DecCol*) (slots + A.slotBytes);                // nColD
	double* constS = (double*) (colS + A.nColD);                   // nColD (Gram mode)
	DecGroup* planS = (DecGroup*) (constS + (GRAM ? A.nColD : 0)); // nGroups
	DecCopy* copyS = (DecCopy*) (planS + A.nGroups);               // nCopies
	DGroup* groupS = (DGroup*) (copyS + A.nCopies);                // nGroups: descriptors, so that a wave task starts from LDS
	int32_t* runBase = (int32_t*) (groupS + A.nGroups);            // nGroups
	int32_t* taskS = runBase + A.nGroups;                          // DEC_WAVES + 1 + nTasks
	const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
	const int i16 = lane & 15, k4 = lane >> 4;
	const DGroup* __restrict__ groups = A.groups;
	const int nGroups = A.nGroups;
	const int64_t nRows = A.nRows;

	const int nTiles = (int) ((nRows + DEC_TILE - 1) / DEC_TILE);
	const int tileBeg = (int) ((int64_t) nTiles * blockIdx.x / gridDim.x);
	const int tileEnd = (int) ((int64_t) nTiles * (blockIdx.x + 1) / gridDim.x);
	if(tileBeg >= tileEnd) return;

	// ---- once per block: plan, column descriptors, dictionaries, B, run cursors
	for(int g = tid; g < nGroups; g += DEC_THREADS) {
		planS[g] = A.plan[g];
		groupS[g] = groups[g];
		runBase[g] = groups[g].type == G_RLE ? rle_find(as_global(groups[g].runStart), groups[g].nRuns, (int32_t) ((int64_t) tileBeg * DEC_TILE)) : 0;
	}
	for(int i = tid; i < A.nCopies; i += DEC_THREADS) copyS[i] = A.copies[i];
	for(int i = tid; i < DEC_WAVES + 1 + A.nTasks; i += DEC_THREADS) taskS[i] = A.tasks[i];
	for(int i = tid; i < A.nColD; i += DEC_THREADS) {
		colS[i] = A.cols[i];
		if(GRAM) constS[i] = A.colConst[i];
	}
	for(int i = tid; i < A.valDoubles; i += DEC_THREADS) smem[i] = 0.0;
	if(!GRAM)
		for(int i = tid; i < A.bDoubles; i += DEC_THREADS) Bs[i] = 0.0;
	__syncthreads();
	for(int g = 0; g < nGroups; g++) {
		const DecGroup P = planS[g];
		const DGroup G = dgroup(groups + (g));
		if(P.slotOff >= 0 && P.dictOff >= 0) {
			const int n = G.nVals * G.nColG;
			for(int i = tid; i < n; i += DEC_THREADS) smem[P.dictOff + i] = G.dict[i];
		}
		if(!GRAM)
			for(int i = tid; i < P.nC * A.q; i += DEC_THREADS) {
				const int h = i / A.q, c = i - h * A.q;
				Bs[(size_t) (P.kOff + h) * 16 + c] = A.B[(size_t) G.cols[h] * A.ld + c];
			}
	}

	// wave task windows: first 64 runs from the run cursor; list windows start empty
	for(int t = taskS[wave]; t < taskS[wave + 1]; t++) {
		const int g = taskS[DEC_WAVES + 1 + t];
		const DecGroup P = planS[g];
		if(P.type == G_RLE) dec_load_runs((int32_t*) ((uint8_t*) smem + P.pad), dgroup(groupS + g), runBase[g], lane);
		else if(P.type == G_SDCZ && lane < 3)
			((int32_t*) ((uint8_t*) smem + P.pad + DEC_TWIN * sizeof(OffState) + 2 * DEC_WIN))[lane] = -(1 << 30);
	}
	dec_wave_sync();

	// Copy list chunks of one tile, flattened: chunk i of a thread is tid + k * DEC_THREADS,
	// so its entry and place in the tile never change. Whole chunks are loaded as 16 bytes
	// one tile ahead; the ragged end of the last tile is copied byte-wise.
	auto chunk_place = [&](int i, const uint8_t*& src, int& dstOff, int& bpr, int& off) {
		int lo = 0, hi = A.nCopies - 1;
		while(lo < hi) {
			const int mid = (lo + hi + 1) >> 1;
			if(copyS[mid].chunk0 <= i) lo = mid; else hi = mid - 1;
		}
		const DecCopy C = copyS[lo];
		off = (i - C.chunk0) * 16;
		bpr = C.bpr;
		src = as_global(C.src + off);
		dstOff = C.dstOff + off;
	};
	uint8_t* const ldsBytes = (uint8_t*) smem;
	auto copy_ragged = [&](const uint8_t* src, int dstOff, int64_t nValid) {
		for(int e = 0; e < 16; e++)
			if(e < nValid) ldsBytes[dstOff + e] = src[e];
	};
	const uint8_t* pfSrc[DEC_PF];
	int pfDst[DEC_PF], pfBpr[DEC_PF], pfOff[DEC_PF];
	u32x4 pf[DEC_PF];
#pragma unroll
	for(int k = 0; k < DEC_PF; k++) {
		pfSrc[k] = nullptr; pfDst[k] = 0; pfBpr[k] = 1; pfOff[k] = 0;
		if(tid + k * DEC_THREADS < A.nChunks) chunk_place(tid + k * DEC_THREADS, pfSrc[k], pfDst[k], pfBpr[k], pfOff[k]);
	}
	// bytes of a tile's share of a copy entry that lie inside the matrix
	auto tile_bytes = [&](int64_t t0, int bpr) { return min((int64_t) DEC_TILE, nRows - t0) * bpr; };
	auto prefetch = [&](int tile) {
		const int64_t t0 = (int64_t) tile * DEC_TILE;
#pragma unroll
		for(int k = 0; k < DEC_PF; k++) {
			pf[k] = u32x4{0, 0, 0, 0};
			if(pfSrc[k] != nullptr && pfOff[k] + 16 <= tile_bytes(t0, pfBpr[k]))
				pf[k] = __builtin_nontemporal_load((const u32x4*) (pfSrc[k] + t0 * pfBpr[k]));
		}
	};
	prefetch(tileBeg);

	// multiply phase state
	// tiles of the Gram matrix held by a wave: the upper triangle, or with XB > 0 (only the product of the first
	// XB column blocks with the others is wanted) those XB x (NB - XB) tiles
	// NAR (the last column block holds at most 4 columns): 16 x 16 tiles only among the NB - 1 full blocks; the
	// rows of the last block come from v_mfma_f64_4x4x4_f64, one instruction per column block (its four 4 x 4 x 4
	// products are the last block's 4 columns against the 4 quarters of a 16-column block), which issues at four
	// times the rate of a 16 x 16 tile and replaces NB of them.
	static_assert(!NAR || (GRAM && XB == 0 && NB >= 2), "narrow last block: full Gram matrices only");
	static_assert(!LM || (GRAM && XB == 0 && NAR == 0), "left multiply: one tile per column block");
	constexpr int NF = NAR ? NB - 1 : NB; // column blocks among which 16 x 16 tiles are computed
	constexpr int NTILES = !GRAM ? 1 : LM ? NB : XB > 0 ? XB * (NB - XB) : NF * (NF + 1) / 2;
	bool badY = false;
	f64x4 gram[NTILES];
	double nar[NAR ? NB : 1]; // lane l: cell (row 16 (NB - 1) + l / 16, column 16 cb + l % 16)
	if(GRAM) {
#pragma unroll
		for(int t = 0; t < NTILES; t++) gram[t] = f64x4{0.0, 0.0, 0.0, 0.0};
#pragma unroll
		for(int cb = 0; cb < (NAR ? NB : 1); cb++) nar[cb] = 0.0;
	}
	const int q = A.q;
	const double cinit = (!GRAM && A.constRow != nullptr && i16 < q) ? A.constRow[i16] : 0.0;
	double* const wstage = stage + (size_t) wave * 16 * RPL * (GRAM ? 0 : q);
	const int KB = A.nColD >> 2;

	int cnt = 0;
	for(int tile = tileBeg; tile < tileEnd; tile++) {
		const int64_t t0 = (int64_t) tile * DEC_TILE;
		const int64_t rEnd = t0 + DEC_TILE;
		__syncthreads(); // previous tile's readers are done with the code and dense tiles
		// ---- copy list: prefetched chunks, then what did not fit the prefetch registers
#pragma unroll
		for(int k = 0; k < DEC_PF; k++) {
			if(pfSrc[k] == nullptr) continue;
			const int64_t tb = tile_bytes(t0, pfBpr[k]);
			if(pfOff[k] + 16 <= tb) *(u32x4*) (ldsBytes + pfDst[k]) = pf[k];
			else copy_ragged(pfSrc[k] + t0 * pfBpr[k], pfDst[k], tb - pfOff[k]);
		}
		for(int i = tid + DEC_PF * DEC_THREADS; i < A.nChunks; i += DEC_THREADS) {
			const uint8_t* src; int dstOff, bpr, off;
			chunk_place(i, src, dstOff, bpr, off);
			const int64_t tb = tile_bytes(t0, bpr);
			if(off + 16 <= tb) *(u32x4*) (ldsBytes + dstOff) = __builtin_nontemporal_load((const u32x4*) (src + t0 * bpr));
			else copy_ragged(src + t0 * bpr, dstOff, tb - off);
		}

		// ---- other dictionary coded groups: the wave's share of the task list, one group at a time
		for(int t = taskS[wave]; t < taskS[wave + 1]; t++) {
			const int g = taskS[DEC_WAVES + 1 + t];
			const DecGroup P = planS[g];
			const DGroup G = dgroup(groupS + g);
			uint8_t* slot = slots + P.slotOff;
			const int w = P.slotW;
			if(P.type == G_DDC) { // code width differs from the tile's: convert
				for(int i = lane; i < DEC_TILE; i += 64)
					if(t0 + i < nRows) dec_store_code(slot, w, i, load_code(G.codes, G.codeWidth, t0 + i));
			}
			else if(P.type == G_RLE) {
				// window of 64 runs in LDS, reloaded when it no longer reaches the end of the tile
				int32_t* win = (int32_t*) (ldsBytes + P.pad);
				int wb = runBase[g];
				while(true) {
					const bool inTable = wb + lane < G.nRuns;
					const int32_t s = win[lane], e = win[64 + lane], code = win[128 + lane];
					const bool ov = inTable && s < rEnd && e > t0;
					unsigned long long valid = __ballot(ov);
					if(__popcll(valid) <= 8) { // long runs: all lanes write each run
						while(valid) {
							const int k = __ffsll((long long) valid) - 1;
							valid &= valid - 1;
							const int sk = max((int) (__shfl(s, k, 64) - t0), 0);
							const int ek = (int) (min((int64_t) __shfl(e, k, 64), rEnd) - t0);
							const int ck = __shfl(code, k, 64);
							for(int i = sk + lane; i < ek; i += 64) dec_store_code(slot, w, i, ck);
						}
					}
					else if(ov) { // short runs: one run per lane
						const int sk = max((int) (s - t0), 0);
						const int ek = (int) (min((int64_t) e, rEnd) - t0);
						for(int i = sk; i < ek; i++) dec_store_code(slot, w, i, code);
					}
					if(__ballot(inTable && e >= rEnd) != 0 || wb + 64 >= G.nRuns) break;
					wb += 64;
					dec_wave_sync();
					dec_load_runs(win, G, wb, lane);
					dec_wave_sync();
				}
				if(lane == 0) runBase[g] = wb;
			}
			else { // SDCZeros: rows without an entry hold the no-value code
				for(int i = lane; i < DEC_TILE; i += 64) dec_store_code(slot, w, i, 0xffff);
				if(G.nOffsets <= 0) continue;
				// same-wave LDS writes are ordered, no barrier needed between fill and scatter
				if(lane == 0 && G.first >= t0 && G.first < rEnd) dec_store_code(slot, w, (int) (G.first - t0), load_code(G.codes, G.codeWidth, 0));
				if(tile < G.nTiles) {
					// windows of the tile index, the delta list and the codes in LDS: a refill every few
					// tiles instead of three dependent global loads per tile
					uint8_t* wbase = ldsBytes + P.pad;
					OffState* tw = (OffState*) wbase;
					uint8_t* dwin = wbase + DEC_TWIN * sizeof(OffState);
					uint8_t* cwin = dwin + DEC_WIN;
					int32_t* wst = (int32_t*) (cwin + DEC_WIN); // dBase, cBase, tBase
					int dBase = wst[0], cBase = wst[1], tBase = wst[2];
					if(tile < tBase || tile >= tBase + DEC_TWIN) {
						tBase = tile;
						dec_wave_sync();
						if(lane < DEC_TWIN) tw[lane] = G.tileIdx[min(tile + lane, G.nTiles - 1)];
						dec_wave_sync();
					}
					const OffState st = tw[tile - tBase];
					int32_t row = st.row, emit = st.emit;
					int64_t i0 = st.idx;
					const int dN = DEC_WIN / G.deltaWidth, cN = DEC_WIN / G.codeWidth;
					while(i0 < G.nDeltas && row < rEnd) {
						if(i0 < dBase || i0 + 256 > dBase + dN) {
							dBase = (int) (i0 & ~(int64_t) 15);
							dec_wave_sync();
							dec_load_window(dwin, (const uint8_t*) G.deltas, (int64_t) dBase * G.deltaWidth, G.nDeltas * G.deltaWidth, lane);
							dec_wave_sync();
						}
						if(emit < cBase || emit + 256 > cBase + cN) {
							cBase = emit & ~15;
							dec_wave_sync();
							dec_load_window(cwin, (const uint8_t*) G.codes, (int64_t) cBase * G.codeWidth, G.nOffsets * G.codeWidth, lane);
							dec_wave_sync();
						}
						int32_t rows[4], didx[4];
						unsigned mask;
						if(G.deltaWidth == 1) sdc_decode256<1>(dwin, G.nDeltas, i0, row, emit, rows, didx, mask, dBase);
						else sdc_decode256<2>(dwin, G.nDeltas, i0, row, emit, rows, didx, mask, dBase);
#pragma unroll
						for(int k = 0; k < 4; k++)
							if((mask & (1u << k)) && rows[k] < rEnd)
								dec_store_code(slot, w, (int) (rows[k] - t0), load_code(cwin, G.codeWidth, didx[k] - cBase));
						i0 += 256;
					}
					if(lane == 0) { wst[0] = dBase; wst[1] = cBase; wst[2] = tBase; }
				}
			}
		}
		__syncthreads();
		// issued behind the wave tasks: loads return in order, so a task's first load would
		// otherwise wait for the whole prefetch
		if(tile + 1 < tileEnd) prefetch(tile + 1);

		if(GRAM) {
			// wave: 128 rows of the tile; lane (k4, i16): rows k4 * 32 .. + 31, column 16 cb + i16
			const int rowsLeft = (int) min((int64_t) DEC_TILE, nRows - t0); // rows of the tile inside the matrix
#pragma unroll 1
			for(int half = 0; half < 2; half++) {
				const int rbase = wave * DEC_WROWS + k4 * 32 + half * 16;
				double cst[NB];
				u32x4 cq[NB][2];
				int lbase[NB], lnC[NB], lsent[NB];
				bool lcoded[NB], ltwo[NB];
				const double* lptr[FLAT ? NB : 1];
#pragma unroll
				for(int cb = 0; cb < NB; cb++) {
					// (narrow block with packed lookups: every lane of the last block works on one of its first four columns)
					const int ci = cb * 16 + (NAR && NB <= 2 && cb == NB - 1 ? i16 & 3 : i16);
					const DecLook L(colS[ci]);
					lbase[cb] = L.base; lnC[cb] = L.nC; lsent[cb] = L.sent; lcoded[cb] = L.coded; ltwo[cb] = L.two;
					if(FLAT) {
						const DecCol D = colS[ci];
						const double* gdict = groupS[D.pad].dict + ((unsigned) D.meta >> 18);
						lptr[cb] = (D.meta & 8) ? gdict : (const double*) smem + L.base;
					}
					cst[cb] = constS[ci];
					const u32x4* cp = (const u32x4*) (slots + (L.coded ? colS[ci].slotOff + rbase * (L.two ? 2 : 1) : 0));
					cq[cb][0] = cp[0];
					cq[cb][1] = cp[1];
				}
				double yv[LM ? 16 : 1];
				if(LM) {
					// row i16 of Y at the lane's 16 matrix rows of this half (rows of Y beyond P and rows behind the end: zeros)
					const double* __restrict__ yp = as_global(A.Y) + (size_t) i16 * nRows + t0 + rbase;
#pragma unroll
					for(int s = 0; s < 16; s++) yv[s] = 0.0;
					if(rowsLeft == DEC_TILE) { // (uniform) all 16 rows exist: 16 bytes per load, around an odd first value where the row of Y starts on one
						if(i16 < A.P) {
							if(((uintptr_t) yp & 15) == 0) {
#pragma unroll
								for(int j = 0; j < 8; j++) {
									const f64x2 v = *(const f64x2*) (yp + 2 * j);
									yv[2 * j] = v[0]; yv[2 * j + 1] = v[1];
								}
							}
							else {
								yv[0] = yp[0];
#pragma unroll
								for(int j = 0; j < 7; j++) {
									const f64x2 v = *(const f64x2*) (yp + 1 + 2 * j);
									yv[1 + 2 * j] = v[0]; yv[2 + 2 * j] = v[1];
								}
								yv[15] = yp[15];
							}
						}
					}
					else {
#pragma unroll
						for(int s = 0; s < 16; s++)
							if(i16 < A.P && rbase + s < rowsLeft) yv[s] = yp[s];
					}
				}
				// SB steps of lookups in flight, then their products
				constexpr int SB = NB <= 2 ? 4 : 2;
				// the narrow block's lookups packed four steps to one (below) pay with few column blocks; with many, the value
				// kept over two batches costs registers that the lookups in flight need
				constexpr bool NPACK = NAR && NB <= 2;
				constexpr int NL = NPACK ? NF : NB; // column blocks looked up per step
				double xn = 0.0; // NAR: lane (k4, i16) holds column i16 % 4 of the last block at step 4 (sb / 4) + i16 / 4
#pragma unroll
				for(int sb = 0; sb < 16; sb += SB) {
					double x[SB][NL];
#pragma unroll
					for(int u = 0; u < SB; u++) {
						const int s = sb + u;
#pragma unroll
						for(int cb = 0; cb < NL; cb++) {
							const int c1 = (int) ((cq[cb][0][s >> 2] >> (8 * (s & 3))) & 0xff);
							const int c2 = (int) ((cq[cb][s >> 3][(s >> 1) & 3] >> (16 * (s & 1))) & 0xffff);
							const int c = ltwo[cb] ? c2 : c1;
							// rows behind the end of the matrix hold stale codes: never used as an index
							// (a column without row data reads a zero that stays zero: no test for it)
							const bool valid = (rbase + s < rowsLeft) & (c != lsent[cb]);
							double v;
							if(FLAT) {
								const double* vp = lptr[cb] + __umul24(lcoded[cb] ? c : rbase + s, lnC[cb]);
								v = *(valid ? vp : (const double*) smem);
							}
							else {
								const int ad = lbase[cb] + __umul24(lcoded[cb] ? c : rbase + s, lnC[cb]);
								v = smem[valid ? ad : 0];
							}
							x[u][cb] = valid ? v : 0.0;
						}
					}
					if(NPACK && (sb & 3) == 0) {
						// the last block's (at most 4) columns of four steps in one lookup: lanes 4 j .. 4 j + 3 of every 16
						// take step sb + j and column i16 % 4 (their descriptors are those of lanes 0 .. 3)
						constexpr int cb = NAR ? NB - 1 : 0;
						const int sHi = sb >> 2, j = i16 >> 2, s = sb + j;
						const int c1 = (int) ((cq[cb][0][sHi] >> (8 * j)) & 0xff);
						const uint32_t lo = cq[cb][sHi >> 1][(2 * sHi) & 3], hi = cq[cb][sHi >> 1][(2 * sHi + 1) & 3]; // codes 4 sHi .. + 3 as 16-bit pieces
						const int c2 = (int) (((j & 2 ? hi : lo) >> (16 * (j & 1))) & 0xffff);
						const int c = ltwo[cb] ? c2 : c1;
						const bool in = rbase + s < rowsLeft;
						const bool valid = in & (c != lsent[cb]);
						double v;
						if(FLAT) {
							const double* vp = lptr[cb] + __umul24(lcoded[cb] ? c : rbase + s, lnC[cb]);
							v = *(valid ? vp : (const double*) smem);
						}
						else {
							const int ad = lbase[cb] + __umul24(lcoded[cb] ? c : rbase + s, lnC[cb]);
							v = smem[valid ? ad : 0];
						}
						v = valid ? v : 0.0;
						xn = in ? cst[cb] + v : 0.0;
					}
#pragma unroll
					for(int u = 0; u < SB; u++) {
						const bool in = rbase + sb + u < rowsLeft;
#pragma unroll
						for(int cb = 0; cb < NL; cb++) x[u][cb] = in ? cst[cb] + x[u][cb] : 0.0;
						int t = 0;
						if(LM) {
							const double y = yv[sb + u];
							badY |= !(__builtin_fabs(y) <= 1.7976931348623157e308);
#pragma unroll
							for(int cb = 0; cb < NB; cb++) gram[cb] = __builtin_amdgcn_mfma_f64_16x16x4f64(y, x[u][cb], gram[cb], 0, 0, 0);
						}
						else
#pragma unroll
						for(int ib = 0; ib < (XB > 0 ? XB : NF); ib++)
#pragma unroll
							for(int jb = (XB > 0 ? XB : ib); jb < NF; jb++, t++)
								gram[t] = __builtin_amdgcn_mfma_f64_16x16x4f64(x[u][ib], x[u][jb], gram[t], 0, 0, 0);
						if(NAR) {
							// operands of the 4 x 4 x 4 form for step sb + u: every lane needs column l % 4 of the last block for
							// its row group, which lane 4 ((sb + u) % 4) + l % 4 of its 16 holds: that bank spread over the others
							// (not packed: every lane looked its own column of the last block up; lanes 0 .. 3 of 16 hold the real ones)
							int a[2], o[2];
							__builtin_memcpy(o, NPACK ? &xn : &x[u][NL - 1], 8);
							a[0] = dec_spread_bank(o[0], NPACK ? (sb + u) & 3 : 0);
							a[1] = dec_spread_bank(o[1], NPACK ? (sb + u) & 3 : 0);
							double an;
							__builtin_memcpy(&an, a, 8);
#pragma unroll
							for(int cb = 0; cb < NF; cb++) nar[cb] = __builtin_amdgcn_mfma_f64_4x4x4f64(an, x[u][cb], nar[cb], 0, 0, 0);
							// last block x last block: all four products are the same 4 x 4 one (the first is kept)
							nar[NAR ? NB - 1 : 0] = __builtin_amdgcn_mfma_f64_4x4x4f64(an, an, nar[NAR ? NB - 1 : 0], 0, 0, 0);
						}
					}
				}
			}
			continue;
		}

		// ---- X %*% B: wave = 128 rows in passes of 16 * RPL; lane (k4, i16): rows i16 * RPL .. of
		// the pass as the A operand of decoded column 4 kb + k4, B[4 kb + k4, i16] as the B operand
		constexpr int PROWS = 16 * RPL;
#pragma unroll 1
		for(int pass = 0; pass < DEC_WROWS / PROWS; pass++) {
			const int pbase = wave * DEC_WROWS + pass * PROWS;
			const int rbase = pbase + i16 * RPL;
			f64x4 acc[RPL];
#pragma unroll
			for(int s = 0; s < RPL; s++) acc[s] = f64x4{cinit, cinit, cinit, cinit};
			bool in[RPL];
#pragma unroll
			for(int s = 0; s < RPL; s++) in[s] = t0 + rbase + s < nRows;
#pragma unroll 2
			for(int kb = 0; kb < KB; kb++) {
				const DecCol D = colS[kb * 4 + k4];
				const double bop = Bs[(kb * 4 + k4) * 16 + i16];
				const DecLook L(D);
				// RPL codes of the column's tile as 16-bit pieces (aligned for either code width)
				const uint16_t* cp = (const uint16_t*) (slots + (L.coded ? D.slotOff + rbase * (L.two ? 2 : 1) : 0));
				uint32_t piece[RPL];
#pragma unroll
				for(int s = 0; s < RPL; s++) piece[s] = cp[s];
				double x[RPL];
#pragma unroll
				for(int s = 0; s < RPL; s++) {
					const int c1 = (int) ((piece[s >> 1] >> (8 * (s & 1))) & 0xff);
					bool valid;
					const int ad = L.addr(L.two ? (int) piece[s] : c1, rbase + s, in[s], valid);
					const double v = smem[ad];
					x[s] = valid ? v : 0.0;
				}
#pragma unroll
				for(int s = 0; s < RPL; s++) acc[s] = __builtin_amdgcn_mfma_f64_16x16x4f64(x[s], bop, acc[s], 0, 0, 0);
			}
			// accumulator register v of lane l: output row 4 v + l / 16 of the step, output column l % 16
			dec_wave_sync(); // the previous pass's readers of the staging area are done
			if(i16 < q) {
#pragma unroll
				for(int s = 0; s < RPL; s++)
#pragma unroll
					for(int v = 0; v < 4; v++) wstage[((4 * v + k4) * RPL + s) * q + i16] = acc[s][v];
			}
			dec_wave_sync();
			const int64_t rowBase = t0 + pbase;
			const int nr = (int) max((int64_t) 0, min((int64_t) PROWS, nRows - rowBase));
			// the pass's rows are one contiguous range of the output: 16 bytes per lane (the range starts on a
			// multiple of 16 bytes: rowBase is a multiple of 16 rows), a single double at an odd end
			if(A.ld == q) {
				const int n = nr * q;
				double* o = A.out + (size_t) rowBase * q;
				for(int i = 2 * lane; i + 1 < n; i += 128) {
					const f64x2 v = *(const f64x2*) (wstage + i);
					cnt += (v[0] != 0.0) + (v[1] != 0.0);
					__builtin_nontemporal_store(v, (f64x2*) (o + i));
				}
				if((n & 1) && lane == 0) {
					const double v = wstage[n - 1];
					cnt += v != 0.0;
					__builtin_nontemporal_store(v, o + n - 1);
				}
			}
			else {
				// q of the output's ld columns (a pass over wide B): pieces of q values per row
				const int n = nr * q;
				double* o = A.out + (size_t) rowBase * A.ld;
				const bool pairs = (q & 1) == 0 && (A.ld & 1) == 0 && ((uintptr_t) A.out & 15) == 0;
				for(int i = 2 * lane; i < n; i += 128) {
					const int r0 = i / q, c0 = i - r0 * q;
					if(pairs) {
						const f64x2 v = *(const f64x2*) (wstage + i);
						cnt += (v[0] != 0.0) + (v[1] != 0.0);
						__builtin_nontemporal_store(v, (f64x2*) (o + (size_t) r0 * A.ld + c0));
					}
					else
						for(int e = 0; e < 2 && i + e < n; e++) {
							const int r = (i + e) / q, c = (i + e) - r * q;
							const double v = wstage[i + e];
							cnt += v != 0.0;
							__builtin_nontemporal_store(v, o + (size_t) r * A.ld + c);
						}
				}
			}
		}
	}
	if(GRAM && LM) {
		// tiles of the block's waves summed in LDS (16 rows of Y x NB * 16 columns), then one global add per cell:
		// accumulator register v of lane l is cell (row 4 v + l / 16 of Y, column 16 cb + l % 16)
		constexpr int NP = NB * 16;
		__syncthreads();
		for(int i = tid; i < 16 * NP; i += DEC_THREADS) stage[i] = 0.0;
		__syncthreads();
#pragma unroll
		for(int cb = 0; cb < NB; cb++)
#pragma unroll
			for(int v = 0; v < 4; v++) unsafeAtomicAdd(&stage[(4 * v + k4) * NP + cb * 16 + i16], gram[cb][v]);
		__syncthreads();
		for(int i = tid; i < 16 * NP; i += DEC_THREADS) {
			const int r = i / NP, c = i - r * NP;
			if(r < A.P && c < A.nCols && stage[i] != 0.0) unsafeAtomicAdd(&A.out[(size_t) r * A.nCols + c], stage[i]);
		}
		if(__ballot(badY) != 0 && lane == 0) atomicOr(A.badY, 1ull);
		return;
	}
	if(GRAM) {
		// Gram tiles of the block's waves summed in LDS, then one global add per cell of the
		// upper triangle. Accumulator register v of lane l is cell (4 v + l / 16, l % 16) of its tile.
		constexpr int NP = NB * 16;
		__syncthreads();
		for(int i = tid; i < NP * NP; i += DEC_THREADS) stage[i] = 0.0;
		__syncthreads();
		int t = 0;
#pragma unroll
		for(int ib = 0; ib < (XB > 0 ? XB : NF); ib++)
#pragma unroll
			for(int jb = (XB > 0 ? XB : ib); jb < NF; jb++, t++)
#pragma unroll
				for(int v = 0; v < 4; v++)
					unsafeAtomicAdd(&stage[(ib * 16 + 4 * v + k4) * NP + jb * 16 + i16], gram[t][v]);
		if(NAR) {
			// cell (16 (NB - 1) + k4, 16 cb + i16): into the upper triangle at its mirror image for the full blocks
#pragma unroll
			for(int cb = 0; cb < NB; cb++) {
				const int r = (NB - 1) * 16 + k4, c = cb * 16 + i16;
				unsafeAtomicAdd(&stage[cb < NB - 1 ? c * NP + r : r * NP + c], nar[cb]);
			}
		}
		__syncthreads();
		double* const dst = A.done != nullptr ? A.acc : A.out;
		for(int i = tid; i < NP * NP; i += DEC_THREADS) {
			const int r = i / NP, c = i - r * NP;
			if(r <= c && c < A.nCols && stage[i] != 0.0) unsafeAtomicAdd(&dst[(size_t) r * A.nCols + c], stage[i]);
		}
		if(A.done != nullptr) gram_tail(A.done, gridDim.x, A.acc, A.out, A.nCols, A.nnz, (unsigned*) stage);
		return;
	}
	count_add(A.nnz, cnt);
}

template <int RPL>
__global__ __launch_bounds__(DEC_THREADS) void k_rmm_decode(const DecArgs A) { decode_body<0, 1, RPL, 0>(A); }

template <int NB, int FLAT, int XB, int NAR = 0>
__global__ __launch_bounds__(DEC_THREADS) void k_tsmm_decode(const DecArgs A) { decode_body<1, NB, 4, FLAT, XB, NAR>(A); }

template <int NB, int FLAT>
__global__ __launch_bounds__(DEC_THREADS) void k_lmm_decode(const DecArgs A) { decode_body<1, NB, 4, FLAT, 0, 0, 1>(A); }

// One code per row for an RLE group (0xff where no run covers the row): thread = 4 rows.
__global__ __launch_bounds__(256) void k_expand_rle(const DGroup* __restrict__ groups, int g, int64_t nRows, uint8_t* __restrict__ codes) {
	const DGroup G = dgroup(groups + g);
	const int64_t rb = ((int64_t) blockIdx.x * 256 + threadIdx.x) * 4;
	if(rb >= nRows) return;
	int j = rle_find(G.runStart, G.nRuns, (int32_t) rb);
	for(int t = 0; t < 4 && rb + t < nRows; t++) {
		while(G.runStart[j + 1] <= rb + t) j++;
		codes[rb + t] = (uint8_t) G.runCode[j]; // -1 (uncovered) becomes 0xff
	}
}

// One code per listed row of an SDCZeros group into a stream preset to 0xff: wave = one tile of the row-tile index.
__global__ __launch_bounds__(256) void k_expand_sdc(const DGroup* __restrict__ groups, int g, int64_t nRows, uint8_t* __restrict__ codes) {
	const DGroup G = dgroup(groups + g);
	const int64_t r0 = ((int64_t) blockIdx.x * 4 + (threadIdx.x >> 6)) * SDC_TILE;
	if(r0 >= nRows) return; // whole waves leave
	const void* src = G.codes;
	const int cw = G.codeWidth;
	sdc_walk_tile(G, r0, SDC_TILE, [&](int rr, int di) { codes[r0 + rr] = (uint8_t) load_code(src, cw, di); });
}

constexpr int RLE_LONG_RUN = 64; // mean rows per run from which a run-length group counts as long

// Expanded code streams make every dictionary-coded group of a block a plain copy in the tile
// fill. Built once, when they cost at most half of what the block itself takes in HBM.
int ensure_expanded(cla_block* b) {
	if(b->expTried) return 0;
	b->expTried = true;
	const int nG = (int) b->groups.size();
	b->expCodes.assign((size_t) nG, nullptr);
	if(!b->opt.expandStreams || b->nRows == 0) return 0;
	std::vector<int> cand;
	for(int g = 0; g < nG; g++) {
		const DGroup& G = b->groups[g].d;
		// (run-length groups with long runs get no copy: the stream kernels follow their runs, cla_runs.hpp)
		const bool shortRuns = G.type == G_RLE && (int64_t) G.nRuns * RLE_LONG_RUN > b->nRows;
		if((shortRuns || (G.type == G_SDCZ && G.nOffsets > 0)) && G.nVals <= 255) cand.push_back(g);
	}
	if(cand.empty() || (int64_t) cand.size() * b->nRows > b->device_bytes_cached / 2) return 0;
	for(int g : cand) {
		const DGroup& G = b->groups[g].d;
		uint8_t* p = nullptr;
		CLA_HIP(hipMalloc((void**) &p, (size_t) b->nRows + 16));
		b->derivedBytes += b->nRows + 16;
		b->expCodes[g] = p;
		if(G.type == G_RLE)
			hipLaunchKernelGGL(k_expand_rle, dim3((unsigned) ((b->nRows + 1023) / 1024)), dim3(256), 0, b->stream, b->dGroups, g, b->nRows, p);
		else {
			CLA_HIP(hipMemsetAsync(p, 0xff, (size_t) b->nRows + 16, b->stream));
			const int64_t nT1 = (b->nRows + SDC_TILE - 1) / SDC_TILE;
			hipLaunchKernelGGL(k_expand_sdc, dim3((unsigned) ((nT1 + 3) / 4)), dim3(256), 0, b->stream, b->dGroups, g, b->nRows, p);
		}
	}
	CLA_HIP(hipGetLastError());
	return 0;
}

// Host side of both kernels: LDS plan, copy list and column descriptors in the block's
// scratch buffer. Returns 1 when the block does not fit (the caller uses another path).
struct DecLaunch {
	DecArgs A;
	size_t lds = 0;
	unsigned grid = 0;
};

// Dictionaries of more than dictLimit doubles stay in global memory (t(X) %*% X only).
// The plan's device image goes into *dImg (an allocation of its own, kept with the plan).
static int dec_build_plan(cla_block* b, bool gram, int q, int rpl, DecLaunch& L, size_t dictLimit, void** dImg, int64_t* imgBytes) {
	const int nG = (int) b->groups.size();
	const int nCols = b->nCols;
	{
		const int rc = ensure_expanded(b);
		if(rc) return rc;
	}
	std::vector<DecGroup> plan((size_t) nG);
	size_t valD = 0, slotB = 0;
	int K = 0;
	for(int g = 0; g < nG; g++) {
		const DGroup& G = b->groups[g].d;
		DecGroup& P = plan[g];
		P.type = G.type; P.nC = G.nColG; P.dictOff = -1; P.slotOff = -1; P.slotW = 0; P.copyIdx = -1; P.pad = 0;
		P.kOff = K;
		K += G.nColG;
		if(G.nColG >= (1 << 14)) return 1;
		if(G.type == G_UNC) {
			P.dictOff = (int32_t) valD;
			valD += (size_t) DEC_TILE * G.nColG;
			continue;
		}
		if(G.type != G_DDC && G.type != G_RLE && !(G.type == G_SDCZ && G.nOffsets > 0)) continue; // no row data
		if(G.nVals > 65535) return 1;
		if((size_t) G.nVals * G.nColG <= dictLimit) {
			P.dictOff = (int32_t) valD;
			valD += (size_t) G.nVals * G.nColG;
		}
		// DDC codes of one or two bytes keep their width (plain copies; no value is set aside for rows without a
		// code); the others are stored with 0xff / 0xffff for such rows
		P.slotW = G.type == G_DDC && G.codeWidth <= 2 ? G.codeWidth : G.nVals <= 255 ? 1 : 2;
		P.slotOff = (int32_t) slotB;
		slotB += (size_t) DEC_TILE * P.slotW + DEC_SLOT_PAD;
	}
	valD = (valD + 1) & ~(size_t) 1;
	const size_t zeroAt = valD; // a value that stays zero: what a column without row data looks up
	valD += 2;
	slotB = (slotB + 16 + 15) & ~(size_t) 15; // the multiply phase may read 16 bytes past the last tile
	const int nColD = gram ? ((nCols + 15) / 16) * 16 : ((K + 3) / 4) * 4;
	const size_t bD = gram ? 0 : (size_t) nColD * 16;
	// (the Gram tile of a block is summed where its dictionaries and dense tiles were, once its rows are done)
	if(gram) valD = std::max(valD, (size_t) nColD * nColD);
	const size_t stageD = gram ? 0 : (size_t) DEC_WAVES * 16 * rpl * q;
	const size_t slotBase = (valD + bD + stageD) * 8;
	// copy list
	std::vector<DecCopy> copies;
	int nChunks = 0;
	for(int g = 0; g < nG; g++) {
		const DGroup& G = b->groups[g].d;
		DecGroup& P = plan[g];
		DecCopy C;
		C.pad = 0;
		if(G.type == G_UNC) {
			if(((uintptr_t) G.dense & 15) != 0) return 1;
			C.src = (const uint8_t*) G.dense; C.bpr = G.nColG * 8; C.dstOff = P.dictOff * 8;
		}
		else if(P.slotOff >= 0 && G.type == G_DDC && G.codeWidth == P.slotW && ((uintptr_t) G.codes & 15) == 0) {
			C.src = (const uint8_t*) G.codes; C.bpr = P.slotW; C.dstOff = (int32_t) (slotBase + P.slotOff);
		}
		else if(P.slotOff >= 0 && b->expCodes[g] != nullptr) { // RLE / SDCZeros with an expanded byte stream
			C.src = b->expCodes[g]; C.bpr = 1; C.dstOff = (int32_t) (slotBase + P.slotOff);
		}
		else continue;
		C.chunk0 = nChunks;
		P.copyIdx = (int32_t) copies.size();
		copies.push_back(C);
		nChunks += DEC_TILE * C.bpr / 16;
	}
	// wave tasks (groups whose tile needs decoding), longest first onto the least loaded wave
	std::vector<std::pair<int, int>> taskCost; // (cost, group)
	for(int g = 0; g < nG; g++) {
		const DecGroup& P = plan[g];
		if(P.slotOff < 0 || P.copyIdx >= 0) continue;
		taskCost.push_back({P.type == G_DDC ? 3 : P.type == G_SDCZ ? 2 : 1, g});
	}
	std::stable_sort(taskCost.begin(), taskCost.end(), [](const std::pair<int, int>& a, const std::pair<int, int>& c) { return a.first > c.first; });
	std::vector<std::vector<int>> waveTasks(DEC_WAVES);
	{
		int load[DEC_WAVES] = {0};
		for(auto& tc : taskCost) {
			int best = 0;
			for(int w = 1; w < DEC_WAVES; w++)
				if(load[w] < load[best]) best = w;
			load[best] += tc.first;
			waveTasks[best].push_back(tc.second);
		}
	}
	std::vector<int32_t> tasks(DEC_WAVES + 1, 0);
	for(int w = 0; w < DEC_WAVES; w++) {
		tasks[w + 1] = tasks[w] + (int32_t) waveTasks[w].size();
		for(int g : waveTasks[w]) tasks.push_back(g);
	}
	size_t ldsEnd = slotBase + slotB + (size_t) nColD * (sizeof(DecCol) + (gram ? 8 : 0)) +
		(size_t) nG * (sizeof(DecGroup) + sizeof(DGroup) + 4) + copies.size() * sizeof(DecCopy) + tasks.size() * 4;
	ldsEnd = (ldsEnd + 15) & ~(size_t) 15;
	for(int g = 0; g < nG; g++) { // windows of the wave tasks
		DecGroup& P = plan[g];
		if(P.slotOff < 0 || P.copyIdx >= 0) continue;
		if(P.type == G_RLE) { P.pad = (int32_t) ldsEnd; ldsEnd += 3 * 64 * 4; }
		else if(P.type == G_SDCZ) { P.pad = (int32_t) ldsEnd; ldsEnd += DEC_TWIN * sizeof(OffState) + 2 * DEC_WIN + 16; }
	}
	L.lds = ldsEnd + 64;
	if(L.lds > (size_t) std::min(g_ldsPerBlock, 160 * 1024) - 1024) return 1;
	// column descriptors: decoded column order (X %*% B) or matrix column order (t(X) %*% X)
	std::vector<DecCol> cols((size_t) nColD, DecCol{0, (int32_t) zeroAt, 0, 0});
	std::vector<double> colConst((size_t) (gram ? nColD : 0), 0.0);
	if(gram)
		for(int c = 0; c < nCols; c++) colConst[c] = b->constV[c];
	std::vector<char> seen((size_t) nCols, 0);
	for(int g = 0; g < nG; g++) {
		const DecGroup& P = plan[g];
		const auto& hc = b->groups[g].cols;
		for(int h = 0; h < P.nC; h++) {
			if(gram && seen[hc[h]]) return 1; // overlapping groups
			seen[hc[h]] = 1;
			DecCol& C = cols[gram ? hc[h] : P.kOff + h];
			const int kind = P.type == G_UNC ? 2 : P.slotOff >= 0 ? (P.type == G_DDC ? 3 : 1) : 0;
			C.slotOff = kind == 1 || kind == 3 ? P.slotOff : 0;
			C.valOff = kind && P.dictOff >= 0 ? P.dictOff : kind ? 0 : (int32_t) zeroAt;
			C.pad = g;
			// (a column without row data looks the zero up whatever the row: no stride, no place in a tuple)
			C.meta = kind == 0 ? 0 : (int32_t) ((uint32_t) kind | (P.slotW == 2 ? 4u : 0u) | ((kind == 1 || kind == 3) && P.dictOff < 0 ? 8u : 0u) | ((uint32_t) P.nC << 4) | ((uint32_t) h << 18));
		}
	}
	const size_t planBytes = plan.size() * sizeof(DecGroup), copyBytes = copies.size() * sizeof(DecCopy);
	const size_t colBytes = cols.size() * sizeof(DecCol), constBytes = colConst.size() * 8;
	const size_t taskBytes = tasks.size() * 4;
	std::vector<uint8_t> img(planBytes + copyBytes + colBytes + constBytes + taskBytes);
	std::memcpy(img.data(), copies.data(), copyBytes); // pointers first: 8-byte aligned
	std::memcpy(img.data() + copyBytes, colConst.data(), constBytes);
	std::memcpy(img.data() + copyBytes + constBytes, cols.data(), colBytes);
	std::memcpy(img.data() + copyBytes + constBytes + colBytes, plan.data(), planBytes);
	std::memcpy(img.data() + copyBytes + constBytes + colBytes + planBytes, tasks.data(), taskBytes);
	uint8_t* d = nullptr;
	CLA_HIP(hipMalloc((void**) &d, img.size() + 64));
	*dImg = d;
	*imgBytes = (int64_t) img.size() + 64;
	CLA_HIP(hipMemcpy(d, img.data(), img.size(), hipMemcpyHostToDevice));
	DecArgs& A = L.A;
	A.groups = b->dGroups;
	A.copies = (const DecCopy*) d;
	A.colConst = (const double*) (d + copyBytes);
	A.cols = (const DecCol*) (d + copyBytes + constBytes);
	A.plan = (const DecGroup*) (d + copyBytes + constBytes + colBytes);
	A.tasks = (const int32_t*) (d + copyBytes + constBytes + colBytes + planBytes);
	A.nTasks = (int) taskCost.size();
	A.nGroups = nG; A.nCopies = (int) copies.size(); A.nChunks = nChunks; A.nColD = nColD;
	A.valDoubles = (int) valD; A.bDoubles = (int) bD; A.stageDoubles = (int) stageD; A.slotBytes = (int) slotB;
	A.B = nullptr; A.q = q; A.ld = q; A.constRow = nullptr; A.Y = nullptr; A.P = 0; A.badY = nullptr; A.out = nullptr; A.nRows = b->nRows; A.nnz = nullptr; A.nCols = nCols;
	A.acc = nullptr; A.done = nullptr;
	const int nTiles = (int) ((b->nRows + DEC_TILE - 1) / DEC_TILE);
	const int blocksPerCU = L.lds <= 76 * 1024 ? 2 : 1;
	L.grid = (unsigned) std::min(nTiles, g_numCU * blocksPerCU);
	return 0;
}

// Plans are kept with the block (they depend on the block, the shape of the product and the options only):
// a call then costs no host planning, no upload and no wait for it.
struct DecPlanEntry {
	bool gram;
	int q, rpl, expand;
	size_t dictLimit;
	int rc;
	DecLaunch L;
	void* dImg;
	int64_t bytes;
};
struct DecPlanCache {
	std::vector<DecPlanEntry> entries;
};

void dir_plan_drop(cla_block* b);
void gdr_plan_drop(cla_block* b);

void dec_plans_drop(cla_block* b) {
	dir_plan_drop(b);
	gdr_plan_drop(b);
	if(b->decPlans == nullptr) return;
	for(auto& e : b->decPlans->entries)
		if(e.dImg) { (void) hipFree(e.dImg); b->derivedBytes -= e.bytes; }
	delete b->decPlans;
	b->decPlans = nullptr;
}

static int dec_prepare(cla_block* b, bool gram, int q, int rpl, DecLaunch& L, size_t dictLimit = (size_t) 1 << 30) {
	if(b->decPlans == nullptr) b->decPlans = new DecPlanCache();
	for(auto& e : b->decPlans->entries)
		if(e.gram == gram && e.q == q && e.rpl == rpl && e.dictLimit == dictLimit && e.expand == b->opt.expandStreams) {
			L = e.L;
			return e.rc;
		}
	DecPlanEntry e;
	e.gram = gram; e.q = q; e.rpl = rpl; e.expand = b->opt.expandStreams; e.dictLimit = dictLimit; e.dImg = nullptr; e.bytes = 0;
	e.rc = dec_build_plan(b, gram, q, rpl, e.L, dictLimit, &e.dImg, &e.bytes);
	if(e.rc < 0) { // an error is not a property of the block: not kept
		if(e.dImg) (void) hipFree(e.dImg);
		return e.rc;
	}
	if(b->decPlans->entries.size() >= 64) { // (products with many different widths of B: start over)
		for(auto& o : b->decPlans->entries)
			if(o.dImg) { (void) hipFree(o.dImg); b->derivedBytes -= o.bytes; }
		b->decPlans->entries.clear();
	}
	if(e.dImg) b->derivedBytes += e.bytes;
	b->decPlans->entries.push_back(e);
	L = e.L;
	return e.rc;
}

// The plan of the decoded Gram matrix: all dictionaries in LDS, else the large ones in global memory (flat).
static int gram_prepare(cla_block* b, DecLaunch& L, bool& flat) {
	flat = false;
	int rc = dec_prepare(b, true, 0, 4, L);
	if(rc == 1) { // large dictionaries stay in global memory
		flat = true;
		rc = dec_prepare(b, true, 0, 4, L, 512);
	}
	if(rc == 1) rc = dec_prepare(b, true, 0, 4, L, 64); // many mid-sized dictionaries: only the small ones in LDS
	return rc;
}

// 0 when launch_tsmm_decode would take the block, 1 when not (LDS), negative on error.
int tsmm_decode_fits(cla_block* b) {
	if(b->groups.empty() || b->nRows == 0 || b->nCols > 64) return 1;
	DecLaunch L;
	bool flat;
	return gram_prepare(b, L, flat);
}

// Column classes of k_rmm_direct: its column list is sorted by class, so that each class runs a loop of its own
// without a test per column.
enum { DSEG_DDC1 = 0, DSEG_DDC2, DSEG_GAP1, DSEG_GAP2, DSEG_DENSE, DSEG_N };
typedef const __attribute__((address_space(4))) double* dec_cdp; // read-only for the kernel's duration: uniform addresses become scalar loads

// ---- X %*% B for narrow B without code tiles: k_rmm_direct
// For blocks whose groups are all plain streams (DDC codes of one or two bytes, the one-code-per-row copies of RLE
// and SDCZeros groups, rows of uncompressed groups) and whose dictionaries fit LDS together. A wave owns slices of
// 128 consecutive rows, lane l rows 2 l and 2 l + 1 of the slice: it loads its two codes of a column straight from
// global memory (64 lanes = one or two full lines), looks the values up in the block's LDS copy of the dictionaries
// and adds value x B[column, j] to its QV sums per row, B's row coming through scalar loads. No barrier after the
// dictionaries are in place: the 16 waves of a block drift apart, so that the loads, the multiply-adds and the stores
// of different waves overlap (the tile kernel's waves walk through fill, multiply and store in step).
constexpr int DIR_THREADS = 1024;
constexpr int DIR_WAVES = DIR_THREADS / 64;
constexpr int DIR_SLICE = 128;   // rows per wave and step
constexpr int DIR_SROWS = 32;    // rows of a slice that go through the wave's staging area at a time

struct DirCol {          // 32 bytes, read through scalar loads
	const uint8_t* src;  // code stream, or the column's first value of an uncompressed group
	int32_t base8;       // bytes from the LDS base: the column's value of tuple 0
	int32_t nC8;         // bytes per tuple; uncompressed: bytes per row
	int32_t orig;        // column of the matrix (row of B); below zero: a filler column
	int32_t r0, r1, r2;
};
struct DirDict {
	const double* src;
	int32_t n, off;      // doubles, doubles from the LDS base
};
struct DirArgs {
	const DirCol* cols;
	const DirDict* dicts;
	const double* zeroRow;
	// run-length columns (never looked up per row): the merged run table's segment starts, its record per slice (segment
	// of the first row, run starts inside), and per segment the columns' part of the output row (k_run_sums, 16 doubles)
	const int32_t* mrtStart;
	const int32_t* sliceRec;
	const double* runSums;
	int nR;
	int nDicts, dictDoubles;
	int segEnd[DSEG_N];
	const double* B;        // first of the QV columns of this launch
	const double* constRow;
	double* out;            // likewise
	int ld;                 // columns of B and of the output (>= QV: wide B goes in chunks of 16 columns)
	int64_t nRows;
	unsigned long long* nnz;
};
typedef const __attribute__((address_space(4))) DirCol* dir_ccp;
typedef unsigned long long dir_u64x4 __attribute__((ext_vector_type(4)));
typedef int32_t dir_i32x8 __attribute__((ext_vector_type(8)));

// HASR: the block has run-length columns. Their part of an output row (plus the constant row) is the same for all rows
// of a segment of the merged run table and comes from k_run_sums: a lane finds its two rows' segments (the slice's
// first one from the table's index, the few run starts inside the slice compared one by one) and adds the segments'
// sums to its rows at the end.
template <int QV, bool HASR>
__global__ __launch_bounds__(DIR_THREADS) void k_rmm_direct(const DirArgs A) {
	constexpr int THREADS = DIR_THREADS, WAVES = THREADS / 64;
	extern __shared__ __align__(16) double smem[];
	const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
	for(int g = 0; g < A.nDicts; g++) {
		const DirDict D = A.dicts[g];
		const double* __restrict__ src = as_global(D.src);
		for(int i = tid; i < D.n; i += THREADS) smem[D.off + i] = src[i];
	}
	if(tid < 2) smem[A.dictDoubles - 2 + tid] = 0.0; // what a filler column looks up
	__syncthreads();
	const uint8_t* const ldsBytes = (const uint8_t*) smem;
	double* const wstage = smem + A.dictDoubles + (size_t) wave * DIR_SROWS * QV;
	const dec_cdp Bc = (dec_cdp) A.B;
	const int64_t nRows = A.nRows;
	const int64_t nSlices = (nRows + DIR_SLICE - 1) / DIR_SLICE;
	int cnt = 0;
	dir_i32x8 rec = {0, 0, 0, 0, 0, 0, 0, 0};
	const int64_t slice0u = (int64_t) blockIdx.x * WAVES + __builtin_amdgcn_readfirstlane(wave); // (a scalar, so that the records come through scalar loads)
	if(HASR && slice0u < nSlices) rec = *(const __attribute__((address_space(4))) dir_i32x8*) (A.sliceRec + 8 * slice0u);
	int64_t sliceU = slice0u;
	for(int64_t slice = (int64_t) blockIdx.x * WAVES + wave; slice < nSlices; slice += (int64_t) gridDim.x * WAVES) {
		const int64_t s0 = slice * DIR_SLICE, row0 = s0 + 2 * lane;
		const bool full = s0 + DIR_SLICE <= nRows; // (uniform)
		const bool in0 = row0 < nRows, in1 = row0 + 1 < nRows;
		double acc[2][QV];
#pragma unroll
		for(int j = 0; j < QV; j++) {
			const double c0 = !HASR && A.constRow != nullptr ? ((dec_cdp) A.constRow)[j] : 0.0; // (HASR: the segments' sums hold the constant row)
			acc[0][j] = c0; acc[1][j] = c0;
		}
		if(HASR) {
			// segments of the lane's two rows: the slice's first one plus the run starts inside the slice that lie at or in
			// front of the row (the slice's record: one scalar load, requested a slice ahead)
			int sid0 = rec[0], sid1 = rec[0];
#pragma unroll
			for(int k = 0; k < 6; k++) {
				sid0 += row0 >= (int64_t) rec[2 + k] ? 1 : 0;
				sid1 += row0 + 1 >= (int64_t) rec[2 + k] ? 1 : 0;
			}
			for(int k = 6; k < rec[1]; k++) { // (uniform, rare) more than six run starts inside the slice
				const int64_t st = ((const __attribute__((address_space(4))) int32_t*) A.mrtStart)[rec[0] + 1 + k];
				sid0 += row0 >= st ? 1 : 0;
				sid1 += row0 + 1 >= st ? 1 : 0;
			}
			{
				const int64_t next = sliceU + (int64_t) gridDim.x * WAVES;
				rec = *(const __attribute__((address_space(4))) dir_i32x8*) (A.sliceRec + 8 * (next < nSlices ? next : sliceU));
				sliceU = next;
			}
			// the rows' sums start from their segments' (requested here, needed by the first column's multiply-adds: the
			// wait falls together with the one for that column's codes)
			const double* __restrict__ r0 = as_global(A.runSums) + (size_t) sid0 * 16, * __restrict__ r1 = as_global(A.runSums) + (size_t) sid1 * 16;
#pragma unroll
			for(int j = 0; j + 1 < QV; j += 2) {
				const f64x2 v0 = *(const f64x2*) (r0 + j), v1 = *(const f64x2*) (r1 + j);
				acc[0][j] = v0[0]; acc[0][j + 1] = v0[1];
				acc[1][j] = v1[0]; acc[1][j + 1] = v1[1];
			}
			if(QV & 1) { acc[0][QV - 1] = r0[QV - 1]; acc[1][QV - 1] = r1[QV - 1]; }
		}
		// NBAT columns of one class at a time; GUARD: the last slice, whose rows may lie behind the end of the matrix
		auto batch = [&](auto kindTag, auto twoTag, auto nTag, auto guardTag, int k) {
			constexpr int KIND = decltype(kindTag)::value;
			constexpr bool TWO = decltype(twoTag)::value;
			constexpr int NBAT = decltype(nTag)::value;
			constexpr bool GUARD = decltype(guardTag)::value;
			double x[NBAT][2];
			dec_cdp brow[NBAT];
			const uint8_t* src[NBAT];
			int base8[NBAT], nC8[NBAT];
			uint32_t cc[NBAT];
			dir_u64x4 D[NBAT];
#pragma unroll
			for(int u = 0; u < NBAT; u++) D[u] = *(const __attribute__((address_space(4))) dir_u64x4*) (A.cols + k + u);
			__builtin_amdgcn_sched_barrier(0);
#pragma unroll
			for(int u = 0; u < NBAT; u++) {
				src[u] = (const uint8_t*) D[u][0];
				base8[u] = (int) (uint32_t) D[u][1]; nC8[u] = (int) (D[u][1] >> 32);
				const int orig = (int) (uint32_t) D[u][2];
				brow[u] = orig < 0 ? (dec_cdp) A.zeroRow : Bc + (size_t) orig * A.ld;
			}
#pragma unroll
			for(int u = 0; u < NBAT; u++) {
				// (the slice's start goes into the uniform part of the address, the lane's part stays small)
				typedef const __attribute__((address_space(1))) uint8_t* gp8;
				if(KIND == 2) {
					const gp8 p = (gp8) src[u] + (size_t) s0 * nC8[u];
					const int lo = __umul24(2 * lane, nC8[u]);
					x[u][0] = !GUARD || in0 ? *(const __attribute__((address_space(1))) double*) (p + lo) : 0.0;
					x[u][1] = !GUARD || in1 ? *(const __attribute__((address_space(1))) double*) (p + lo + nC8[u]) : 0.0;
				}
				else if(TWO) {
					const gp8 p = (gp8) src[u] + (size_t) s0 * 2;
					if(!GUARD || in1) cc[u] = *(const __attribute__((address_space(1))) uint32_t*) (p + 4 * lane);
					else cc[u] = in0 ? *(const __attribute__((address_space(1))) uint16_t*) (p + 4 * lane) : 0u;
				}
				else {
					const gp8 p = (gp8) src[u] + (size_t) s0;
					if(!GUARD || in1) cc[u] = *(const __attribute__((address_space(1))) uint16_t*) (p + 2 * lane);
					else cc[u] = in0 ? *(p + 2 * lane) : 0u;
				}
			}
			__builtin_amdgcn_sched_barrier(0);
			if(KIND != 2) {
				bool valid[NBAT][2];
#pragma unroll
				for(int u = 0; u < NBAT; u++)
#pragma unroll
					for(int r = 0; r < 2; r++) {
						const int c = TWO ? (int) ((cc[u] >> (16 * r)) & 0xffff) : (int) ((cc[u] >> (8 * r)) & 0xff);
						valid[u][r] = (!GUARD || (r == 0 ? in0 : in1)) & (KIND == 3 || c != 0xff);
						x[u][r] = *(const double*) (ldsBytes + (base8[u] + __umul24(KIND == 3 && !GUARD ? c : valid[u][r] ? c : 0, nC8[u])));
					}
				__builtin_amdgcn_sched_barrier(0);
				if(KIND == 1) {
#pragma unroll
					for(int u = 0; u < NBAT; u++)
#pragma unroll
						for(int r = 0; r < 2; r++) x[u][r] = valid[u][r] ? x[u][r] : 0.0;
				}
			}
#pragma unroll
			for(int u = 0; u < NBAT; u++)
#pragma unroll
				for(int j = 0; j < QV; j++) {
					const double bv = brow[u][j];
					acc[0][j] = __builtin_fma(x[u][0], bv, acc[0][j]);
					acc[1][j] = __builtin_fma(x[u][1], bv, acc[1][j]);
				}
		};
		auto seg = [&](auto kindTag, auto twoTag, int k0, int k1) {
			int k = k0; // (every class holds an even number of columns)
			if(full) {
				// (columns in flight: eight next to at most 2 x 12 sums, two next to more: C5 with 13 / 15 columns of B 1.86 / 2.02
				// instead of 2.14 / 2.67 ms)
				if constexpr(QV <= 12) {
#pragma unroll 1
					for(; k + 8 <= k1; k += 8) batch(kindTag, twoTag, std::integral_constant<int, 8>(), std::false_type(), k);
					if(k + 4 <= k1) { batch(kindTag, twoTag, std::integral_constant<int, 4>(), std::false_type(), k); k += 4; }
				}
#pragma unroll 1
				for(; k + 2 <= k1; k += 2) batch(kindTag, twoTag, std::integral_constant<int, 2>(), std::false_type(), k);
			}
			else {
#pragma unroll 1
				for(; k + 2 <= k1; k += 2) batch(kindTag, twoTag, std::integral_constant<int, 2>(), std::true_type(), k);
			}
		};
		seg(std::integral_constant<int, 3>(), std::false_type(), 0, A.segEnd[DSEG_DDC1]);
		seg(std::integral_constant<int, 3>(), std::true_type(), A.segEnd[DSEG_DDC1], A.segEnd[DSEG_DDC2]);
		seg(std::integral_constant<int, 1>(), std::false_type(), A.segEnd[DSEG_DDC2], A.segEnd[DSEG_GAP1]);
		seg(std::integral_constant<int, 2>(), std::false_type(), A.segEnd[DSEG_GAP2], A.segEnd[DSEG_DENSE]);
		// through the wave's staging area, 32 rows (16 lanes) at a time: full-line stores of consecutive output rows
#pragma unroll 1
		for(int part = 0; part < DIR_SLICE / DIR_SROWS; part++) {
			dec_wave_sync(); // the readers of the staging area are done
			if((lane >> 4) == part) {
				double* w = wstage + (size_t) (lane & 15) * 2 * QV;
#pragma unroll
				for(int j = 0; j < QV; j++) { w[j] = acc[0][j]; w[QV + j] = acc[1][j]; }
			}
			dec_wave_sync();
			const int64_t rowBase = s0 + part * DIR_SROWS;
			const int nr = (int) max((int64_t) 0, min((int64_t) DIR_SROWS, nRows - rowBase));
			const int n = nr * QV;
			if(A.ld == QV) { // (uniform) the rows are one contiguous range of the output
				double* o = A.out + (size_t) rowBase * QV; // (a multiple of 16 bytes: rowBase is even)
#pragma unroll
				for(int i = 2 * lane; i < DIR_SROWS * QV; i += 128) {
					if(i + 1 < n) {
						const f64x2 v = *(const f64x2*) (wstage + i);
						cnt += (v[0] != 0.0) + (v[1] != 0.0);
						__builtin_nontemporal_store(v, (f64x2*) (o + i));
					}
					else if(i < n) {
						const double v = wstage[i];
						cnt += v != 0.0;
						__builtin_nontemporal_store(v, o + i);
					}
				}
			}
			else { // QV of the output's ld columns: pieces of QV values per row (pairs where QV is even and the output allows 16-byte stores)
				double* o = A.out + (size_t) rowBase * A.ld;
				const bool pairs = (QV & 1) == 0 && (A.ld & 1) == 0 && ((uintptr_t) A.out & 15) == 0;
#pragma unroll
				for(int i = 2 * lane; i < DIR_SROWS * QV; i += 128) {
					const int r0 = i / QV, c0 = i - r0 * QV;
					if(pairs) {
						if(i + 1 < n) {
							const f64x2 v = *(const f64x2*) (wstage + i);
							cnt += (v[0] != 0.0) + (v[1] != 0.0);
							__builtin_nontemporal_store(v, (f64x2*) (o + (size_t) r0 * A.ld + c0));
						}
					}
					else {
#pragma unroll
						for(int e = 0; e < 2; e++)
							if(i + e < n) {
								const int r = (i + e) / QV, c = (i + e) - r * QV;
								const double v = wstage[i + e];
								cnt += v != 0.0;
								__builtin_nontemporal_store(v, o + (size_t) r * A.ld + c);
							}
					}
				}
			}
		}
	}
	count_add(A.nnz, cnt);
}

struct DirPlan {
	int rc = 1;            // 0 usable, 1 the block does not qualify
	void* dImg = nullptr;
	int64_t bytes = 0;
	DirArgs A;
	std::vector<RunCol> runs; // run-length columns that are followed by run, and their merged run table
	Mrt mrt;
};

static int dir_build_plan(cla_block* b, DirPlan& P) {
	P.rc = 1;
	const int nG = (int) b->groups.size();
	{
		const int rc = ensure_expanded(b);
		if(rc) return rc;
	}
	std::vector<DirDict> dicts;
	std::vector<RunCol> runs;
	std::vector<DirCol> cols[DSEG_N];
	size_t valD = 0;
	for(int g = 0; g < nG; g++) {
		const DGroup& G = b->groups[g].d;
		const auto& hc = b->groups[g].cols;
		if(G.nColG >= (1 << 14)) return 0;
		if(G.type == G_UNC) {
			if(((uintptr_t) G.dense & 7) != 0) return 0;
			for(int h = 0; h < G.nColG; h++) cols[DSEG_DENSE].push_back(DirCol{(const uint8_t*) (G.dense + h), 0, G.nColG * 8, hc[h], 0, 0, 0});
			continue;
		}
		if(G.type != G_DDC && G.type != G_RLE && !(G.type == G_SDCZ && G.nOffsets > 0)) continue; // no row data
		const uint8_t* src;
		int cls;
		if(G.type == G_DDC) {
			if(G.codeWidth > 2 || ((uintptr_t) G.codes & 3) != 0) return 0;
			src = (const uint8_t*) G.codes;
			cls = G.codeWidth == 2 ? DSEG_DDC2 : DSEG_DDC1;
		}
		else {
			if(b->expCodes[g] == nullptr) {
				if(G.type != G_RLE) return 0;
				// a run-length group of long runs: its columns are followed by run (the constant row carries the columns' constants)
				for(int h = 0; h < G.nColG; h++) runs.push_back(RunCol{G.runStart, G.runCode, G.dict, 0.0, G.nRuns, G.nColG, h, hc[h]});
				continue;
			}
			src = b->expCodes[g];
			cls = DSEG_GAP1;
		}
		dicts.push_back(DirDict{G.dict, G.nVals * G.nColG, (int32_t) valD});
		for(int h = 0; h < G.nColG; h++) cols[cls].push_back(DirCol{src, (int32_t) (8 * (valD + h)), G.nColG * 8, hc[h], 0, 0, 0});
		valD += (size_t) G.nVals * G.nColG;
		if(valD * 8 > (size_t) 150 * 1024) return 0;
	}
	valD = (valD + 1) & ~(size_t) 1;
	const size_t zeroAt = valD; // two zeros behind the dictionaries
	valD += 2;
	std::vector<DirCol> all;
	for(int sgm = 0; sgm < DSEG_N; sgm++) {
		for(const DirCol& C : cols[sgm]) all.push_back(C);
		if((cols[sgm].size() & 1) != 0) { // classes of even size: a filler column (a real stream, the zero behind the dictionaries, a row of zeros for B)
			DirCol F = cols[sgm].back();
			if(sgm == DSEG_DENSE) return 0; // (a dense filler would need a stream of its own: odd numbers of dense columns take the tile kernel)
			F.base8 = (int32_t) (8 * zeroAt); F.nC8 = 0; F.orig = -1;
			all.push_back(F);
		}
		P.A.segEnd[sgm] = (int) all.size();
	}
	if(all.empty() || runs.size() > (size_t) RC_MAX || (!runs.empty() && b->nRows >= ((int64_t) 1 << 31) - 2 * DIR_SLICE)) return 0;
	const size_t colBytes = all.size() * sizeof(DirCol), dictBytes = dicts.size() * sizeof(DirDict);
	std::vector<uint8_t> img(colBytes + dictBytes + 16 * 8, 0);
	std::memcpy(img.data(), all.data(), colBytes);
	if(dictBytes) std::memcpy(img.data() + colBytes, dicts.data(), dictBytes);
	uint8_t* d = nullptr;
	CLA_HIP(hipMalloc((void**) &d, img.size() + 64));
	P.dImg = d;
	P.bytes = (int64_t) img.size() + 64;
	CLA_HIP(hipMemcpy(d, img.data(), img.size(), hipMemcpyHostToDevice));
	P.A.cols = (const DirCol*) d;
	P.A.dicts = (const DirDict*) (d + colBytes);
	P.A.zeroRow = (const double*) (d + colBytes + dictBytes);
	P.A.nR = (int) runs.size();
	P.A.mrtStart = nullptr; P.A.sliceRec = nullptr; P.A.runSums = nullptr;
	if(!runs.empty()) {
		const int rc = mrt_build(b, runs, DIR_SLICE, P.mrt);
		if(rc) return rc < 0 ? rc : 0;
		P.runs = runs;
		P.bytes += P.mrt.bytes;
		P.A.mrtStart = P.mrt.start; P.A.sliceRec = P.mrt.sliceRec; P.A.runSums = P.mrt.sums;
	}
	P.A.nDicts = (int) dicts.size();
	P.A.dictDoubles = (int) valD;
	P.A.nRows = b->nRows;
	P.rc = 0;
	return 0;
}

void dir_plan_drop(cla_block* b) {
	if(b->dirPlan == nullptr) return;
	if(b->dirPlan->dImg) { (void) hipFree(b->dirPlan->dImg); b->derivedBytes -= b->dirPlan->bytes; }
	mrt_free(b->dirPlan->mrt);
	delete b->dirPlan;
	b->dirPlan = nullptr;
}

static int dir_plan_get(cla_block* b) {
	if(b->dirPlan == nullptr) {
		b->dirPlan = new DirPlan();
		const int rc = dir_build_plan(b, *b->dirPlan);
		if(rc < 0) { dir_plan_drop(b); return rc; }
		if(b->dirPlan->dImg) b->derivedBytes += b->dirPlan->bytes;
	}
	return b->dirPlan->rc;
}

// Returns 1 when the block does not qualify (the caller takes the tile kernel).
static int launch_rmm_direct(cla_block* b, const double* dB, int q, const double* dConstRow, double* dOut, unsigned long long* dNnz) {
	{
		const int rc = dir_plan_get(b);
		if(rc) return rc;
	}
	DirArgs A = b->dirPlan->A;
	const size_t ldsMax = ((size_t) A.dictDoubles + (size_t) DIR_WAVES * DIR_SROWS * std::min(q, 16)) * 8;
	if(ldsMax > (size_t) std::min(g_ldsPerBlock, 160 * 1024) - 1024) return 1;
	A.nnz = dNnz; A.ld = q;
	const int64_t nSlices = (b->nRows + DIR_SLICE - 1) / DIR_SLICE;
	const unsigned grid = (unsigned) std::min<int64_t>((nSlices + DIR_WAVES - 1) / DIR_WAVES, g_numCU);
	// B wider than 16 columns: 16 columns per pass over the block (whole 128-byte lines of the output rows; 12 columns
	// per pass take less time per column to compute and twice as long to store: C5, 64 columns: 23 against 10 ms)
	const int chunk = 16;
	for(int c0 = 0; c0 < q; c0 += chunk) {
		const int qv = std::min(chunk, q - c0);
		const size_t lds = ((size_t) A.dictDoubles + (size_t) DIR_WAVES * DIR_SROWS * qv) * 8;
		A.B = dB + c0; A.constRow = dConstRow ? dConstRow + c0 : nullptr; A.out = dOut + c0;
		const double algo = (double) b->device_bytes_cached + (double) b->nRows * qv * 8;
		if(A.nR > 0) {
			const int rc = launch_run_sums(b, b->dirPlan->runs, b->dirPlan->mrt, A.B, q, qv, A.constRow);
			if(rc) return rc;
		}
		Prof pf(b, "k_rmm_direct", grid, DIR_THREADS, (long) lds, algo);
		switch(qv) {
#define DIR_CASE(QV)                                                                                         \
	case QV:                                                                                                 \
		if(A.nR > 0) {                                                                                       \
			CLA_HIP(allow_full_lds((const void*) k_rmm_direct<QV, true>));                                   \
			hipLaunchKernelGGL((k_rmm_direct<QV, true>), dim3(grid), dim3(DIR_THREADS), lds, b->stream, A);  \
		}                                                                                                    \
		else {                                                                                               \
			CLA_HIP(allow_full_lds((const void*) k_rmm_direct<QV, false>));                                  \
			hipLaunchKernelGGL((k_rmm_direct<QV, false>), dim3(grid), dim3(DIR_THREADS), lds, b->stream, A); \
		}                                                                                                    \
		break;
			DIR_CASE(1) DIR_CASE(2) DIR_CASE(3) DIR_CASE(4) DIR_CASE(5) DIR_CASE(6) DIR_CASE(7) DIR_CASE(8)
			DIR_CASE(9) DIR_CASE(10) DIR_CASE(11) DIR_CASE(12) DIR_CASE(13) DIR_CASE(14) DIR_CASE(15) DIR_CASE(16)
#undef DIR_CASE
			default: return -CLA_ERR_INVALID;
		}
	}
	CLA_HIP(hipGetLastError());
	return 0;
}

// Returns 1 when the block/shape is not eligible (caller uses the generic path).
int launch_rmm_decode(cla_block* b, const double* dB, int q, const double* dConstRow, double* dOut,
	unsigned long long* dNnz) {
	if(b->groups.empty() || b->nRows == 0 || q < 1) return 1;
	// (16 columns: no padding of B left for the tile kernel to lose, and the stream kernel short of registers: C5 2.1 against 2.5 ms)
	// (... unless run-length columns are followed by run: the tile kernel would expand them tile by tile, 2.4 against 2.2 ms)
	bool tilesFirst = q == DEC_QMAX;
	if(tilesFirst && b->opt.rmmDirect && dir_plan_get(b) == 0 && b->dirPlan->A.nR > 0) tilesFirst = false;
	if(b->opt.rmmDirect && !tilesFirst) {
		const int rc = launch_rmm_direct(b, dB, q, dConstRow, dOut, dNnz);
		if(rc != 1) return rc;
	}
	// (B wider than 16 columns: 16 columns per pass over the block, as in the stream kernel; not where offset lists
	// carry most of the block: their own tile kernel works per entry, this one per row)
	if(q > DEC_QMAX) {
		int nLists = 0, nOther = 0;
		for(auto& g : b->groups) {
			if(g.d.type == G_SDCZ) nLists += g.d.nOffsets > 0;
			else nOther += g.d.type == G_UNC || g.d.nVals > 0;
		}
		if(nOther == 0 || nLists > nOther) return 1;
	}
	for(int c0 = 0; c0 < q; c0 += DEC_QMAX) {
		const int qv = std::min(DEC_QMAX, q - c0);
		DecLaunch L;
		int rpl = 4; // rows per lane and pass: the smaller output staging area when LDS is short
		int rc = dec_prepare(b, false, qv, rpl, L);
		if(rc == 1) rc = dec_prepare(b, false, qv, rpl = 2, L);
		if(rc == 1 && c0 == 0 && tilesFirst && b->opt.rmmDirect) return launch_rmm_direct(b, dB, q, dConstRow, dOut, dNnz);
		if(rc) return rc;
		L.A.B = dB + c0; L.A.ld = q; L.A.constRow = dConstRow ? dConstRow + c0 : nullptr; L.A.out = dOut + c0; L.A.nnz = dNnz;
		double algo = (double) b->device_bytes_cached + (double) b->nRows * qv * 8;
		Prof pf(b, "k_rmm_decode", L.grid, DEC_THREADS, (long) L.lds, algo);
		if(rpl == 4) {
			CLA_HIP(allow_full_lds((const void*) k_rmm_decode<4>));
			hipLaunchKernelGGL(k_rmm_decode<4>, dim3(L.grid), dim3(DEC_THREADS), L.lds, b->stream, L.A);
		}
		else {
			CLA_HIP(allow_full_lds((const void*) k_rmm_decode<2>));
			hipLaunchKernelGGL(k_rmm_decode<2>, dim3(L.grid), dim3(DEC_THREADS), L.lds, b->stream, L.A);
		}
	}
	CLA_HIP(hipGetLastError());
	return 0;
}

// dOut (p x nCols, zeroed) += Y %*% D of the decoded rows, constants included; *dBad is set when Y holds a value that is
// not finite (the result is then not the reference's: a row that a group does not cover stays out of that group's sums
// there, here it is a decoded zero). Returns 1 when the block is not eligible (more than 64 columns, LDS plan too large).
int launch_lmm_decode(cla_block* b, const double* dY, int p, double* dOut, unsigned long long* dBad) {
	const int nCols = b->nCols;
	if(b->groups.empty() || b->nRows == 0 || nCols > 64 || p < 1 || p > 16) return 1;
	const int NB = (nCols + 15) / 16;
	DecLaunch L;
	bool flat = false;
	int rc = gram_prepare(b, L, flat);
	if(rc) return rc;
	L.A.out = dOut; L.A.Y = dY; L.A.P = p; L.A.badY = dBad;
	Prof pf(b, "k_lmm_decode", L.grid, DEC_THREADS, (long) L.lds, (double) b->device_bytes_cached + (double) b->nRows * p * 8);
#define LM_LAUNCH(NBV, FL)                                                                                      \
	do {                                                                                                        \
		CLA_HIP(allow_full_lds((const void*) k_lmm_decode<NBV, FL>));                                           \
		hipLaunchKernelGGL((k_lmm_decode<NBV, FL>), dim3(L.grid), dim3(DEC_THREADS), L.lds, b->stream, L.A); \
	} while(0)
	if(!flat) { if(NB == 1) LM_LAUNCH(1, 0); else if(NB == 2) LM_LAUNCH(2, 0); else if(NB == 3) LM_LAUNCH(3, 0); else LM_LAUNCH(4, 0); }
	else { if(NB == 1) LM_LAUNCH(1, 1); else if(NB == 2) LM_LAUNCH(2, 1); else if(NB == 3) LM_LAUNCH(3, 1); else LM_LAUNCH(4, 1); }
#undef LM_LAUNCH
	CLA_HIP(hipGetLastError());
	return 0;
}

// dOut (nCols x nCols, zeroed) += upper triangle of t(D) %*% D of the decoded rows, constants
// included. Returns 1 when the block is not eligible (more than 64 columns, LDS plan too large).
// dNnz != nullptr: the kernel is the call's only one (dOut need not be zero; it is written whole, mirrored, and its
// non-zeros are counted into *dNnz by the last block, gram_tail), else the caller has zeroed dOut, mirrors and counts.
int launch_tsmm_decode(cla_block* b, double* dOut, unsigned long long* dNnz) {
	const int nCols = b->nCols;
	if(b->groups.empty() || b->nRows == 0 || nCols > 64) return 1;
	if(dNnz != nullptr && (b->crossBlocks > 0 || b->crossSplit > 0)) return 1; // (only a part of the Gram matrix is wanted: no one-kernel form)
	{
		const int rc = launch_tsmm_direct(b, dOut, dNnz);
		if(rc != 1) return rc;
	}
	const int NB = (nCols + 15) / 16;
	// only the product of the first crossBlocks column blocks with the others is wanted (a pair of column chunks
	// whose own Gram matrices nobody reads): shapes 1 x 1, 1 x 2, 2 x 1, 2 x 2 blocks, anything else in full
	int XB = b->crossBlocks;
	if(XB < 1 || XB > 2 || NB - XB < 1 || NB - XB > 2) XB = 0;
	DecLaunch L;
	bool flat = false;
	int rc = gram_prepare(b, L, flat);
	if(rc) return rc;
	L.A.out = dOut;
	if(dNnz != nullptr) {
		if((rc = ensure_gram_acc(b))) return rc;
		L.A.acc = b->dGramAcc; L.A.done = (unsigned*) (b->dCounters + 7); L.A.nnz = dNnz;
	}
	Prof pf(b, "k_tsmm_decode", L.grid, DEC_THREADS, (long) L.lds, (double) b->device_bytes_cached);
	// a last column block of at most 4 columns: its rows on the 4 x 4 x 4 matrix instruction
	const bool narrow = XB == 0 && NB >= 2 && nCols - 16 * (NB - 1) <= 4 && b->opt.tsmmNarrow;
#define GRAM_LAUNCH(NBV, FL, XBV)                                                                               \
	do {                                                                                                        \
		if(XBV == 0 && NBV >= 2 && narrow) {                                                                    \
			constexpr int NARV = XBV == 0 && NBV >= 2 ? 1 : 0;                                                  \
			CLA_HIP(allow_full_lds((const void*) k_tsmm_decode<NBV, FL, XBV, NARV>)); \
			hipLaunchKernelGGL((k_tsmm_decode<NBV, FL, XBV, NARV>), dim3(L.grid), dim3(DEC_THREADS), L.lds, b->stream, L.A); \
		}                                                                                                       \
		else {                                                                                                  \
			CLA_HIP(allow_full_lds((const void*) k_tsmm_decode<NBV, FL, XBV>)); \
			hipLaunchKernelGGL((k_tsmm_decode<NBV, FL, XBV>), dim3(L.grid), dim3(DEC_THREADS), L.lds, b->stream, L.A); \
		}                                                                                                       \
	} while(0)
#define GRAM_SHAPES(FL)                                        \
	do {                                                       \
		if(XB == 0) {                                          \
			if(NB == 1) GRAM_LAUNCH(1, FL, 0);                 \
			else if(NB == 2) GRAM_LAUNCH(2, FL, 0);            \
			else if(NB == 3) GRAM_LAUNCH(3, FL, 0);            \
			else GRAM_LAUNCH(4, FL, 0);                        \
		}                                                      \
		else if(NB == 2) GRAM_LAUNCH(2, FL, 1);                \
		else if(NB == 3 && XB == 1) GRAM_LAUNCH(3, FL, 1);     \
		else if(NB == 3) GRAM_LAUNCH(3, FL, 2);                \
		else GRAM_LAUNCH(4, FL, 2);                            \
	} while(0)
	if(!flat) GRAM_SHAPES(0);
	else GRAM_SHAPES(1);
#undef GRAM_SHAPES
#undef GRAM_LAUNCH
	CLA_HIP(hipGetLastError());
	return 0;
}

} // namespace cla
