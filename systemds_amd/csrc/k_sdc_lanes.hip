// SDCZeros mat-vecs on lane-major lists (gfx950).
//
//   k_lane_convert    one-time rewrite of the listed groups' offset and code lists into lane-major windows
//   k_lmm_sdc_lanes   out[col(g)] += sum over the listed rows of Y[row] * dict_g[code]   (t(v) %*% X)
//   k_rmm_sdc_lanes   out[row] += T_g[code] for every listed row                          (X %*% u)
//
// The groups are cut into slabs (a slab's dictionaries fit LDS; at most 256 groups). Rows are cut into windows of
// LN_WIN. For a (slab, window) every group's entries inside the window are stored in chunks of 16 bytes that hold
// seven entries - the row of the first (relative to the window), six row deltas, seven codes, one byte each, and
// the group's index inside the slab (its tag) - and the chunks of all groups of the slab, in group order, are dealt
// to the lanes of a wave in equal contiguous shares: with `rows` chunks per lane, chunk p of the window goes to lane
// p / rows as its chunk p % rows, and the lanes' chunks lie side by side. One 16-byte load per lane brings a chunk
// row, fully coalesced, and a window takes as many chunk rows as its chunks need (no group waits for a longer
// one; the last chunk row is filled up with unused chunks). A lane works through its share in order: it meets a
// few groups per window, each in consecutive chunks, and keeps the sum of the group at hand in registers.
//
// Chunk: word 0 = first row (14 bits; 0x3fff: unused chunk) | window index modulo LN_G << 14 | delta 1 << 16 |
// delta 2 << 24, word 1 = deltas 3..6, words 2 and 3 = codes 0..6 and, in the last byte, the tag. A gap of more
// than 255 rows inside a chunk takes entries of (255, spare) first, where the spare code nVals maps to a 0.0 behind
// the group's dictionary (or table); a chunk's unused entries are (0, spare).
//
// Left multiply: every wave holds the Y window it works on in LDS, with a 0.0 behind it at index LN_WIN; every
// entry adds Y[min(row, LN_WIN)] * dict[code] to the lane's sum (spare entries add Y[row] * 0.0; a window of Y with
// non-finite values takes the variant that sends spare entries to the 0.0 instead); where the tag changes, the sum
// goes to the group's accumulator in LDS. Right multiply: LN_G output windows sit in LDS, every entry with a tuple
// adds T[code] at its row with an LDS atomic; the slabs take turns, their tables in LDS in two buffers.
#include "../../include/cla_hip.h"
#include "cla_device.hpp"
#include <algorithm>
#include <numeric>
#include <vector>

namespace cla {

constexpr int LN_TPW = 1;                  // row tiles (SDC_TILE rows) per window
constexpr int LN_WIN = LN_TPW * SDC_TILE;  // rows per window
constexpr int LN_E = 7;                    // entries per chunk
constexpr int LN_TAGS = 256;               // groups per slab (a chunk's tag is a byte)
constexpr int LN_DICT_MAX = 6656;          // dictionary entries (spares included) of a slab in LDS (left: next to LN_LW windows of Y; right: two buffers next to the output windows)
constexpr int LN_YT = LN_WIN + 64;         // left: Y window + 64 slots of 0.0 behind it
constexpr int LN_LW = 12;                  // left: waves per block at most, each on windows of its own
constexpr int LN_LK = 8;                   // left: chunk rows requested ahead
constexpr int LN_RW = 16;                  // right: waves per block
constexpr int LN_G = 4;                    // right: output windows per block and round
constexpr int LN_RK = 6;                   // right: chunk rows per wave and (slab, round) requested a turn ahead
constexpr int LN_TMAX = (LN_DICT_MAX + LN_RW * 64 - 1) / (LN_RW * 64); // right: table entries per thread
constexpr uint32_t LN_NOROW = 0x3fffu;     // first row of an unused chunk
static_assert(LN_WIN < (int) LN_NOROW && LN_G == 4, "a chunk's first row is 14 bits next to the window's index modulo 4");

struct LaneDesc { // a group of a slab, 16 bytes
	int32_t g;        // index of the group in the block
	int32_t dictOff;  // its dictionary inside the slab's (nVals entries and the 0.0 of the spare code)
	int32_t spare;    // = nVals
	int32_t col0;     // the column of a single-column group
};

struct LaneSlab { // 48 bytes
	int32_t l0, n;             // groups desc[l0 .. l0 + n)
	int32_t dictOff, dictLen;  // their dictionaries inside the concatenation
	int32_t w, pad;            // lanes per chunk row (a power of two)
	int64_t dataOff;           // first chunk of the slab, in 16-byte units
	int64_t chunkOff;          // the slab's nWin + 1 chunk-row starts inside chunkStart
	int64_t cntOff;            // the slab's chunk counts per (window, group) inside the conversion's count array
};

// ---------------------------------------------------------------------------------------------
// Conversion. thread = (window, group of the slab): walks the group's list inside the window from the row-tile
// index and counts its chunks (FILL == false: into cnt, and the window's total into winTotal) or writes them
// (FILL == true) where the counts of the groups in front of it put them; the slab's last group also writes the
// unused chunks that fill the window's last chunk row.
// ---------------------------------------------------------------------------------------------
template <bool FILL>
__global__ __launch_bounds__(256) void k_lane_convert(const DGroup* __restrict__ groups, const LaneDesc* __restrict__ desc,
	const LaneSlab* __restrict__ slabs, int64_t nRows, int nWin, uint8_t* __restrict__ cnt, uint32_t* __restrict__ winTotal,
	const uint32_t* __restrict__ chunkStart, u32x4* __restrict__ data) {
	const LaneSlab S = slabs[blockIdx.y];
	const int win = blockIdx.x * 4 + (threadIdx.x >> 6);
	if(win >= nWin) return;
	uint8_t* myCnt = cnt + S.cntOff + (int64_t) win * S.n;
	for(int l = threadIdx.x & 63; l < S.n; l += 64) {
		const LaneDesc L = desc[S.l0 + l];
		const DGroup G = dgroup(groups + L.g);
		const int64_t r0 = (int64_t) win * LN_WIN, rEnd = r0 + LN_WIN;
		const uint32_t spare = (uint32_t) L.spare;
		const uint32_t spare4 = spare * 0x01010101u;
		const uint32_t wbits = (uint32_t) (win & (LN_G - 1)) << 14;
		uint32_t cs = 0, rows = 1, p0 = 0, total = 0;
		if(FILL) {
			cs = chunkStart[S.chunkOff + win];
			rows = chunkStart[S.chunkOff + win + 1] - cs;
			for(int k = 0; k < S.n; k++) {
				const uint32_t c = myCnt[k];
				p0 += k < l ? c : 0;
				total += c;
			}
		}
		u32x4* dst = data + S.dataOff + (int64_t) cs * S.w;
		auto place = [&](uint32_t p) { return dst + (int64_t) (p % rows) * S.w + p / rows; }; // chunk p of the window
		int nE = 0, prev = -1; // entries so far, row of the previous entry
		uint64_t dby = 0, cby = 0;
		auto flush = [&]() { // the chunk that holds entries nE - (nE % LN_E) .. (whole or partial)
			const int p = nE % LN_E == 0 ? LN_E : nE % LN_E;
			for(int t = p; t < LN_E; t++) cby |= (uint64_t) spare << (8 * t);
			cby |= (uint64_t) l << 56;
			u32x4 v = {(uint32_t) dby | wbits, (uint32_t) (dby >> 32), (uint32_t) cby, (uint32_t) (cby >> 32)};
			*place(p0 + (uint32_t) ((nE - 1) / LN_E)) = v;
			dby = 0; cby = 0;
		};
		auto put = [&](int row, uint32_t c) {
			if(FILL) {
				const int p = nE % LN_E;
				if(p == 0) dby = (uint64_t) (uint32_t) row;
				else dby |= (uint64_t) (uint32_t) (row - prev) << (8 * (p + 1));
				cby |= (uint64_t) c << (8 * p);
			}
			prev = row;
			nE++;
			if(FILL && nE % LN_E == 0) flush();
		};
		// the lists come in aligned pieces of 16 bytes (a piece behind the end of a list lies in the slack of its allocation)
		struct Piece {
			u32x4 v;
			int64_t at = -1;
		} pd, pc;
		auto word = [](const Piece& P, int k) { return k == 0 ? P.v.x : k == 1 ? P.v.y : k == 2 ? P.v.z : P.v.w; };
		auto fetch = [](Piece& P, const void* src, int64_t piece) {
			if(piece != P.at) {
				P.at = piece;
				P.v = *(const u32x4*) ((const uint8_t*) src + (piece << 4));
			}
		};
		auto entry = [&](int rel, int di) {
			while(nE % LN_E != 0 && rel - prev > 255) put(prev + 255, spare);
			uint32_t c = 0;
			if(FILL) { // (the groups of this form have codes of one byte)
				fetch(pc, G.codes, (int64_t) di >> 4);
				c = (word(pc, (di >> 2) & 3) >> (8 * (di & 3))) & 0xffu;
			}
			put(rel, c);
		};
		if(G.first >= r0 && G.first < rEnd) entry((int) (G.first - r0), 0);
		if(win * LN_TPW < G.nTiles) {
			const OffState st = G.tileIdx[win * LN_TPW];
			int64_t i = st.idx;
			int32_t row = st.row, emit = st.emit;
			const int maxV = G.deltaWidth == 1 ? 255 : 65535;
			for(; i < G.nDeltas; i++) {
				int v;
				if(G.deltaWidth == 1) {
					fetch(pd, G.deltas, i >> 4);
					v = (int) ((word(pd, (int) (i >> 2) & 3) >> (8 * (int) (i & 3))) & 0xffu);
				}
				else {
					fetch(pd, G.deltas, i >> 3);
					v = (int) ((word(pd, (int) (i >> 1) & 3) >> (16 * (int) (i & 1))) & 0xffffu);
				}
				const int64_t nr = (int64_t) row + (v == 0 ? maxV : v);
				if(nr >= rEnd) break;
				row = (int32_t) nr;
				if(v != 0) {
					if(nr >= r0) entry((int) (nr - r0), emit); // (the state in front of a window holds no row of it)
					emit++;
				}
			}
		}
		const uint32_t nCh = (uint32_t) (nE + LN_E - 1) / LN_E;
		if(FILL) {
			if(nE % LN_E != 0) flush();
			if(l == S.n - 1) {
				const u32x4 none = {LN_NOROW | wbits, 0u, spare4, (spare4 & 0x00ffffffu) | (uint32_t) l << 24};
				for(uint32_t p = total; p < rows * (uint32_t) S.w; p++) *place(p) = none;
			}
		}
		else {
			myCnt[l] = (uint8_t) nCh;
			if(nCh) atomicAdd(&winTotal[(int64_t) blockIdx.y * nWin + win], nCh);
		}
	}
}

// The seven rows (relative to the window; behind it for unused chunks) and codes of a chunk.
__device__ __forceinline__ void ln_decode(const u32x4 v, uint32_t (&row)[LN_E], uint32_t (&code)[LN_E]) {
	row[0] = v.x & LN_NOROW;
	row[1] = row[0] + ((v.x >> 16) & 0xffu);
	row[2] = row[1] + (v.x >> 24);
#pragma unroll
	for(int t = 3; t < LN_E; t++) row[t] = row[t - 1] + ((v.y >> (8 * (t - 3))) & 0xffu);
#pragma unroll
	for(int t = 0; t < LN_E; t++) code[t] = ((t < 4 ? v.z : v.w) >> (8 * (t & 3))) & 0xffu;
}

// ---------------------------------------------------------------------------------------------
// Left multiply. block = (share of the windows, slab, row of Y); every wave works on windows of its own, which
// the block's waves take from the block's share one by one.
// ---------------------------------------------------------------------------------------------
struct LnSum { // the group a lane is at: its tag, dictionary, spare code, sum so far
	uint32_t tag;
	const double* dict;
	uint32_t spare;
	double acc[4];
};

template <bool CAREFUL>
__device__ __forceinline__ void ln_lmm_chunk(const u32x4 v, const double* yt, const double* dictL, const uint32_t* descS,
	double* accS, bool live, LnSum& s) {
	const uint32_t tag = v.w >> 24;
	if(tag != s.tag) { // (a few times per window and lane)
		if(live && s.tag < (uint32_t) LN_TAGS) unsafeAtomicAdd(&accS[s.tag], (s.acc[0] + s.acc[1]) + (s.acc[2] + s.acc[3]));
		s.acc[0] = s.acc[1] = s.acc[2] = s.acc[3] = 0.0;
		s.tag = tag;
		const uint32_t d = descS[tag];
		s.dict = dictL + (d & 0xffffu);
		s.spare = d >> 16;
	}
	uint32_t row[LN_E], code[LN_E];
	ln_decode(v, row, code);
	double yv[LN_E], dv[LN_E];
#pragma unroll
	for(int t = 0; t < LN_E; t++) {
		uint32_t idx = min(row[t], (uint32_t) LN_WIN);
		if(CAREFUL) idx = code[t] == s.spare ? (uint32_t) LN_WIN : idx;
		yv[t] = yt[idx];
		dv[t] = s.dict[code[t]];
	}
#pragma unroll
	for(int t = 0; t < LN_E; t++) s.acc[t & 3] = __builtin_fma(yv[t], dv[t], s.acc[t & 3]);
}

__global__ __launch_bounds__(LN_LW * 64) void k_lmm_sdc_lanes(const LaneDesc* __restrict__ desc,
	const LaneSlab* __restrict__ slabs, int nSlabs, const double* __restrict__ dictAll, const uint32_t* __restrict__ descPk,
	int dictLds, const uint32_t* __restrict__ chunkStart, const u32x4* __restrict__ data, const double* __restrict__ Y,
	int64_t nRows, int nWin, double* __restrict__ out, int nCols, unsigned* __restrict__ done, unsigned long long* __restrict__ nnz) {
	extern __shared__ double smem[];
	const int tid = threadIdx.x, lane = tid & 63, nWaves = blockDim.x >> 6;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6); // (uniform: the chunk starts below come by scalar loads)
	double* dictL = smem;                                     // the slab's dictionaries
	double* accS = smem + dictLds;                             // the groups' sums (LN_TAGS)
	uint32_t* descS = (uint32_t*) (accS + LN_TAGS);            // per group: dictionary offset | spare code << 16 (LN_TAGS)
	int32_t* nextS = (int32_t*) (descS + LN_TAGS);             // the block's next window (2 slots: 8 bytes)
	double* yt = (double*) (nextS + 2) + wave * LN_YT;         // this wave's Y window
	// Blocks go round the 8 XCDs by their index. The slabs of a share of the windows read the same part of Y: they sit 8
	// block indices apart, on one XCD and at work at the same time, so that its L2 fetches that part of Y once.
	const int nParts = gridDim.x / nSlabs;
	const int period = 8 * nSlabs, grp = blockIdx.x / period, in = blockIdx.x % period;
	const int inLast = nParts - grp * 8 < 8 ? nParts - grp * 8 : 8; // shares of the last, partial period
	const int slab = in / inLast, part = grp * 8 + in % inLast;
	const LaneSlab S = slabs[slab];
	// the block's share of the windows
	const int wBeg = (int) ((int64_t) nWin * part / nParts), wEnd = (int) ((int64_t) nWin * (part + 1) / nParts);
	for(int k0 = tid; k0 < S.dictLen; k0 += 8 * blockDim.x) { // eight loads in flight per thread
		double v[8];
#pragma unroll
		for(int j = 0; j < 8; j++) v[j] = dictAll[S.dictOff + min(k0 + j * (int) blockDim.x, S.dictLen - 1)];
#pragma unroll
		for(int j = 0; j < 8; j++)
			if(k0 + j * (int) blockDim.x < S.dictLen) dictL[k0 + j * (int) blockDim.x] = v[j];
	}
	for(int k = tid; k < LN_TAGS; k += blockDim.x) {
		accS[k] = 0.0;
		descS[k] = descPk[S.l0 + min(k, S.n - 1)];
	}
	if(tid == 0) nextS[0] = wBeg + nWaves; // (the waves start on windows wBeg + wave)
	yt[LN_WIN + lane] = 0.0;
	__syncthreads();
	const bool live = lane < S.w; // lanes behind the chunk row's width repeat its last lane, their sums are dropped
	const int w = S.w;
	const double* y = Y + (size_t) blockIdx.y * nRows;
	const uint32_t* cst = chunkStart + S.chunkOff;
	const u32x4* base = data + S.dataOff + min(lane, w - 1);
	LnSum sum;
	sum.tag = 0xffffffffu; sum.dict = dictL; sum.spare = 0;
	sum.acc[0] = sum.acc[1] = sum.acc[2] = sum.acc[3] = 0.0;
	// A unit is up to LN_LK chunk rows of a window. Requested a unit ahead: its chunk rows and, in front of a window's
	// first unit, the lane's share of the Y window. Two sets of chunk rows take turns; a unit's work is straight-line code
	// on its set (no loads inside: the compiler's wait counts are exact).
	struct Ahead {
		u32x4 buf[LN_LK];
		uint32_t c0, c1;  // the unit's chunk rows (c0 < c1 <= c0 + LN_LK)
		uint32_t cw1;     // end of its window's chunk rows
		int win;          // its window; -1: no unit
		bool first;       // the window's first unit
	};
	double yreg[LN_WIN / 64]; // Y of the window whose first unit was requested last
	auto request_rows = [&](Ahead& A) {
#pragma unroll
		for(int j = 0; j < LN_LK; j++) A.buf[j] = __builtin_nontemporal_load(base + (int64_t) min(A.c0 + j, A.c1 - 1) * w);
	};
	auto request_window = [&](Ahead& A, int win) { // win < wEnd: the window's first unit
		A.win = win; A.first = true;
		A.c0 = cst[win];
		A.cw1 = cst[win + 1]; // (every window holds a chunk row)
		A.c1 = min(A.c0 + LN_LK, A.cw1);
		request_rows(A);
		const int64_t r0 = (int64_t) win * LN_WIN;
#pragma unroll
		for(int k = 0; k < LN_WIN / 64; k++) yreg[k] = y[min(r0 + k * 64 + lane, nRows - 1)]; // unconditional: a load under a branch is waited for at the branch's end
	};
	auto request_next = [&](const Ahead& A, Ahead& B) { // the unit behind A
		if(A.c1 < A.cw1) {
			B.win = A.win; B.first = false;
			B.c0 = A.c1; B.cw1 = A.cw1;
			B.c1 = min(B.c0 + LN_LK, B.cw1);
			request_rows(B);
		}
		else {
			int nw = 0;
			if(lane == 0) nw = atomicAdd(&nextS[0], 1);
			nw = __builtin_amdgcn_readfirstlane(nw);
			if(nw < wEnd) request_window(B, nw);
			else B.win = -1;
		}
	};
	bool careful = false;
	auto work = [&](Ahead& A, Ahead& B) { // A holds a unit, B takes the one behind it
		if(A.first) {
			const int64_t r0 = (int64_t) A.win * LN_WIN;
			bool bad = false;
			__builtin_amdgcn_wave_barrier(); // (the previous window's reads are done: LDS serves a wave's accesses in order)
#pragma unroll
			for(int k = 0; k < LN_WIN / 64; k++) {
				const double v = r0 + k * 64 + lane < nRows ? yreg[k] : 0.0;
				bad |= !isfinite(v);
				yt[k * 64 + lane] = v;
			}
			careful = __builtin_amdgcn_ballot_w64(bad) != 0;
			__builtin_amdgcn_wave_barrier();
		}
		const uint32_t c0 = A.c0, c1 = A.c1;
		u32x4 cur[LN_LK];
#pragma unroll
		for(int j = 0; j < LN_LK; j++) cur[j] = A.buf[j];
		request_next(A, B);
#pragma unroll
		for(int j = 0; j < LN_LK; j++) {
			if(c0 + j < c1) {
				if(careful) ln_lmm_chunk<true>(cur[j], yt, dictL, descS, accS, live, sum);
				else ln_lmm_chunk<false>(cur[j], yt, dictL, descS, accS, live, sum);
			}
		}
	};
	if(wBeg + wave < wEnd) {
		Ahead A, B;
		request_window(A, wBeg + wave);
		for(;;) {
			work(A, B);
			if(B.win < 0) break;
			work(B, A);
			if(A.win < 0) break;
		}
	}
	if(live && sum.tag < (uint32_t) LN_TAGS) unsafeAtomicAdd(&accS[sum.tag], (sum.acc[0] + sum.acc[1]) + (sum.acc[2] + sum.acc[3]));
	__syncthreads();
	for(int k = tid; k < S.n; k += blockDim.x) unsafeAtomicAdd(&out[(size_t) blockIdx.y * nCols + desc[S.l0 + k].col0], accS[k]);
	lmm_tail(done, gridDim.x * gridDim.y, out, (int) gridDim.y * nCols, nnz);
}

// ---------------------------------------------------------------------------------------------
// Right multiply with one output column. block = run of windows, in rounds of LN_G windows whose output sits in
// LDS. In a round the slabs take turns; the block's waves share the chunk rows of the slab's LN_G windows (a chunk
// stands for itself: it carries its rows, its window and its group). The tables of the next turn's slab (T gathered
// through tblIndex, -1 = the 0.0 of a spare code) and its groups' table offsets are fetched during a turn and stored
// into the other buffer behind it. accumulate == 0: a window starts from constRow (or zero) and is the whole
// result; accumulate != 0: it starts from what other groups already wrote.
// ---------------------------------------------------------------------------------------------
template <bool RESIDENT>
__global__ __launch_bounds__(LN_RW * 64) void k_rmm_sdc_lanes(const LaneSlab* __restrict__ slabs, int nSlabs,
	const uint32_t* __restrict__ descPk, const int32_t* __restrict__ tblIndex, int dictLds, int dictTotal,
	const uint32_t* __restrict__ chunkStart, const u32x4* __restrict__ data, const double* __restrict__ T, int constRow,
	int accumulate, double* __restrict__ out, int64_t nRows, int nWin, int winPerBlock, unsigned long long* __restrict__ nnz) {
	extern __shared__ double smem[];
	double* tblAll = smem;                 // RESIDENT: the tables of all slabs (dictTotal entries); else two buffers of dictLds entries
	double* ot = smem + (RESIDENT ? dictTotal : 2 * dictLds); // LN_G windows of output
	uint32_t* descS = (uint32_t*) (ot + LN_G * LN_WIN + 64);  // two buffers of LN_TAGS: table offset | spare code << 16 per group of the slab
	const int tid = threadIdx.x, lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	constexpr int THREADS = LN_RW * 64, OPT = LN_G * LN_WIN / THREADS;
	const int wBeg = min((int) blockIdx.x * winPerBlock, nWin), wEnd = min(wBeg + winPerBlock, nWin);
	if(wBeg >= wEnd) return;
	const double init = !accumulate && constRow >= 0 ? T[constRow] : 0.0;
	const int nRounds = (wEnd - wBeg + LN_G - 1) / LN_G, nTurns = nRounds * nSlabs;
	double treg[LN_TMAX];
	uint32_t dreg = 0;
	auto tbl_request = [&](int s) {
		const LaneSlab S = slabs[s];
		if(!RESIDENT) {
#pragma unroll
			for(int k = 0; k < LN_TMAX; k++) {
				const int e = k * THREADS + tid;
				const int32_t ti = tblIndex[S.dictOff + min(e, S.dictLen - 1)];
				treg[k] = T[max(ti, 0)];
				treg[k] = ti >= 0 ? treg[k] : 0.0;
			}
		}
		dreg = descPk[S.l0 + min(tid, S.n - 1)];
	};
	auto tbl_store = [&](int turn) {
		const int buf = nSlabs > 1 ? turn & 1 : 0; // (one slab: its tables stay)
		if(!RESIDENT) {
			double* tb = tblAll + buf * dictLds;
#pragma unroll
			for(int k = 0; k < LN_TMAX; k++)
				if(k * THREADS + tid < dictLds) tb[k * THREADS + tid] = treg[k];
		}
		if(tid < LN_TAGS) descS[buf * LN_TAGS + tid] = dreg;
	};
	struct Ahead {
		u32x4 buf[LN_RK];
		uint32_t c0, c1; // this wave's first chunk row of the turn, end of the turn's chunk rows
	};
	auto request = [&](Ahead& A, int turn) { // turn < nTurns
		const int s = turn % nSlabs, wg = wBeg + (turn / nSlabs) * LN_G;
		const LaneSlab S = slabs[s];
		const uint32_t* cst = chunkStart + S.chunkOff;
		A.c0 = cst[wg] + wave;
		A.c1 = cst[min(wg + LN_G, wEnd)];
		const u32x4* base = data + S.dataOff + min(lane, S.w - 1);
#pragma unroll
		for(int j = 0; j < LN_RK; j++) A.buf[j] = *(base + (int64_t) min(A.c0 + j * LN_RW, A.c1 - 1) * S.w);
	};
	auto add_chunk = [&](const u32x4 v, const double* tbl, const uint32_t* dsc) {
		const uint32_t off = ((v.x >> 14) & 3u) * (uint32_t) LN_WIN; // the chunk's window inside the round (rounds start at multiples of LN_G)
		const uint32_t d = dsc[v.w >> 24];
		const double* tg = tbl + (d & 0xffffu);
		const uint32_t spare = d >> 16;
		uint32_t row[LN_E], code[LN_E];
		ln_decode(v, row, code);
		double tv[LN_E];
#pragma unroll
		for(int t = 0; t < LN_E; t++) tv[t] = tg[code[t]];
		// (LDS adds of doubles take about a cycle per lane: spare entries stay out of them; an entry with a tuple
		// lies inside its window)
#pragma unroll
		for(int t = 0; t < LN_E; t++)
			if(code[t] != spare) unsafeAtomicAdd(&ot[row[t] + off], tv[t]);
	};
	int cntNz = 0;
	auto work = [&](Ahead& A, Ahead& B, int turn) {
		const int s = turn % nSlabs, round = turn / nSlabs, wg = wBeg + round * LN_G;
		if(s == 0) { // a new round: the output windows start from their initial values
#pragma unroll
			for(int k = 0; k < OPT; k++) {
				const int64_t r = (int64_t) wg * LN_WIN + k * THREADS + tid;
				ot[k * THREADS + tid] = accumulate ? out[min(r, nRows - 1)] : init;
			}
			__syncthreads();
		}
		const int next = turn + 1 < nTurns ? turn + 1 : turn;
		if(nSlabs > 1) tbl_request(next % nSlabs);
		request(B, next);
		const LaneSlab S = slabs[s];
		const int buf = nSlabs > 1 ? turn & 1 : 0;
		const double* tbl = tblAll + (RESIDENT ? S.dictOff : buf * dictLds);
		const uint32_t* dsc = descS + buf * LN_TAGS;
		const u32x4* base = data + S.dataOff + min(lane, S.w - 1);
		const uint32_t c0 = A.c0, c1 = A.c1;
		if(lane < S.w) {
#pragma unroll
			for(int j = 0; j < LN_RK; j++)
				if(c0 + j * LN_RW < c1) add_chunk(A.buf[j], tbl, dsc);
			for(uint32_t c = c0 + LN_RK * LN_RW; c < c1; c += LN_RW) add_chunk(*(base + (int64_t) c * S.w), tbl, dsc);
		}
		if(nSlabs > 1) tbl_store(turn + 1); // the other buffers were last read before the previous barrier
		if(nSlabs > 1 || s == nSlabs - 1) __syncthreads();
		if(s == nSlabs - 1) { // the round's windows are complete
#pragma unroll
			for(int k = 0; k < OPT; k++) {
				const int64_t r = (int64_t) wg * LN_WIN + k * THREADS + tid;
				if(r < nRows && r < (int64_t) wEnd * LN_WIN) {
					const double v = ot[k * THREADS + tid];
					cntNz += v != 0.0;
					out[r] = v;
				}
			}
			// (the next round's initial values are written by the same threads to the same slots)
		}
	};
	if(RESIDENT) {
		for(int k = tid; k < dictTotal; k += THREADS) {
			const int32_t ti = tblIndex[k];
			tblAll[k] = ti >= 0 ? T[ti] : 0.0;
		}
	}
	tbl_request(0);
	tbl_store(0);
	Ahead A, B;
	request(A, 0);
	// (the first round's barrier behind the initial values also orders the first tables)
	for(int turn = 0; turn < nTurns; turn += 2) {
		work(A, B, turn);
		if(turn + 1 < nTurns) work(B, A, turn + 1);
	}
	count_add(nnz, cntNz);
}

// ---------------------------------------------------------------------------------------------
// Host side: the lane-major form of the block's listed groups (whole-block plan), built once.
// ---------------------------------------------------------------------------------------------
static int lanes_plan(cla_block* b) {
	if(b->laneState != 0) return 0;
	b->laneState = -1;
	const std::vector<int32_t>& list = b->sdcList;
	const int nL = (int) list.size();
	const int nWin = (int) ((b->nRows + LN_WIN - 1) / LN_WIN);
	if(nL == 0 || nWin == 0 || b->nRows >= ((int64_t) 1 << 31) - LN_WIN) return 0;
	double rawBytes = 0;
	bool singleCols = true;
	for(int g : list) {
		const DGroup& G = b->groups[g].d;
		if(G.codeWidth != 1 || G.nVals > 255) return 0; // a slot's code is a byte, nVals is the spare code
		singleCols &= G.nColG == 1;
		rawBytes += (double) G.nDeltas * G.deltaWidth + (double) G.nOffsets;
	}
	// slabs of equal group counts within the tags of a chunk and the LDS budget (the left multiply's waves, each with
	// a window of Y, next to the dictionaries; the right multiply's two table buffers next to its output windows)
	std::vector<int32_t> order(list.begin(), list.end());
	std::vector<int32_t> dictOffAll(nL + 1, 0);
	for(int l = 0; l < nL; l++) dictOffAll[l + 1] = dictOffAll[l] + b->groups[order[l]].d.nVals + 1;
	std::vector<LaneSlab> slabs;
	for(int nS = 1; nS <= nL; nS++) {
		const int per = (nL + nS - 1) / nS;
		if(per > LN_TAGS) continue;
		slabs.clear();
		bool fits = true;
		for(int l0 = 0; l0 < nL && fits; l0 += per) {
			const int n = std::min(per, nL - l0);
			LaneSlab s{l0, n, dictOffAll[l0], dictOffAll[l0 + n] - dictOffAll[l0], 64, 0, 0, 0, 0};
			fits = s.dictLen <= LN_DICT_MAX;
			slabs.push_back(s);
		}
		if(fits) break;
		slabs.clear();
	}
	if(slabs.empty() || slabs.size() > 65535) return 0;
	const int nS = (int) slabs.size();
	std::vector<LaneDesc> descs(nL);
	std::vector<uint32_t> descPk(nL);
	std::vector<int32_t> tblIndex(dictOffAll[nL], -1);
	int dictLds = 0;
	int64_t cntBytes = 0;
	for(int s = 0; s < nS; s++) {
		slabs[s].chunkOff = (int64_t) s * (nWin + 1);
		slabs[s].cntOff = cntBytes;
		cntBytes += (int64_t) nWin * slabs[s].n;
		dictLds = std::max(dictLds, slabs[s].dictLen);
		for(int l = slabs[s].l0; l < slabs[s].l0 + slabs[s].n; l++) {
			const DGroup& G = b->groups[order[l]].d;
			descs[l] = LaneDesc{order[l], dictOffAll[l] - slabs[s].dictOff, G.nVals, b->groups[order[l]].cols[0]};
			descPk[l] = (uint32_t) descs[l].dictOff | (uint32_t) G.nVals << 16;
			for(int k = 0; k < G.nVals; k++) tblIndex[dictOffAll[l] + k] = G.tblOff + k;
		}
	}
	hipStream_t st = b->stream;
	auto up16 = [](size_t n) { return (n + 15) / 16 * 16; };
	const size_t descBytes = sizeof(LaneDesc) * (size_t) nL, slabBytes = sizeof(LaneSlab) * (size_t) nS;
	const size_t dictBytes = sizeof(double) * (size_t) dictOffAll[nL], idxBytes = up16(sizeof(int32_t) * (size_t) dictOffAll[nL]);
	const size_t pkBytes = up16(sizeof(uint32_t) * (size_t) nL);
	const size_t csBytes = sizeof(uint32_t) * (size_t) nS * (nWin + 1);
	char* meta = nullptr;
	CLA_HIP(hipMalloc((void**) &meta, descBytes + slabBytes + dictBytes + idxBytes + pkBytes + csBytes));
	b->dLaneMeta = meta;
	LaneDesc* dDesc = (LaneDesc*) meta;
	LaneSlab* dSlabs = (LaneSlab*) (meta + descBytes);
	double* dDict = (double*) (meta + descBytes + slabBytes);
	int32_t* dIdx = (int32_t*) (meta + descBytes + slabBytes + dictBytes);
	uint32_t* dPk = (uint32_t*) (meta + descBytes + slabBytes + dictBytes + idxBytes);
	uint32_t* dCs = (uint32_t*) (meta + descBytes + slabBytes + dictBytes + idxBytes + pkBytes);
	CLA_HIP(hipMemcpyAsync(dDesc, descs.data(), descBytes, hipMemcpyHostToDevice, st));
	CLA_HIP(hipMemcpyAsync(dSlabs, slabs.data(), slabBytes, hipMemcpyHostToDevice, st));
	CLA_HIP(hipMemcpyAsync(dIdx, tblIndex.data(), sizeof(int32_t) * tblIndex.size(), hipMemcpyHostToDevice, st));
	CLA_HIP(hipMemcpyAsync(dPk, descPk.data(), sizeof(uint32_t) * (size_t) nL, hipMemcpyHostToDevice, st));
	CLA_HIP(hipMemsetAsync(dDict, 0, dictBytes, st));
	for(int l = 0; l < nL && singleCols; l++) {
		const DGroup& G = b->groups[order[l]].d;
		CLA_HIP(hipMemcpyAsync(dDict + dictOffAll[l], G.dict, sizeof(double) * (size_t) G.nVals, hipMemcpyDeviceToDevice, st));
	}
	// pass 1: chunks per (window, group) and per (slab, window); the width of a slab's chunk rows from its windows'
	// mean (64 lanes unless the windows hold too few chunks to fill two such rows); chunk rows per window and their
	// prefix sums on the host
	struct Tmp {
		void* p = nullptr;
		~Tmp() { if(p) (void) hipFree(p); }
	} tmpCnt, tmpTot;
	CLA_HIP(hipMalloc(&tmpCnt.p, (size_t) std::max<int64_t>(cntBytes, 1)));
	CLA_HIP(hipMalloc(&tmpTot.p, sizeof(uint32_t) * (size_t) nS * nWin));
	uint32_t* dTot = (uint32_t*) tmpTot.p;
	CLA_HIP(hipMemsetAsync(dTot, 0, sizeof(uint32_t) * (size_t) nS * nWin, st));
	const dim3 grid((unsigned) ((nWin + 3) / 4), (unsigned) nS);
	hipLaunchKernelGGL(k_lane_convert<false>, grid, dim3(256), 0, st, b->dGroups, dDesc, dSlabs, b->nRows, nWin, (uint8_t*) tmpCnt.p, dTot,
		nullptr, nullptr);
	CLA_HIP(hipGetLastError());
	std::vector<uint32_t> tot((size_t) nS * nWin), cs((size_t) nS * (nWin + 1));
	CLA_HIP(hipMemcpyAsync(tot.data(), dTot, sizeof(uint32_t) * tot.size(), hipMemcpyDeviceToHost, st));
	CLA_HIP(hipStreamSynchronize(st)); // (also: the host vectors above have been read)
	int64_t total16 = 0;
	for(int s = 0; s < nS; s++) {
		uint64_t chunks = 0;
		for(int w = 0; w < nWin; w++) chunks += tot[(size_t) s * nWin + w];
		int width = 64;
		while(width > 1 && chunks < (uint64_t) 2 * width * nWin) width /= 2;
		slabs[s].w = width;
		slabs[s].dataOff = total16;
		uint64_t c = 0;
		for(int w = 0; w < nWin; w++) {
			cs[(size_t) s * (nWin + 1) + w] = (uint32_t) c;
			c += std::max<uint32_t>(1, (tot[(size_t) s * nWin + w] + width - 1) / width);
		}
		if(c > 0xffffffffull) return 0;
		cs[(size_t) s * (nWin + 1) + nWin] = (uint32_t) c;
		total16 += (int64_t) c * width;
	}
	// (very short lists leave most of a window's only chunk row unused: not worth more than thrice the lists' own size)
	if((double) total16 * 16 > 3.0 * rawBytes + (double) (64 << 20)) return 0;
	size_t freeB = 0, totalB = 0;
	CLA_HIP(hipMemGetInfo(&freeB, &totalB));
	if((size_t) total16 * 16 + ((size_t) 1 << 30) > freeB) return 0;
	CLA_HIP(hipMalloc((void**) &b->dLaneData, (size_t) std::max<int64_t>(total16, 1) * 16));
	b->derivedBytes += (int64_t) (descBytes + slabBytes + dictBytes + idxBytes + pkBytes + csBytes) + total16 * 16;
	CLA_HIP(hipMemcpyAsync(dSlabs, slabs.data(), slabBytes, hipMemcpyHostToDevice, st));
	CLA_HIP(hipMemcpyAsync(dCs, cs.data(), csBytes, hipMemcpyHostToDevice, st));
	hipLaunchKernelGGL(k_lane_convert<true>, grid, dim3(256), 0, st, b->dGroups, dDesc, dSlabs, b->nRows, nWin, (uint8_t*) tmpCnt.p, nullptr,
		dCs, (u32x4*) b->dLaneData);
	CLA_HIP(hipGetLastError());
	CLA_HIP(hipStreamSynchronize(st)); // `slabs`, `cs` and the count arrays go out of scope
	b->laneSlabs = nS;
	b->laneDictLds = dictLds;
	b->laneDictTotal = dictOffAll[nL];
	b->laneOff[0] = descBytes; b->laneOff[1] = descBytes + slabBytes; b->laneOff[2] = descBytes + slabBytes + dictBytes;
	b->laneOff[3] = descBytes + slabBytes + dictBytes + idxBytes;
	b->laneOff[4] = descBytes + slabBytes + dictBytes + idxBytes + pkBytes;
	b->laneLmm = singleCols;
	b->laneState = 1;
	return 0;
}

// t(Y) %*% X of all listed groups straight into dOut. Returns 1 when the block's lists do not fit these kernels
// (codes beyond a byte, groups of several columns, dictionaries beyond LDS, lists too short), 0 when done.
int launch_lmm_sdc_lanes(cla_block* b, const double* dY, int p, double* dOut) {
	int rc = lanes_plan(b);
	if(rc) return rc;
	if(b->laneState != 1 || !b->laneLmm || p > 65535) return 1;
	// as many waves (each with a Y window of its own) as fit next to the slab's dictionaries
	const size_t ldsMax = (size_t) std::min(g_ldsPerBlock, 160 * 1024);
	const size_t fixed = sizeof(double) * ((size_t) b->laneDictLds + LN_TAGS) + sizeof(uint32_t) * LN_TAGS + 8;
	if(fixed + sizeof(double) * LN_YT > ldsMax) return 1;
	const int waves = (int) std::min<size_t>(LN_LW, (ldsMax - fixed) / (sizeof(double) * LN_YT));
	const size_t lds = fixed + sizeof(double) * (size_t) waves * LN_YT;
	const int nWin = (int) ((b->nRows + LN_WIN - 1) / LN_WIN), nS = b->laneSlabs;
	// about one block per CU (what its LDS allows): a share of the windows each, which its waves take one by one
	const int64_t parts = std::max<int64_t>(1, std::min<int64_t>((int64_t) g_numCU / ((int64_t) nS * p), (nWin + waves - 1) / waves));
	char* meta = (char*) b->dLaneMeta;
	double algo = (double) b->nRows * 8 * p;
	for(int g : b->sdcList) algo += (double) p * ((double) b->groups[g].d.nDeltas * b->groups[g].d.deltaWidth + (double) b->groups[g].d.nOffsets);
	// (the block's only groups are the listed ones: this kernel's sums are the whole result)
	const bool tail = b->lmmTailWanted && b->sdcList.size() == b->groups.size();
	Prof pf(b, "k_lmm_sdc_lanes", (long) parts * nS * p, waves * 64, (long) lds, algo);
	CLA_HIP(allow_full_lds((const void*) k_lmm_sdc_lanes));
	hipLaunchKernelGGL(k_lmm_sdc_lanes, dim3((unsigned) (parts * nS), p), dim3(waves * 64), lds, b->stream, (const LaneDesc*) meta,
		(const LaneSlab*) (meta + b->laneOff[0]), nS, (const double*) (meta + b->laneOff[1]), (const uint32_t*) (meta + b->laneOff[3]),
		b->laneDictLds, (const uint32_t*) (meta + b->laneOff[4]), (const u32x4*) b->dLaneData, dY, b->nRows, nWin, dOut, b->nCols,
		tail ? (unsigned*) (b->dCounters + 6) : nullptr, b->dCounters);
	b->lmmTailDone = tail;
	CLA_HIP(hipGetLastError());
	return 0;
}

// X %*% u of all listed groups (tables in b->dTables). Returns 1 when the lists do not fit, 0 when done.
int launch_rmm_sdc_lanes(cla_block* b, int constRow, int accumulate, double* dOut, unsigned long long* dNnz) {
	int rc = lanes_plan(b);
	if(rc) return rc;
	if(b->laneState != 1) return 1;
	// the tables of all slabs in LDS if they fit next to the output windows, else two buffers for the slab at work and the next
	const size_t ldsMax = (size_t) std::min(g_ldsPerBlock, 160 * 1024);
	const size_t otBytes = sizeof(double) * ((size_t) LN_G * LN_WIN + 64) + 2 * sizeof(uint32_t) * LN_TAGS;
	const bool resident = sizeof(double) * (size_t) b->laneDictTotal + otBytes <= ldsMax;
	const size_t lds = otBytes + sizeof(double) * (resident ? (size_t) b->laneDictTotal : 2 * (size_t) b->laneDictLds);
	if(lds > ldsMax) return 1;
	const int nWin = (int) ((b->nRows + LN_WIN - 1) / LN_WIN), nS = b->laneSlabs;
	// one block per CU; whole rounds of LN_G windows
	int wpb = (int) std::max<int64_t>(LN_G, ((int64_t) nWin + g_numCU - 1) / g_numCU);
	wpb = (wpb + LN_G - 1) / LN_G * LN_G;
	const unsigned grid = (unsigned) ((nWin + wpb - 1) / wpb);
	char* meta = (char*) b->dLaneMeta;
	double algo = (double) b->nRows * 8 * (accumulate ? 2 : 1);
	for(int g : b->sdcList) algo += (double) b->groups[g].d.nDeltas * b->groups[g].d.deltaWidth + (double) b->groups[g].d.nOffsets;
	Prof pf(b, "k_rmm_sdc_lanes", (long) grid, LN_RW * 64, (long) lds, algo);
	auto go = [&](auto kernel) {
		CLA_HIP(allow_full_lds((const void*) kernel));
		hipLaunchKernelGGL(kernel, dim3(grid), dim3(LN_RW * 64), lds, b->stream, (const LaneSlab*) (meta + b->laneOff[0]), nS,
			(const uint32_t*) (meta + b->laneOff[3]), (const int32_t*) (meta + b->laneOff[2]), b->laneDictLds, b->laneDictTotal,
			(const uint32_t*) (meta + b->laneOff[4]), (const u32x4*) b->dLaneData, (const double*) b->dTables, constRow, accumulate,
			dOut, b->nRows, nWin, wpb, dNnz);
		return 0;
	};
	if((rc = resident ? go(k_rmm_sdc_lanes<true>) : go(k_rmm_sdc_lanes<false>))) return rc;
	CLA_HIP(hipGetLastError());
	return 0;
}

} // namespace cla
