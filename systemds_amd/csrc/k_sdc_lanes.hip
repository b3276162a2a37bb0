// SDCZeros mat-vecs with one lane per group (gfx950).
//
//   k_lane_convert    one-time rewrite of the listed groups' offset and code lists into lane-major windows
//   k_lmm_sdc_lanes   out[col(g)] += sum over the listed rows of Y[row] * dict_g[code]   (t(v) %*% X)
//   k_rmm_sdc_lanes   out[row] += T_g[code] for every listed row                          (X %*% u)
//
// The groups are sorted by list length and cut into slabs of up to 64; lane l of a wave owns
// the slab's group l. Rows are cut into windows of LN_WIN. For a (slab, window) every lane's
// entries inside the window are stored in chunks of 16 bytes that hold seven entries - the row
// of the first (16 bits, relative to the window), six row deltas and seven codes, one byte
// each - and the chunks of the slab's lanes lie side by side: one 16-byte load per lane brings
// seven entries of every group of the slab, fully coalesced. A chunk row stands for itself
// (it carries its rows), so the right multiply's waves share the chunk rows of a block's
// windows among them; a lane decodes its entries with a running row - no prefix sums across
// lanes, no bins, no cross-lane traffic.
//
// Chunk of a lane: word 0 = first row | delta 1 << 16 | delta 2 << 24, word 1 = deltas 3..6, words 2 and 3 = codes
// 0..6 and, in the last byte, the window's index modulo LN_G (its place in a round of the right multiply). A gap of more than 255 rows inside a chunk takes entries of (255, spare) first, where the spare code nVals
// maps to a 0.0 behind the group's dictionary (or table); a chunk's unused entries are (0, spare), a lane's unused
// chunks start at row 0xffff. The chunk rows of a window are as many as its longest lane needs (sorting the groups
// by list length keeps that close to what the others need).
//
// Left multiply: every wave holds the Y window it works on in LDS, with a 0.0 behind it at index LN_WIN; every
// entry adds Y[min(row, LN_WIN)] * dict[code] to the lane's sum (spare entries add Y[row] * 0.0; a
// window of Y with non-finite values takes the variant that sends spare entries to the 0.0 instead). Right
// multiply: LN_G output windows sit in LDS, every entry with a tuple adds T[code] at its row with an LDS atomic; the slabs take turns, their tables in LDS in two buffers.
#include "../../include/cla_hip.h"
#include "cla_device.hpp"
#include <algorithm>
#include <numeric>
#include <vector>

namespace cla {

constexpr int LN_TPW = 1;                  // row tiles (SDC_TILE rows) per window
constexpr int LN_WIN = LN_TPW * SDC_TILE;  // rows per window
constexpr int LN_E = 7;                    // entries per chunk
constexpr int LN_DICT_MAX = 6016;          // dictionary entries (spares included) of a slab in LDS (right: two buffers next to the output windows)
constexpr int LN_YT = LN_WIN + 64;         // left: Y window + 64 slots of 0.0 behind it
constexpr int LN_LW = 8;                   // left: waves per block, each on windows of its own
constexpr int LN_LK = 12;                  // left: chunk rows of a window requested a window ahead
constexpr int LN_RW = 16;                  // right: waves per block
constexpr int LN_G = 4;                    // right: output windows per block and round
constexpr int LN_RK = 6;                   // right: chunk rows per wave and (slab, round) requested a turn ahead
constexpr int LN_TMAX = (LN_DICT_MAX + LN_RW * 64 - 1) / (LN_RW * 64); // right: table entries per thread
static_assert(LN_WIN <= 0x7fff, "a chunk's first row is 16 bits, 0xffff marks an unused chunk");

struct LaneDesc { // a lane's group, 16 bytes
	int32_t g;        // index of the group in the block
	int32_t dictOff;  // its dictionary inside the slab's (nVals entries and the 0.0 of the spare code)
	int32_t spare;    // = nVals
	int32_t col0;     // the column of a single-column group
};

struct LaneSlab { // 32 bytes
	int32_t l0, n;             // lanes desc[l0 .. l0 + n)
	int32_t dictOff, dictLen;  // their dictionaries inside the concatenation
	int64_t dataOff;           // first chunk of the slab, in 16-byte units
	int64_t chunkOff;          // the slab's nWin + 1 chunk-row starts inside chunkStart
};

// ---------------------------------------------------------------------------------------------
// Conversion. thread = (window, lane of the slab): walks the group's list inside the window from the row-tile
// index and counts its entries (FILL == false: maximum over the slab's lanes into slotMax) or writes its chunks
// (FILL == true).
// ---------------------------------------------------------------------------------------------
template <bool FILL>
__global__ __launch_bounds__(256) void k_lane_convert(const DGroup* __restrict__ groups, const LaneDesc* __restrict__ desc,
	const LaneSlab* __restrict__ slabs, int64_t nRows, int nWin, uint32_t* __restrict__ slotMax,
	const uint32_t* __restrict__ chunkStart, u32x4* __restrict__ data) {
	const LaneSlab S = slabs[blockIdx.y];
	const int lane = threadIdx.x & 63;
	const int win = blockIdx.x * 4 + (threadIdx.x >> 6);
	if(win >= nWin || lane >= S.n) return;
	const LaneDesc L = desc[S.l0 + lane];
	const DGroup G = dgroup(groups + L.g);
	const int64_t r0 = (int64_t) win * LN_WIN, rEnd = r0 + LN_WIN;
	const uint32_t spare = (uint32_t) L.spare;
	const uint32_t spare4 = spare * 0x01010101u;
	uint32_t cs = 0, nChunks = 0;
	if(FILL) {
		cs = chunkStart[S.chunkOff + win];
		nChunks = chunkStart[S.chunkOff + win + 1] - cs;
	}
	u32x4* dst = data + S.dataOff + (int64_t) cs * S.n + lane;
	int cnt = 0, prev = -1; // prev: row of the previous entry
	uint64_t dby = 0, cby = 0;
	auto flush = [&]() { // the chunk that holds entries cnt - (cnt % LN_E) .. (whole or partial)
		const int p = cnt % LN_E == 0 ? LN_E : cnt % LN_E;
		for(int t = p; t < LN_E; t++) cby |= (uint64_t) spare << (8 * t);
		cby |= (uint64_t) (win & (LN_G - 1)) << 56;
		u32x4 v = {(uint32_t) dby, (uint32_t) (dby >> 32), (uint32_t) cby, (uint32_t) (cby >> 32)};
		dst[(int64_t) ((cnt - 1) / LN_E) * S.n] = v;
		dby = 0; cby = 0;
	};
	auto put = [&](int row, uint32_t c) {
		if(FILL) {
			const int p = cnt % LN_E;
			if(p == 0) dby = (uint64_t) (uint32_t) row;
			else dby |= (uint64_t) (uint32_t) (row - prev) << (8 * (p + 1));
			cby |= (uint64_t) c << (8 * p);
		}
		prev = row;
		cnt++;
		if(FILL && cnt % LN_E == 0) flush();
	};
	auto entry = [&](int rel, int di) {
		while(cnt % LN_E != 0 && rel - prev > 255) put(prev + 255, spare);
		put(rel, (uint32_t) load_code(G.codes, G.codeWidth, di));
	};
	if(G.first >= r0 && G.first < rEnd) entry((int) (G.first - r0), 0);
	if(win * LN_TPW < G.nTiles) {
		const OffState st = G.tileIdx[win * LN_TPW];
		int64_t i = st.idx;
		int32_t row = st.row, emit = st.emit;
		const int maxV = G.deltaWidth == 1 ? 255 : 65535;
		for(; i < G.nDeltas; i++) {
			const int v = G.deltaWidth == 1 ? (int) ((const uint8_t*) G.deltas)[i] : (int) ((const uint16_t*) G.deltas)[i];
			const int64_t nr = (int64_t) row + (v == 0 ? maxV : v);
			if(nr >= rEnd) break;
			row = (int32_t) nr;
			if(v != 0) {
				if(nr >= r0) entry((int) (nr - r0), emit); // (the state in front of a window holds no row of it)
				emit++;
			}
		}
	}
	if(FILL) {
		if(cnt % LN_E != 0) flush();
		const u32x4 none = {0xffffu, 0u, spare4, (spare4 & 0x00ffffffu) | (uint32_t) (win & (LN_G - 1)) << 24};
		for(uint32_t k = (uint32_t) (cnt + LN_E - 1) / LN_E; k < nChunks; k++) dst[(int64_t) k * S.n] = none;
	}
	else atomicMax(&slotMax[(int64_t) blockIdx.y * nWin + win], (uint32_t) cnt);
}

// The seven rows (relative to the window; may lie behind it for unused chunks) and codes of a chunk.
__device__ __forceinline__ void ln_decode(const u32x4 v, uint32_t (&row)[LN_E], uint32_t (&code)[LN_E]) {
	row[0] = v.x & 0xffffu;
	row[1] = row[0] + ((v.x >> 16) & 0xffu);
	row[2] = row[1] + (v.x >> 24);
#pragma unroll
	for(int t = 3; t < LN_E; t++) row[t] = row[t - 1] + ((v.y >> (8 * (t - 3))) & 0xffu);
#pragma unroll
	for(int t = 0; t < LN_E; t++) code[t] = ((t < 4 ? v.z : v.w) >> (8 * (t & 3))) & 0xffu;
}

// ---------------------------------------------------------------------------------------------
// Left multiply. block = (run of windows, slab, row of Y); every wave works on windows of its own.
// ---------------------------------------------------------------------------------------------
template <bool CAREFUL>
__device__ __forceinline__ void ln_lmm_chunk(const u32x4 v, const double* yt, const double* dict, uint32_t spare,
	double (&acc)[4]) {
	uint32_t row[LN_E], code[LN_E];
	ln_decode(v, row, code);
	double yv[LN_E], dv[LN_E];
#pragma unroll
	for(int t = 0; t < LN_E; t++) {
		uint32_t idx = min(row[t], (uint32_t) LN_WIN);
		if(CAREFUL) idx = code[t] == spare ? (uint32_t) LN_WIN : idx;
		yv[t] = yt[idx];
		dv[t] = dict[code[t]];
	}
#pragma unroll
	for(int t = 0; t < LN_E; t++) acc[t & 3] = __builtin_fma(yv[t], dv[t], acc[t & 3]);
}

__global__ __launch_bounds__(LN_LW * 64) void k_lmm_sdc_lanes(const LaneDesc* __restrict__ desc,
	const LaneSlab* __restrict__ slabs, int nSlabs, const double* __restrict__ dictAll, int dictLds,
	const uint32_t* __restrict__ chunkStart, const u32x4* __restrict__ data, const double* __restrict__ Y, int64_t nRows,
	int nWin, int winPerWave, double* __restrict__ out, int nCols) {
	extern __shared__ double smem[];
	double* dictL = smem; // the slab's dictionaries
	const int tid = threadIdx.x, lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6); // (uniform: the chunk starts below come by scalar loads)
	double* yt = smem + dictLds + wave * LN_YT; // this wave's Y window
	// Blocks go round the 8 XCDs by their index. The slabs of a run of windows read the same part of Y: they sit 8
	// block indices apart, on one XCD and close in time, so that its L2 fetches that part of Y once.
	const int nRuns = gridDim.x / nSlabs;
	const int period = 8 * nSlabs, grp = blockIdx.x / period, in = blockIdx.x % period;
	const int inLast = nRuns - grp * 8 < 8 ? nRuns - grp * 8 : 8; // runs of the last, partial period
	const int slab = in / inLast, run = grp * 8 + in % inLast;
	const LaneSlab S = slabs[slab];
	for(int k = tid; k < S.dictLen; k += LN_LW * 64) dictL[k] = dictAll[S.dictOff + k];
	yt[LN_WIN + lane] = 0.0;
	__syncthreads();
	const int ln = min(lane, S.n - 1); // lanes behind the slab's last repeat it, their sums are dropped
	const LaneDesc L = desc[S.l0 + ln];
	const double* dict = dictL + L.dictOff;
	const uint32_t spare = (uint32_t) L.spare;
	const double* y = Y + (size_t) blockIdx.y * nRows;
	const uint32_t* cst = chunkStart + S.chunkOff;
	const u32x4* base = data + S.dataOff + ln;
	const int n = S.n;
	double acc[4] = {0.0, 0.0, 0.0, 0.0};
	// this wave's windows: w0, w0 + LN_LW, ... below w1 (the block's waves read one stretch of the lists together)
	const int w1 = min((run + 1) * LN_LW * winPerWave, nWin), w0 = min(run * LN_LW * winPerWave + wave, w1);
	// Requested a window ahead: the window's first LN_LK chunk rows, the lane's share of the Y window, the chunk
	// range. Two sets take turns. The window's work is straight-line code on the set (no loads inside: the compiler's
	// wait counts are exact); chunk rows behind the first LN_LK (dense lists) come in a plain loop at the end.
	struct Ahead {
		u32x4 buf[LN_LK];
		double y[LN_WIN / 64];
		uint32_t c0, c1;
	};
	auto request = [&](Ahead& A, int win) { // win < w1
		A.c0 = cst[win];
		A.c1 = cst[win + 1];
#pragma unroll
		for(int j = 0; j < LN_LK; j++) A.buf[j] = *(base + (int64_t) min(A.c0 + j, A.c1 - 1) * n); // (every window holds a chunk row)
		const int64_t r0 = (int64_t) win * LN_WIN;
#pragma unroll
		for(int k = 0; k < LN_WIN / 64; k++) A.y[k] = y[min(r0 + k * 64 + lane, nRows - 1)]; // unconditional: a load under a branch is waited for at the branch's end
	};
	auto work = [&](Ahead& A, Ahead& B, int win) { // A holds the requests of `win`, B takes those of the wave's next window
		const int64_t r0 = (int64_t) win * LN_WIN;
		bool bad = false;
#pragma unroll
		for(int k = 0; k < LN_WIN / 64; k++) {
			const double v = r0 + k * 64 + lane < nRows ? A.y[k] : 0.0;
			bad |= !isfinite(v);
			yt[k * 64 + lane] = v;
		}
		const bool careful = __builtin_amdgcn_ballot_w64(bad) != 0;
		__builtin_amdgcn_wave_barrier(); // LDS serves a wave's accesses in order: the reads below see the window
		const uint32_t c0 = A.c0, c1 = A.c1;
		u32x4 cur[LN_LK];
#pragma unroll
		for(int j = 0; j < LN_LK; j++) cur[j] = A.buf[j];
		request(B, win + LN_LW < w1 ? win + LN_LW : win);
#pragma unroll
		for(int j = 0; j < LN_LK; j++) {
			if(c0 + j < c1) {
				if(careful) ln_lmm_chunk<true>(cur[j], yt, dict, spare, acc);
				else ln_lmm_chunk<false>(cur[j], yt, dict, spare, acc);
			}
		}
		for(uint32_t c = c0 + LN_LK; c < c1; c++) {
			const u32x4 v = *(base + (int64_t) c * n);
			if(careful) ln_lmm_chunk<true>(v, yt, dict, spare, acc);
			else ln_lmm_chunk<false>(v, yt, dict, spare, acc);
		}
	};
	if(w0 < w1) {
		Ahead A, B;
		request(A, w0);
		for(int win = w0; win < w1; win += 2 * LN_LW) {
			work(A, B, win);
			if(win + LN_LW < w1) work(B, A, win + LN_LW);
		}
	}
	if(lane < n) unsafeAtomicAdd(&out[(size_t) blockIdx.y * nCols + L.col0], (acc[0] + acc[1]) + (acc[2] + acc[3]));
}

// ---------------------------------------------------------------------------------------------
// Right multiply with one output column. block = run of windows, in rounds of LN_G windows whose output sits in
// LDS. In a round the slabs take turns; the block's waves share the chunk rows of the slab's LN_G windows. The
// tables of the next turn's slab (T gathered through tblIndex, -1 = the 0.0 of a spare code) are fetched during a
// turn and stored into the other table buffer behind it. accumulate == 0: a window starts from constRow (or zero)
// and is the whole result; accumulate != 0: it starts from what other groups already wrote.
// ---------------------------------------------------------------------------------------------
template <bool RESIDENT>
__global__ __launch_bounds__(LN_RW * 64) void k_rmm_sdc_lanes(const LaneDesc* __restrict__ desc,
	const LaneSlab* __restrict__ slabs, int nSlabs, const int32_t* __restrict__ tblIndex, int dictLds, int dictTotal,
	const uint32_t* __restrict__ chunkStart, const u32x4* __restrict__ data, const double* __restrict__ T, int constRow,
	int accumulate, double* __restrict__ out, int64_t nRows, int nWin, int winPerBlock, unsigned long long* __restrict__ nnz) {
	extern __shared__ double smem[];
	double* tblAll = smem;                 // RESIDENT: the tables of all slabs (dictTotal entries); else two buffers of dictLds entries
	double* ot = smem + (RESIDENT ? dictTotal : 2 * dictLds); // LN_G windows of output
	const int tid = threadIdx.x, lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	constexpr int THREADS = LN_RW * 64, OPT = LN_G * LN_WIN / THREADS;
	const int wBeg = min((int) blockIdx.x * winPerBlock, nWin), wEnd = min(wBeg + winPerBlock, nWin);
	if(wBeg >= wEnd) return;
	const double init = !accumulate && constRow >= 0 ? T[constRow] : 0.0;
	const int nRounds = (wEnd - wBeg + LN_G - 1) / LN_G, nTurns = nRounds * nSlabs;
	double treg[LN_TMAX];
	auto tbl_request = [&](int s) {
		const LaneSlab S = slabs[s];
#pragma unroll
		for(int k = 0; k < LN_TMAX; k++) {
			const int e = k * THREADS + tid;
			const int32_t ti = tblIndex[S.dictOff + min(e, S.dictLen - 1)];
			treg[k] = T[max(ti, 0)];
			treg[k] = ti >= 0 ? treg[k] : 0.0;
		}
	};
	auto tbl_store = [&](int turn) {
		double* tb = tblAll + (nSlabs > 1 ? turn & 1 : 0) * dictLds; // (one slab: its tables stay)
#pragma unroll
		for(int k = 0; k < LN_TMAX; k++)
			if(k * THREADS + tid < dictLds) tb[k * THREADS + tid] = treg[k];
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
		const u32x4* base = data + S.dataOff + min(lane, S.n - 1);
#pragma unroll
		for(int j = 0; j < LN_RK; j++) A.buf[j] = *(base + (int64_t) min(A.c0 + j * LN_RW, A.c1 - 1) * S.n);
	};
	auto add_chunk = [&](const u32x4 v, const double* tbl, uint32_t spare) {
		const uint32_t off = (v.w >> 24) * (uint32_t) LN_WIN; // the chunk row's window inside the round (rounds start at multiples of LN_G)
		uint32_t row[LN_E], code[LN_E];
		ln_decode(v, row, code);
		double tv[LN_E];
#pragma unroll
		for(int t = 0; t < LN_E; t++) tv[t] = tbl[code[t]];
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
		if(!RESIDENT && nSlabs > 1) tbl_request(next % nSlabs);
		request(B, next);
		const LaneSlab S = slabs[s];
		const LaneDesc L = desc[S.l0 + min(lane, S.n - 1)];
		const double* tbl = tblAll + (RESIDENT ? S.dictOff : (nSlabs > 1 ? turn & 1 : 0) * dictLds) + L.dictOff;
		const uint32_t spare = (uint32_t) L.spare;
		const u32x4* base = data + S.dataOff + min(lane, S.n - 1);
		const uint32_t c0 = A.c0, c1 = A.c1;
		if(lane < S.n) {
#pragma unroll
			for(int j = 0; j < LN_RK; j++)
				if(c0 + j * LN_RW < c1) add_chunk(A.buf[j], tbl, spare);
			for(uint32_t c = c0 + LN_RK * LN_RW; c < c1; c += LN_RW) add_chunk(*(base + (int64_t) c * S.n), tbl, spare);
		}
		if(!RESIDENT && nSlabs > 1) tbl_store(turn + 1); // the other buffer was last read before the previous barrier
		if(!RESIDENT || s == nSlabs - 1) __syncthreads(); // (resident tables: the waves only meet at the ends of a round)
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
	else {
		tbl_request(0);
		tbl_store(0);
	}
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
	// lanes in the order of list length, slabs of equal lane counts within the 64 lanes and the LDS budget
	std::vector<int32_t> order(list.begin(), list.end());
	std::stable_sort(order.begin(), order.end(), [&](int32_t x, int32_t y) { return b->groups[x].d.nOffsets > b->groups[y].d.nOffsets; });
	std::vector<int32_t> dictOffAll(nL + 1, 0);
	for(int l = 0; l < nL; l++) dictOffAll[l + 1] = dictOffAll[l] + b->groups[order[l]].d.nVals + 1;
	std::vector<LaneSlab> slabs;
	for(int nS = (nL + 63) / 64; nS <= nL; nS++) {
		const int per = (nL + nS - 1) / nS;
		slabs.clear();
		bool fits = true;
		for(int l0 = 0; l0 < nL && fits; l0 += per) {
			const int n = std::min(per, nL - l0);
			LaneSlab s{l0, n, dictOffAll[l0], dictOffAll[l0 + n] - dictOffAll[l0], 0, 0};
			fits = s.dictLen <= LN_DICT_MAX;
			slabs.push_back(s);
		}
		if(fits) break;
		slabs.clear();
	}
	if(slabs.empty() || slabs.size() > 65535) return 0;
	const int nS = (int) slabs.size();
	std::vector<LaneDesc> descs(nL);
	std::vector<int32_t> tblIndex(dictOffAll[nL], -1);
	int dictLds = 0;
	for(int s = 0; s < nS; s++) {
		slabs[s].chunkOff = (int64_t) s * (nWin + 1);
		dictLds = std::max(dictLds, slabs[s].dictLen);
		for(int l = slabs[s].l0; l < slabs[s].l0 + slabs[s].n; l++) {
			const DGroup& G = b->groups[order[l]].d;
			descs[l] = LaneDesc{order[l], dictOffAll[l] - slabs[s].dictOff, G.nVals, b->groups[order[l]].cols[0]};
			for(int k = 0; k < G.nVals; k++) tblIndex[dictOffAll[l] + k] = G.tblOff + k;
		}
	}
	hipStream_t st = b->stream;
	const size_t descBytes = sizeof(LaneDesc) * (size_t) nL, slabBytes = sizeof(LaneSlab) * (size_t) nS;
	const size_t dictBytes = sizeof(double) * (size_t) dictOffAll[nL], idxBytes = (sizeof(int32_t) * (size_t) dictOffAll[nL] + 15) / 16 * 16;
	const size_t csBytes = sizeof(uint32_t) * (size_t) nS * (nWin + 1);
	char* meta = nullptr;
	CLA_HIP(hipMalloc((void**) &meta, descBytes + slabBytes + dictBytes + idxBytes + csBytes));
	b->dLaneMeta = meta;
	LaneDesc* dDesc = (LaneDesc*) meta;
	LaneSlab* dSlabs = (LaneSlab*) (meta + descBytes);
	double* dDict = (double*) (meta + descBytes + slabBytes);
	int32_t* dIdx = (int32_t*) (meta + descBytes + slabBytes + dictBytes);
	uint32_t* dCs = (uint32_t*) (meta + descBytes + slabBytes + dictBytes + idxBytes);
	CLA_HIP(hipMemcpyAsync(dDesc, descs.data(), descBytes, hipMemcpyHostToDevice, st));
	CLA_HIP(hipMemcpyAsync(dSlabs, slabs.data(), slabBytes, hipMemcpyHostToDevice, st));
	CLA_HIP(hipMemcpyAsync(dIdx, tblIndex.data(), sizeof(int32_t) * tblIndex.size(), hipMemcpyHostToDevice, st));
	CLA_HIP(hipMemsetAsync(dDict, 0, dictBytes, st));
	for(int l = 0; l < nL && singleCols; l++) {
		const DGroup& G = b->groups[order[l]].d;
		CLA_HIP(hipMemcpyAsync(dDict + dictOffAll[l], G.dict, sizeof(double) * (size_t) G.nVals, hipMemcpyDeviceToDevice, st));
	}
	// pass 1: slots per (slab, window) = the maximum over the slab's lanes; chunk starts by a prefix sum on the host
	CLA_HIP(hipMemsetAsync(dCs, 0, csBytes, st));
	const dim3 grid((unsigned) ((nWin + 3) / 4), (unsigned) nS);
	hipLaunchKernelGGL(k_lane_convert<false>, grid, dim3(256), 0, st, b->dGroups, dDesc, dSlabs, b->nRows, nWin, dCs, nullptr, nullptr);
	CLA_HIP(hipGetLastError());
	std::vector<uint32_t> slotMax((size_t) nS * nWin), cs((size_t) nS * (nWin + 1));
	CLA_HIP(hipMemcpyAsync(slotMax.data(), dCs, sizeof(uint32_t) * slotMax.size(), hipMemcpyDeviceToHost, st));
	CLA_HIP(hipStreamSynchronize(st)); // (also: the host vectors above have been read)
	int64_t total16 = 0;
	for(int s = 0; s < nS; s++) {
		slabs[s].dataOff = total16;
		uint64_t c = 0;
		for(int w = 0; w < nWin; w++) {
			cs[(size_t) s * (nWin + 1) + w] = (uint32_t) c;
			c += std::max<uint32_t>(1, (slotMax[(size_t) s * nWin + w] + LN_E - 1) / LN_E); // at least one chunk row: the kernels' loads are unconditional
		}
		if(c > 0xffffffffull) return 0;
		cs[(size_t) s * (nWin + 1) + nWin] = (uint32_t) c;
		total16 += (int64_t) c * slabs[s].n;
	}
	// lists of very different lengths inside a slab pad each other: not worth more than thrice the lists' own size
	if((double) total16 * 16 > 3.0 * rawBytes + (double) (64 << 20)) return 0;
	size_t freeB = 0, totalB = 0;
	CLA_HIP(hipMemGetInfo(&freeB, &totalB));
	if((size_t) total16 * 16 + ((size_t) 1 << 30) > freeB) return 0;
	CLA_HIP(hipMalloc((void**) &b->dLaneData, (size_t) std::max<int64_t>(total16, 1) * 16));
	b->derivedBytes += (int64_t) (descBytes + slabBytes + dictBytes + idxBytes + csBytes) + total16 * 16;
	CLA_HIP(hipMemcpyAsync(dSlabs, slabs.data(), slabBytes, hipMemcpyHostToDevice, st));
	CLA_HIP(hipMemcpyAsync(dCs, cs.data(), csBytes, hipMemcpyHostToDevice, st));
	hipLaunchKernelGGL(k_lane_convert<true>, grid, dim3(256), 0, st, b->dGroups, dDesc, dSlabs, b->nRows, nWin, nullptr, dCs,
		(u32x4*) b->dLaneData);
	CLA_HIP(hipGetLastError());
	CLA_HIP(hipStreamSynchronize(st)); // `slabs` and `cs` go out of scope
	b->laneSlabs = nS;
	b->laneDictLds = dictLds;
	b->laneDictTotal = dictOffAll[nL];
	b->laneOff[0] = descBytes; b->laneOff[1] = descBytes + slabBytes; b->laneOff[2] = descBytes + slabBytes + dictBytes;
	b->laneOff[3] = descBytes + slabBytes + dictBytes + idxBytes;
	b->laneLmm = singleCols;
	b->laneState = 1;
	return 0;
}

// t(Y) %*% X of all listed groups straight into dOut. Returns 1 when the block's lists do not fit these kernels
// (codes beyond a byte, groups of several columns, dictionaries beyond LDS, lists too uneven), 0 when done.
int launch_lmm_sdc_lanes(cla_block* b, const double* dY, int p, double* dOut) {
	int rc = lanes_plan(b);
	if(rc) return rc;
	if(b->laneState != 1 || !b->laneLmm || p > 65535) return 1;
	const size_t lds = sizeof(double) * ((size_t) b->laneDictLds + LN_LW * LN_YT);
	if(lds > (size_t) std::min(g_ldsPerBlock, 160 * 1024)) return 1;
	const int nWin = (int) ((b->nRows + LN_WIN - 1) / LN_WIN), nS = b->laneSlabs;
	// about one block per CU (what its registers and LDS allow), every wave a share of the block's run of windows
	const int64_t runs = std::max<int64_t>(1, (int64_t) g_numCU / ((int64_t) nS * p));
	const int wpw = (int) std::max<int64_t>(1, (nWin + runs * LN_LW - 1) / (runs * LN_LW));
	const unsigned nRuns = (unsigned) ((nWin + wpw * LN_LW - 1) / (wpw * LN_LW));
	char* meta = (char*) b->dLaneMeta;
	double algo = (double) b->nRows * 8 * p;
	for(int g : b->sdcList) algo += (double) p * ((double) b->groups[g].d.nDeltas * b->groups[g].d.deltaWidth + (double) b->groups[g].d.nOffsets);
	Prof pf(b, "k_lmm_sdc_lanes", (long) nRuns * nS * p, LN_LW * 64, (long) lds, algo);
	CLA_HIP(allow_full_lds((const void*) k_lmm_sdc_lanes));
	hipLaunchKernelGGL(k_lmm_sdc_lanes, dim3(nRuns * nS, p), dim3(LN_LW * 64), lds, b->stream, (const LaneDesc*) meta,
		(const LaneSlab*) (meta + b->laneOff[0]), nS, (const double*) (meta + b->laneOff[1]), b->laneDictLds,
		(const uint32_t*) (meta + b->laneOff[3]), (const u32x4*) b->dLaneData, dY, b->nRows, nWin, wpw, dOut, b->nCols);
	CLA_HIP(hipGetLastError());
	return 0;
}

// X %*% u of all listed groups (tables in b->dTables). Returns 1 when the lists do not fit, 0 when done.
int launch_rmm_sdc_lanes(cla_block* b, int constRow, int accumulate, double* dOut, unsigned long long* dNnz) {
	int rc = lanes_plan(b);
	if(rc) return rc;
	if(b->laneState != 1) return 1;
	// the tables of all slabs in LDS if they fit next to the output windows, else two buffers for the slab at work and the next
	const size_t ldsMax = (size_t) std::min(g_ldsPerBlock, 160 * 1024), otBytes = sizeof(double) * ((size_t) LN_G * LN_WIN + 64);
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
		hipLaunchKernelGGL(kernel, dim3(grid), dim3(LN_RW * 64), lds, b->stream, (const LaneDesc*) meta,
			(const LaneSlab*) (meta + b->laneOff[0]), nS, (const int32_t*) (meta + b->laneOff[2]), b->laneDictLds, b->laneDictTotal,
			(const uint32_t*) (meta + b->laneOff[3]), (const u32x4*) b->dLaneData, (const double*) b->dTables, constRow, accumulate,
			dOut, b->nRows, nWin, wpb, dNnz);
		return 0;
	};
	if((rc = resident ? go(k_rmm_sdc_lanes<true>) : go(k_rmm_sdc_lanes<false>))) return rc;
	CLA_HIP(hipGetLastError());
	return 0;
}

} // namespace cla
