// SDCZeros mat-vecs with one lane per group (gfx950).
//
//   k_lane_convert    one-time rewrite of the listed groups' offset and code lists into lane-major windows
//   k_lmm_sdc_lanes   out[col(g)] += sum over the listed rows of Y[row] * dict_g[code]   (t(v) %*% X)
//   k_rmm_sdc_lanes   out[row] += T_g[code] for every listed row                          (X %*% u)
//
// The groups are sorted by list length and cut into slabs of up to 64; a wave owns a slab, lane l
// owns the slab's group l. Rows are cut into windows of LN_WIN. For a (slab, window) every lane's
// entries inside the window are stored as slots of (row delta, code), one byte each, eight slots
// per 16-byte chunk, the chunks of the slab's lanes side by side: one 16-byte load per lane brings
// eight entries of every group of the slab, fully coalesced, and a lane decodes its list with a
// running row - no prefix sums across lanes, no bins, no cross-lane traffic.
//
// Slot encoding: delta 1..255 = rows since the previous slot (since row -1 of the window for the first), code =
// tuple index; a gap of more than 255 rows takes slots of (255, spare) first, where the spare code nVals maps to a
// 0.0 behind the group's dictionary (or table); lanes with fewer slots than the longest of the slab are padded
// with (0, spare). The windows' chunk counts are the maxima over the slab's lanes (sorting by list length keeps
// them close to the lanes' own counts).
//
// Left multiply: the Y window sits in LDS with a 0.0 at index LN_WIN, every slot adds
// Y[min(row, LN_WIN)] * dict[code] to the lane's sum (spare slots add Y[row] * 0.0; a window of Y with non-finite
// values takes the variant that sends spare slots to the 0.0 instead). Right multiply: the output window sits in
// LDS, every slot adds T[code] at its row with an LDS atomic (spare slots add their 0.0 to a dump slot per lane); the slabs take turns on the block's windows, their tables staged in LDS one after the other.
#include "../../include/cla_hip.h"
#include "cla_device.hpp"
#include <algorithm>
#include <numeric>
#include <vector>

namespace cla {

constexpr int LN_WIN = SDC_TILE;        // rows per window
constexpr int LN_DICT_MAX = 6144;       // dictionary entries (spares included) of a slab in LDS
constexpr int LN_YT = LN_WIN + 64;      // window + 64 slots behind it (left: 0.0; right: one dump slot per lane)
constexpr int LN_PF = 4;                // right multiply: chunks a lane keeps requested ahead
constexpr int LN_NC = 12;               // left multiply: chunks of a window requested a window ahead

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
	int64_t chunkOff;          // the slab's nWin + 1 chunk starts inside chunkStart
};

// ---------------------------------------------------------------------------------------------
// Conversion. thread = (window, lane of the slab): walks the group's list inside the window from the row-tile
// index and counts (FILL == false: maximum over the slab's lanes into slotMax) or writes (FILL == true) its slots.
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
	uint32_t cs = 0, nChunks = 0;
	if(FILL) {
		cs = chunkStart[S.chunkOff + win];
		nChunks = chunkStart[S.chunkOff + win + 1] - cs;
	}
	u32x4* dst = data + S.dataOff + (int64_t) cs * S.n + lane;
	int cnt = 0, prev = -1;
	uint64_t dby = 0, cby = 0;
	auto slot = [&](uint32_t d, uint32_t c) {
		if(FILL) {
			dby |= (uint64_t) d << (8 * (cnt & 7));
			cby |= (uint64_t) c << (8 * (cnt & 7));
			if((cnt & 7) == 7) {
				u32x4 v = {(uint32_t) dby, (uint32_t) (dby >> 32), (uint32_t) cby, (uint32_t) (cby >> 32)};
				dst[(int64_t) (cnt >> 3) * S.n] = v;
				dby = 0; cby = 0;
			}
		}
		cnt++;
	};
	auto entry = [&](int rel, int di) {
		int gap = rel - prev;
		while(gap > 255) { slot(255u, spare); gap -= 255; }
		slot((uint32_t) gap, (uint32_t) load_code(G.codes, G.codeWidth, di));
		prev = rel;
	};
	if(G.first >= r0 && G.first < rEnd) entry((int) (G.first - r0), 0);
	if(win < G.nTiles) {
		const OffState st = G.tileIdx[win];
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
		while(cnt < (int) nChunks * 8) slot(0u, spare);
	}
	else atomicMax(&slotMax[(int64_t) blockIdx.y * nWin + win], (uint32_t) cnt);
}

// ---------------------------------------------------------------------------------------------
// Left multiply.
// ---------------------------------------------------------------------------------------------
// Eight slots of one lane. r = row of the previous slot, relative to the window.
template <bool CAREFUL>
__device__ __forceinline__ void ln_lmm_chunk(const u32x4 v, int& r, const double* yt, const double* dict, uint32_t spare,
	double (&acc)[4]) {
	uint32_t idx[8], code[8];
#pragma unroll
	for(int t = 0; t < 8; t++) {
		const uint32_t dw = t < 4 ? v.x : v.y, cw = t < 4 ? v.z : v.w;
		r += (int) ((dw >> (8 * (t & 3))) & 0xffu);
		code[t] = (cw >> (8 * (t & 3))) & 0xffu;
		idx[t] = min((uint32_t) r, (uint32_t) LN_WIN);
		if(CAREFUL) idx[t] = code[t] == spare ? (uint32_t) LN_WIN : idx[t];
	}
	double yv[8], dv[8];
#pragma unroll
	for(int t = 0; t < 8; t++) {
		yv[t] = yt[idx[t]];
		dv[t] = dict[code[t]];
	}
#pragma unroll
	for(int t = 0; t < 8; t++) acc[t & 3] = __builtin_fma(yv[t], dv[t], acc[t & 3]);
}

template <int WAVES>
__global__ __launch_bounds__(WAVES * 64) void k_lmm_sdc_lanes(const LaneDesc* __restrict__ desc,
	const LaneSlab* __restrict__ slabs, int nSlabs, const double* __restrict__ dictAll, int dictLds,
	const uint32_t* __restrict__ chunkStart, const u32x4* __restrict__ data, const double* __restrict__ Y, int64_t nRows,
	int nWin, int winPerWave, double* __restrict__ out, int nCols) {
	extern __shared__ double smem[];
	double* dictL = smem; // the slab's dictionaries
	const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
	double* yt = smem + dictLds + wave * LN_YT;
	// Blocks go round the 8 XCDs by their index. The slabs of a run of windows read the same part of Y: they sit 8
	// block indices apart, on one XCD and close in time, so that its L2 fetches that part of Y once.
	const int nRuns = gridDim.x / nSlabs;
	const int period = 8 * nSlabs, grp = blockIdx.x / period, in = blockIdx.x % period;
	const int inLast = nRuns - grp * 8 < 8 ? nRuns - grp * 8 : 8; // runs of the last, partial period
	const int slab = in / inLast, run = grp * 8 + in % inLast;
	const LaneSlab S = slabs[slab];
	for(int k = tid; k < S.dictLen; k += WAVES * 64) dictL[k] = dictAll[S.dictOff + k];
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
	const int waveU = __builtin_amdgcn_readfirstlane(wave); // (uniform: the chunk starts below come by scalar loads)
	// this wave's windows: w0, w0 + WAVES, ... below w1 (the block's waves read one stretch of the lists together)
	const int w1 = min((run + 1) * WAVES * winPerWave, nWin), w0 = min(run * WAVES * winPerWave + waveU, w1);
	// Requested a window ahead: the window's first LN_NC chunks, the lane's share of the Y window, the chunk range.
	// Two sets take turns. The window's work is straight-line code on the set (no loads inside: the compiler's
	// wait counts are exact); chunks behind the first LN_NC (dense lists) come in a plain loop at the end.
	struct Ahead {
		u32x4 buf[LN_NC];
		double y[LN_WIN / 64];
		uint32_t c0, c1;
	};
	auto request = [&](Ahead& A, int win) { // win < w1
		A.c0 = cst[win];
		A.c1 = cst[win + 1];
#pragma unroll
		for(int j = 0; j < LN_NC; j++) A.buf[j] = *(base + (int64_t) min(A.c0 + j, A.c1 - 1) * n); // (every window holds a chunk)
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
		u32x4 cur[LN_NC];
#pragma unroll
		for(int j = 0; j < LN_NC; j++) cur[j] = A.buf[j];
		request(B, win + WAVES < w1 ? win + WAVES : win);
		int r = -1;
#pragma unroll
		for(int j = 0; j < LN_NC; j++) {
			if(c0 + j < c1) {
				if(careful) ln_lmm_chunk<true>(cur[j], r, yt, dict, spare, acc);
				else ln_lmm_chunk<false>(cur[j], r, yt, dict, spare, acc);
			}
		}
		for(uint32_t c = c0 + LN_NC; c < c1; c++) {
			const u32x4 v = *(base + (int64_t) c * n);
			if(careful) ln_lmm_chunk<true>(v, r, yt, dict, spare, acc);
			else ln_lmm_chunk<false>(v, r, yt, dict, spare, acc);
		}
	};
	if(w0 < w1) {
		Ahead A, B;
		request(A, w0);
		for(int win = w0; win < w1; win += 2 * WAVES) {
			work(A, B, win);
			if(win + WAVES < w1) work(B, A, win + WAVES);
		}
	}
	if(lane < n) unsafeAtomicAdd(&out[(size_t) blockIdx.y * nCols + L.col0], (acc[0] + acc[1]) + (acc[2] + acc[3]));
}

// ---------------------------------------------------------------------------------------------
// Right multiply with one output column. block = run of windows; per round every wave takes one window, and the
// slabs take turns: tables of slab s into LDS (T gathered through tblIndex, -1 = the 0.0 of a spare code), every
// wave adds the slab's slots of its window. accumulate == 0: a window starts from constRow (or zero) and is the
// whole result; accumulate != 0: it starts from what other groups already wrote.
// ---------------------------------------------------------------------------------------------
template <int WAVES>
__global__ __launch_bounds__(WAVES * 64) void k_rmm_sdc_lanes(const LaneDesc* __restrict__ desc,
	const LaneSlab* __restrict__ slabs, int nSlabs, const int32_t* __restrict__ tblIndex, int dictLds,
	const uint32_t* __restrict__ chunkStart, const u32x4* __restrict__ data, const double* __restrict__ T, int constRow,
	int accumulate, double* __restrict__ out, int64_t nRows, int nWin, int winPerBlock, unsigned long long* __restrict__ nnz) {
	extern __shared__ double smem[];
	double* tblL = smem;
	const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
	double* ot = smem + dictLds + wave * LN_YT;
	const int wBeg = blockIdx.x * winPerBlock, wEnd = min(wBeg + winPerBlock, nWin);
	const double init = !accumulate && constRow >= 0 ? T[constRow] : 0.0;
	int cntNz = 0;
	for(int wb = wBeg; wb < wEnd; wb += WAVES) { // the same trip count for every wave: barriers inside
		const int win = wb + wave;
		const bool on = win < wEnd;
		const int64_t r0 = (int64_t) win * LN_WIN;
		if(on && accumulate) {
#pragma unroll
			for(int k = 0; k < LN_WIN / 64; k++) ot[k * 64 + lane] = out[min(r0 + k * 64 + lane, nRows - 1)]; // (unconditional loads)
		}
		else if(on) {
#pragma unroll
			for(int k = 0; k < LN_WIN / 64; k++) ot[k * 64 + lane] = init;
		}
		for(int s = 0; s < nSlabs; s++) {
			const LaneSlab S = slabs[s];
			__syncthreads(); // the previous slab's tables are no longer read
			for(int k = tid; k < S.dictLen; k += WAVES * 64) {
				const int32_t ti = tblIndex[S.dictOff + k];
				tblL[k] = ti >= 0 ? T[ti] : 0.0;
			}
			__syncthreads();
			if(!on) continue;
			const int ln = min(lane, S.n - 1);
			const LaneDesc L = desc[S.l0 + ln];
			const double* tbl = tblL + L.dictOff;
			const uint32_t spare = (uint32_t) L.spare;
			const uint32_t* cst = chunkStart + S.chunkOff;
			const u32x4* base = data + S.dataOff + ln;
			const int n = S.n;
			const uint32_t c0 = __builtin_amdgcn_readfirstlane(cst[win]), c1 = __builtin_amdgcn_readfirstlane(cst[win + 1]);
			u32x4 buf[LN_PF];
#pragma unroll
			for(int j = 0; j < LN_PF; j++) buf[j] = __builtin_nontemporal_load(base + (int64_t) min(c0 + j, c1 - 1) * n);
			int r = -1;
			const uint32_t dump = (uint32_t) (LN_WIN + lane);
			for(uint32_t c = c0; c < c1; c += LN_PF) {
#pragma unroll
				for(int j = 0; j < LN_PF; j++) {
					const u32x4 v = buf[j];
					buf[j] = __builtin_nontemporal_load(base + (int64_t) min(c + j + LN_PF, c1 - 1) * n);
					if(c + j < c1 && lane < n) {
						double tv[8];
						uint32_t idx[8];
#pragma unroll
						for(int t = 0; t < 8; t++) {
							const uint32_t dw = t < 4 ? v.x : v.y, cw = t < 4 ? v.z : v.w;
							r += (int) ((dw >> (8 * (t & 3))) & 0xffu);
							const uint32_t code = (cw >> (8 * (t & 3))) & 0xffu;
							idx[t] = code != spare ? (uint32_t) r : dump; // (a slot with a tuple lies inside the window)
							tv[t] = tbl[code];
						}
#pragma unroll
						for(int t = 0; t < 8; t++) unsafeAtomicAdd(&ot[idx[t]], tv[t]);
					}
				}
			}
		}
		if(on) {
			__builtin_amdgcn_wave_barrier();
#pragma unroll
			for(int k = 0; k < LN_WIN / 64; k++) {
				const int64_t r = r0 + k * 64 + lane;
				if(r < nRows) {
					const double v = ot[k * 64 + lane];
					cntNz += v != 0.0;
					out[r] = v;
				}
			}
		}
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
			c += std::max<uint32_t>(1, (slotMax[(size_t) s * nWin + w] + 7) / 8); // at least one chunk: the kernels' loads are unconditional
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
	b->laneOff[0] = descBytes; b->laneOff[1] = descBytes + slabBytes; b->laneOff[2] = descBytes + slabBytes + dictBytes;
	b->laneOff[3] = descBytes + slabBytes + dictBytes + idxBytes;
	b->laneLmm = singleCols;
	b->laneState = 1;
	return 0;
}

// Waves per block (one block per CU): as many of 16, 12, 8, 4 as `most` and the LDS windows next to the dictionaries allow.
static int lanes_waves(const cla_block* b, int most, size_t* lds) {
	const size_t ldsMax = (size_t) std::min(g_ldsPerBlock, 160 * 1024);
	const size_t fixed = sizeof(double) * (size_t) b->laneDictLds, perWave = sizeof(double) * LN_YT;
	int waves = 4;
	for(int w : {16, 12, 8})
		if(w <= most && fixed + w * perWave <= ldsMax) { waves = w; break; }
	*lds = fixed + waves * perWave;
	return *lds <= ldsMax ? waves : 0;
}

// t(Y) %*% X of all listed groups straight into dOut. Returns 1 when the block's lists do not fit these kernels
// (codes beyond a byte, groups of several columns, dictionaries beyond LDS, lists too uneven), 0 when done.
int launch_lmm_sdc_lanes(cla_block* b, const double* dY, int p, double* dOut) {
	int rc = lanes_plan(b);
	if(rc) return rc;
	if(b->laneState != 1 || !b->laneLmm || p > 65535) return 1;
	size_t lds = 0;
	const int waves = lanes_waves(b, 8, &lds); // (the kernel's registers allow two waves per SIMD)
	if(waves == 0) return 1;
	const int nWin = (int) ((b->nRows + LN_WIN - 1) / LN_WIN), nS = b->laneSlabs;
	// about one block per CU, every wave a run of windows
	const int64_t runs = std::max<int64_t>(1, (int64_t) g_numCU / ((int64_t) nS * p));
	const int wpw = (int) std::max<int64_t>(1, (nWin + runs * waves - 1) / (runs * waves));
	const unsigned nRuns = (unsigned) ((nWin + wpw * waves - 1) / (wpw * waves));
	char* meta = (char*) b->dLaneMeta;
	double algo = (double) b->nRows * 8 * p;
	for(int g : b->sdcList) algo += (double) p * ((double) b->groups[g].d.nDeltas * b->groups[g].d.deltaWidth + (double) b->groups[g].d.nOffsets);
	Prof pf(b, "k_lmm_sdc_lanes", (long) nRuns * nS * p, waves * 64, (long) lds, algo);
	auto go = [&](auto kernel) {
		CLA_HIP(hipFuncSetAttribute((const void*) kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds));
		hipLaunchKernelGGL(kernel, dim3(nRuns * nS, p), dim3(waves * 64), lds, b->stream, (const LaneDesc*) meta,
			(const LaneSlab*) (meta + b->laneOff[0]), nS, (const double*) (meta + b->laneOff[1]), b->laneDictLds,
			(const uint32_t*) (meta + b->laneOff[3]), (const u32x4*) b->dLaneData, dY, b->nRows, nWin, wpw, dOut, b->nCols);
		return 0;
	};
	rc = waves == 8 ? go(k_lmm_sdc_lanes<8>) : go(k_lmm_sdc_lanes<4>);
	if(rc) return rc;
	CLA_HIP(hipGetLastError());
	return 0;
}

// X %*% u of all listed groups (tables in b->dTables). Returns 1 when the lists do not fit, 0 when done.
int launch_rmm_sdc_lanes(cla_block* b, int constRow, int accumulate, double* dOut, unsigned long long* dNnz) {
	int rc = lanes_plan(b);
	if(rc) return rc;
	if(b->laneState != 1) return 1;
	size_t lds = 0;
	const int waves = lanes_waves(b, 16, &lds);
	if(waves == 0) return 1;
	const int nWin = (int) ((b->nRows + LN_WIN - 1) / LN_WIN), nS = b->laneSlabs;
	// one block per CU and round; whole rounds of the block's waves
	int wpb = (int) std::max<int64_t>(waves, ((int64_t) nWin + g_numCU - 1) / g_numCU);
	wpb = (wpb + waves - 1) / waves * waves;
	const unsigned grid = (unsigned) ((nWin + wpb - 1) / wpb);
	char* meta = (char*) b->dLaneMeta;
	double algo = (double) b->nRows * 8 * (accumulate ? 2 : 1);
	for(int g : b->sdcList) algo += (double) b->groups[g].d.nDeltas * b->groups[g].d.deltaWidth + (double) b->groups[g].d.nOffsets;
	Prof pf(b, "k_rmm_sdc_lanes", (long) grid, waves * 64, (long) lds, algo);
	auto go = [&](auto kernel) {
		CLA_HIP(hipFuncSetAttribute((const void*) kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds));
		hipLaunchKernelGGL(kernel, dim3(grid), dim3(waves * 64), lds, b->stream, (const LaneDesc*) meta,
			(const LaneSlab*) (meta + b->laneOff[0]), nS, (const int32_t*) (meta + b->laneOff[2]), b->laneDictLds,
			(const uint32_t*) (meta + b->laneOff[3]), (const u32x4*) b->dLaneData, (const double*) b->dTables, constRow, accumulate,
			dOut, b->nRows, nWin, wpb, dNnz);
		return 0;
	};
	rc = waves == 16 ? go(k_rmm_sdc_lanes<16>) : waves == 12 ? go(k_rmm_sdc_lanes<12>) : waves == 8 ? go(k_rmm_sdc_lanes<8>) : go(k_rmm_sdc_lanes<4>);
	if(rc) return rc;
	CLA_HIP(hipGetLastError());
	return 0;
}

} // namespace cla
