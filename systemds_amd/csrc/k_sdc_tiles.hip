// Row-tile kernels for SDCZeros groups (gfx950): all offset lists of a block are
// walked tile by tile, so the dense operand (a tile of Y for the left multiply,
// a tile of the output for the right multiply) is staged in LDS once and shared
// by every group, instead of being gathered from / scattered to HBM per entry.
//
//   k_lmm_sdc_tiles   bins[g][code] += Y[i, row] for every listed row (t(v) %*% X)
//   k_rmm_sdc_tiles   out[row, :] += T_g[code, :] for every listed row (X %*% u); tables from L2
//   k_sdc_pack        one-time rewrite of the lists into one word per entry (code, row in tile)
//   k_rmm_sdc_packed  X %*% u on the packed lists, software-pipelined over a wave's groups
//   k_lmm_sdc_packed  t(v) %*% X on the packed lists for single-column groups of <= 64 tuples
//
// A tile is ST = 4 * SDC_TILE rows; the iterator state in front of a tile comes
// from the row-tile index built at finalize.
#include "../../include/cla_hip.h"
#include "cla_device.hpp"
#include <algorithm>

namespace cla {

constexpr int ST = 4 * SDC_TILE;   // rows per tile
constexpr int ST_THREADS = 512;    // 8 waves; each wave walks one (group, tile) list segment at a time

// ---------------------------------------------------------------------------
// Left multiply, SDCZeros groups sdcList[l0 .. l1): block = range of tiles, row i of Y
// = blockIdx.y. LDS: the Y tile and private bins of all groups of the slab.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(ST_THREADS) void k_lmm_sdc_tiles(const DGroup* __restrict__ groups,
	const int32_t* __restrict__ sdcList, const int32_t* __restrict__ binOff, int l0, int l1, const double* __restrict__ Y,
	int64_t nRows, int tilesPerBlock, double* __restrict__ pre, int totalVals) {
	extern __shared__ double smem[];
	double* ytile = smem;          // ST
	double* bins = smem + ST;      // binOff[l1] - binOff[l0]
	const int tid = threadIdx.x, wave = tid >> 6;
	const int i = blockIdx.y;
	const int nBins = binOff[l1] - binOff[l0];
	const int b0 = binOff[l0];
	for(int k = tid; k < nBins; k += ST_THREADS) bins[k] = 0.0;
	const int nTiles = (int) ((nRows + ST - 1) / ST);
	const int t0 = blockIdx.x * tilesPerBlock, t1 = min(t0 + tilesPerBlock, nTiles);
	const double* y = Y + (size_t) i * nRows;
	for(int tile = t0; tile < t1; tile++) {
		const int64_t r0 = (int64_t) tile * ST;
		__syncthreads();
		for(int t = tid; t < ST; t += ST_THREADS) ytile[t] = r0 + t < nRows ? y[r0 + t] : 0.0;
		__syncthreads();
		for(int l = l0 + wave; l < l1; l += ST_THREADS / 64) {
			const DGroup G = dgroup(groups + (sdcList[l]));
			double* bg = bins + (binOff[l] - b0);
			const void* codes = G.codes;
			const int cw = G.codeWidth;
			sdc_walk_tile(G, r0, ST, [&](int rr, int di) { unsafeAtomicAdd(&bg[load_code(codes, cw, di)], ytile[rr]); });
		}
	}
	__syncthreads();
	for(int l = l0; l < l1; l++) {
		const DGroup G = dgroup(groups + (sdcList[l]));
		const double* bg = bins + (binOff[l] - b0);
		double* dst = pre + (size_t) i * totalVals + G.tblOff;
		for(int k = tid; k < G.nVals; k += ST_THREADS) {
			const double v = bg[k];
			if(v != 0.0) unsafeAtomicAdd(&dst[k], v);
		}
	}
}

// ---------------------------------------------------------------------------
// Right multiply with q output columns, SDCZeros groups sdcList[0 .. nL): block =
// one tile of the output columns [q0, q0 + qc). LDS: the output tile [ST x qc] and the tables of a
// slab of groups. accumulate == 0: the tile starts from constRow (or zero) and is the whole
// result; accumulate != 0: the tile starts from what other groups already wrote.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(ST_THREADS) void k_rmm_sdc_tiles(const DGroup* __restrict__ groups,
	const int32_t* __restrict__ sdcList, const int32_t* __restrict__ binOff, int nL, int slabLen, const double* __restrict__ T,
	int q, int q0, int qc, int constRow, int accumulate, int tileRows, double* __restrict__ out, int64_t nRows,
	unsigned long long* __restrict__ nnz, int ldsTables) {
	extern __shared__ double smem[];
	double* otile = smem;                        // tileRows * qc
	double* tbl = smem + (size_t) tileRows * qc; // tables of the current slab, qc doubles per tuple
	const int tid = threadIdx.x, wave = tid >> 6;
	const int tile = blockIdx.x;
	const int64_t r0 = (int64_t) tile * tileRows;
	const int nr = (int) min((int64_t) tileRows, nRows - r0);
	for(int t = tid; t < tileRows * qc; t += ST_THREADS) {
		double v = 0.0;
		const int rr = t / qc, c = t - rr * qc;
		if(rr < nr) v = accumulate ? out[(size_t) (r0 + rr) * q + q0 + c] : (constRow >= 0 ? T[(size_t) constRow * q + q0 + c] : 0.0);
		otile[t] = v;
	}
	for(int l0 = 0; l0 < nL; l0 += slabLen) {
		const int l1 = min(l0 + slabLen, nL);
		const int b0 = binOff[l0];
		__syncthreads();
		if(ldsTables) {
			for(int l = l0; l < l1; l++) {
				const DGroup G = dgroup(groups + (sdcList[l]));
				double* tg = tbl + (size_t) (binOff[l] - b0) * qc;
				const double* src = T + (size_t) G.tblOff * q + q0;
				for(int k = tid; k < G.nVals * qc; k += ST_THREADS) tg[k] = src[(size_t) (k / qc) * q + k % qc];
			}
			__syncthreads();
		}
		for(int l = l0 + wave; l < l1; l += ST_THREADS / 64) {
			const DGroup G = dgroup(groups + (sdcList[l]));
			const double* tg = ldsTables ? tbl + (size_t) (binOff[l] - b0) * qc : T + (size_t) G.tblOff * q + q0;
			const int ts = ldsTables ? qc : q; // doubles between two tuples of the table
			const void* codes = G.codes;
			const int cw = G.codeWidth;
			sdc_walk_tile(G, r0, tileRows, [&](int rr, int di) {
				const int code = load_code(codes, cw, di);
				for(int c = 0; c < qc; c++) unsafeAtomicAdd(&otile[(size_t) rr * qc + c], tg[(size_t) code * ts + c]);
			});
		}
	}
	__syncthreads();
	int cnt = 0;
	for(int t = tid; t < nr * qc; t += ST_THREADS) {
		const double v = otile[t];
		const int rr = t / qc, c = t - rr * qc;
		cnt += v != 0.0;
		out[(size_t) (r0 + rr) * q + q0 + c] = v;
	}
	count_add(nnz, cnt);
}

// What a list walk needs of a group, in one 48-byte read.
struct SdcDesc {
	const void* deltas;
	const void* codes;
	const OffState* tileIdx;
	int32_t nDeltas, nOffsets, first, tblOff, nTiles;
	int32_t widths; // delta width | code width << 8
	int32_t nVals, col0; // col0: the column of a single-column group
	const double* dict;
	const uint32_t* packed; // the group's entries as (code << 16 | row & 4095), in list order
};

// Tasks (list segments) whose loads a wave keeps in flight in the packed-list kernels.
constexpr int SDC_P = 4;

template <class T>
__device__ __forceinline__ T bcast_lane(T v, int l) {
	static_assert(sizeof(T) == 4 || sizeof(T) == 8, "readlane moves 32-bit pieces");
	if(sizeof(T) == 4) {
		int x;
		__builtin_memcpy(&x, &v, 4);
		x = __builtin_amdgcn_readlane(x, l);
		__builtin_memcpy(&v, &x, 4);
	}
	else {
		int x[2];
		__builtin_memcpy(x, &v, 8);
		x[0] = __builtin_amdgcn_readlane(x[0], l);
		x[1] = __builtin_amdgcn_readlane(x[1], l);
		__builtin_memcpy(&v, x, 8);
	}
	return v;
}

// ---------------------------------------------------------------------------
// Packed entry lists: at first use every listed group's offsets and codes are rewritten once
// into one word per entry, code << 16 | row inside its 4096-row tile, in list order. A tile's
// entries are then the range [entries before the tile, entries before the next tile) (both from
// the row-tile index) and need no decoding: no prefix sums, no skip entries, no special first
// row. Costs 4 bytes per entry in HBM next to the 2 of the reference's own form.
// ---------------------------------------------------------------------------
static_assert(ST == 4096, "packed entries hold 12-bit rows");

__global__ __launch_bounds__(256) void k_sdc_pack(const DGroup* __restrict__ groups, int g, int64_t nRows,
	uint32_t* __restrict__ packed) {
	const DGroup G = dgroup(groups + g);
	const int tile = blockIdx.x * 4 + (threadIdx.x >> 6);
	const int64_t r0 = (int64_t) tile * SDC_TILE;
	if(r0 >= nRows) return; // whole waves leave
	const void* codes = G.codes;
	const int cw = G.codeWidth;
	sdc_walk_tile(G, r0, SDC_TILE, [&](int rr, int di) { packed[di] = ((uint32_t) load_code(codes, cw, di) << 16) | (uint32_t) ((r0 + rr) & (ST - 1)); });
}

// lane t of a wave: entry range of task t's group inside the tile [r0, r0 + ST)
__device__ __forceinline__ void sdc_tile_range(const SdcDesc& D, int64_t r0, int& start, int& cnt) {
	const int ti = (int) (r0 / SDC_TILE);
	const OffState* idx = as_global(D.tileIdx);
	const int s0 = D.first < r0 ? (ti < D.nTiles ? idx[ti].emit : D.nOffsets) : 0;
	const int s1 = D.first < r0 + ST ? (ti + ST / SDC_TILE < D.nTiles ? idx[ti + ST / SDC_TILE].emit : D.nOffsets) : 0;
	start = s0;
	cnt = s1 - s0;
}

// Right multiply with one output column on packed lists. A wave owns the groups l = wave,
// wave + 8, ...; lane t keeps descriptor and entry range of the wave's task t. The task loop
// runs three stages on consecutive tasks: (A) request four packed entries per lane and the
// group's table entry `lane`; (B) look the table values up (by lane permute for groups of at
// most 64 tuples, from L2 otherwise); (C) add into the output tile in LDS. Every wait is for
// loads issued one iteration earlier, which the other waves of the CU cover.
__global__ __launch_bounds__(ST_THREADS) void k_rmm_sdc_packed(const SdcDesc* __restrict__ desc, int nL,
	const double* __restrict__ T, int constRow, int accumulate, double* __restrict__ out, int64_t nRows,
	unsigned long long* __restrict__ nnz) {
	extern __shared__ double otile[]; // ST
	const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
	const int64_t r0 = (int64_t) blockIdx.x * ST;
	const int nr = (int) min((int64_t) ST, nRows - r0);
	for(int t = tid; t < ST; t += ST_THREADS) {
		double v = 0.0;
		if(t < nr) v = accumulate ? out[r0 + t] : (constRow >= 0 ? T[constRow] : 0.0);
		otile[t] = v;
	}
	__syncthreads();
	const int nT = wave < nL ? (nL - wave + ST_THREADS / 64 - 1) / (ST_THREADS / 64) : 0;
	for(int t0 = 0; t0 < nT; t0 += 64) {
		const int nHere = min(64, nT - t0);
		SdcDesc D;
		D.deltas = nullptr; D.codes = nullptr; D.tileIdx = nullptr;
		D.nDeltas = 0; D.nOffsets = 0; D.first = -1; D.tblOff = 0; D.nTiles = 0; D.widths = 0x101; D.nVals = 0; D.col0 = 0; D.dict = nullptr; D.packed = nullptr;
		int start = 0, cnt = 0;
		if(lane < nHere) {
			D = desc[wave + (ST_THREADS / 64) * (t0 + lane)];
			sdc_tile_range(D, r0, start, cnt);
		}
		// Common case, every task of the batch a segment of at most 256 entries of a group with at most 64
		// tuples: the loads (list segment, table entry `lane`) of SDC_P tasks are kept in flight. Every load
		// of this loop is unconditional (tasks past the end repeat the last one with no entries, lanes past
		// a table's end read its last entry): a load under a branch makes the compiler wait for all
		// outstanding loads at the join, which is what limited the one-task-ahead form to a memory latency
		// per task.
		const bool simple = __builtin_amdgcn_ballot_w64(lane < nHere && (cnt > 256 || D.nVals > 64 || D.nVals < 1)) == 0;
		if(simple) {
			const int last = nHere - 1;
			u32x4 eR[SDC_P];
			double tblR[SDC_P];
			auto issue = [&](int slot, int t) {
				const uint32_t* pk = as_global(bcast_lane(D.packed, t)) + bcast_lane(start, t);
				const int nv = bcast_lane(D.nVals, t);
				eR[slot] = *(const u32x4*) (pk + lane * 4); // (256 entries of slack behind the last list)
				tblR[slot] = T[bcast_lane(D.tblOff, t) + min(lane, nv - 1)];
			};
#pragma unroll
			for(int j = 0; j < SDC_P; j++) issue(j, min(j, last));
			for(int t = 0; t < nHere; t += SDC_P) {
#pragma unroll
				for(int j = 0; j < SDC_P; j++) {
					const int tb = t + j;
					const u32x4 eB = eR[j];
					const double tblB = tblR[j];
					issue(j, min(tb + SDC_P, last));
					const int n = tb < nHere ? bcast_lane(cnt, min(tb, last)) : 0;
#pragma unroll
					for(int k = 0; k < 4; k++) {
						const double tv = __shfl(tblB, (int) (eB[k] >> 16) & 63, 64);
						if(lane * 4 + k < n) unsafeAtomicAdd(&otile[eB[k] & (ST - 1)], tv);
					}
				}
			}
		}
		else {
			u32x4 eA = {0, 0, 0, 0};
			double tblA = 0.0;
			int rowsC[4] = {0, 0, 0, 0};
			double tvC[4] = {0.0, 0.0, 0.0, 0.0};
			unsigned maskC = 0;
			for(int t = 0; t < nHere + 2; t++) {
				const u32x4 eB = eA;
				const double tblB = tblA;
				if(t < nHere) { // ---- stage A: task t
					const uint32_t* pk = as_global(bcast_lane(D.packed, t)) + bcast_lane(start, t);
					const int nv = bcast_lane(D.nVals, t);
					eA = *(const u32x4*) (pk + lane * 4); // dword aligned; entries beyond the task's count are masked in stage B
					tblA = nv <= 64 && lane < nv ? T[bcast_lane(D.tblOff, t) + lane] : 0.0;
				}
				if(t >= 2) { // ---- stage C: task t - 2
	#pragma unroll
					for(int k = 0; k < 4; k++)
						if(maskC & (1u << k)) unsafeAtomicAdd(&otile[rowsC[k]], tvC[k]);
				}
				maskC = 0;
				if(t >= 1 && t - 1 < nHere) { // ---- stage B: task t - 1
					const int tb = t - 1;
					const int n = bcast_lane(cnt, tb);
					const double* tg = T + bcast_lane(D.tblOff, tb);
					const bool inRegs = bcast_lane(D.nVals, tb) <= 64;
	#pragma unroll
					for(int k = 0; k < 4; k++) {
						const bool on = lane * 4 + k < n;
						const int code = (int) (eB[k] >> 16);
						const double tv = inRegs ? __shfl(tblB, code & 63, 64) : (on ? tg[code] : 0.0);
						rowsC[k] = (int) (eB[k] & (ST - 1));
						tvC[k] = tv;
						if(on) maskC |= 1u << k;
					}
					if(n > 256) { // dense lists: the rest of the tile's entries, straight
						const uint32_t* pk = as_global(bcast_lane(D.packed, tb)) + bcast_lane(start, tb);
						for(int j = 256 + lane; j < n; j += 64) {
							const uint32_t e = pk[j];
							unsafeAtomicAdd(&otile[e & (ST - 1)], tg[e >> 16]);
						}
					}
				}
			}
	
		}
	}
	__syncthreads();
	int cntNz = 0;
	for(int t = tid; t < nr; t += ST_THREADS) {
		const double v = otile[t];
		cntNz += v != 0.0;
		out[r0 + t] = v;
	}
	count_add(nnz, cntNz);
}

// Left multiply on packed lists for single-column groups with at most 64 tuples: the group's
// dictionary sits in registers (entry `lane`), every entry contributes Y[row] * dict[code] (row
// from the Y tile in LDS, dictionary value by lane permute), the wave sums the products (DPP) and
// lane t keeps the total of task t. No bins, no LDS atomics, one launch for all groups; the
// totals go straight into the output. block = (range of tiles, row i of Y).
__global__ __launch_bounds__(ST_THREADS) void k_lmm_sdc_packed(const SdcDesc* __restrict__ desc, int nL,
	const double* __restrict__ Y, int64_t nRows, int tilesPerBlock, double* __restrict__ out, int nCols) {
	extern __shared__ double ytile[]; // ST
	const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
	const int irow = blockIdx.y;
	const double* y = Y + (size_t) irow * nRows;
	const int nTilesAll = (int) ((nRows + ST - 1) / ST);
	const int tile0 = blockIdx.x * tilesPerBlock, tile1 = min(tile0 + tilesPerBlock, nTilesAll);
	const int nT = wave < nL ? (nL - wave + ST_THREADS / 64 - 1) / (ST_THREADS / 64) : 0;
	const int nTmax = (nL + ST_THREADS / 64 - 1) / (ST_THREADS / 64); // the same trip count for every wave: barriers inside
	for(int t0 = 0; t0 < max(nTmax, 1); t0 += 64) {
		const int nHere = max(0, min(64, nT - t0));
		SdcDesc D;
		D.deltas = nullptr; D.codes = nullptr; D.tileIdx = nullptr;
		D.nDeltas = 0; D.nOffsets = 0; D.first = -1; D.tblOff = 0; D.nTiles = 0; D.widths = 0x101; D.nVals = 0; D.col0 = 0; D.dict = nullptr; D.packed = nullptr;
		if(lane < nHere) D = desc[wave + (ST_THREADS / 64) * (t0 + lane)];
		double accT = 0.0; // lane t: total of task t over the block's tiles
		for(int tile = tile0; tile < tile1; tile++) {
			const int64_t r0 = (int64_t) tile * ST;
			__syncthreads(); // the previous tile's readers are done
			for(int t = tid; t < ST; t += ST_THREADS) ytile[t] = r0 + t < nRows ? y[r0 + t] : 0.0;
			__syncthreads();
			int start = 0, cnt = 0;
			if(lane < nHere) sdc_tile_range(D, r0, start, cnt);
			// (see k_rmm_sdc_packed: unconditional loads, SDC_P tasks in flight)
			const bool simple = nHere > 0 && __builtin_amdgcn_ballot_w64(lane < nHere && (cnt > 256 || D.nVals < 1)) == 0;
			if(simple) {
				const int last = nHere - 1;
				u32x4 eR[SDC_P];
				double dictR[SDC_P];
				auto issue = [&](int slot, int t) {
					const uint32_t* pk = as_global(bcast_lane(D.packed, t)) + bcast_lane(start, t);
					eR[slot] = *(const u32x4*) (pk + lane * 4);
					dictR[slot] = as_global(bcast_lane(D.dict, t))[min(lane, bcast_lane(D.nVals, t) - 1)];
				};
#pragma unroll
				for(int j = 0; j < SDC_P; j++) issue(j, min(j, last));
				for(int t = 0; t < nHere; t += SDC_P) {
#pragma unroll
					for(int j = 0; j < SDC_P; j++) {
						const int tb = t + j;
						const u32x4 eB = eR[j];
						const double dictB = dictR[j];
						issue(j, min(tb + SDC_P, last));
						const int n = tb < nHere ? bcast_lane(cnt, min(tb, last)) : 0;
						double part = 0.0;
#pragma unroll
						for(int k = 0; k < 4; k++) {
							const double d = __shfl(dictB, (int) (eB[k] >> 16) & 63, 64);
							const double yv = ytile[eB[k] & (ST - 1)];
							part += lane * 4 + k < n ? yv * d : 0.0;
						}
						const double total = wave_sum_f64_all(part);
						if(lane == tb) accT += total;
					}
				}
			}
			else {
				u32x4 eA = {0, 0, 0, 0};
				double dictA = 0.0;
				for(int t = 0; t < nHere + 1; t++) {
					const u32x4 eB = eA;
					const double dictB = dictA;
					if(t < nHere) { // ---- stage A: task t
						const uint32_t* pk = as_global(bcast_lane(D.packed, t)) + bcast_lane(start, t);
						eA = *(const u32x4*) (pk + lane * 4);
						dictA = lane < bcast_lane(D.nVals, t) ? as_global(bcast_lane(D.dict, t))[lane] : 0.0;
					}
					if(t >= 1) { // ---- stage B: task t - 1
						const int tb = t - 1;
						const int n = bcast_lane(cnt, tb);
						double part = 0.0;
	#pragma unroll
						for(int k = 0; k < 4; k++) {
							const double d = __shfl(dictB, (int) (eB[k] >> 16) & 63, 64);
							if(lane * 4 + k < n) part += ytile[eB[k] & (ST - 1)] * d;
						}
						if(n > 256) {
							const uint32_t* pk = as_global(bcast_lane(D.packed, tb)) + bcast_lane(start, tb);
							for(int j0 = 256; j0 < n; j0 += 64) { // uniform trip count: the permute needs every lane
								const uint32_t e = j0 + lane < n ? pk[j0 + lane] : 0u;
								const double d = __shfl(dictB, (int) (e >> 16) & 63, 64);
								if(j0 + lane < n) part += ytile[e & (ST - 1)] * d;
							}
						}
						const double total = wave_sum_f64_all(part);
						if(lane == tb) accT += total;
					}
				}
		
			}
		}
		if(lane < nHere && accT != 0.0) unsafeAtomicAdd(&out[(size_t) irow * nCols + D.col0], accT);
	}
}

// Host side: list of SDCZeros groups and the prefix sums of their nVals, kept on the block
// (host and device copy) and rebuilt only when the requested group selection changes.
static int sdc_upload_desc(cla_block* b, bool wholeBlock) {
	std::vector<SdcDesc> descs;
	int64_t packedOff = 0;
	for(int g : b->sdcList) {
		const DGroup& G = b->groups[g].d;
		SdcDesc d;
		d.deltas = G.deltas; d.codes = G.codes; d.tileIdx = G.tileIdx;
		d.nDeltas = (int32_t) G.nDeltas; d.nOffsets = (int32_t) G.nOffsets; d.first = G.first; d.tblOff = G.tblOff; d.nTiles = G.nTiles;
		d.widths = G.deltaWidth | (G.codeWidth << 8);
		d.nVals = G.nVals; d.col0 = b->groups[g].cols[0]; d.dict = G.dict;
		d.packed = wholeBlock && b->dSdcPacked ? b->dSdcPacked + packedOff : nullptr; // packed lists belong to the whole-block plan
		packedOff += G.nOffsets;
		descs.push_back(d);
	}
	if(!descs.empty()) {
		CLA_HIP(hipMemcpyAsync(b->dSdcDesc, descs.data(), descs.size() * sizeof(SdcDesc), hipMemcpyHostToDevice, b->stream));
		CLA_HIP(hipStreamSynchronize(b->stream)); // `descs` goes out of scope
	}
	return 0;
}

static int sdc_plan(cla_block* b, int onlyGroup, int32_t** dList, int32_t** dBinOff, bool wantPacked = false) {
	const size_t nG = b->groups.size();
	if(b->dSdcPlan == nullptr) CLA_HIP(hipMalloc((void**) &b->dSdcPlan, (2 * nG + 2) * sizeof(int32_t)));
	if(b->dSdcDesc == nullptr) CLA_HIP(hipMalloc(&b->dSdcDesc, std::max<size_t>(nG, 1) * sizeof(SdcDesc)));
	if(b->sdcPlanGroup != onlyGroup) {
		b->sdcList.clear();
		b->sdcBinOff.assign(1, 0);
		for(int g = 0; g < (int) nG; g++) {
			const DGroup& G = b->groups[g].d;
			if(G.type != G_SDCZ || G.nOffsets == 0 || (onlyGroup >= 0 && onlyGroup != g)) continue;
			b->sdcList.push_back(g);
			b->sdcBinOff.push_back(b->sdcBinOff.back() + G.nVals);
		}
		b->sdcPlanGroup = -2; // invalid until both copies have been issued
		int rc = sdc_upload_desc(b, onlyGroup < 0);
		if(rc) return rc;
		if(!b->sdcList.empty()) {
			CLA_HIP(hipMemcpyAsync(b->dSdcPlan, b->sdcList.data(), b->sdcList.size() * 4, hipMemcpyHostToDevice, b->stream));
			CLA_HIP(hipMemcpyAsync(b->dSdcPlan + nG, b->sdcBinOff.data(), b->sdcBinOff.size() * 4, hipMemcpyHostToDevice, b->stream));
			// the host vectors are rewritten by the next selection: the copies must have read them
			CLA_HIP(hipStreamSynchronize(b->stream));
		}
		b->sdcPlanGroup = onlyGroup;
	}
	// packed entries of all listed groups (whole-block plans only, when a packed kernel asks), 256 entries of slack
	// behind the last
	if(wantPacked && onlyGroup < 0 && !b->sdcList.empty() && b->dSdcPacked == nullptr && !b->sdcPackFailed) {
		int64_t totalEntries = 0;
		bool packable = true;
		for(int g : b->sdcList) {
			totalEntries += b->groups[g].d.nOffsets;
			packable &= b->groups[g].d.nVals <= 65536;
		}
		b->sdcPackFailed = !packable;
		if(packable) {
			CLA_HIP(hipMalloc((void**) &b->dSdcPacked, sizeof(uint32_t) * (size_t) (totalEntries + 256)));
			b->derivedBytes += (int64_t) sizeof(uint32_t) * (totalEntries + 256);
			CLA_HIP(hipMemsetAsync(b->dSdcPacked + totalEntries, 0, sizeof(uint32_t) * 256, b->stream));
			const int nT1 = (int) ((b->nRows + SDC_TILE - 1) / SDC_TILE);
			int64_t off = 0;
			for(int g : b->sdcList) {
				hipLaunchKernelGGL(k_sdc_pack, dim3((unsigned) ((nT1 + 3) / 4)), dim3(256), 0, b->stream, b->dGroups, g, b->nRows,
					b->dSdcPacked + off);
				off += b->groups[g].d.nOffsets;
			}
			CLA_HIP(hipGetLastError());
			int rc = sdc_upload_desc(b, true);
			if(rc) return rc;
		}
	}
	*dList = b->dSdcPlan;
	*dBinOff = b->dSdcPlan + nG;
	return 0;
}

int sdc_plan_all(cla_block* b) {
	int32_t *dList = nullptr, *dBinOff = nullptr;
	return sdc_plan(b, -1, &dList, &dBinOff);
}

// Returns 1 if some SDC group cannot use the tile kernel (caller falls back), 0 when done.
int launch_lmm_sdc_tiles(cla_block* b, const double* dY, int p, double* dPre, int onlyGroup, double* dOut) {
	int32_t *dList = nullptr, *dBinOff = nullptr;
	int rc = sdc_plan(b, onlyGroup, &dList, &dBinOff);
	if(rc) return rc;
	struct { const std::vector<int32_t>&list, &binOff; } plan{b->sdcList, b->sdcBinOff};
	if(plan.list.empty()) return 0;
	// whole-block call on single-column groups: one lane per group on lane-major lists, products straight
	// into dOut (the groups' part of dPre stays zero)
	// (not with a non-finite dictionary value: the kernels below sum Y[row] * dict[code] over the rows, the reference
	// sums Y per tuple first, and the two differ where an infinity meets values of Y of both signs)
	if(dOut != nullptr && onlyGroup < 0 && b->opt.sdcLanes && !b->dictNonFinite) {
		const int r = launch_lmm_sdc_lanes(b, dY, p, dOut);
		if(r <= 0) return r;
	}
	// all listed groups single-column with at most 64 tuples, whole-block call: packed lists, products
	// straight into dOut
	bool packed = dOut != nullptr && onlyGroup < 0 && b->opt.sdcPacked && !b->dictNonFinite;
	for(int g : plan.list) packed &= b->groups[g].d.nColG == 1 && b->groups[g].d.nVals <= 64;
	if(packed && (rc = sdc_plan(b, onlyGroup, &dList, &dBinOff, true))) return rc;
	packed &= b->dSdcPacked != nullptr;
	if(packed) {
		const int nTiles = (int) ((b->nRows + ST - 1) / ST);
		int tpb = std::max(1, (nTiles * p + 4 * g_numCU - 1) / (4 * g_numCU));
		tpb = std::min(tpb, std::max(1, nTiles));
		const unsigned grid = (unsigned) ((nTiles + tpb - 1) / tpb);
		double algo = (double) b->nRows * 8 * p;
		for(int g : plan.list) algo += (double) p * ((double) b->groups[g].d.nDeltas * b->groups[g].d.deltaWidth + (double) b->groups[g].d.nOffsets * b->groups[g].d.codeWidth);
		const size_t lds = (size_t) ST * 8;
		Prof pf(b, "k_lmm_sdc_packed", (long) grid * p, ST_THREADS, (long) lds, algo);
		CLA_HIP(allow_full_lds((const void*) k_lmm_sdc_packed));
		hipLaunchKernelGGL(k_lmm_sdc_packed, dim3(grid, p), dim3(ST_THREADS), lds, b->stream, (const SdcDesc*) b->dSdcDesc,
			(int) plan.list.size(), dY, b->nRows, tpb, dOut, b->nCols);
		CLA_HIP(hipGetLastError());
		return 0;
	}
	const size_t ldsMax = (size_t) std::min(g_ldsPerBlock, 160 * 1024) - 2048;
	// bins of a slab of groups next to the Y tile; small slabs keep LDS per block low
	// enough for three blocks per CU, which hides the latency of the list walks
	size_t binBudget = 18 * 1024;
	binBudget = std::min(binBudget, ldsMax - (size_t) ST * 8);
	for(size_t l = 0; l < plan.list.size(); l++)
		binBudget = std::max(binBudget, (size_t) (plan.binOff[l + 1] - plan.binOff[l]) * 8);
	binBudget = std::min(binBudget, ldsMax - (size_t) ST * 8);
	for(size_t l = 0; l < plan.list.size(); l++)
		if((size_t) (plan.binOff[l + 1] - plan.binOff[l]) * 8 > binBudget) return 1;
	const int nTiles = (int) ((b->nRows + ST - 1) / ST);
	// slabs of groups whose bins fit next to the Y tile
	size_t l0 = 0;
	while(l0 < plan.list.size()) {
		size_t l1 = l0;
		while(l1 < plan.list.size() && (size_t) (plan.binOff[l1 + 1] - plan.binOff[l0]) * 8 <= binBudget) l1++;
		const size_t lds = (size_t) ST * 8 + (size_t) (plan.binOff[l1] - plan.binOff[l0]) * 8;
		// about four blocks per CU and Y row: bins are flushed once per block
		int tpb = std::max(1, (nTiles * p + 4 * g_numCU - 1) / (4 * g_numCU));
		tpb = std::min(tpb, std::max(1, nTiles));
		const unsigned grid = (unsigned) ((nTiles + tpb - 1) / tpb);
		double algo = (double) b->nRows * 8 * p;
		for(size_t l = l0; l < l1; l++) {
			const DGroup& G = b->groups[plan.list[l]].d;
			algo += (double) p * ((double) G.nDeltas * G.deltaWidth + (double) G.nOffsets * G.codeWidth);
		}
		b->preUsed = true;
		Prof pf(b, "k_lmm_sdc_tiles", (long) grid * p, ST_THREADS, (long) lds, algo);
		CLA_HIP(allow_full_lds((const void*) k_lmm_sdc_tiles));
		hipLaunchKernelGGL(k_lmm_sdc_tiles, dim3(grid, p), dim3(ST_THREADS), lds, b->stream, b->dGroups, dList, dBinOff,
			(int) l0, (int) l1, dY, b->nRows, tpb, dPre, b->totalVals);
		l0 = l1;
	}
	CLA_HIP(hipGetLastError());
	return 0;
}

// Returns 1 if the tile kernel cannot be used (caller falls back), 0 when done.
int launch_rmm_sdc_tiles(cla_block* b, int q, int constRow, int accumulate, double* dOut, unsigned long long* dNnz) {
	int32_t *dList = nullptr, *dBinOff = nullptr;
	int rc = sdc_plan(b, -1, &dList, &dBinOff);
	if(rc) return rc;
	struct { const std::vector<int32_t>&list, &binOff; } plan{b->sdcList, b->sdcBinOff};
	if(plan.list.empty() || b->nRows == 0) return 1;
	if(q == 1 && b->opt.sdcRows) { // one lane per row on row lists
		const int r = launch_rmm_sdc_rows(b, constRow, accumulate, dOut, dNnz);
		if(r <= 0) return r;
	}
	if(q == 1 && b->opt.sdcLanes) { // one lane per group on lane-major lists
		const int r = launch_rmm_sdc_lanes(b, constRow, accumulate, dOut, dNnz);
		if(r <= 0) return r;
	}
	if(q == 1 && b->opt.sdcPacked && (rc = sdc_plan(b, -1, &dList, &dBinOff, true))) return rc;
	const size_t ldsMax = (size_t) std::min(g_ldsPerBlock, 160 * 1024) - 2048;
	// columns per pass: all of them when a tile of SDC_TILE rows fits LDS, else chunks of that many columns
	// (each pass walks the lists again)
	int qc = q;
	while((size_t) SDC_TILE * qc * 8 + 4096 > ldsMax && qc > 1) qc = (qc + 1) / 2;
	// rows per tile: a multiple of the tile-index granularity whose output tile takes at most ~half of LDS
	int tileRows = ST;
	while(tileRows > SDC_TILE && (size_t) tileRows * qc * 8 > ldsMax / 2) tileRows /= 2;
	if((size_t) tileRows * qc * 8 + 4096 > ldsMax) return 1;
	size_t maxVals = 1;
	for(size_t l = 0; l < plan.list.size(); l++) maxVals = std::max(maxVals, (size_t) (plan.binOff[l + 1] - plan.binOff[l]));
	// Tables are read from global memory (they stay in L2): without table slabs in LDS the
	// waves of a block never meet at a barrier between the list walks, and only the output
	// tile takes LDS (C4: 1.95 ms with one 100 KB slab in LDS, 0.72 ms with 8 KB slabs,
	// 0.58 ms with none).
	size_t tblBudget = 8 * 1024;
	const bool ldsTables = false;
	tblBudget = std::max(tblBudget, maxVals * qc * 8);
	tblBudget = std::min(tblBudget, ldsMax - (size_t) tileRows * qc * 8);
	// groups per slab: uniform count so that every slab's tables fit
	const size_t slabLen = tblBudget / (maxVals * qc * 8);
	if(slabLen < 1) return 1;
	const int nTiles = (int) ((b->nRows + tileRows - 1) / tileRows);
	const int sl = ldsTables ? (int) std::min(slabLen, plan.list.size()) : (int) plan.list.size();
	size_t tblDoubles = 0;
	for(size_t l0 = 0; ldsTables && l0 < plan.list.size(); l0 += sl)
		tblDoubles = std::max(tblDoubles, (size_t) (plan.binOff[std::min(l0 + sl, plan.list.size())] - plan.binOff[l0]) * qc);
	const size_t lds = (size_t) tileRows * qc * 8 + tblDoubles * 8;
	double algo = (double) b->nRows * q * 8 * (accumulate ? 2 : 1);
	for(int g : plan.list) {
		const DGroup& G = b->groups[g].d;
		algo += (double) G.nDeltas * G.deltaWidth + (double) G.nOffsets * G.codeWidth;
	}
	const bool noPacked = !b->opt.sdcPacked;
	if(q == 1 && !ldsTables && tileRows == ST && !noPacked && b->dSdcPacked != nullptr) {
		const size_t ldsP = (size_t) ST * 8;
		Prof pf(b, "k_rmm_sdc_packed", nTiles, ST_THREADS, (long) ldsP, algo);
		CLA_HIP(allow_full_lds((const void*) k_rmm_sdc_packed));
		hipLaunchKernelGGL(k_rmm_sdc_packed, dim3(nTiles), dim3(ST_THREADS), ldsP, b->stream, (const SdcDesc*) b->dSdcDesc,
			(int) plan.list.size(), b->dTables, constRow, accumulate, dOut, b->nRows, dNnz);
	}
	else {
		CLA_HIP(allow_full_lds((const void*) k_rmm_sdc_tiles));
		for(int q0 = 0; q0 < q; q0 += qc) {
			Prof pf(b, "k_rmm_sdc_tiles", nTiles, ST_THREADS, (long) lds, algo * std::min(qc, q - q0) / q);
			hipLaunchKernelGGL(k_rmm_sdc_tiles, dim3(nTiles), dim3(ST_THREADS), lds, b->stream, b->dGroups, dList, dBinOff,
				(int) plan.list.size(), sl, b->dTables, q, q0, std::min(qc, q - q0), constRow, accumulate, tileRows, dOut, b->nRows, dNnz,
				ldsTables ? 1 : 0);
		}
	}
	CLA_HIP(hipGetLastError());
	return 0;
}

} // namespace cla
