// Row-tile kernels for SDCZeros groups (gfx950): all offset lists of a block are
// walked tile by tile, so the dense operand (a tile of Y for the left multiply,
// a tile of the output for the right multiply) is staged in LDS once and shared
// by every group, instead of being gathered from / scattered to HBM per entry.
//
//   k_lmm_sdc_tiles   bins[g][code] += Y[i, row] for every listed row (t(v) %*% X)
//   k_rmm_sdc_tiles   out[row, :] += T_g[code, :] for every listed row (X %*% u); tables from L2
//
// A tile is ST = 4 * SDC_TILE rows; the iterator state in front of a tile comes
// from the row-tile index built at finalize.
#include "../../include/cla_hip.h"
#include "cla_device.hpp"
#include <algorithm>

namespace cla {

constexpr int ST = 4 * SDC_TILE;   // rows per tile
constexpr int ST_THREADS = 512;    // 8 waves; each wave walks one (group, tile) list segment at a time

// Walks the entries of group G with rows in [r0, r0 + ST) and calls f(row - r0, dataIdx)
// on the owning lane. Must be called by all 64 lanes of a wave.
template <typename F>
__device__ __forceinline__ void sdc_walk_tile(const DGroup& G, int64_t r0, int tileRows, F f) {
	// r0 and tileRows are multiples of SDC_TILE
	if(G.nOffsets <= 0) return;
	const int lane = threadIdx.x & 63;
	const int64_t rEnd = r0 + tileRows;
	if(lane == 0 && G.first >= r0 && G.first < rEnd) f((int) (G.first - r0), 0);
	const int ti = (int) (r0 / SDC_TILE);
	if(ti >= G.nTiles) return;
	const OffState st = G.tileIdx[ti];
	int32_t row = st.row, emit = st.emit;
	int64_t i0 = st.idx;
	while(i0 < G.nDeltas && row < rEnd) {
		int32_t rows[4], didx[4];
		unsigned mask;
		if(G.deltaWidth == 1) sdc_decode256<1>(G.deltas, G.nDeltas, i0, row, emit, rows, didx, mask);
		else sdc_decode256<2>(G.deltas, G.nDeltas, i0, row, emit, rows, didx, mask);
#pragma unroll
		for(int k = 0; k < 4; k++)
			if((mask & (1u << k)) && rows[k] < rEnd) f((int) (rows[k] - r0), didx[k]);
		i0 += 256;
	}
}

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
// one tile. LDS: the output tile [ST x q] and the tables of a slab of groups.
// accumulate == 0: the tile starts from constRow (or zero) and is the whole
// result; accumulate != 0: the tile starts from what other groups already wrote.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(ST_THREADS) void k_rmm_sdc_tiles(const DGroup* __restrict__ groups,
	const int32_t* __restrict__ sdcList, const int32_t* __restrict__ binOff, int nL, int slabLen, const double* __restrict__ T,
	int q, int constRow, int accumulate, int tileRows, double* __restrict__ out, int64_t nRows,
	unsigned long long* __restrict__ nnz, int ldsTables) {
	extern __shared__ double smem[];
	double* otile = smem;                       // tileRows * q
	double* tbl = smem + (size_t) tileRows * q; // tables of the current slab, q doubles per tuple
	const int tid = threadIdx.x, wave = tid >> 6;
	const int tile = blockIdx.x;
	const int64_t r0 = (int64_t) tile * tileRows;
	const int nr = (int) min((int64_t) tileRows, nRows - r0);
	for(int t = tid; t < tileRows * q; t += ST_THREADS) {
		double v = 0.0;
		if(t < nr * q) v = accumulate ? out[(size_t) r0 * q + t] : (constRow >= 0 ? T[(size_t) constRow * q + (t % q)] : 0.0);
		otile[t] = v;
	}
	for(int l0 = 0; l0 < nL; l0 += slabLen) {
		const int l1 = min(l0 + slabLen, nL);
		const int b0 = binOff[l0];
		__syncthreads();
		if(ldsTables) {
			for(int l = l0; l < l1; l++) {
				const DGroup G = dgroup(groups + (sdcList[l]));
				double* tg = tbl + (size_t) (binOff[l] - b0) * q;
				const double* src = T + (size_t) G.tblOff * q;
				for(int k = tid; k < G.nVals * q; k += ST_THREADS) tg[k] = src[k];
			}
			__syncthreads();
		}
		for(int l = l0 + wave; l < l1; l += ST_THREADS / 64) {
			const DGroup G = dgroup(groups + (sdcList[l]));
			const double* tg = ldsTables ? tbl + (size_t) (binOff[l] - b0) * q : T + (size_t) G.tblOff * q;
			const void* codes = G.codes;
			const int cw = G.codeWidth;
			sdc_walk_tile(G, r0, tileRows, [&](int rr, int di) {
				const int code = load_code(codes, cw, di);
				for(int c = 0; c < q; c++) unsafeAtomicAdd(&otile[(size_t) rr * q + c], tg[(size_t) code * q + c]);
			});
		}
	}
	__syncthreads();
	int cnt = 0;
	for(int t = tid; t < nr * q; t += ST_THREADS) {
		const double v = otile[t];
		cnt += v != 0.0;
		out[(size_t) r0 * q + t] = v;
	}
	count_add(nnz, cnt);
}

// Host side: list of SDCZeros groups and the prefix sums of their nVals, kept on the block
// (host and device copy) and rebuilt only when the requested group selection changes.
static int sdc_plan(cla_block* b, int onlyGroup, int32_t** dList, int32_t** dBinOff) {
	const size_t nG = b->groups.size();
	if(b->dSdcPlan == nullptr) CLA_HIP(hipMalloc((void**) &b->dSdcPlan, (2 * nG + 2) * sizeof(int32_t)));
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
		if(!b->sdcList.empty()) {
			CLA_HIP(hipMemcpyAsync(b->dSdcPlan, b->sdcList.data(), b->sdcList.size() * 4, hipMemcpyHostToDevice, b->stream));
			CLA_HIP(hipMemcpyAsync(b->dSdcPlan + nG, b->sdcBinOff.data(), b->sdcBinOff.size() * 4, hipMemcpyHostToDevice, b->stream));
			// the host vectors are rewritten by the next selection: the copies must have read them
			CLA_HIP(hipStreamSynchronize(b->stream));
		}
		b->sdcPlanGroup = onlyGroup;
	}
	*dList = b->dSdcPlan;
	*dBinOff = b->dSdcPlan + nG;
	return 0;
}

// Returns 1 if some SDC group cannot use the tile kernel (caller falls back), 0 when done.
int launch_lmm_sdc_tiles(cla_block* b, const double* dY, int p, double* dPre, int onlyGroup) {
	int32_t *dList = nullptr, *dBinOff = nullptr;
	int rc = sdc_plan(b, onlyGroup, &dList, &dBinOff);
	if(rc) return rc;
	struct { const std::vector<int32_t>&list, &binOff; } plan{b->sdcList, b->sdcBinOff};
	if(plan.list.empty()) return 0;
	const size_t ldsMax = (size_t) std::min(g_ldsPerBlock, 160 * 1024) - 2048;
	// bins of a slab of groups next to the Y tile; small slabs keep LDS per block low
	// enough for three blocks per CU, which hides the latency of the list walks
	size_t binBudget = 18 * 1024;
	if(const char* e = getenv("CLA_LMM_SDC_BIN_KB")) binBudget = (size_t) atoi(e) * 1024;
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
		Prof pf(b, "k_lmm_sdc_tiles", (long) grid * p, ST_THREADS, (long) lds, algo);
		CLA_HIP(hipFuncSetAttribute((const void*) k_lmm_sdc_tiles, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds));
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
	const size_t ldsMax = (size_t) std::min(g_ldsPerBlock, 160 * 1024) - 2048;
	// rows per tile: a multiple of the tile-index granularity whose output tile takes at most ~half of LDS
	int tileRows = ST;
	while(tileRows > SDC_TILE && (size_t) tileRows * q * 8 > ldsMax / 2) tileRows /= 2;
	if((size_t) tileRows * q * 8 + 4096 > ldsMax) return 1;
	size_t maxVals = 1;
	for(size_t l = 0; l < plan.list.size(); l++) maxVals = std::max(maxVals, (size_t) (plan.binOff[l + 1] - plan.binOff[l]));
	// Tables are read from global memory (they stay in L2): without table slabs in LDS the
	// waves of a block never meet at a barrier between the list walks, and only the output
	// tile takes LDS (C4: 1.95 ms with one 100 KB slab in LDS, 0.72 ms with 8 KB slabs,
	// 0.58 ms with none). CLA_RMM_SDC_TBL_KB > 0 brings the slabs back.
	size_t tblBudget = 8 * 1024;
	bool ldsTables = false;
	if(const char* e = getenv("CLA_RMM_SDC_TBL_KB")) {
		tblBudget = (size_t) std::max(1, atoi(e)) * 1024;
		ldsTables = atoi(e) > 0;
	}
	tblBudget = std::max(tblBudget, maxVals * q * 8);
	tblBudget = std::min(tblBudget, ldsMax - (size_t) tileRows * q * 8);
	// groups per slab: uniform count so that every slab's tables fit
	const size_t slabLen = tblBudget / (maxVals * q * 8);
	if(slabLen < 1) return 1;
	const int nTiles = (int) ((b->nRows + tileRows - 1) / tileRows);
	const int sl = ldsTables ? (int) std::min(slabLen, plan.list.size()) : (int) plan.list.size();
	size_t tblDoubles = 0;
	for(size_t l0 = 0; ldsTables && l0 < plan.list.size(); l0 += sl)
		tblDoubles = std::max(tblDoubles, (size_t) (plan.binOff[std::min(l0 + sl, plan.list.size())] - plan.binOff[l0]) * q);
	const size_t lds = (size_t) tileRows * q * 8 + tblDoubles * 8;
	double algo = (double) b->nRows * q * 8 * (accumulate ? 2 : 1);
	for(int g : plan.list) {
		const DGroup& G = b->groups[g].d;
		algo += (double) G.nDeltas * G.deltaWidth + (double) G.nOffsets * G.codeWidth;
	}
	{
		Prof pf(b, "k_rmm_sdc_tiles", nTiles, ST_THREADS, (long) lds, algo);
		CLA_HIP(hipFuncSetAttribute((const void*) k_rmm_sdc_tiles, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds));
		hipLaunchKernelGGL(k_rmm_sdc_tiles, dim3(nTiles), dim3(ST_THREADS), lds, b->stream, b->dGroups, dList, dBinOff,
			(int) plan.list.size(), sl, b->dTables, q, constRow, accumulate, tileRows, dOut, b->nRows, dNnz, ldsTables ? 1 : 0);
	}
	CLA_HIP(hipGetLastError());
	return 0;
}

} // namespace cla
