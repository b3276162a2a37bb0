// Right multiply X %*% B for narrow B (2 <= q <= 16) on blocks of any group mix:
// every thread decodes one row of X group by group (dictionary copies in LDS) and
// accumulates value x B[col, :] with B rows as scalar operands. Codes, offset lists,
// runs and dense columns are read once, the output tile is staged in LDS and written
// with full-line stores. (Wide B on all-DDC blocks uses k_rmm_mfma instead.)
#include "../../include/cla_hip.h"
#include "cla_device.hpp"
#include <algorithm>

namespace cla {

constexpr int DEC_THREADS = 512;       // rows per half tile, one row per thread
constexpr int DEC_TILE = SDC_TILE;     // rows per tile = granularity of the offset tile index
constexpr int DEC_QMAX = 16;

struct DecPlan {
	int32_t dictOff;   // offset (doubles) of the group's dictionary copy in LDS, -1 = not dictionary coded
	int32_t sdcSlot;   // SDCZeros: index of the group's code tile in LDS, else -1
};

template <int Q>
__global__ __launch_bounds__(DEC_THREADS) void k_rmm_decode(const DGroup* __restrict__ groups, int nGroups,
	const DecPlan* __restrict__ plan, int dictDoubles, int nSdc, const double* __restrict__ B, int q,
	const double* __restrict__ constRow, double* __restrict__ out, int64_t nRows, unsigned long long* __restrict__ nnz) {
	extern __shared__ double smem[];
	double* dictS = smem;                                   // dictDoubles
	double* otile = dictS + dictDoubles;                    // DEC_THREADS * Q (padded row stride Q + 1 when Q even)
	int32_t* sdcCodes = (int32_t*) (otile + (size_t) DEC_THREADS * (Q + 1)); // nSdc * DEC_TILE
	int32_t* runBase = sdcCodes + (size_t) nSdc * DEC_TILE; // nGroups
	const int tid = threadIdx.x, wave = tid >> 6;
	constexpr int OS = Q + 1; // LDS row stride of the output tile (odd: conflict-free column access)

	// dictionary copies, once per block
	for(int g = 0; g < nGroups; g++) {
		const int off = plan[g].dictOff;
		if(off < 0) continue;
		const DGroup& G = groups[g];
		const int n = G.nVals * G.nColG;
		for(int i = tid; i < n; i += DEC_THREADS) dictS[off + i] = G.dict[i];
	}
	double cadd[Q];
#pragma unroll
	for(int c = 0; c < Q; c++) cadd[c] = (constRow != nullptr && c < q) ? constRow[c] : 0.0;

	const int nTiles = (int) ((nRows + DEC_TILE - 1) / DEC_TILE);
	int cnt = 0;
	for(int tile = blockIdx.x; tile < nTiles; tile += gridDim.x) {
		const int64_t t0 = (int64_t) tile * DEC_TILE;
		__syncthreads();
		for(int i = tid; i < nSdc * DEC_TILE; i += DEC_THREADS) sdcCodes[i] = -1;
		// one binary search per RLE group and tile
		for(int g = tid; g < nGroups; g += DEC_THREADS)
			if(groups[g].type == G_RLE) runBase[g] = rle_find(groups[g].runStart, groups[g].nRuns, (int32_t) t0);
		__syncthreads();
		// SDCZeros lists of this tile -> per-row codes in LDS (one wave per group)
		for(int g = wave; g < nGroups; g += DEC_THREADS / 64) {
			const int slot = plan[g].sdcSlot;
			if(slot < 0) continue;
			const DGroup& G = groups[g];
			if(G.nOffsets <= 0) continue;
			int32_t* ct = sdcCodes + (size_t) slot * DEC_TILE;
			const int64_t rEnd = t0 + DEC_TILE;
			if((tid & 63) == 0 && G.first >= t0 && G.first < rEnd) ct[G.first - t0] = load_code(G.codes, G.codeWidth, 0);
			if(tile < G.nTiles) {
				const OffState st = G.tileIdx[tile];
				int32_t row = st.row, emit = st.emit;
				int64_t i0 = st.idx;
				while(i0 < G.nDeltas && row < rEnd) {
					int32_t rows[4], didx[4];
					unsigned mask;
					if(G.deltaWidth == 1) sdc_decode256<1>(G.deltas, G.nDeltas, i0, row, emit, rows, didx, mask);
					else sdc_decode256<2>(G.deltas, G.nDeltas, i0, row, emit, rows, didx, mask);
#pragma unroll
					for(int k = 0; k < 4; k++)
						if((mask & (1u << k)) && rows[k] < rEnd) ct[rows[k] - t0] = load_code(G.codes, G.codeWidth, didx[k]);
					i0 += 256;
				}
			}
		}
		__syncthreads();
		for(int half = 0; half < DEC_TILE / DEC_THREADS; half++) {
			const int rt = half * DEC_THREADS + tid; // row inside the tile
			const int64_t r = t0 + rt;
			double acc[Q];
#pragma unroll
			for(int c = 0; c < Q; c++) acc[c] = 0.0;
			if(r < nRows) {
				for(int g = 0; g < nGroups; g++) {
					const DGroup& G = groups[g];
					const int nC = G.nColG;
					const double* vals = nullptr;
					if(G.type == G_DDC) vals = dictS + plan[g].dictOff + (size_t) load_code(G.codes, G.codeWidth, r) * nC;
					else if(G.type == G_RLE) {
						int j = runBase[g];
						while(G.runStart[j + 1] <= r) j++;
						const int code = G.runCode[j];
						if(code >= 0) vals = dictS + plan[g].dictOff + (size_t) code * nC;
					}
					else if(G.type == G_SDCZ) {
						const int code = sdcCodes[(size_t) plan[g].sdcSlot * DEC_TILE + rt];
						if(code >= 0) vals = dictS + plan[g].dictOff + (size_t) code * nC;
					}
					else
						vals = G.dense + (size_t) r * nC;
					if(vals == nullptr) continue;
					for(int h = 0; h < nC; h++) {
						const double a = vals[h];
						const double* brow = B + (size_t) G.cols[h] * q; // uniform: scalar loads
#pragma unroll
						for(int c = 0; c < Q; c++)
							if(c < q) acc[c] += a * brow[c];
					}
				}
			}
			__syncthreads(); // previous half's stores have read the tile
#pragma unroll
			for(int c = 0; c < Q; c++) otile[tid * OS + c] = acc[c] + cadd[c];
			__syncthreads();
			// coalesced write of the half tile: rows [t0 + half*DEC_THREADS, +DEC_THREADS) x q
			const int64_t rowBase = t0 + (int64_t) half * DEC_THREADS;
			const int nr = (int) max((int64_t) 0, min((int64_t) DEC_THREADS, nRows - rowBase));
			for(int i = tid; i < nr * q; i += DEC_THREADS) {
				const int rr = i / q, c = i - rr * q;
				const double v = otile[rr * OS + c];
				cnt += v != 0.0;
				__builtin_nontemporal_store(v, out + (size_t) rowBase * q + i);
			}
		}
	}
	count_add(nnz, cnt);
}

// Returns 1 when the block/shape is not eligible (caller uses the generic path).
int launch_rmm_decode(cla_block* b, const double* dB, int q, const double* dConstRow, double* dOut,
	unsigned long long* dNnz) {
	const int nG = (int) b->groups.size();
	if(nG == 0 || b->nRows == 0 || q < 2 || q > DEC_QMAX) return 1;
	std::vector<DecPlan> plan((size_t) nG);
	size_t dictD = 0;
	int nSdc = 0;
	for(int g = 0; g < nG; g++) {
		const DGroup& G = b->groups[g].d;
		plan[g].dictOff = -1; plan[g].sdcSlot = -1;
		if(G.type == G_UNC) continue;
		plan[g].dictOff = (int32_t) dictD;
		dictD += (size_t) G.nVals * G.nColG;
		if(G.type == G_SDCZ) plan[g].sdcSlot = nSdc++;
	}
	const int Q = q <= 4 ? 4 : q <= 8 ? 8 : q <= 12 ? 12 : 16;
	const size_t lds = dictD * 8 + (size_t) DEC_THREADS * (Q + 1) * 8 + (size_t) nSdc * DEC_TILE * 4 + (size_t) nG * 4 + 64;
	if(lds > (size_t) std::min(g_ldsPerBlock, 160 * 1024) - 1024) return 1;
	int rc = ensure_scratch(b, plan.size() * sizeof(DecPlan) + 64);
	if(rc) return rc;
	DecPlan* dPlan = (DecPlan*) b->dScratch;
	CLA_HIP(hipMemcpyAsync(dPlan, plan.data(), plan.size() * sizeof(DecPlan), hipMemcpyHostToDevice, b->stream));
	CLA_HIP(hipStreamSynchronize(b->stream));
	const int nTiles = (int) ((b->nRows + DEC_TILE - 1) / DEC_TILE);
	const int blocksPerCU = lds <= 76 * 1024 ? 2 : 1;
	const unsigned grid = (unsigned) std::min(nTiles, g_numCU * blocksPerCU);
	double algo = (double) b->device_bytes_cached + (double) b->nRows * q * 8;
	Prof pf(b, "k_rmm_decode", grid, DEC_THREADS, (long) lds, algo);
#define DEC_LAUNCH(QV)                                                                                          \
	do {                                                                                                        \
		CLA_HIP(hipFuncSetAttribute((const void*) k_rmm_decode<QV>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds)); \
		hipLaunchKernelGGL(k_rmm_decode<QV>, dim3(grid), dim3(DEC_THREADS), lds, b->stream, b->dGroups, nG, dPlan, (int) dictD, \
			nSdc, dB, q, dConstRow, dOut, b->nRows, dNnz);                                                      \
	} while(0)
	if(Q == 4) DEC_LAUNCH(4);
	else if(Q == 8) DEC_LAUNCH(8);
	else if(Q == 12) DEC_LAUNCH(12);
	else DEC_LAUNCH(16);
#undef DEC_LAUNCH
	CLA_HIP(hipGetLastError());
	return 0;
}

} // namespace cla
