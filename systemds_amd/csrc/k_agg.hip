// Unary aggregates of a compressed block (sum, sum of squares, min, max; all cells, per
// row, per column) without decompressing: the column-wise forms come from the exact
// integer counts per dictionary entry (AColGroupCompressed.unaryAggregateOperations,
// CG/AColGroupCompressed.java:137-205: computeColSums / computeColSumsSq / computeColMxx
// over `counts x dictionary`), the row-wise sums from the right-multiply gather with a
// table of per-tuple row aggregates (computeRowSums with a pre-aggregated dictionary,
// CG/AColGroupCompressed.java:71, driver C/lib/CLALibCompAgg.java:78-127, 527-545).
//   k_agg_cols_dict    per dictionary group and column: counts x f(dictionary)
//   k_agg_cols_dense   uncompressed groups: partial column aggregates per row chunk
//   k_agg_finish       constants, untouched columns, reduction over all cells, non-zero count
// What has no such form goes through decompressed row chunks, as the reference's decompressing
// aggregate does (CLALibCompAgg.decompressingAggregate / UAOverlappingTask, C/lib/CLALibCompAgg.java:
// 419-452, 605-720: rows [rl, ru) of all groups into a temporary dense block, then the dense operator):
// everything but sums on overlapping groups (requireDecompression, :220-232), row minima and maxima,
// row sums of squares next to an uncompressed group.
//   k_agg_chunk_rows   one value per row of a decompressed chunk
//   k_agg_chunk_cols   partial column aggregates per 4096 rows of a decompressed chunk
//   k_agg_chunk_finish folds the partials, reduces to one cell for all cells, counts non-zero cells
#include "../../include/cla_hip.h"
#include "cla_device.hpp"
#include <vector>

namespace cla {

__device__ __forceinline__ double agg_identity(int op) {
	return op == CLA_AGG_MIN ? __builtin_inf() : op == CLA_AGG_MAX ? -__builtin_inf() : 0.0;
}
// (min / max as Math.min / Math.max, which the reference's Builtin MIN / MAX use (functionobjects/Builtin.java:259-264,
// 308-312): a NaN operand gives NaN, where fmin / fmax would drop it)
__device__ __forceinline__ double agg_combine(int op, double a, double v) {
	if(op == CLA_AGG_MIN) return a != a || v != v ? __builtin_nan("") : fmin(a, v);
	if(op == CLA_AGG_MAX) return a != a || v != v ? __builtin_nan("") : fmax(a, v);
	return a + v;
}

__device__ __forceinline__ double block_reduce(int op, double v, double* red) {
#pragma unroll
	for(int d = 32; d > 0; d >>= 1) v = agg_combine(op, v, __shfl_down(v, d, WAVE));
	__syncthreads();
	if((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
	__syncthreads();
	double r = red[0];
	for(int w = 1; w < (int) (blockDim.x >> 6); w++) r = agg_combine(op, r, red[w]);
	return r;
}

// block = one dictionary group; c = constant part of the column (SDC default, 0 otherwise).
// sum:    sum_k cnt[k] d[k,j]                      (+ nRows c in the finish)
// sum sq: sum_k cnt[k] (d[k,j] + c)^2 + (nRows - rows with an entry) c^2: terms of one sign, no cancellation
//         where the cells are small next to c
// min/max over entries that occur, and 0 when some row of the group has no entry (+ c in the finish)
__global__ __launch_bounds__(256) void k_agg_cols_dict(const DGroup* __restrict__ groups, const int32_t* __restrict__ countsAll,
	const double* __restrict__ constV, int64_t nRows, int op, double* __restrict__ out) {
	__shared__ double red[4];
	const DGroup G = dgroup(groups + blockIdx.x);
	if(G.type == G_UNC || G.nVals == 0) return;
	const int32_t* counts = countsAll + G.tblOff;
	const int nC = G.nColG, tid = threadIdx.x;
	double covered = 0.0;
	for(int k = tid; k < G.nVals; k += 256) covered += (double) counts[k];
	covered = block_reduce(CLA_AGG_SUM, covered, red);
	for(int j = 0; j < nC; j++) {
		const double c = constV[G.cols[j]];
		double a = agg_identity(op);
		for(int k = tid; k < G.nVals; k += 256) {
			const double cnt = (double) counts[k], d = G.dict[(size_t) k * nC + j];
			if(op == CLA_AGG_SUM) a += cnt * d;
			else if(op == CLA_AGG_SUMSQ) a += cnt * ((d + c) * (d + c));
			else if(counts[k] > 0) a = agg_combine(op, a, d);
		}
		a = block_reduce(op, a, red);
		if(tid == 0) {
			if(op == CLA_AGG_SUM) unsafeAtomicAdd(&out[G.cols[j]], a); // linear: overlapping groups add up
			else {
				if((op == CLA_AGG_MIN || op == CLA_AGG_MAX) && covered < (double) nRows) a = agg_combine(op, a, 0.0);
				if(op == CLA_AGG_SUMSQ) a += ((double) nRows - covered) * (c * c);
				out[G.cols[j]] = a;
			}
		}
	}
}

// grid (row chunks, columns of the group): partial[chunk * nC + j]
// (sum of squares: with the column's filtered constant c, (v + c)^2)
__global__ __launch_bounds__(256) void k_agg_cols_dense(const double* __restrict__ dense, int64_t nRows, int nC, int64_t rowsPerBlock,
	int op, const int32_t* __restrict__ cols, const double* __restrict__ constV, double* __restrict__ partial) {
	__shared__ double red[4];
	const int j = blockIdx.y;
	const double c = op == CLA_AGG_SUMSQ ? constV[cols[j]] : 0.0;
	const int64_t r0 = (int64_t) blockIdx.x * rowsPerBlock, r1 = min(nRows, r0 + rowsPerBlock);
	double a = agg_identity(op);
	for(int64_t r = r0 + threadIdx.x; r < r1; r += 256) {
		const double v = dense[(size_t) r * nC + j];
		a = op == CLA_AGG_SUMSQ ? a + (v + c) * (v + c) : agg_combine(op, a, v);
	}
	a = block_reduce(op, a, red);
	if(threadIdx.x == 0) partial[(size_t) blockIdx.x * nC + j] = a;
}

// one block: folds the partials of an uncompressed group into its columns
__global__ __launch_bounds__(256) void k_agg_cols_dense_fold(const double* __restrict__ partial, int nChunks, int nC,
	const int32_t* __restrict__ cols, int op, double* __restrict__ out) {
	__shared__ double red[4];
	for(int j = 0; j < nC; j++) {
		double a = agg_identity(op);
		for(int i = threadIdx.x; i < nChunks; i += 256) a = agg_combine(op, a, partial[(size_t) i * nC + j]);
		a = block_reduce(op, a, red);
		if(threadIdx.x == 0) {
			if(op == CLA_AGG_SUM) unsafeAtomicAdd(&out[cols[j]], a);
			else out[cols[j]] = a;
		}
	}
}

// one block. touched[c] != 0: column c belongs to a group with row data. Adds the constants,
// gives columns without row data their constant, reduces to one cell for dir == ALL (result
// in out[0] .. there) and counts the non-zero cells of the result.
__global__ __launch_bounds__(256) void k_agg_finish(double* __restrict__ colAgg, const uint8_t* __restrict__ touched,
	const double* __restrict__ constV, int nCols, int64_t nRows, int op, int dir, double* __restrict__ out,
	unsigned long long* __restrict__ nnz) {
	__shared__ double red[4];
	const double n = (double) nRows;
	double all = agg_identity(op);
	int cnt = 0;
	for(int c = threadIdx.x; c < nCols; c += 256) {
		const double k = constV[c];
		double v = colAgg[c];
		if(op == CLA_AGG_SUM) v += n * k;
		else if(op == CLA_AGG_SUMSQ) v = touched[c] ? v : n * k * k;
		else v = touched[c] ? v + k : k;
		if(nRows == 0) v = op == CLA_AGG_MIN || op == CLA_AGG_MAX ? agg_identity(op) : 0.0;
		if(dir == CLA_AGG_COL) { out[c] = v; cnt += v != 0.0; }
		all = agg_combine(op, all, v);
	}
	all = block_reduce(op, all, red);
	if(dir == CLA_AGG_ALL && threadIdx.x == 0) { out[0] = all; cnt = all != 0.0; }
	count_add(nnz, cnt);
}

// ---------------------------------------------------------------------------
// Aggregates of a decompressed chunk of rows (dense, row-major, nCols wide)
// ---------------------------------------------------------------------------
__device__ __forceinline__ double agg_term(int op, double v) { return op == CLA_AGG_SUMSQ ? v * v : v; }

// a wave per row
__global__ __launch_bounds__(256) void k_agg_chunk_rows(const double* __restrict__ dense, int64_t rows, int nCols, int op,
	double* __restrict__ out, unsigned long long* __restrict__ nnz) {
	const int64_t r = (int64_t) blockIdx.x * 4 + (threadIdx.x >> 6);
	const int lane = threadIdx.x & 63;
	int cnt = 0;
	if(r < rows) {
		double a = agg_identity(op);
		for(int c = lane; c < nCols; c += 64) a = agg_combine(op, a, agg_term(op, dense[(size_t) r * nCols + c]));
#pragma unroll
		for(int d = 32; d > 0; d >>= 1) a = agg_combine(op, a, __shfl_down(a, d, WAVE));
		if(lane == 0) { out[r] = a; cnt = a != 0.0; }
	}
	count_add(nnz, cnt);
}

constexpr int AGG_CHUNK_ROWS = 4096;

// block = 4096 rows: a thread keeps one column (of a pass of at most 256 columns) and walks the rows that
// 256 threads do not cover side by side; partial[block * nCols + c]
__global__ __launch_bounds__(256) void k_agg_chunk_cols(const double* __restrict__ dense, int64_t rows, int nCols, int op,
	double* __restrict__ partial) {
	__shared__ double red[256];
	const int tid = threadIdx.x;
	const int64_t rBeg = (int64_t) blockIdx.x * AGG_CHUNK_ROWS, rEnd = min(rows, rBeg + AGG_CHUNK_ROWS);
	const int perPass = min(nCols, 256), side = 256 / perPass;
	const int rr = tid / perPass, cc = tid - rr * perPass;
	for(int cb = 0; cb < nCols; cb += perPass) {
		const int c = cb + cc;
		double a = agg_identity(op);
		if(rr < side && c < nCols)
			for(int64_t r = rBeg + rr; r < rEnd; r += side) a = agg_combine(op, a, agg_term(op, dense[(size_t) r * nCols + c]));
		__syncthreads();
		red[tid] = a;
		__syncthreads();
		if(rr == 0 && c < nCols) {
			for(int k = 1; k < side; k++) a = agg_combine(op, a, red[k * perPass + cc]);
			partial[(size_t) blockIdx.x * nCols + c] = a;
		}
	}
}

// one block
__global__ __launch_bounds__(256) void k_agg_chunk_finish(const double* __restrict__ partial, int nParts, int nCols, int op, int dir,
	double* __restrict__ out, unsigned long long* __restrict__ nnz) {
	__shared__ double red[4];
	double all = agg_identity(op);
	int cnt = 0;
	for(int c = threadIdx.x; c < nCols; c += 256) {
		double v = agg_identity(op);
		for(int i = 0; i < nParts; i++) v = agg_combine(op, v, partial[(size_t) i * nCols + c]);
		if(dir == CLA_AGG_COL) { out[c] = v; cnt += v != 0.0; }
		all = agg_combine(op, all, v);
	}
	all = block_reduce(op, all, red);
	if(dir == CLA_AGG_ALL && threadIdx.x == 0) { out[0] = all; cnt = all != 0.0; }
	count_add(nnz, cnt);
}

// The aggregate of the decompressed block, chunk of rows by chunk of rows (at most 256 MiB decompressed at a time).
static int launch_aggregate_decompressed(cla_block* b, int op, int dir, double* dOut, unsigned long long* dNnz) {
	const int nCols = b->nCols;
	const int64_t nRows = b->nRows;
	hipStream_t st = b->stream;
	clear_stats(b);
	CLA_HIP(hipMemsetAsync(dNnz, 0, sizeof(unsigned long long), st));
	const int64_t chunkRows = std::min<int64_t>(nRows, std::max<int64_t>(AGG_CHUNK_ROWS,
		((int64_t) 256 << 20) / ((int64_t) sizeof(double) * nCols) / AGG_CHUNK_ROWS * AGG_CHUNK_ROWS));
	const int64_t nParts = (nRows + AGG_CHUNK_ROWS - 1) / AGG_CHUNK_ROWS;
	const size_t denseBytes = (sizeof(double) * (size_t) chunkRows * nCols + 255) & ~(size_t) 255;
	const size_t partBytes = dir == CLA_AGG_ROW ? 0 : sizeof(double) * (size_t) nParts * nCols;
	int rc = ensure_scratch(b, denseBytes + partBytes);
	if(rc) return rc;
	double* dDense = (double*) b->dScratch;
	double* dPartial = (double*) ((uint8_t*) b->dScratch + denseBytes);
	for(int64_t r0 = 0; r0 < nRows; r0 += chunkRows) {
		const int64_t r1 = std::min(nRows, r0 + chunkRows), rows = r1 - r0;
		if((rc = launch_decompress_rows(b, r0, r1, dDense))) return rc;
		if(dir == CLA_AGG_ROW) {
			Prof pf(b, "k_agg_chunk_rows", (long) ((rows + 3) / 4), 256, 0, (double) rows * nCols * 8);
			hipLaunchKernelGGL(k_agg_chunk_rows, dim3((unsigned) ((rows + 3) / 4)), dim3(256), 0, st, dDense, rows, nCols, op, dOut + r0, dNnz);
		}
		else {
			const unsigned grid = (unsigned) ((rows + AGG_CHUNK_ROWS - 1) / AGG_CHUNK_ROWS);
			Prof pf(b, "k_agg_chunk_cols", grid, 256, 0, (double) rows * nCols * 8);
			hipLaunchKernelGGL(k_agg_chunk_cols, dim3(grid), dim3(256), 0, st, dDense, rows, nCols, op,
				dPartial + (size_t) (r0 / AGG_CHUNK_ROWS) * nCols);
		}
	}
	if(dir != CLA_AGG_ROW) {
		Prof pf(b, "k_agg_chunk_finish", 1, 256, 0, 0);
		hipLaunchKernelGGL(k_agg_chunk_finish, dim3(1), dim3(256), 0, st, dPartial, (int) nParts, nCols, op, dir, dOut, dNnz);
	}
	CLA_HIP(hipGetLastError());
	return 0;
}

__global__ __launch_bounds__(256) void k_fill(double* __restrict__ p, int64_t n, double v) {
	const int64_t i = (int64_t) blockIdx.x * 256 + threadIdx.x;
	if(i < n) p[i] = v;
}

int ensure_counts(cla_block* b) {
	if(b->dCountsAll != nullptr) return 0;
	int32_t* dc = nullptr;
	CLA_HIP(hipMalloc((void**) &dc, sizeof(int32_t) * (size_t) std::max(b->totalVals, 1)));
	b->derivedBytes += (int64_t) sizeof(int32_t) * std::max(b->totalVals, 1);
	CLA_HIP(hipMemsetAsync(dc, 0, sizeof(int32_t) * (size_t) std::max(b->totalVals, 1), b->stream));
	for(int g = 0; g < (int) b->groups.size(); g++) {
		const int type = b->groups[g].d.type;
		if(type != G_DDC && type != G_SDCZ && type != G_RLE) continue; // no code stream
		const int rc = launch_counts(b, g, dc + b->groups[g].d.tblOff);
		if(rc) { (void) hipFree(dc); return rc; }
	}
	b->dCountsAll = dc;
	return 0;
}

int launch_aggregate(cla_block* b, int op, int dir, double* dOut, unsigned long long* dNnz) {
	const int nG = (int) b->groups.size();
	const int nCols = b->nCols;
	const int64_t nRows = b->nRows;
	hipStream_t st = b->stream;
	if(op < CLA_AGG_SUM || op > CLA_AGG_MAX || dir < CLA_AGG_ALL || dir > CLA_AGG_COL) {
		set_error("aggregate: unknown operation %d / direction %d", op, dir);
		return -CLA_ERR_INVALID;
	}
	// everything but the plain sum needs each cell to come from one group
	std::vector<uint8_t> touched((size_t) std::max(nCols, 1), 0);
	bool overlap = false;
	for(auto& g : b->groups) {
		const bool rowData = g.d.type == G_UNC || g.d.nVals > 0;
		for(int c : g.cols) {
			if(touched[c] && rowData) overlap = true;
			if(rowData) touched[c] = 1;
		}
	}
	if(nRows > 0 && nCols > 0) {
		// (row sums of squares from tables: a tuple's table entry is (d + c)^2 - c^2 under the constant row's c^2, which
		// cancels where an offset list's default c is large against the values; such blocks are decompressed instead)
		bool listOverDefault = false;
		if(op == CLA_AGG_SUMSQ && dir == CLA_AGG_ROW)
			for(auto& g : b->groups)
				if(g.d.type == G_SDCZ && g.d.nOffsets > 0)
					for(int c : g.cols) listOverDefault |= b->constV[c] != 0.0;
		const bool rowNoTable = dir == CLA_AGG_ROW && (op == CLA_AGG_MIN || op == CLA_AGG_MAX || (op == CLA_AGG_SUMSQ && (b->hasUnc || listOverDefault)));
		if((overlap && op != CLA_AGG_SUM) || rowNoTable) return launch_aggregate_decompressed(b, op, dir, dOut, dNnz);
	}
	if(dir == CLA_AGG_ROW) {
		// rowSums(X) = X %*% 1; the squares use per-tuple tables sum_j ((d + c)^2 - c^2) instead of dict x B
		if(b->dOnes == nullptr) {
			CLA_HIP(hipMalloc((void**) &b->dOnes, sizeof(double) * (size_t) std::max(nCols, 1)));
			if(nCols > 0) hipLaunchKernelGGL(k_fill, dim3((unsigned) ((nCols + 255) / 256)), dim3(256), 0, st, b->dOnes, (int64_t) nCols, 1.0);
		}
		return launch_rmm(b, b->dOnes, 1, dOut, dNnz, op == CLA_AGG_SUMSQ ? 1 : 0);
	}
	clear_stats(b);
	CLA_HIP(hipMemsetAsync(dNnz, 0, sizeof(unsigned long long), st));
	int rc = ensure_counts(b);
	if(rc) return rc;
	// scratch: column aggregates | touched flags | partials of one uncompressed group at a time
	const int64_t rowsPerBlock = 64 * 1024;
	const int nChunks = (int) std::max<int64_t>((nRows + rowsPerBlock - 1) / rowsPerBlock, 1);
	int maxDenseCols = 0;
	for(auto& g : b->groups)
		if(g.d.type == G_UNC) maxDenseCols = std::max(maxDenseCols, g.d.nColG);
	const size_t aggBytes = (sizeof(double) * (size_t) std::max(nCols, 1) + 255) & ~(size_t) 255;
	const size_t flagBytes = ((size_t) std::max(nCols, 1) + 255) & ~(size_t) 255;
	if((rc = ensure_scratch(b, aggBytes + flagBytes + sizeof(double) * (size_t) nChunks * std::max(maxDenseCols, 1)))) return rc;
	double* dAgg = (double*) b->dScratch;
	uint8_t* dTouched = (uint8_t*) b->dScratch + aggBytes;
	double* dPartial = (double*) ((uint8_t*) b->dScratch + aggBytes + flagBytes);
	CLA_HIP(hipMemsetAsync(dAgg, 0, aggBytes, st));
	CLA_HIP(hipMemcpyAsync(dTouched, touched.data(), (size_t) std::max(nCols, 1), hipMemcpyHostToDevice, st));
	if(nG > 0 && nRows > 0) {
		Prof pf(b, "k_agg_cols_dict", nG, 256, 0, 0);
		hipLaunchKernelGGL(k_agg_cols_dict, dim3(nG), dim3(256), 0, st, b->dGroups, b->dCountsAll, b->dConstV, nRows, op, dAgg);
	}
	for(int g = 0; g < nG && nRows > 0; g++) {
		const DGroup& G = b->groups[g].d;
		if(G.type != G_UNC) continue;
		Prof pf(b, "k_agg_cols_dense", (long) nChunks * G.nColG, 256, 0, (double) nRows * G.nColG * 8);
		hipLaunchKernelGGL(k_agg_cols_dense, dim3(nChunks, G.nColG), dim3(256), 0, st, G.dense, nRows, G.nColG, rowsPerBlock, op, G.cols, b->dConstV, dPartial);
		hipLaunchKernelGGL(k_agg_cols_dense_fold, dim3(1), dim3(256), 0, st, dPartial, nChunks, G.nColG, G.cols, op, dAgg);
	}
	{
		Prof pf(b, "k_agg_finish", 1, 256, 0, 0);
		hipLaunchKernelGGL(k_agg_finish, dim3(1), dim3(256), 0, st, dAgg, dTouched, b->dConstV, nCols, nRows, op, dir, dOut, dNnz);
	}
	CLA_HIP(hipGetLastError());
	CLA_HIP(hipStreamSynchronize(st)); // `touched` is read by the copy above
	return 0;
}

} // namespace cla
