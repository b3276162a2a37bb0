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
#include "../../include/cla_hip.h"
#include "cla_device.hpp"
#include <vector>

namespace cla {

__device__ __forceinline__ double agg_identity(int op) {
	return op == CLA_AGG_MIN ? __builtin_inf() : op == CLA_AGG_MAX ? -__builtin_inf() : 0.0;
}
__device__ __forceinline__ double agg_combine(int op, double a, double v) {
	return op == CLA_AGG_MIN ? fmin(a, v) : op == CLA_AGG_MAX ? fmax(a, v) : a + v;
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
// sum sq: sum_k cnt[k] ((d[k,j] + c)^2 - c^2)      (+ nRows c^2 in the finish)
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
			else if(op == CLA_AGG_SUMSQ) a += cnt * ((d + c) * (d + c) - c * c);
			else if(counts[k] > 0) a = agg_combine(op, a, d);
		}
		a = block_reduce(op, a, red);
		if(tid == 0) {
			if(op == CLA_AGG_SUM) unsafeAtomicAdd(&out[G.cols[j]], a); // linear: overlapping groups add up
			else {
				if((op == CLA_AGG_MIN || op == CLA_AGG_MAX) && covered < (double) nRows) a = agg_combine(op, a, 0.0);
				out[G.cols[j]] = a;
			}
		}
	}
}

// grid (row chunks, columns of the group): partial[chunk * nC + j]
// (sum of squares: the column's filtered constant c enters as (v + c)^2 - c^2, like the dictionary form; n c^2 is added at the end)
__global__ __launch_bounds__(256) void k_agg_cols_dense(const double* __restrict__ dense, int64_t nRows, int nC, int64_t rowsPerBlock,
	int op, const int32_t* __restrict__ cols, const double* __restrict__ constV, double* __restrict__ partial) {
	__shared__ double red[4];
	const int j = blockIdx.y;
	const double c = op == CLA_AGG_SUMSQ ? constV[cols[j]] : 0.0;
	const int64_t r0 = (int64_t) blockIdx.x * rowsPerBlock, r1 = min(nRows, r0 + rowsPerBlock);
	double a = agg_identity(op);
	for(int64_t r = r0 + threadIdx.x; r < r1; r += 256) {
		const double v = dense[(size_t) r * nC + j];
		a = op == CLA_AGG_SUMSQ ? a + ((v + c) * (v + c) - c * c) : agg_combine(op, a, v);
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
		else if(op == CLA_AGG_SUMSQ) v += n * k * k;
		else v = touched[c] ? v + k : k;
		if(nRows == 0) v = op == CLA_AGG_MIN || op == CLA_AGG_MAX ? agg_identity(op) : 0.0;
		if(dir == CLA_AGG_COL) { out[c] = v; cnt += v != 0.0; }
		all = agg_combine(op, all, v);
	}
	all = block_reduce(op, all, red);
	if(dir == CLA_AGG_ALL && threadIdx.x == 0) { out[0] = all; cnt = all != 0.0; }
	count_add(nnz, cnt);
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
	if(overlap && op != CLA_AGG_SUM) {
		set_error("aggregate: overlapping column groups support sums only");
		return -CLA_ERR_UNSUPPORTED;
	}
	if(dir == CLA_AGG_ROW) {
		if(op == CLA_AGG_MIN || op == CLA_AGG_MAX) {
			set_error("aggregate: row minima and maxima are not on the device path");
			return -CLA_ERR_UNSUPPORTED;
		}
		if(op == CLA_AGG_SUMSQ && b->hasUnc) {
			set_error("aggregate: row sums of squares with an uncompressed group are not on the device path");
			return -CLA_ERR_UNSUPPORTED;
		}
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
