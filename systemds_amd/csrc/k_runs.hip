// Merged run table of the run-length columns of a block (columns of ColGroupRLE groups whose runs are long):
// all columns' run starts merged into one sorted list of segments, on each of which every such column is constant
// (the reference walks each group's runs per row range, CG/ColGroupRLE.java:104-141; here the row-parallel kernels
// need "which value does column a hold at row r" without a search per row).
//   start[s]            first row of segment s (nSeg + 1 entries, the last = nRows); a column's run that starts where
//                       another's does gives a segment of no rows
//   codes[s * nR + a]   tuple of column a on segment s (-1: no run covers the rows)
//   sliceRec[8 i ..]    per slice of sliceRows rows: segment of its first row, number of run starts inside the slice
//                       (behind its first row), the first six of them (RC_NEVER where there are fewer)
// The place of a run start in the merged order is the number of run starts in front of it, which a thread finds by
// one binary search per other column: no sort.
#include "../../include/cla_hip.h"
#include "cla_runs.hpp"
#include <vector>

namespace cla {

struct MrtCols {
	RunCol c[RC_MAX];
	int32_t first[RC_MAX + 1]; // column a's runs are threads first[a] .. first[a + 1] - 1
	int nR;
};

// number of run starts of the column that are <= row (INCL) or < row
template <bool INCL>
__device__ __forceinline__ int mrt_count(const int32_t* __restrict__ start, int nRuns, int32_t row) {
	int lo = 0, hi = nRuns; // first index whose start is beyond (INCL) / not below the row
	while(lo < hi) {
		const int mid = (lo + hi) >> 1;
		const int32_t s = start[mid];
		if(INCL ? s <= row : s < row) lo = mid + 1; else hi = mid;
	}
	return lo;
}

__global__ __launch_bounds__(256) void k_mrt_segments(const MrtCols M, int32_t* __restrict__ start, int32_t* __restrict__ codes) {
	const int t = blockIdx.x * 256 + threadIdx.x;
	if(t >= M.first[M.nR]) return;
	int a = 0;
	while(t >= M.first[a + 1]) a++;
	const int j = t - M.first[a];
	const int32_t s = as_global(M.c[a].runStart)[j];
	int rank = j;
	int idx[RC_MAX];
	for(int b = 0; b < M.nR; b++) {
		if(b == a) { idx[b] = j; continue; }
		const int32_t* st = as_global(M.c[b].runStart);
		const int le = mrt_count<true>(st, M.c[b].nRuns, s);
		rank += b < a ? le : mrt_count<false>(st, M.c[b].nRuns, s);
		idx[b] = le - 1; // (every column's first run starts at row 0)
	}
	start[rank] = s;
	for(int b = 0; b < M.nR; b++) codes[(size_t) rank * M.nR + b] = as_global(M.c[b].runCode)[idx[b]];
}

__global__ __launch_bounds__(256) void k_mrt_slices(const MrtCols M, int64_t nSlices, int sliceRows, int64_t nRows, const int32_t* __restrict__ start,
	int32_t* __restrict__ sliceRec) {
	const int64_t i = (int64_t) blockIdx.x * 256 + threadIdx.x;
	if(i >= nSlices) return;
	const int32_t row = (int32_t) (i * sliceRows), last = (int32_t) min((i + 1) * sliceRows, nRows) - 1;
	int n0 = 0, n1 = 0;
	for(int b = 0; b < M.nR; b++) {
		n0 += mrt_count<true>(as_global(M.c[b].runStart), M.c[b].nRuns, row);
		n1 += mrt_count<true>(as_global(M.c[b].runStart), M.c[b].nRuns, last);
	}
	int32_t* r = sliceRec + i * 8;
	r[0] = n0 - 1;
	r[1] = n1 - n0;
	for(int k = 0; k < 6; k++) r[2 + k] = k < n1 - n0 ? start[n0 + k] : RC_NEVER;
}

// Per product: sums[s * 16 + j] = constRow[j] + sum over the run-length columns of their value on segment s times
// B[column, j], for the q <= 16 columns of B at hand (columns in list order, one multiply-add each).
__global__ __launch_bounds__(256) void k_run_sums(const MrtCols M, int nSeg, const int32_t* __restrict__ codes, const double* __restrict__ B, int ld,
	int q, const double* __restrict__ constRow, double* __restrict__ sums) {
	// rows of B of the run-length columns and the constant row, once per block
	__shared__ double Bs[(RC_MAX + 1) * 16];
	for(int i = threadIdx.x; i < (RC_MAX + 1) * 16; i += 256) {
		const int a = i >> 4, j = i & 15;
		double v = 0.0;
		if(j < q) {
			if(a < M.nR) v = B[(size_t) M.c[a].col * ld + j];
			else if(a == RC_MAX && constRow != nullptr) v = constRow[j];
		}
		Bs[i] = v;
	}
	__syncthreads();
	// thread = (segment, quarter of the 16 output columns): the segment's values once per thread
	const int64_t t = (int64_t) blockIdx.x * 256 + threadIdx.x;
	const int s = (int) (t >> 2), j0 = (int) (t & 3) * 4;
	if(s >= nSeg) return;
	double val[RC_MAX];
#pragma unroll
	for(int b = 0; b < RC_MAX; b++) {
		val[b] = 0.0;
		if(b < M.nR) {
			const int code = codes[(size_t) s * M.nR + b];
			if(code >= 0) val[b] = as_global(M.c[b].dict)[(size_t) code * M.c[b].nC + M.c[b].h];
		}
	}
	double r[4];
#pragma unroll
	for(int u = 0; u < 4; u++) {
		r[u] = Bs[RC_MAX * 16 + j0 + u];
#pragma unroll
		for(int b = 0; b < RC_MAX; b++)
			if(b < M.nR) r[u] = __builtin_fma(val[b], Bs[b * 16 + j0 + u], r[u]); // (a run without a tuple is a decoded 0, multiplied like any other value)
	}
	double* o = sums + (size_t) s * 16 + j0;
	*(f64x2*) o = f64x2{r[0], r[1]};
	*(f64x2*) (o + 2) = f64x2{r[2], r[3]};
}

static MrtCols mrt_cols(const std::vector<RunCol>& runs) {
	MrtCols M;
	M.nR = (int) runs.size();
	M.first[0] = 0;
	for(int a = 0; a < RC_MAX; a++) {
		if(a < M.nR) M.c[a] = runs[a];
		else M.c[a] = RunCol{nullptr, nullptr, nullptr, 0.0, 0, 1, 0, 0};
		M.first[a + 1] = M.first[a] + (a < M.nR ? runs[a].nRuns : 0);
	}
	return M;
}

// Builds the table for the given columns (device pointers inside) and slices of sliceRows rows.
int mrt_build(cla_block* b, const std::vector<RunCol>& runs, int sliceRows, Mrt& T) {
	T = Mrt();
	if(runs.empty() || runs.size() > (size_t) RC_MAX) return 1;
	const MrtCols M = mrt_cols(runs);
	T.nR = M.nR;
	T.nSeg = M.first[M.nR];
	T.sliceRows = sliceRows;
	T.nSlices = (b->nRows + sliceRows - 1) / sliceRows;
	const size_t startBytes = sizeof(int32_t) * ((size_t) T.nSeg + 1), codeBytes = sizeof(int32_t) * (size_t) T.nSeg * T.nR;
	const size_t sliceBytes = sizeof(int32_t) * 8 * (size_t) T.nSlices, sumBytes = sizeof(double) * 16 * (size_t) T.nSeg;
	auto up = [](size_t n) { return (n + 255) & ~(size_t) 255; };
	uint8_t* d = nullptr;
	CLA_HIP(hipMalloc((void**) &d, up(startBytes) + up(codeBytes) + up(sliceBytes) + up(sumBytes)));
	T.base = d;
	T.bytes = (int64_t) (up(startBytes) + up(codeBytes) + up(sliceBytes) + up(sumBytes));
	T.start = (int32_t*) d;
	T.codes = (int32_t*) (d + up(startBytes));
	T.sliceRec = (int32_t*) (d + up(startBytes) + up(codeBytes));
	T.sums = (double*) (d + up(startBytes) + up(codeBytes) + up(sliceBytes));
	const int32_t nRows32 = (int32_t) b->nRows;
	CLA_HIP(hipMemcpyAsync(T.start + T.nSeg, &nRows32, sizeof(int32_t), hipMemcpyHostToDevice, b->stream));
	CLA_HIP(hipStreamSynchronize(b->stream)); // (the source of the copy is a local)
	{
		Prof pf(b, "k_mrt_segments", (T.nSeg + 255) / 256, 256, 0, 0);
		hipLaunchKernelGGL(k_mrt_segments, dim3((unsigned) ((T.nSeg + 255) / 256)), dim3(256), 0, b->stream, M, T.start, T.codes);
	}
	{
		Prof pf(b, "k_mrt_slices", (long) ((T.nSlices + 255) / 256), 256, 0, 0);
		hipLaunchKernelGGL(k_mrt_slices, dim3((unsigned) ((T.nSlices + 255) / 256)), dim3(256), 0, b->stream, M, T.nSlices, sliceRows, b->nRows, T.start, T.sliceRec);
	}
	CLA_HIP(hipGetLastError());
	return 0;
}

void mrt_free(Mrt& T) {
	if(T.base) (void) hipFree(T.base);
	T = Mrt();
}

// sums of the table for B (q <= 16 columns, row stride ld) and the constant row (may be null)
int launch_run_sums(cla_block* b, const std::vector<RunCol>& runs, const Mrt& T, const double* dB, int ld, int q, const double* dConstRow) {
	const MrtCols M = mrt_cols(runs);
	const int64_t n = (int64_t) T.nSeg * 4;
	Prof pf(b, "k_run_sums", (long) ((n + 255) / 256), 256, 0, 0);
	hipLaunchKernelGGL(k_run_sums, dim3((unsigned) ((n + 255) / 256)), dim3(256), 0, b->stream, M, T.nSeg, T.codes, dB, ld, q, dConstRow, T.sums);
	CLA_HIP(hipGetLastError());
	return 0;
}

} // namespace cla
