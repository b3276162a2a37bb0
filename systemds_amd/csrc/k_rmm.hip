// Right multiply X %*% B on a compressed block (gfx950).
//
//   k_preagg          T_g = dict_g x B[cols_g, :]   (Dictionary.preaggValuesFromDense)
//   k_rmm_q1_ddc      row-parallel gather-accumulate for mat-vec, tables in LDS
//   k_rmm_rows        generic row-parallel gather for any q / DDC, RLE, uncompressed
//   k_rmm_sdc_scatter offset-list scatter for SDCZeros groups
//   k_count_nnz       non-zero count of the result
#include "../../include/cla_hip.h"
#include "cla_device.hpp"

namespace cla {

// ---------------------------------------------------------------------------
// K1: per group dictionary x B pre-aggregation. One thread per (tuple k, output
// column c). Products and sums are rounded separately (no FMA) in column order
// h, and zero dictionary cells are skipped, as the reference does, so the
// tables are bit-identical to a scalar CPU evaluation.
// grid.y = group index; grid.y == nGroups computes constV x B.
// ---------------------------------------------------------------------------
__global__ void k_preagg(const DGroup* __restrict__ groups, int nGroups, const double* __restrict__ B, int q,
	int nCols, const double* __restrict__ constV, double* __restrict__ T, int totalVals) {
	const int g = blockIdx.y;
	const int idx = blockIdx.x * blockDim.x + threadIdx.x;
	if(g == nGroups) {
		if(constV == nullptr || idx >= q) return;
		double acc = 0;
		for(int c0 = 0; c0 < nCols; c0++) {
			const double a = constV[c0];
			if(a != 0) acc = __dadd_rn(acc, __dmul_rn(a, B[(size_t) c0 * q + idx]));
		}
		T[(size_t) totalVals * q + idx] = acc;
		return;
	}
	const DGroup G = groups[g];
	if(G.type == G_UNC || idx >= G.nVals * q) return;
	const int k = idx / q, c = idx - k * q;
	double acc = 0;
	for(int h = 0; h < G.nColG; h++) {
		const double v = G.dict[(size_t) k * G.nColG + h];
		if(v != 0) acc = __dadd_rn(acc, __dmul_rn(v, B[(size_t) G.cols[h] * q + c]));
	}
	T[(size_t) (G.tblOff + k) * q + c] = acc;
}

// ---------------------------------------------------------------------------
// K2 (mat-vec): all groups DDC with the same code width CW.
// A thread owns RPT = 16 consecutive rows and keeps their sums in registers;
// the pre-aggregated tables of a slab of groups are staged in LDS. Code streams
// are read with 16-byte loads (a wave reads 1 KiB x CW contiguous per group),
// NB groups in flight per thread. Groups are visited in list order, so every
// output cell is summed in the same order as the CPU algorithm.
// ---------------------------------------------------------------------------
template <int CW>
struct CodeVec;
template <>
struct CodeVec<1> {
	uint4 v;
	__device__ __forceinline__ void load(const void* codes, int64_t row0) { v = *(const uint4*) ((const uint8_t*) codes + row0); }
	__device__ __forceinline__ int get(int i) const {
		const uint32_t w = i < 4 ? v.x : i < 8 ? v.y : i < 12 ? v.z : v.w;
		return (w >> (8 * (i & 3))) & 0xffu;
	}
};
template <>
struct CodeVec<2> {
	uint4 v[2];
	__device__ __forceinline__ void load(const void* codes, int64_t row0) {
		const uint4* p = (const uint4*) ((const uint16_t*) codes + row0);
		v[0] = p[0]; v[1] = p[1];
	}
	__device__ __forceinline__ int get(int i) const {
		const uint4 q = v[i >> 3];
		const int j = i & 7;
		const uint32_t w = j < 2 ? q.x : j < 4 ? q.y : j < 6 ? q.z : q.w;
		return (w >> (16 * (j & 1))) & 0xffffu;
	}
};
template <>
struct CodeVec<4> {
	uint4 v[4];
	__device__ __forceinline__ void load(const void* codes, int64_t row0) {
		const uint4* p = (const uint4*) ((const int32_t*) codes + row0);
		v[0] = p[0]; v[1] = p[1]; v[2] = p[2]; v[3] = p[3];
	}
	__device__ __forceinline__ int get(int i) const {
		const uint4 q = v[i >> 2];
		const int j = i & 3;
		return (int) (j == 0 ? q.x : j == 1 ? q.y : j == 2 ? q.z : q.w);
	}
};

constexpr int Q1_RPT = 16;

template <int CW, int THREADS>
__global__ __launch_bounds__(THREADS) void k_rmm_q1_ddc(const DGroup* __restrict__ groups,
	const int32_t* __restrict__ slabStart, int nSlabs, const double* __restrict__ T, int constIdx,
	double* __restrict__ out, int64_t nRows, unsigned long long* __restrict__ nnz) {
	extern __shared__ double tbl[];
	constexpr int NB = CW == 1 ? 8 : CW == 2 ? 4 : 2;
	const int tid = threadIdx.x;
	const int64_t row0 = ((int64_t) blockIdx.x * THREADS + tid) * Q1_RPT;
	const bool full = row0 + Q1_RPT <= nRows;
	const bool any = row0 < nRows;
	double acc[Q1_RPT];
#pragma unroll
	for(int i = 0; i < Q1_RPT; i++) acc[i] = 0.0;

	for(int s = 0; s < nSlabs; s++) {
		const int g0 = slabStart[s], g1 = slabStart[s + 1];
		const int t0 = groups[g0].tblOff;
		const int t1 = groups[g1 - 1].tblOff + groups[g1 - 1].nVals;
		__syncthreads();
		for(int i = tid; i < t1 - t0; i += THREADS) tbl[i] = T[t0 + i];
		__syncthreads();
		if(full) {
			int g = g0;
			for(; g + NB <= g1; g += NB) {
				CodeVec<CW> cv[NB];
#pragma unroll
				for(int j = 0; j < NB; j++) cv[j].load(groups[g + j].codes, row0);
#pragma unroll
				for(int j = 0; j < NB; j++) {
					const double* t = tbl + (groups[g + j].tblOff - t0);
#pragma unroll
					for(int i = 0; i < Q1_RPT; i++) acc[i] += t[cv[j].get(i)];
				}
			}
			for(; g < g1; g++) {
				CodeVec<CW> cv;
				cv.load(groups[g].codes, row0);
				const double* t = tbl + (groups[g].tblOff - t0);
#pragma unroll
				for(int i = 0; i < Q1_RPT; i++) acc[i] += t[cv.get(i)];
			}
		}
		else if(any) {
			for(int g = g0; g < g1; g++) {
				const double* t = tbl + (groups[g].tblOff - t0);
				const void* codes = groups[g].codes;
#pragma unroll
				for(int i = 0; i < Q1_RPT; i++)
					if(row0 + i < nRows) acc[i] += t[load_code(codes, CW, row0 + i)];
			}
		}
	}

	int cnt = 0;
	if(any) {
		const double cadd = constIdx >= 0 ? T[constIdx] : 0.0;
		if(constIdx >= 0) {
#pragma unroll
			for(int i = 0; i < Q1_RPT; i++) acc[i] += cadd;
		}
		if(full) {
#pragma unroll
			for(int i = 0; i < Q1_RPT; i += 2) {
				cnt += (acc[i] != 0.0) + (acc[i + 1] != 0.0);
				*(double2*) (out + row0 + i) = make_double2(acc[i], acc[i + 1]);
			}
		}
		else {
#pragma unroll
			for(int i = 0; i < Q1_RPT; i++)
				if(row0 + i < nRows) { cnt += acc[i] != 0.0; out[row0 + i] = acc[i]; }
		}
	}
	count_add(nnz, cnt);
}

// ---------------------------------------------------------------------------
// Generic row-parallel gather: one thread per output cell (r, c), groups in list
// order; handles DDC, RLE (merged run table) and uncompressed groups. SDCZeros
// groups are added afterwards by k_rmm_sdc_scatter.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_rmm_rows(const DGroup* __restrict__ groups, int nGroups,
	const double* __restrict__ T, const double* __restrict__ B, int q, int constRow, double* __restrict__ out,
	int64_t nRows) {
	const int64_t idx = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
	if(idx >= nRows * q) return;
	const int64_t r = idx / q;
	const int c = (int) (idx - r * q);
	double acc = 0.0;
	for(int g = 0; g < nGroups; g++) {
		const DGroup& G = groups[g];
		if(G.type == G_DDC) {
			const int code = load_code(G.codes, G.codeWidth, r);
			acc += T[(size_t) (G.tblOff + code) * q + c];
		}
		else if(G.type == G_RLE) {
			const int code = G.runCode[rle_find(G.runStart, G.nRuns, (int32_t) r)];
			if(code >= 0) acc += T[(size_t) (G.tblOff + code) * q + c];
		}
		else if(G.type == G_UNC) {
			double s = 0.0;
			for(int h = 0; h < G.nColG; h++) {
				const double a = G.dense[(size_t) r * G.nColG + h];
				if(a != 0) s = __dadd_rn(s, __dmul_rn(a, B[(size_t) G.cols[h] * q + c]));
			}
			acc += s;
		}
	}
	if(constRow >= 0) acc += T[(size_t) constRow * q + c];
	out[idx] = acc;
}

// One block per chunk of SDC_CK delta entries of one SDCZeros group: decode the
// rows with a wave prefix sum and add the group's table row to the output rows.
template <int W>
__global__ __launch_bounds__(256) void k_rmm_sdc_scatter(const DGroup* __restrict__ groups, int g,
	const double* __restrict__ T, int q, double* __restrict__ out) {
	const DGroup& G = groups[g];
	const int chunk = blockIdx.x;
	const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
	const double* Tg = T + (size_t) G.tblOff * q;
	if(chunk == 0 && threadIdx.x == 0 && G.nOffsets > 0) {
		const int code = load_code(G.codes, G.codeWidth, 0);
		for(int c = 0; c < q; c++) unsafeAtomicAdd(out + (size_t) G.first * q + c, Tg[(size_t) code * q + c]);
	}
	if(chunk >= G.nCkpt) return;
	const OffState st = G.ckpt[chunk];
	// each wave decodes its 256 entries; it first needs the state behind the
	// preceding waves' entries, so waves w > 0 re-scan the preceding 256-entry
	// pieces (at most three).
	int32_t row = st.row, emit = st.emit;
	int32_t rows[4], didx[4];
	unsigned mask;
	const int64_t base = (int64_t) chunk * SDC_CK;
	for(int w = 0; w < wave; w++) sdc_decode256<W>(G.deltas, G.nDeltas, base + w * 256, row, emit, rows, didx, mask);
	sdc_decode256<W>(G.deltas, G.nDeltas, base + wave * 256, row, emit, rows, didx, mask);
	(void) lane;
#pragma unroll
	for(int k = 0; k < 4; k++) {
		if(mask & (1u << k)) {
			const int code = load_code(G.codes, G.codeWidth, didx[k]);
			for(int c = 0; c < q; c++) unsafeAtomicAdd(out + (size_t) rows[k] * q + c, Tg[(size_t) code * q + c]);
		}
	}
}

__global__ __launch_bounds__(256) void k_count_nnz(const double* __restrict__ x, int64_t n,
	unsigned long long* __restrict__ nnz) {
	int cnt = 0;
	for(int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t) gridDim.x * blockDim.x)
		cnt += x[i] != 0.0;
	count_add(nnz, cnt);
}

int launch_rmm(cla_block* b, const double* dB, int q, double* dOut, unsigned long long* dNnz) {
	const int nG = (int) b->groups.size();
	const int64_t nRows = b->nRows;
	hipStream_t st = b->stream;
	clear_stats(b);
	int rc = ensure_tables(b, (size_t) (b->totalVals + 1) * q);
	if(rc) return rc;
	CLA_HIP(hipMemsetAsync(dNnz, 0, sizeof(unsigned long long), st));

	// K1
	{
		const int maxWork = (b->maxVals > 1 ? b->maxVals : 1) * q;
		dim3 grid((maxWork + 255) / 256 > (q + 255) / 256 ? (maxWork + 255) / 256 : (q + 255) / 256, nG + 1);
		Prof pf(b, "k_preagg", (long) grid.x * grid.y, 256, 0, 0);
		hipLaunchKernelGGL(k_preagg, grid, dim3(256), 0, st, b->dGroups, nG, dB, q, b->nCols,
			b->hasConst ? b->dConstV : nullptr, b->dTables, b->totalVals);
	}
	const int constRow = b->hasConst ? b->totalVals : -1;
	if(nRows == 0) return 0;

	bool allDdc = nG > 0;
	int cw = nG > 0 ? b->groups[0].d.codeWidth : 0;
	for(auto& g : b->groups)
		if(g.d.type != G_DDC || g.d.codeWidth != cw) allDdc = false;

	if(q == 1 && allDdc && b->slabLdsBytes > 0) {
		constexpr int THREADS = 256;
		const int64_t rowsPerBlock = (int64_t) THREADS * Q1_RPT;
		const unsigned grid = (unsigned) ((nRows + rowsPerBlock - 1) / rowsPerBlock);
		const int nSlabs = (int) b->slabStart.size() - 1;
		const size_t lds = (size_t) b->slabLdsBytes;
		double codeBytes = 0;
		for(auto& g : b->groups) codeBytes += (double) nRows * g.d.codeWidth;
		const double bytes = codeBytes + (double) nRows * 8 + (double) b->totalVals * 8;
#define LAUNCH_Q1(CWV)                                                                                          \
	do {                                                                                                        \
		auto kern = k_rmm_q1_ddc<CWV, THREADS>;                                                                 \
		CLA_HIP(hipFuncSetAttribute((const void*) kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds)); \
		hipLaunchKernelGGL(kern, dim3(grid), dim3(THREADS), lds, st, b->dGroups, b->dSlabStart, nSlabs,         \
			b->dTables, constRow, dOut, nRows, dNnz);                                                           \
	} while(0)
		{
			Prof pf(b, "k_rmm_q1_ddc", grid, THREADS, (long) lds, bytes);
			if(cw == 1) LAUNCH_Q1(1);
			else if(cw == 2) LAUNCH_Q1(2);
			else LAUNCH_Q1(4);
		}
#undef LAUNCH_Q1
		CLA_HIP(hipGetLastError());
		return 0;
	}

	// generic path
	{
		const int64_t n = nRows * q;
		const unsigned grid = (unsigned) ((n + 255) / 256);
		{
			Prof pf(b, "k_rmm_rows", grid, 256, 0, 0);
			hipLaunchKernelGGL(k_rmm_rows, dim3(grid), dim3(256), 0, st, b->dGroups, nG, b->dTables, dB, q, constRow,
				dOut, nRows);
		}
		for(int g = 0; g < nG; g++) {
			const DGroup& G = b->groups[g].d;
			if(G.type != G_SDCZ || G.nOffsets == 0) continue;
			const unsigned sg = (unsigned) (G.nCkpt > 1 ? G.nCkpt : 1);
			Prof pf(b, "k_rmm_sdc_scatter", sg, 256, 0, 0);
			if(G.deltaWidth == 1)
				hipLaunchKernelGGL(k_rmm_sdc_scatter<1>, dim3(sg), dim3(256), 0, st, b->dGroups, g, b->dTables, q, dOut);
			else
				hipLaunchKernelGGL(k_rmm_sdc_scatter<2>, dim3(sg), dim3(256), 0, st, b->dGroups, g, b->dTables, q, dOut);
		}
		const unsigned cg = (unsigned) ((n + 256 * 8 - 1) / (256 * 8));
		Prof pf(b, "k_count_nnz", cg, 256, 0, 0);
		hipLaunchKernelGGL(k_count_nnz, dim3(cg > 65535 * 16 ? 65535 * 16 : cg), dim3(256), 0, st, dOut, n, dNnz);
	}
	CLA_HIP(hipGetLastError());
	return 0;
}

} // namespace cla
