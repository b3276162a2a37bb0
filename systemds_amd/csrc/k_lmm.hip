// Left multiply Y %*% X on a compressed block (gfx950).
//
//   k_lmm_preagg_rows   per-code aggregation of Y over DDC / RLE groups (row parallel),
//                       block-private fp64 bins in LDS, flushed with global atomics
//   k_lmm_preagg_sdc    the same for SDCZeros groups, parallel over offset-list chunks
//   k_lmm_unc           uncompressed groups: Y %*% U on the matrix cores
//   k_lmm_rowsum        rowSums(Y) for the constant correction
//   k_lmm_post          preAgg x dictionary into the output columns
//   k_lmm_finish        + rowSum (x) constV, non-zero count
#include "../../include/cla_hip.h"
#include "cla_device.hpp"

namespace cla {

constexpr int LMM_RPT = 16;        // rows per thread
constexpr int LMM_THREADS = 256;
constexpr int LMM_BIN_BYTES = 32 * 1024;

// Slab = consecutive groups [g0, g1) whose bins fit LDS; binOff[g - g0] = offset of
// the group's bins inside the LDS slab. One block covers `rowsPerBlock` rows.
__global__ __launch_bounds__(LMM_THREADS) void k_lmm_preagg_rows(const DGroup* __restrict__ groups, int g0, int g1,
	const double* __restrict__ Y, int64_t nRows, int64_t rowsPerBlock, double* __restrict__ pre, int totalVals,
	int direct) {
	// direct != 0: the group's bins do not fit LDS, aggregate straight into `pre` in HBM
	extern __shared__ double ldsBins[];
	const int i = blockIdx.y; // row of Y
	const int base = groups[g0].tblOff;
	const int nBins = groups[g1 - 1].tblOff + groups[g1 - 1].nVals - base;
	double* bins = direct ? pre + (size_t) i * totalVals + base : ldsBins;
	if(!direct) {
		for(int k = threadIdx.x; k < nBins; k += LMM_THREADS) bins[k] = 0.0;
		__syncthreads();
	}
	const double* y = Y + (size_t) i * nRows;
	const int64_t rb = (int64_t) blockIdx.x * rowsPerBlock;
	const int64_t re = min(rb + rowsPerBlock, nRows);
	for(int64_t r0 = rb + (int64_t) threadIdx.x * LMM_RPT; r0 < re; r0 += (int64_t) LMM_THREADS * LMM_RPT) {
		const int n = (int) min((int64_t) LMM_RPT, re - r0);
		double yv[LMM_RPT];
#pragma unroll
		for(int t = 0; t < LMM_RPT; t++) yv[t] = t < n ? y[r0 + t] : 0.0;
		for(int g = g0; g < g1; g++) {
			const DGroup G = dgroup(groups + (g));
			double* bg = bins + (G.tblOff - base);
			if(G.type == G_DDC) {
				if(n == LMM_RPT && G.codeWidth == 1) {
					const uint4 c = *(const uint4*) ((const uint8_t*) G.codes + r0);
					const uint32_t w[4] = {c.x, c.y, c.z, c.w};
#pragma unroll
					for(int t = 0; t < LMM_RPT; t++) unsafeAtomicAdd(&bg[(w[t >> 2] >> (8 * (t & 3))) & 0xff], yv[t]);
				}
				else {
					for(int t = 0; t < n; t++) unsafeAtomicAdd(&bg[load_code(G.codes, G.codeWidth, r0 + t)], yv[t]);
				}
			}
			else if(G.type == G_RLE) {
				// walk the merged run table, adding each run's partial sum once
				int j = rle_find(G.runStart, G.nRuns, (int32_t) r0);
				int t = 0;
				while(t < n) {
					const int64_t runEnd = G.runStart[j + 1];
					const int code = G.runCode[j];
					double s = 0.0;
					while(t < n && r0 + t < runEnd) s += yv[t++];
					if(code >= 0) unsafeAtomicAdd(&bg[code], s);
					j++;
				}
			}
		}
	}
	if(direct) return;
	__syncthreads();
	double* dst = pre + (size_t) i * totalVals + base;
	for(int k = threadIdx.x; k < nBins; k += LMM_THREADS) {
		const double v = bins[k];
		if(v != 0.0) unsafeAtomicAdd(&dst[k], v);
	}
}

// SDCZeros: one block walks `chunksPerBlock` chunks of SDC_CK offset entries of one
// group; bins[code] += Y[i, row].
template <int W>
__global__ __launch_bounds__(256) void k_lmm_preagg_sdc(const DGroup* __restrict__ groups, int g, const double* __restrict__ Y,
	int64_t nRows, int chunksPerBlock, double* __restrict__ pre, int totalVals, int direct) {
	extern __shared__ double ldsBins[];
	const DGroup G = dgroup(groups + (g));
	const int i = blockIdx.y;
	const double* y = Y + (size_t) i * nRows;
	double* bins = direct ? pre + (size_t) i * totalVals + G.tblOff : ldsBins;
	if(!direct) {
		for(int k = threadIdx.x; k < G.nVals; k += 256) bins[k] = 0.0;
		__syncthreads();
	}
	if(blockIdx.x == 0 && threadIdx.x == 0 && G.nOffsets > 0)
		unsafeAtomicAdd(&bins[load_code(G.codes, G.codeWidth, 0)], y[G.first]);
	const int wave = threadIdx.x >> 6;
	const int c0 = blockIdx.x * chunksPerBlock;
	const int c1 = min(c0 + chunksPerBlock, G.nCkpt);
	for(int c = c0; c < c1; c++) {
		const OffState st = G.ckpt[c];
		int32_t row = st.row, emit = st.emit;
		int32_t rows[4], didx[4];
		unsigned mask;
		const int64_t base = (int64_t) c * SDC_CK;
		for(int w = 0; w < wave; w++) sdc_decode256<W>(G.deltas, G.nDeltas, base + w * 256, row, emit, rows, didx, mask);
		sdc_decode256<W>(G.deltas, G.nDeltas, base + wave * 256, row, emit, rows, didx, mask);
#pragma unroll
		for(int k = 0; k < 4; k++)
			if(mask & (1u << k)) unsafeAtomicAdd(&bins[load_code(G.codes, G.codeWidth, didx[k])], y[rows[k]]);
	}
	if(direct) return;
	__syncthreads();
	double* dst = pre + (size_t) i * totalVals + G.tblOff;
	for(int k = threadIdx.x; k < G.nVals; k += 256) {
		const double v = bins[k];
		if(v != 0.0) unsafeAtomicAdd(&dst[k], v);
	}
}

// uncompressed group: out[i, cols[j]] += sum_r Y[i,r] * U[r,j] on v_mfma_f64_16x16x4_f64. Block = (range of rows,
// 16 rows of Y, LU_NBJ blocks of 16 columns of the group); wave w takes rows 4 w .. 4 w + 3 of every 16; lane
// (k4, i16) holds Y[16 ib + i16, row k4] and U[row k4, 16 jb + i16]. The group is read once per 16 rows of Y, in
// pieces of 128 bytes per row (the scalar form it replaces read it once per row of Y and column: 1.6 ms per row of Y
// on 1M rows x 90 columns).
constexpr int LU_NBJ = 4;
typedef double lu_f64x4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void k_lmm_unc(const DGroup* __restrict__ groups, int g, const double* __restrict__ Y, int p,
	int64_t nRows, int64_t rowsPerBlock, double* __restrict__ out, int nCols) {
	__shared__ double red[LU_NBJ * 256];
	const DGroup G = dgroup(groups + (g));
	const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
	const int i16 = lane & 15, k4 = lane >> 4;
	const int nC = G.nColG, nb = (nC + 15) / 16;
	const int ib = blockIdx.y, jb0 = blockIdx.z * LU_NBJ;
	const int nj = min(LU_NBJ, nb - jb0);
	const int yi = ib * 16 + i16;
	const bool yIn = yi < p;
	const double* y = as_global(Y) + (size_t) (yIn ? yi : 0) * nRows;
	const int64_t r0 = (int64_t) blockIdx.x * rowsPerBlock, r1 = min(nRows, r0 + rowsPerBlock);
	lu_f64x4 acc[LU_NBJ];
#pragma unroll
	for(int j = 0; j < LU_NBJ; j++) acc[j] = lu_f64x4{0.0, 0.0, 0.0, 0.0};
	for(int64_t r = r0 + wave * 4; r < r1; r += 16) {
		const int64_t row = r + k4;
		const bool in = row < r1;
		const double a = in && yIn ? y[row] : 0.0;
		const double* drow = G.dense + (size_t) (in ? row : r0) * nC;
#pragma unroll
		for(int j = 0; j < LU_NBJ; j++) {
			if(j >= nj) break;
			const int cbj = (jb0 + j) * 16 + i16;
			const double bv = in && cbj < nC ? drow[cbj] : 0.0;
			acc[j] = __builtin_amdgcn_mfma_f64_16x16x4f64(a, bv, acc[j], 0, 0, 0);
		}
	}
	for(int i = tid; i < LU_NBJ * 256; i += 256) red[i] = 0.0;
	__syncthreads();
#pragma unroll
	for(int j = 0; j < LU_NBJ; j++)
#pragma unroll
		for(int v = 0; v < 4; v++)
			if(j < nj) unsafeAtomicAdd(&red[j * 256 + (4 * v + k4) * 16 + i16], acc[j][v]);
	__syncthreads();
	for(int i = tid; i < nj * 256; i += 256) {
		const int j = i >> 8, rr = (i >> 4) & 15, cc = i & 15;
		const int gr = ib * 16 + rr, gc = (jb0 + j) * 16 + cc;
		if(gr < p && gc < nC && red[i] != 0.0) unsafeAtomicAdd(&out[(size_t) gr * nCols + G.cols[gc]], red[i]);
	}
}

__global__ __launch_bounds__(256) void k_lmm_rowsum(const double* __restrict__ Y, int64_t nRows, int64_t rowsPerBlock,
	double* __restrict__ rs) {
	__shared__ double red[4];
	const int i = blockIdx.y;
	const double* y = Y + (size_t) i * nRows;
	const int64_t rb = (int64_t) blockIdx.x * rowsPerBlock, re = min(rb + rowsPerBlock, nRows);
	double s = 0.0;
	for(int64_t r = rb + threadIdx.x; r < re; r += 256) s += y[r];
	s = wave_sum_f64(s);
	if((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
	__syncthreads();
	if(threadIdx.x == 0) unsafeAtomicAdd(&rs[i], red[0] + red[1] + red[2] + red[3]);
}

// K9: out[i, cols_g[j]] += sum_k pre[i, tblOff_g + k] * dict_g[k, j]; block = (group, i)
__global__ __launch_bounds__(256) void k_lmm_post(const DGroup* __restrict__ groups, const double* __restrict__ pre,
	int totalVals, double* __restrict__ out, int nCols) {
	__shared__ double red[4];
	const DGroup G = dgroup(groups + (blockIdx.x));
	if(G.type == G_UNC) return;
	const int i = blockIdx.y;
	const double* p = pre + (size_t) i * totalVals + G.tblOff;
	for(int j = 0; j < G.nColG; j++) {
		double s = 0.0;
		for(int k = threadIdx.x; k < G.nVals; k += 256) s += p[k] * G.dict[(size_t) k * G.nColG + j];
		s = wave_sum_f64(s);
		if((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
		__syncthreads();
		if(threadIdx.x == 0) unsafeAtomicAdd(&out[(size_t) i * nCols + G.cols[j]], red[0] + red[1] + red[2] + red[3]);
		__syncthreads();
	}
}

// out[i, c] += rowSum[i] * constV[c] (skipped for rowSum == 0, as the reference does); nnz
__global__ __launch_bounds__(256) void k_lmm_finish(double* __restrict__ out, int p, int nCols, const double* __restrict__ rs,
	const double* __restrict__ constV, unsigned long long* __restrict__ nnz) {
	const int64_t idx = (int64_t) blockIdx.x * 256 + threadIdx.x;
	int cnt = 0;
	if(idx < (int64_t) p * nCols) {
		const int i = (int) (idx / nCols), c = (int) (idx - (int64_t) i * nCols);
		double v = out[idx];
		if(rs != nullptr) {
			const double vl = rs[i];
			if(vl != 0.0) v += vl * constV[c];
			out[idx] = v;
		}
		cnt = v != 0.0;
	}
	count_add(nnz, cnt);
}

// dOut != nullptr (whole-block calls): groups whose products can be summed directly write into dOut
// and leave their part of dPre zero.
static int run_preagg(cla_block* b, const double* dY, int p, double* dPre, int onlyGroup, double* dOut) {
	const int nG = (int) b->groups.size();
	const int64_t nRows = b->nRows;
	hipStream_t st = b->stream;
	// all groups DDC with byte codes in one arena: one persistent kernel for the whole block
	if(onlyGroup < 0) {
		const int r = launch_lmm_u8(b, dY, p, dPre);
		if(r == 0) b->preUsed = true;
		if(r <= 0) return r;
	}
	// row-parallel groups (DDC, RLE) in LDS-sized slabs
	int64_t rowsPerBlock = 64 * 1024;
	while(rowsPerBlock > 4096 && (nRows + rowsPerBlock - 1) / rowsPerBlock * p < (int64_t) g_numCU * 2) rowsPerBlock /= 2;
	const unsigned gridRows = (unsigned) std::max<int64_t>((nRows + rowsPerBlock - 1) / rowsPerBlock, 1);
	int g = 0;
	while(g < nG) {
		const DGroup& G = b->groups[g].d;
		const bool rowPar = (G.type == G_DDC || G.type == G_RLE) && (onlyGroup < 0 || onlyGroup == g);
		if(!rowPar) { g++; continue; }
		const int direct = (size_t) G.nVals * 8 > (size_t) 60 * 1024;
		int g1 = g;
		size_t bytes = 0;
		const size_t budget = (size_t) G.nVals * 8 > LMM_BIN_BYTES ? (size_t) G.nVals * 8 : LMM_BIN_BYTES;
		while(g1 < nG) {
			const DGroup& H = b->groups[g1].d;
			if(!((H.type == G_DDC || H.type == G_RLE) && (onlyGroup < 0 || onlyGroup == g1))) break;
			if(bytes + (size_t) H.nVals * 8 > budget) break;
			bytes += (size_t) H.nVals * 8;
			g1++;
			if(direct) break;
		}
		if(nRows > 0) {
			b->preUsed = true;
			const size_t lds = direct ? 0 : bytes;
			Prof pf(b, "k_lmm_preagg_rows", (long) gridRows * p, LMM_THREADS, (long) lds, 0);
			CLA_HIP(allow_full_lds((const void*) k_lmm_preagg_rows));
			hipLaunchKernelGGL(k_lmm_preagg_rows, dim3(gridRows, p), dim3(LMM_THREADS), lds, st, b->dGroups, g, g1, dY,
				nRows, rowsPerBlock, dPre, b->totalVals, direct);
		}
		g = g1;
	}
	// SDCZeros groups: all lists walked tile by tile with the Y tile in LDS; the
	// per-group chunk kernel below only serves dictionaries too large for LDS bins
	{
		const int r = nRows > 0 ? launch_lmm_sdc_tiles(b, dY, p, dPre, onlyGroup, dOut) : 0;
		if(r < 0) return r;
		if(r == 0) { CLA_HIP(hipGetLastError()); return 0; }
	}
	for(g = 0; g < nG; g++) {
		const DGroup& G = b->groups[g].d;
		if(G.type != G_SDCZ || G.nOffsets == 0 || (onlyGroup >= 0 && onlyGroup != g)) continue;
		const int direct = (size_t) G.nVals * 8 > (size_t) 60 * 1024;
		int cpb = 1;
		while(cpb < 16 && (G.nCkpt + cpb - 1) / cpb * p > g_numCU * 8) cpb *= 2;
		const unsigned grid = (unsigned) std::max((G.nCkpt + cpb - 1) / cpb, 1);
		const size_t bytes = direct ? 0 : (size_t) G.nVals * 8;
		const double algo = (double) G.nDeltas * G.deltaWidth + (double) G.nOffsets * (G.codeWidth + 8.0);
		b->preUsed = true;
		Prof pf(b, "k_lmm_preagg_sdc", (long) grid * p, 256, (long) bytes, algo);
		if(G.deltaWidth == 1) {
			CLA_HIP(allow_full_lds((const void*) k_lmm_preagg_sdc<1>));
			hipLaunchKernelGGL(k_lmm_preagg_sdc<1>, dim3(grid, p), dim3(256), bytes, st, b->dGroups, g, dY, nRows, cpb, dPre,
				b->totalVals, direct);
		}
		else {
			CLA_HIP(allow_full_lds((const void*) k_lmm_preagg_sdc<2>));
			hipLaunchKernelGGL(k_lmm_preagg_sdc<2>, dim3(grid, p), dim3(256), bytes, st, b->dGroups, g, dY, nRows, cpb, dPre,
				b->totalVals, direct);
		}
	}
	CLA_HIP(hipGetLastError());
	return 0;
}

int launch_preagg(cla_block* b, int group, const double* dY, int p, double* dPre) {
	clear_stats(b);
	const DGroup& G = b->groups[group].d;
	if(G.type == G_UNC) { set_error("preagg: group %d is uncompressed", group); return -CLA_ERR_UNSUPPORTED; }
	// aggregate into a full-width scratch (p x totalVals) and slice the group's bins out
	int rc = ensure_tables(b, (size_t) p * b->totalVals);
	if(rc) return rc;
	CLA_HIP(hipMemsetAsync(b->dTables, 0, sizeof(double) * (size_t) p * b->totalVals, b->stream));
	if((rc = run_preagg(b, dY, p, b->dTables, group, nullptr))) return rc;
	CLA_HIP(hipMemcpy2DAsync(dPre, sizeof(double) * (size_t) G.nVals, b->dTables + G.tblOff,
		sizeof(double) * (size_t) b->totalVals, sizeof(double) * (size_t) G.nVals, (size_t) p, hipMemcpyDeviceToDevice,
		b->stream));
	return 0;
}

int launch_lmm(cla_block* b, const double* dY, int p, double* dOut, unsigned long long* dNnz) {
	const int nG = (int) b->groups.size();
	const int64_t nRows = b->nRows;
	hipStream_t st = b->stream;
	clear_stats(b);
	// mixed blocks of few columns: one pass on the decoded Gram kernel
	{
		const int j = launch_lmm_joint(b, dY, p, dOut, dNnz);
		if(j <= 0) return j;
	}
	int rc = ensure_tables(b, (size_t) p * b->totalVals + (size_t) p + 8);
	if(rc) return rc;
	double* dPre = b->dTables;
	double* dRs = b->dTables + (size_t) p * b->totalVals;
	CLA_HIP(hipMemsetAsync(dOut, 0, sizeof(double) * (size_t) p * b->nCols, st));
	// Blocks that one kernel serves whole (byte-code DDC groups of one column; SDCZeros lists only) and that have no
	// constants to add: that kernel also counts the result's non-zeros, and nothing else runs.
	b->preUsed = false;
	b->lmmTailWanted = !b->hasConst && dNnz == b->dCounters && (int64_t) p * b->nCols < ((int64_t) 1 << 30);
	b->lmmTailDone = false;
	int dot = nRows > 0 ? launch_lmm_u8_dot(b, dY, p, dOut) : 1;
	if(dot < 0) return dot;
	if(dot != 0 && nRows > 0 && b->lmmTailWanted && b->opt.sdcLanes && !b->dictNonFinite && b->hasSdc && !b->hasUnc && !b->hasRle) {
		bool onlyLists = true;
		for(int g = 0; g < nG && onlyLists; g++) onlyLists = b->groups[g].d.type == G_SDCZ && b->groups[g].d.nOffsets > 0;
		if(onlyLists) {
			if((rc = sdc_plan_all(b))) return rc;
			const int r = launch_lmm_sdc_lanes(b, dY, p, dOut);
			if(r < 0) return r;
		}
	}
	b->lmmTailWanted = false;
	if(b->lmmTailDone) {
		CLA_HIP(hipGetLastError());
		return 0;
	}
	CLA_HIP(hipMemsetAsync(dPre, 0, sizeof(double) * ((size_t) p * b->totalVals + (size_t) p), st));
	CLA_HIP(hipMemsetAsync(dNnz, 0, sizeof(unsigned long long), st));
	if(dot != 0 && (rc = run_preagg(b, dY, p, dPre, -1, dOut))) return rc;

	int64_t rowsPerBlock = 256 * 1024;
	while(rowsPerBlock > 8192 && (nRows + rowsPerBlock - 1) / rowsPerBlock * p < (int64_t) g_numCU * 2) rowsPerBlock /= 2;
	const unsigned gridRows = (unsigned) std::max<int64_t>((nRows + rowsPerBlock - 1) / rowsPerBlock, 1);
	for(int g = 0; g < nG; g++) {
		const DGroup& G = b->groups[g].d;
		if(G.type != G_UNC || nRows == 0 || G.nColG == 0) continue;
		const int nbY = (p + 15) / 16, nbC = ((G.nColG + 15) / 16 + LU_NBJ - 1) / LU_NBJ;
		int64_t rpb = 16384;
		while(rpb > 1024 && (nRows + rpb - 1) / rpb * nbY * nbC < (int64_t) g_numCU * 8) rpb /= 2;
		const dim3 grid((unsigned) ((nRows + rpb - 1) / rpb), (unsigned) nbY, (unsigned) nbC);
		Prof pf(b, "k_lmm_unc", (long) grid.x * grid.y * grid.z, 256, 0, (double) nRows * G.nColG * 8);
		hipLaunchKernelGGL(k_lmm_unc, grid, dim3(256), 0, st, b->dGroups, g, dY, p, nRows, rpb, dOut, b->nCols);
	}
	if(b->hasConst && nRows > 0) {
		Prof pf(b, "k_lmm_rowsum", (long) gridRows * p, 256, 0, 0);
		hipLaunchKernelGGL(k_lmm_rowsum, dim3(gridRows, p), dim3(256), 0, st, dY, nRows, rowsPerBlock, dRs);
	}
	if(nG > 0 && dot != 0 && b->preUsed) {
		Prof pf(b, "k_lmm_post", (long) nG * p, 256, 0, 0);
		hipLaunchKernelGGL(k_lmm_post, dim3(nG, p), dim3(256), 0, st, b->dGroups, dPre, b->totalVals, dOut, b->nCols);
	}
	{
		const int64_t n = (int64_t) p * b->nCols;
		Prof pf(b, "k_lmm_finish", (long) ((n + 255) / 256), 256, 0, 0);
		hipLaunchKernelGGL(k_lmm_finish, dim3((unsigned) ((n + 255) / 256)), dim3(256), 0, st, dOut, p, b->nCols,
			b->hasConst ? dRs : nullptr, b->dConstV, dNnz);
	}
	CLA_HIP(hipGetLastError());
	return 0;
}

// CLALibMMChain.mmChain: tmp = X %*% v ; tmp *= w (XtwXv) or tmp -= w (XtXvy) ; out = t(tmp) %*% X.
__global__ __launch_bounds__(256) void k_mul_inplace(double* __restrict__ x, const double* __restrict__ w, int64_t n) {
	const int64_t i = (int64_t) blockIdx.x * 256 + threadIdx.x;
	if(i < n) x[i] *= w[i];
}

__global__ __launch_bounds__(256) void k_sub_inplace(double* __restrict__ x, const double* __restrict__ y, int64_t n) {
	const int64_t i = (int64_t) blockIdx.x * 256 + threadIdx.x;
	if(i < n) x[i] -= y[i];
}

int launch_mmchain(cla_block* b, const double* dV, const double* dW, int ctype, double* dOut, unsigned long long* dNnz) {
	const int64_t nRows = b->nRows;
	// the intermediate vector has a workspace of its own: the multiplies below may resize the shared scratch
	const size_t need = (size_t) std::max<int64_t>(nRows, 1);
	if(need > b->chainCap) {
		if(b->dChain) CLA_HIP(hipFree(b->dChain));
		b->dChain = nullptr; b->chainCap = 0;
		CLA_HIP(hipMalloc((void**) &b->dChain, need * sizeof(double)));
		b->chainCap = need;
	}
	double* tmp = b->dChain;
	int rc;
	if((rc = launch_rmm(b, dV, 1, tmp, dNnz))) return rc;
	b->nnzSlot = 0; // the left multiply below counts the result's non-zeros into dNnz
	std::vector<KernelStat> first;
	first.swap(b->lastStats);
	if(ctype == 1 && nRows > 0)
		hipLaunchKernelGGL(k_mul_inplace, dim3((unsigned) ((nRows + 255) / 256)), dim3(256), 0, b->stream, tmp, dW, nRows);
	if(ctype == 2 && nRows > 0)
		hipLaunchKernelGGL(k_sub_inplace, dim3((unsigned) ((nRows + 255) / 256)), dim3(256), 0, b->stream, tmp, dW, nRows);
	rc = launch_lmm(b, tmp, 1, dOut, dNnz);
	b->lastStats.insert(b->lastStats.begin(), first.begin(), first.end());
	return rc;
}

} // namespace cla
