// t(X) %*% X on a compressed block, integer co-occurrence and additive
// decompression (gfx950).
//
//   tile_codes          materialises the per-row codes of one group for a tile of
//                       SDC_TILE rows in LDS (-1 = row not covered): DDC direct,
//                       RLE by run walk, SDCZeros from the row-tile index
//   k_tsmm_pair         P[code_t(r), :] += dict_s[code_s(r), :] in LDS (the reference's
//                       preAggregateThatIndexStructure), contracted with dict_t per block
//   k_tsmm_self         counts x dict (x) dict, and column sums for the correction layer
//   k_tsmm_dense        scalar form (option tsmm_mfma = 0): decode row tiles and accumulate the Gram matrix
//   k_tsmm_finish       correction layer, mirror upper -> lower, non-zero count
//   k_cooc_*            exact integer co-occurrence counts
//   k_decompress_*      additive decompression into a dense block
#include "../../include/cla_hip.h"
#include "cla_device.hpp"

namespace cla {

constexpr int TT = SDC_TILE;      // rows per tile
constexpr int TSMM_THREADS = 256; // 4 rows per thread per tile

// Fills codes[0..TT) for rows [tile*TT, tile*TT+TT) of group G. All threads of the
// block must call it; ends with a barrier.
__device__ void tile_codes(const DGroup& G, int tile, int64_t nRows, int32_t* __restrict__ codes) {
	const int64_t r0 = (int64_t) tile * TT;
	const int tid = threadIdx.x;
	const int TSMM_THREADS = blockDim.x; // any multiple of 64, at least 256
	if(G.type == G_DDC) {
		for(int t = tid; t < TT; t += TSMM_THREADS) codes[t] = r0 + t < nRows ? load_code(G.codes, G.codeWidth, r0 + t) : -1;
	}
	else if(G.type == G_RLE) {
		// threads 0..255 expand 4 consecutive rows each from the merged run table
		const int64_t rb = r0 + tid * 4;
		if(tid >= TT / 4) {}
		else if(rb < nRows) {
			int j = rle_find(G.runStart, G.nRuns, (int32_t) rb);
			for(int t = 0; t < 4; t++) {
				const int64_t r = rb + t;
				if(r >= nRows) { codes[tid * 4 + t] = -1; continue; }
				while(G.runStart[j + 1] <= r) j++;
				codes[tid * 4 + t] = G.runCode[j];
			}
		}
		else
			for(int t = 0; t < 4; t++) codes[tid * 4 + t] = -1;
	}
	else if(G.type == G_SDCZ) {
		for(int t = tid; t < TT; t += TSMM_THREADS) codes[t] = -1;
		__syncthreads();
		if(G.nOffsets > 0) {
			const int64_t rEnd = r0 + TT;
			if(tid == 0 && G.first >= r0 && G.first < rEnd) codes[G.first - r0] = load_code(G.codes, G.codeWidth, 0);
			// wave 0 walks the list from the tile's iterator state
			if(tid < 64 && tile < G.nTiles) {
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
						if((mask & (1u << k)) && rows[k] < rEnd && rows[k] >= r0)
							codes[rows[k] - r0] = load_code(G.codes, G.codeWidth, didx[k]);
					i0 += 256;
				}
			}
		}
	}
	else {
		for(int t = tid; t < TT; t += TSMM_THREADS) codes[t] = -1;
	}
	__syncthreads();
}

__device__ __forceinline__ void add_upper_atomic(double* out, int nCols, int row, int col, double v) {
	// DictLibMatrixMult.addToUpperTriangle: lower-triangle cells are mirrored, a
	// diagonal cell (only reachable with overlapping groups) receives the value twice
	if(row == col) unsafeAtomicAdd(&out[(size_t) row * nCols + col], v + v);
	else if(row > col) unsafeAtomicAdd(&out[(size_t) col * nCols + row], v);
	else unsafeAtomicAdd(&out[(size_t) row * nCols + col], v);
}

// ---------------------------------------------------------------------------
// Pair term. `t` = target group (its codes select the accumulator row), `s` =
// source group (its dictionary tuples are accumulated). LDS: P[nVals_t x nC_s],
// optionally a copy of dict_s, and the two code tiles. Each block owns a
// contiguous range of tiles, then contracts t(dict_t) . P and adds the
// nC_t x nC_s result into the upper triangle.
// ---------------------------------------------------------------------------
constexpr int PAIR_THREADS = 1024;

// one row of a DDC-DDC pair: P[a, :] += dict_s[c, :]
__device__ __forceinline__ void pair_add(double* __restrict__ P, const double* __restrict__ dsrc, int nCs, int a, int c) {
	const double* v = dsrc + (size_t) c * nCs;
	double* p = P + (size_t) a * nCs;
	if(nCs == 2) {
		const double2 vv = *(const double2*) v;
		unsafeAtomicAdd(&p[0], vv.x);
		unsafeAtomicAdd(&p[1], vv.y);
	}
	else
		for(int j = 0; j < nCs; j++) unsafeAtomicAdd(&p[j], v[j]);
}

__global__ __launch_bounds__(PAIR_THREADS) void k_tsmm_pair(const DGroup* __restrict__ groups,
	const int4* __restrict__ pairs, int64_t nRows, int tilesPerBlock, double* __restrict__ out, int nCols) {
	constexpr int TSMM_THREADS = PAIR_THREADS;
	extern __shared__ double smem[];
	const int4 pr = pairs[blockIdx.y]; // (target, source, dictInLds, 0)
	const DGroup Gt = dgroup(groups + (pr.x));
	const DGroup Gs = dgroup(groups + (pr.y));
	const int dictInLds = pr.z;
	const int nCs = Gs.nColG, nCt = Gt.nColG;
	double* P = smem;                                             // nVals_t * nCs
	double* dS = P + (size_t) Gt.nVals * nCs;                      // nVals_s * nCs (optional)
	int32_t* ca = (int32_t*) (dS + (dictInLds ? (size_t) Gs.nVals * nCs : 0));
	int32_t* cb = ca + TT;
	const int tid = threadIdx.x;
	for(int i = tid; i < Gt.nVals * nCs; i += TSMM_THREADS) P[i] = 0.0;
	if(dictInLds)
		for(int i = tid; i < Gs.nVals * nCs; i += TSMM_THREADS) dS[i] = Gs.dict[i];
	const double* dsrc = dictInLds ? dS : Gs.dict;
	const int nTiles = (int) ((nRows + TT - 1) / TT);
	const int t0 = blockIdx.x * tilesPerBlock, t1 = min(t0 + tilesPerBlock, nTiles);
	__syncthreads();
	if(Gt.type == G_DDC && Gs.type == G_DDC) {
		// both code streams are read directly, 8 rows per thread and step
		const int64_t rb = (int64_t) t0 * TT, re = min((int64_t) t1 * TT, nRows);
		const int wt = Gt.codeWidth, ws = Gs.codeWidth;
		for(int64_t r0 = rb + (int64_t) tid * 8; r0 < re; r0 += (int64_t) TSMM_THREADS * 8) {
			if(r0 + 8 <= re && wt == 2 && ws == 2) {
				const u32x4 ua = __builtin_nontemporal_load((const u32x4*) ((const uint16_t*) Gt.codes + r0));
				const u32x4 ub = __builtin_nontemporal_load((const u32x4*) ((const uint16_t*) Gs.codes + r0));
				const uint32_t wa[4] = {ua.x, ua.y, ua.z, ua.w}, wb[4] = {ub.x, ub.y, ub.z, ub.w};
#pragma unroll
				for(int t = 0; t < 8; t++)
					pair_add(P, dsrc, nCs, (wa[t >> 1] >> (16 * (t & 1))) & 0xffff, (wb[t >> 1] >> (16 * (t & 1))) & 0xffff);
			}
			else if(r0 + 8 <= re && wt == 1 && ws == 1) {
				const uint2 ua = *(const uint2*) ((const uint8_t*) Gt.codes + r0);
				const uint2 ub = *(const uint2*) ((const uint8_t*) Gs.codes + r0);
				const uint32_t wa[2] = {ua.x, ua.y}, wb[2] = {ub.x, ub.y};
#pragma unroll
				for(int t = 0; t < 8; t++)
					pair_add(P, dsrc, nCs, (wa[t >> 2] >> (8 * (t & 3))) & 0xff, (wb[t >> 2] >> (8 * (t & 3))) & 0xff);
			}
			else {
				for(int t = 0; t < 8 && r0 + t < re; t++)
					pair_add(P, dsrc, nCs, load_code(Gt.codes, wt, r0 + t), load_code(Gs.codes, ws, r0 + t));
			}
		}
		__syncthreads();
	}
	else {
		for(int tile = t0; tile < t1; tile++) {
			tile_codes(Gt, tile, nRows, ca);
			tile_codes(Gs, tile, nRows, cb);
			for(int t = tid; t < TT; t += TSMM_THREADS) {
				const int a = ca[t], c = cb[t];
				if(a >= 0 && c >= 0) pair_add(P, dsrc, nCs, a, c);
			}
			__syncthreads();
		}
	}
	// contraction: S[i, j] = sum_a dict_t[a, i] * P[a, j]
	__shared__ double red[PAIR_THREADS / 64];
	for(int i = 0; i < nCt; i++)
		for(int j = 0; j < nCs; j++) {
			double s = 0.0;
			for(int a = tid; a < Gt.nVals; a += TSMM_THREADS) s += Gt.dict[(size_t) a * nCt + i] * P[(size_t) a * nCs + j];
			s = wave_sum_f64(s);
			if((tid & 63) == 0) red[tid >> 6] = s;
			__syncthreads();
			if(tid == 0) {
				double tot = 0.0;
				for(int w = 0; w < TSMM_THREADS / 64; w++) tot += red[w];
				add_upper_atomic(out, nCols, Gt.cols[i], Gs.cols[j], tot);
			}
			__syncthreads();
		}
}

// ---------------------------------------------------------------------------
// Pair term in dot form for two DDC groups whose dictionaries both fit LDS:
// S[i, j] = sum_r dict_t[code_t(r), i] * dict_s[code_s(r), j], accumulated in registers,
// no LDS atomics (an LDS fp64 add costs about four LDS reads on this device). Equal to the
// pre-aggregate form t(dict_t) . P up to rounding. Blocks are ordered row chunk first,
// pair second, so that the code streams of one chunk of rows are served from the
// last-level cache for all pairs.
// ---------------------------------------------------------------------------
constexpr int PD_THREADS = 1024;
constexpr int PD_RPT = 8; // rows per thread and step: one 8- or 16-byte load per stream
constexpr int PD_DEPTH = 4;

template <int CW, int NCT, int NCS>
__global__ __launch_bounds__(PD_THREADS) void k_tsmm_pair_dot(const DGroup* __restrict__ groups, const int4* __restrict__ pairs,
	int nPairs, int64_t nRows, int64_t chunkRows, int blocksPerChunkPair, double* __restrict__ out, int nCols) {
	extern __shared__ double smem[];
	const int tid = threadIdx.x;
	// blockIdx.x = (chunk * nPairs + pair) * blocksPerChunkPair + part
	const int part = blockIdx.x % blocksPerChunkPair;
	const int cp = blockIdx.x / blocksPerChunkPair;
	const int pairIdx = cp % nPairs, chunk = cp / nPairs;
	const int4 pr = pairs[pairIdx];
	const DGroup Gt = dgroup(groups + (pr.x));
	const DGroup Gs = dgroup(groups + (pr.y));
	double* dT = smem;                                   // nVals_t * NCT
	double* dS = smem + (((size_t) Gt.nVals * NCT + 1) & ~(size_t) 1); // nVals_s * NCS, 16-byte aligned
	for(int i = tid; i < Gt.nVals * NCT; i += PD_THREADS) dT[i] = Gt.dict[i];
	for(int i = tid; i < Gs.nVals * NCS; i += PD_THREADS) dS[i] = Gs.dict[i];
	const int64_t cb = (int64_t) chunk * chunkRows, ce = min(cb + chunkRows, nRows);
	const int64_t per = ((ce - cb + blocksPerChunkPair - 1) / blocksPerChunkPair + PD_RPT - 1) / PD_RPT * PD_RPT;
	const int64_t rb = cb + (int64_t) part * per, re = min(rb + per, ce);
	const uint8_t* ct = (const uint8_t*) Gt.codes;
	const uint8_t* cs = (const uint8_t*) Gs.codes;
	double acc[NCT][NCS];
#pragma unroll
	for(int i = 0; i < NCT; i++)
#pragma unroll
		for(int j = 0; j < NCS; j++) acc[i][j] = 0.0;
	__syncthreads();
	auto row = [&](int a, int c) {
		double vt[NCT], vs[NCS];
#pragma unroll
		for(int i = 0; i < NCT; i++) vt[i] = dT[a * NCT + i];
#pragma unroll
		for(int j = 0; j < NCS; j++) vs[j] = dS[c * NCS + j];
#pragma unroll
		for(int i = 0; i < NCT; i++)
#pragma unroll
			for(int j = 0; j < NCS; j++) acc[i][j] = __builtin_fma(vt[i], vs[j], acc[i][j]);
	};
	// Whole steps (every thread 8 rows) with a ring of PD_DEPTH code requests in flight per
	// stream, then the rows that do not fill a step.
	CodeVec<CW, PD_RPT> at[PD_DEPTH], as[PD_DEPTH];
	const int64_t step = (int64_t) PD_THREADS * PD_RPT;
	const int nFull = re > rb ? (int) ((re - rb) / step) : 0;
	const uint8_t* pt = ct + (rb + (int64_t) tid * PD_RPT) * CW;
	const uint8_t* ps = cs + (rb + (int64_t) tid * PD_RPT) * CW;
#pragma unroll
	for(int d = 0; d < PD_DEPTH; d++)
		if(d < nFull) { at[d].load(pt + (int64_t) d * step * CW); as[d].load(ps + (int64_t) d * step * CW); }
	for(int it = 0; it < nFull; it += PD_DEPTH) {
#pragma unroll
		for(int d = 0; d < PD_DEPTH; d++) {
			if(it + d >= nFull) break;
#pragma unroll
			for(int t = 0; t < PD_RPT; t++) row(at[d].get(t), as[d].get(t));
			if(it + d + PD_DEPTH < nFull) {
				at[d].load(pt + (int64_t) (it + d + PD_DEPTH) * step * CW);
				as[d].load(ps + (int64_t) (it + d + PD_DEPTH) * step * CW);
			}
		}
	}
	for(int64_t r = rb + (int64_t) nFull * step + tid; r < re; r += PD_THREADS) row(load_code(ct, CW, r), load_code(cs, CW, r));
	// block reduction, then one add per cell into the upper triangle
	__shared__ double red[PD_THREADS / 64];
#pragma unroll
	for(int i = 0; i < NCT; i++)
#pragma unroll
		for(int j = 0; j < NCS; j++) {
			const double s = wave_sum_f64(acc[i][j]);
			__syncthreads();
			if((tid & 63) == 0) red[tid >> 6] = s;
			__syncthreads();
			if(tid == 0) {
				double tot = 0.0;
				for(int w = 0; w < PD_THREADS / 64; w++) tot += red[w];
				if(tot != 0.0) add_upper_atomic(out, nCols, Gt.cols[i], Gs.cols[j], tot);
			}
		}
}

template <int CW>
static void launch_pair_dot_cw(int nct, int ncs, dim3 grid, size_t lds, hipStream_t st, const DGroup* g, const int4* pairs, int nPairs,
	int64_t nRows, int64_t chunkRows, int bpcp, double* out, int nCols) {
#define PD_CASE(A, B)                                                                                           \
	if(nct == A && ncs == B) {                                                                                  \
		auto kern = k_tsmm_pair_dot<CW, A, B>;                                                                  \
		(void) allow_full_lds((const void*) kern);  \
		hipLaunchKernelGGL(kern, grid, dim3(PD_THREADS), lds, st, g, pairs, nPairs, nRows, chunkRows, bpcp, out, nCols); \
	}
	PD_CASE(1, 1) PD_CASE(1, 2) PD_CASE(2, 1) PD_CASE(2, 2)
#undef PD_CASE
}

// Self term (AColGroupCompressed.tsmmDense) + column sums of the group:
// out[cols[i], cols[j]] += sum_k cnt[k] d[k,i] d[k,j], j >= i; colSum[cols[j]] += sum_k cnt[k] d[k,j]
__global__ __launch_bounds__(256) void k_tsmm_self(const DGroup* __restrict__ groups, const int32_t* __restrict__ countsAll,
	double* __restrict__ out, int nCols, double* __restrict__ colSum) {
	__shared__ double red[4];
	const DGroup G = dgroup(groups + (blockIdx.y));
	if(G.type == G_UNC) return;
	const int32_t* counts = countsAll + G.tblOff;
	const int nC = G.nColG, tid = threadIdx.x;
	for(int i = 0; i < nC; i++) {
		for(int j = i; j <= nC; j++) { // j == nC: column sum of column i
			double s = 0.0;
			for(int k = tid; k < G.nVals; k += 256) {
				const double v = G.dict[(size_t) k * nC + i] * (double) counts[k];
				s += j < nC ? v * G.dict[(size_t) k * nC + j] : v;
			}
			s = wave_sum_f64(s);
			if((tid & 63) == 0) red[tid >> 6] = s;
			__syncthreads();
			if(tid == 0) {
				const double tot = red[0] + red[1] + red[2] + red[3];
				if(j < nC) {
					const int r = G.cols[i], c = G.cols[j];
					unsafeAtomicAdd(&out[(size_t) min(r, c) * nCols + max(r, c)], tot);
				}
				else
					unsafeAtomicAdd(&colSum[G.cols[i]], tot);
			}
			__syncthreads();
		}
	}
}

// ---------------------------------------------------------------------------
// Dense fallback (any uncompressed group, or at least as many groups as columns):
// decode DT rows into LDS and accumulate the upper triangle of t(D) %*% D.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_tsmm_dense(const DGroup* __restrict__ groups, int nGroups,
	const double* __restrict__ constV, int64_t nRows, int nCols, int DT, int tilesPerBlock, double* __restrict__ out) {
	extern __shared__ double D[]; // DT x nCols
	const int tid = threadIdx.x;
	const int nPairs = nCols * (nCols + 1) / 2;
	const int64_t nTiles = (nRows + DT - 1) / DT;
	const int64_t t0 = (int64_t) blockIdx.x * tilesPerBlock, t1 = min(t0 + tilesPerBlock, nTiles);
	// pairs owned by this thread (strided), partial sums kept in registers for up to 8 pairs
	constexpr int MAXP = 24;
	double acc[MAXP];
#pragma unroll
	for(int k = 0; k < MAXP; k++) acc[k] = 0.0;
	for(int64_t tile = t0; tile < t1; tile++) {
		const int64_t r0 = tile * DT;
		const int nr = (int) min((int64_t) DT, nRows - r0);
		for(int i = tid; i < DT * nCols; i += 256) D[i] = (i / nCols) < nr ? constV[i % nCols] : 0.0;
		__syncthreads();
		for(int g = 0; g < nGroups; g++) {
			const DGroup G = dgroup(groups + (g));
			if(G.type == G_DDC || G.type == G_RLE) {
				for(int t = tid; t < nr; t += 256) {
					const int64_t r = r0 + t;
					const int code = G.type == G_DDC ? load_code(G.codes, G.codeWidth, r)
					                                 : G.runCode[rle_find(G.runStart, G.nRuns, (int32_t) r)];
					if(code >= 0)
						for(int j = 0; j < G.nColG; j++) D[t * nCols + G.cols[j]] += G.dict[(size_t) code * G.nColG + j];
				}
			}
			else if(G.type == G_UNC) {
				for(int t = tid; t < nr * G.nColG; t += 256) {
					const int rr = t / G.nColG, j = t - rr * G.nColG;
					D[rr * nCols + G.cols[j]] += G.dense[(size_t) (r0 + rr) * G.nColG + j];
				}
			}
			else if(G.type == G_SDCZ && G.nOffsets > 0) {
				// thread 0.. walk: rows of the list inside [r0, r0+nr) via the coarse tile index
				if(tid < 64) {
					const int64_t rEnd = r0 + nr;
					if(tid == 0 && G.first >= r0 && G.first < rEnd) {
						const int code = load_code(G.codes, G.codeWidth, 0);
						for(int j = 0; j < G.nColG; j++) D[(G.first - r0) * nCols + G.cols[j]] += G.dict[(size_t) code * G.nColG + j];
					}
					const int ti = (int) (r0 / SDC_TILE);
					if(ti < G.nTiles) {
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
								if((mask & (1u << k)) && rows[k] >= r0 && rows[k] < rEnd) {
									const int code = load_code(G.codes, G.codeWidth, didx[k]);
									for(int j = 0; j < G.nColG; j++)
										D[(rows[k] - r0) * nCols + G.cols[j]] += G.dict[(size_t) code * G.nColG + j];
								}
							i0 += 256;
						}
					}
				}
			}
			__syncthreads();
		}
		int slot = 0;
		for(int pr = tid; pr < nPairs && slot < MAXP; pr += 256, slot++) {
			// pair index -> (i, j), j >= i
			int i = 0, rem = pr;
			while(rem >= nCols - i) { rem -= nCols - i; i++; }
			const int j = i + rem;
			double s = 0.0;
			for(int t = 0; t < nr; t++) s += D[t * nCols + i] * D[t * nCols + j];
			acc[slot] += s;
		}
		__syncthreads();
	}
	int slot = 0;
	for(int pr = tid; pr < nPairs && slot < MAXP; pr += 256, slot++) {
		int i = 0, rem = pr;
		while(rem >= nCols - i) { rem -= nCols - i; i++; }
		const int j = i + rem;
		if(acc[slot] != 0.0) unsafeAtomicAdd(&out[(size_t) i * nCols + j], acc[slot]);
	}
}

// correction layer (CLALibTSMM.addCorrectionLayer), mirror, nnz; single block
__global__ __launch_bounds__(256) void k_tsmm_finish(double* __restrict__ out, int nCols, const double* __restrict__ constV,
	const double* __restrict__ colSum, double nRowsD, int applyCorrection, unsigned long long* __restrict__ nnz) {
	int cnt = 0;
	for(int idx = threadIdx.x + blockIdx.x * 256; idx < nCols * nCols; idx += 256 * gridDim.x) {
		const int i = idx / nCols, j = idx - i * nCols;
		if(j < i) continue;
		double v = out[idx];
		if(applyCorrection) {
			const double v1l = constV[i];
			const double v2l = colSum[i] + constV[i] * nRowsD;
			v += v1l * colSum[j] + v2l * constV[j];
		}
		out[idx] = v;
		out[(size_t) j * nCols + i] = v;
		cnt += v != 0.0 ? (i == j ? 1 : 2) : 0;
	}
	count_add(nnz, cnt);
}

__global__ void k_count_nnz2(const double* __restrict__ x, int64_t n, unsigned long long* __restrict__ nnz);

// ---------------------------------------------------------------------------
// t(D) %*% D of a dense row-major matrix on the matrix cores: the last resort for blocks no compressed form
// takes (overlapping groups, uncompressed groups wider than a column chunk among many columns, pair
// accumulators beyond LDS), after decompressing the block, which is what the reference does in these cases
// (CLALibTSMM.java:73-77). Block = (range of rows, column block ib, group of GD_NBJ column blocks jb >= ib);
// wave w takes rows 4 w .. 4 w + 3 of every 16; lane (k4, i16) holds D[row k4, 16 cb + i16] as both operands
// of v_mfma_f64_16x16x4_f64. Accumulator register v of lane l is cell (4 v + l / 16, l % 16) of its tile.
// Only tiles on or above the diagonal are computed; the caller mirrors.
// ---------------------------------------------------------------------------
constexpr int GD_NBJ = 8;
typedef double gd_f64x4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void k_gram_dense(const double* __restrict__ D, int64_t nRows, int nCols, int64_t rowsPerBlock,
	double* __restrict__ out) {
	__shared__ double red[GD_NBJ * 256];
	const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
	const int i16 = lane & 15, k4 = lane >> 4;
	const int nb = (nCols + 15) / 16;
	const int ib = blockIdx.y, jb0 = ib + blockIdx.z * GD_NBJ;
	if(jb0 >= nb) return;
	const int nj = min(GD_NBJ, nb - jb0);
	const int64_t r0 = (int64_t) blockIdx.x * rowsPerBlock, r1 = min(nRows, r0 + rowsPerBlock);
	gd_f64x4 acc[GD_NBJ];
#pragma unroll
	for(int j = 0; j < GD_NBJ; j++) acc[j] = gd_f64x4{0.0, 0.0, 0.0, 0.0};
	const int ca = ib * 16 + i16;
	for(int64_t r = r0 + wave * 4; r < r1; r += 16) {
		const int64_t row = r + k4;
		const bool in = row < r1;
		const double* drow = D + (size_t) (in ? row : r0) * nCols;
		const double a = in && ca < nCols ? drow[ca] : 0.0;
#pragma unroll
		for(int j = 0; j < GD_NBJ; j++) {
			if(j >= nj) break;
			const int cbj = (jb0 + j) * 16 + i16;
			const double bv = in && cbj < nCols ? drow[cbj] : 0.0;
			acc[j] = __builtin_amdgcn_mfma_f64_16x16x4f64(a, bv, acc[j], 0, 0, 0);
		}
	}
	for(int i = tid; i < GD_NBJ * 256; i += 256) red[i] = 0.0;
	__syncthreads();
#pragma unroll
	for(int j = 0; j < GD_NBJ; j++)
#pragma unroll
		for(int v = 0; v < 4; v++)
			if(j < nj) unsafeAtomicAdd(&red[j * 256 + (4 * v + k4) * 16 + i16], acc[j][v]);
	__syncthreads();
	for(int i = tid; i < nj * 256; i += 256) {
		const int j = i >> 8, rr = (i >> 4) & 15, cc = i & 15;
		const int gr = ib * 16 + rr, gc = (jb0 + j) * 16 + cc;
		if(gr <= gc && gc < nCols && red[i] != 0.0) unsafeAtomicAdd(&out[(size_t) gr * nCols + gc], red[i]);
	}
}

// The same for at most 16 NB columns with all tiles on or above the diagonal in one block: a row's values are loaded
// once (NB loads for NB (NB + 1) / 2 matrix instructions) where the kernel above loads them once per column block of
// the grid (4M x 60: 1.75 ms there).
template <int NB>
__global__ __launch_bounds__(256) void k_gram_dense_all(const double* __restrict__ D, int64_t nRows, int nCols, int64_t rowsPerBlock,
	double* __restrict__ out) {
	constexpr int NT = NB * (NB + 1) / 2;
	__shared__ double red[NT * 256];
	const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
	const int i16 = lane & 15, k4 = lane >> 4;
	const int64_t r0 = (int64_t) blockIdx.x * rowsPerBlock, r1 = min(nRows, r0 + rowsPerBlock);
	gd_f64x4 acc[NT];
#pragma unroll
	for(int t = 0; t < NT; t++) acc[t] = gd_f64x4{0.0, 0.0, 0.0, 0.0};
#pragma unroll 2
	for(int64_t r = r0 + wave * 4; r < r1; r += 16) {
		const int64_t row = r + k4;
		const bool in = row < r1;
		const double* drow = D + (size_t) (in ? row : r0) * nCols;
		double v[NB];
#pragma unroll
		for(int c = 0; c < NB; c++) {
			const int col = c * 16 + i16;
			v[c] = in && col < nCols ? drow[col] : 0.0;
		}
		int t = 0;
#pragma unroll
		for(int i = 0; i < NB; i++)
#pragma unroll
			for(int j = i; j < NB; j++) {
				acc[t] = __builtin_amdgcn_mfma_f64_16x16x4f64(v[i], v[j], acc[t], 0, 0, 0);
				t++;
			}
	}
	for(int i = tid; i < NT * 256; i += 256) red[i] = 0.0;
	__syncthreads();
#pragma unroll
	for(int t = 0; t < NT; t++)
#pragma unroll
		for(int v = 0; v < 4; v++) unsafeAtomicAdd(&red[t * 256 + (4 * v + k4) * 16 + i16], acc[t][v]);
	__syncthreads();
	int t = 0;
	for(int i = 0; i < NB; i++)
		for(int j = i; j < NB; j++) {
			const int rr = tid >> 4, cc = tid & 15;
			const int gr = i * 16 + rr, gc = j * 16 + cc;
			const double s = red[t * 256 + tid];
			if(gr <= gc && gc < nCols && s != 0.0) unsafeAtomicAdd(&out[(size_t) gr * nCols + gc], s);
			t++;
		}
}

// dOut (zeroed) = t(X) %*% X through the decompressed block. -CLA_ERR_UNSUPPORTED when the dense copy does
// not fit the free device memory.
static int launch_tsmm_decompressed(cla_block* b, double* dOut, unsigned long long* dNnz, const char* why) {
	// chunks of rows decompressed into the block's scratch buffer (at most 512 MiB), their Gram matrices added up
	(void) why;
	const int nCols = b->nCols;
	const int64_t nRows = b->nRows;
	hipStream_t st = b->stream;
	int rc = 0;
	if(nRows > 0 && nCols > 0) {
		int64_t rowsPerChunk = std::max<int64_t>((int64_t) 512 * 1024 * 1024 / ((int64_t) nCols * 8) / 1024 * 1024, 1024);
		rowsPerChunk = std::min(rowsPerChunk, (nRows + 1023) / 1024 * 1024);
		if((rc = ensure_scratch(b, sizeof(double) * (size_t) rowsPerChunk * nCols))) return rc;
		double* dense = (double*) b->dScratch;
		const int nb = (nCols + 15) / 16;
		for(int64_t r0 = 0; r0 < nRows; r0 += rowsPerChunk) {
			const int64_t rows = std::min(rowsPerChunk, nRows - r0);
			if((rc = launch_decompress_rows(b, r0, r0 + rows, dense))) return rc;
			int64_t rowsPerBlock = 16384;
			if(nb <= 4) { // all tiles of a range of rows in one block
				while(rowsPerBlock > 1024 && (rows + rowsPerBlock - 1) / rowsPerBlock < (int64_t) g_numCU * 4) rowsPerBlock /= 2;
				const unsigned grid = (unsigned) ((rows + rowsPerBlock - 1) / rowsPerBlock);
				Prof pf(b, "k_gram_dense", grid, 256, 0, (double) rows * nCols * 8);
				if(nb == 1) hipLaunchKernelGGL(k_gram_dense_all<1>, dim3(grid), dim3(256), 0, st, dense, rows, nCols, rowsPerBlock, dOut);
				else if(nb == 2) hipLaunchKernelGGL(k_gram_dense_all<2>, dim3(grid), dim3(256), 0, st, dense, rows, nCols, rowsPerBlock, dOut);
				else if(nb == 3) hipLaunchKernelGGL(k_gram_dense_all<3>, dim3(grid), dim3(256), 0, st, dense, rows, nCols, rowsPerBlock, dOut);
				else hipLaunchKernelGGL(k_gram_dense_all<4>, dim3(grid), dim3(256), 0, st, dense, rows, nCols, rowsPerBlock, dOut);
				continue;
			}
			while(rowsPerBlock > 1024 && (rows + rowsPerBlock - 1) / rowsPerBlock * nb < (int64_t) g_numCU * 4) rowsPerBlock /= 2;
			const dim3 grid((unsigned) ((rows + rowsPerBlock - 1) / rowsPerBlock), (unsigned) nb, (unsigned) ((nb + GD_NBJ - 1) / GD_NBJ));
			Prof pf(b, "k_gram_dense", (long) grid.x * grid.y * grid.z, 256, 0, (double) rows * nCols * 8);
			hipLaunchKernelGGL(k_gram_dense, grid, dim3(256), 0, st, dense, rows, nCols, rowsPerBlock, dOut);
		}
	}
	{
		Prof pf(b, "k_tsmm_finish", 1, 256, 0, 0);
		hipLaunchKernelGGL(k_tsmm_finish, dim3(1), dim3(256), 0, st, dOut, nCols, b->dConstV, b->dConstV, (double) nRows, 0, dNnz);
	}
	CLA_HIP(hipGetLastError());
	return 0;
}

int launch_tsmm(cla_block* b, double* dOut, unsigned long long* dNnz) {
	const int nG = (int) b->groups.size();
	const int nCols = b->nCols;
	const int64_t nRows = b->nRows;
	hipStream_t st = b->stream;
	clear_stats(b);
	auto clear = [&]() -> int {
		CLA_HIP(hipMemsetAsync(dOut, 0, sizeof(double) * (size_t) nCols * nCols, st));
		CLA_HIP(hipMemsetAsync(dNnz, 0, sizeof(unsigned long long), st));
		return 0;
	};
	// Overlapping column groups (the result of an overlapping right multiply): every compressed form here
	// assumes one group per column, and such blocks typically hold more groups than columns, where the
	// reference decompresses as well (CLALibTSMM.java:73-77).
	{
		int rc0;
		std::vector<char> seen((size_t) nCols, 0);
		for(auto& g : b->groups)
			for(int c : g.cols) {
				if(seen[c]) {
					if((rc0 = clear())) return rc0;
					return launch_tsmm_decompressed(b, dOut, dNnz, "overlapping column groups");
				}
				seen[c] = 1;
			}
	}
	int rc;
	// Decoded Gram matrix on the matrix cores (one pass over all groups) against one pass per
	// pair of groups: the first costs about as much per 16 x 16 tile of the result and row as
	// the second per eight pairs and row.
	const bool forceDecode = b->opt.tsmmRoute == 2, forcePairs = b->opt.tsmmRoute == 1;
	const int nb = (nCols + 15) / 16;
	// a joint block (cbind of two blocks, only the cross product wanted) pairs left groups with right groups only
	const int split = b->crossSplit;
	const int64_t nPairs = split > 0 ? (int64_t) split * (nG - split) : (int64_t) nG * (nG - 1) / 2;
	const bool gramCheaper = nCols <= 64 && nPairs >= (int64_t) 8 * nb * (nb + 1) / 2;
	// the per-pair path keeps the smaller accumulator nVals_t x nCol_s of a pair in LDS; where that cannot fit
	// (two very large dictionaries meet) the block is decoded instead when it is narrow enough
	bool pairsFit = true;
	for(int g = 0; g < nG && pairsFit; g++)
		for(int h = g + 1; h < nG; h++) {
			if(split > 0 && (g < split) == (h < split)) continue;
			const DGroup& A = b->groups[g].d;
			const DGroup& B = b->groups[h].d;
			if(A.type == G_UNC || B.type == G_UNC) continue;
			const size_t acc = std::min((size_t) A.nVals * B.nColG, (size_t) B.nVals * A.nColG) * 8;
			if(acc + (size_t) 2 * TT * 4 > (size_t) 150 * 1024) { pairsFit = false; break; }
		}
	const bool mustDecode = b->hasUnc || forceDecode || (!pairsFit && nCols <= 64);
	// As many groups as columns: the reference decompresses (CLALibTSMM.java:73-77); here that is the decoded
	// Gram matrix up to 64 columns. Wider blocks without uncompressed groups go per pair (the scalar
	// decompressing fallback is slower and ends at 110 columns) unless the option tsmm_wide_dense asks for it.
	const bool wideDense = nCols > 64 && nG >= nCols && (!pairsFit || b->opt.tsmmWideDense);
	const bool dense = split > 0 ? mustDecode || (nCols <= 64 && (nG >= nCols || gramCheaper) && !forcePairs)
	                             : mustDecode || wideDense || (nCols <= 64 && (nG >= nCols || gramCheaper) && !forcePairs);
	// More than 64 columns: the decoded Gram matrices of pairs of 32-column chunks (about 1.4 ms per pair of
	// chunks on 10M rows) against one pass per pair of groups (3-16 us each): chunks when there are a hundred
	// times more pairs of groups than pairs of chunks, or when there is no per-pair form.
	// The decoded Gram matrix of a whole block of at most 64 columns as the call's only kernel: its blocks add into an
	// accumulator kept with the block, and the last one to finish writes the output (both triangles) and the count of
	// its non-zeros and clears the accumulator again: no fill in front of the kernel, no kernel behind it.
	bool decodeTried = false;
	if(dense && nCols <= 64 && split == 0 && b->crossBlocks == 0 && nRows > 0 && b->opt.tsmmMfma && b->opt.tsmmOneKernel) {
		decodeTried = true;
		rc = launch_tsmm_decode(b, dOut, dNnz);
		if(rc <= 0) return rc;
	}
	if((rc = clear())) return rc;
	const int64_t mAll = (nCols + 31) / 32, mLeft = split > 0 ? std::max<int64_t>(1, mAll / 2) : 0;
	const int64_t nJoints = split > 0 ? mLeft * std::max<int64_t>(1, mAll - mLeft) : mAll * (mAll - 1) / 2;
	const bool chunkCheaper = !forcePairs && pairsFit && nPairs >= 100 * nJoints;
	if((dense || chunkCheaper) && nCols > 64 && nRows > 0 && b->opt.tsmmChunks) {
		// decoded Gram matrices of pairs of column chunks
		rc = launch_tsmm_chunked(b, dOut);
		if(rc < 0) return rc;
		if(rc == 0) {
			if(split == 0) { // (a joint block's caller takes its part and counts there)
				const int64_t nn = (int64_t) nCols * nCols;
				const unsigned cg = (unsigned) std::min<int64_t>((nn + 255) / 256, 1024);
				Prof pf(b, "k_count_nnz", cg, 256, 0, 0);
				hipLaunchKernelGGL(k_count_nnz2, dim3(cg), dim3(256), 0, st, dOut, nn, dNnz);
				CLA_HIP(hipGetLastError());
			}
			return 0;
		}
	}
	if(dense && split > 0 && nCols > 64)
		return launch_tsmm_decompressed(b, dOut, dNnz, "a group of more than 32 columns without a per-pair form among more than 64 joint columns");
	if(dense) {
		// t(D) %*% D of the decoded rows, constants included (no correction layer needed)
		const bool noMfma = !b->opt.tsmmMfma;
		rc = (noMfma || nRows == 0 || decodeTried) ? 1 : launch_tsmm_decode(b, dOut);
		if(rc < 0) return rc;
		if(rc == 0) {
			Prof pf(b, "k_tsmm_finish", 1, 256, 0, 0);
			hipLaunchKernelGGL(k_tsmm_finish, dim3(1), dim3(256), 0, st, dOut, nCols, b->dConstV, b->dConstV, (double) nRows, 0, dNnz);
			CLA_HIP(hipGetLastError());
			return 0;
		}
		// (the decode kernel does not take the block: its code tiles, list windows or dictionaries exceed LDS. Chunks of
		// rows decompressed through LDS tiles, their Gram matrices on the matrix cores: 4 M rows x 60 columns of two-byte
		// codes in 3 ms; the scalar form below, 6.7 ms, stays for the option tsmm_mfma = 0)
		if(!noMfma && nRows > 0)
			return launch_tsmm_decompressed(b, dOut, dNnz, "the decode plan exceeds LDS");
		int DT = 256;
		while(DT > 8 && (size_t) DT * nCols * 8 > (size_t) 96 * 1024) DT /= 2;
		if((size_t) DT * nCols * 8 > (size_t) 96 * 1024 || (int64_t) nCols * (nCols + 1) / 2 > 24 * 256)
			return launch_tsmm_decompressed(b, dOut, dNnz, "more than 110 columns with a group of more than 32 columns that has no per-pair form");
		if(DT > SDC_TILE) DT = SDC_TILE;
		const int64_t nTiles = (nRows + DT - 1) / DT;
		int tpb = 1;
		while(nTiles / tpb > (int64_t) g_numCU * 16) tpb *= 2;
		const unsigned grid = (unsigned) std::max<int64_t>((nTiles + tpb - 1) / tpb, 1);
		const size_t lds = (size_t) DT * nCols * 8;
		if(nRows > 0) {
			Prof pf(b, "k_tsmm_dense", grid, 256, (long) lds, 0);
			CLA_HIP(allow_full_lds((const void*) k_tsmm_dense));
			hipLaunchKernelGGL(k_tsmm_dense, dim3(grid), dim3(256), lds, st, b->dGroups, nG, b->dConstV, nRows, nCols, DT,
				tpb, dOut);
		}
		Prof pf(b, "k_tsmm_finish", 1, 256, 0, 0);
		hipLaunchKernelGGL(k_tsmm_finish, dim3(1), dim3(256), 0, st, dOut, nCols, b->dConstV, b->dConstV, (double) nRows, 0, dNnz);
		CLA_HIP(hipGetLastError());
		return 0;
	}

	// scratch: colSum (nCols doubles) | pair list (one int4 per pair of groups)
	const size_t sumBytes = (sizeof(double) * (size_t) nCols + 255) & ~(size_t) 255;
	const size_t pairBytes = sizeof(int4) * ((size_t) nG * (nG > 0 ? nG - 1 : 0) / 2 + 1);
	if((rc = ensure_scratch(b, sumBytes + pairBytes))) return rc;
	double* dColSum = (double*) b->dScratch;
	int4* dPairs = (int4*) ((char*) b->dScratch + sumBytes);
	CLA_HIP(hipMemsetAsync(dColSum, 0, sizeof(double) * (size_t) nCols, st));
	if((rc = ensure_counts(b))) return rc;
	if(nG > 0) {
		Prof pf(b, "k_tsmm_self", nG, 256, 0, 0);
		hipLaunchKernelGGL(k_tsmm_self, dim3(1, nG), dim3(256), 0, st, b->dGroups, b->dCountsAll, dOut, nCols, dColSum);
	}
	const int nTiles = (int) ((nRows + TT - 1) / TT);
	// Pairs of DDC groups with one or two columns each, equal code width and both dictionaries
	// in LDS take the dot-form kernel (one launch per shape); the others the pre-aggregate kernel.
	struct DotShape { int cw, nct, ncs; std::vector<int4> list; };
	std::vector<DotShape> dots;
	std::vector<int4> pairs;
	size_t ldsMax = 0, dotLds = 0;
	for(int g = 0; g < nG && nRows > 0; g++)
		for(int h = g + 1; h < nG; h++) {
			if(split > 0 && (g < split) == (h < split)) continue;
			const DGroup& A = b->groups[g].d;
			const DGroup& B = b->groups[h].d;
			const size_t bothDicts = ((size_t) A.nVals * A.nColG + (size_t) B.nVals * B.nColG + 2) * 8;
			if(A.type == G_DDC && B.type == G_DDC && A.codeWidth == B.codeWidth && A.codeWidth <= 2 && A.nColG <= 2 && B.nColG <= 2 &&
				bothDicts <= (size_t) 150 * 1024 && b->opt.tsmmPairDot) {
				size_t k = 0;
				while(k < dots.size() && !(dots[k].cw == A.codeWidth && dots[k].nct == A.nColG && dots[k].ncs == B.nColG)) k++;
				if(k == dots.size()) dots.push_back(DotShape{A.codeWidth, A.nColG, B.nColG, {}});
				dots[k].list.push_back(make_int4(g, h, 0, 0));
				dotLds = std::max(dotLds, bothDicts);
				continue;
			}
			// target = side with the smaller accumulator nVals_t * nC_s
			const bool gTarget = (size_t) A.nVals * B.nColG <= (size_t) B.nVals * A.nColG;
			const int gt = gTarget ? g : h, gs = gTarget ? h : g;
			const DGroup& T = b->groups[gt].d;
			const DGroup& S = b->groups[gs].d;
			const size_t pBytes = (size_t) T.nVals * S.nColG * 8;
			const size_t dBytes = (size_t) S.nVals * S.nColG * 8;
			const size_t cBytes = (size_t) 2 * TT * 4;
			if(pBytes + cBytes > (size_t) 150 * 1024) {
				// (what the kernels above have added to dOut is dropped)
				CLA_HIP(hipMemsetAsync(dOut, 0, sizeof(double) * (size_t) nCols * nCols, st));
				return launch_tsmm_decompressed(b, dOut, dNnz, "a pair of groups whose pre-aggregate exceeds LDS");
			}
			const int dictInLds = pBytes + dBytes + cBytes <= (size_t) 150 * 1024;
			ldsMax = std::max(ldsMax, pBytes + (dictInLds ? dBytes : 0) + cBytes);
			pairs.push_back(make_int4(gt, gs, dictInLds, 0));
		}
	if(!dots.empty()) {
		// one list on the device: the shapes one after the other, then the remaining pairs
		std::vector<int4> all;
		for(auto& d : dots) all.insert(all.end(), d.list.begin(), d.list.end());
		const size_t nDot = all.size();
		all.insert(all.end(), pairs.begin(), pairs.end());
		CLA_HIP(hipMemcpyAsync(dPairs, all.data(), sizeof(int4) * all.size(), hipMemcpyHostToDevice, st));
		CLA_HIP(hipStreamSynchronize(st)); // `all` is a local: the copy must have read it
		// rows per chunk: the code streams of one chunk (all DDC groups) stay in the last-level cache
		double bytesPerRow = 0;
		for(auto& g : b->groups)
			if(g.d.type == G_DDC) bytesPerRow += g.d.codeWidth;
		int64_t chunkRows = (int64_t) (128.0 * 1024 * 1024 / std::max(bytesPerRow, 1.0));
		chunkRows = std::max<int64_t>(chunkRows / 8192 * 8192, 8192);
		const int nChunks = (int) ((nRows + chunkRows - 1) / chunkRows);
		size_t off = 0;
		for(auto& d : dots) {
			const int nP = (int) d.list.size();
			int bpcp = 1;
			while((int64_t) nChunks * nP * bpcp < (int64_t) g_numCU * 4 && chunkRows / (bpcp * 2) >= 64 * 1024) bpcp *= 2;
			const dim3 grid((unsigned) ((int64_t) nChunks * nP * bpcp));
			Prof pf(b, "k_tsmm_pair_dot", (long) grid.x, PD_THREADS, (long) dotLds, (double) nRows * 2 * d.cw * nP);
			if(d.cw == 1)
				launch_pair_dot_cw<1>(d.nct, d.ncs, grid, dotLds, st, b->dGroups, dPairs + off, nP, nRows, chunkRows, bpcp, dOut, nCols);
			else
				launch_pair_dot_cw<2>(d.nct, d.ncs, grid, dotLds, st, b->dGroups, dPairs + off, nP, nRows, chunkRows, bpcp, dOut, nCols);
			off += nP;
		}
		dPairs += nDot;
	}
	if(!pairs.empty()) {
		if(dots.empty()) {
			CLA_HIP(hipMemcpyAsync(dPairs, pairs.data(), sizeof(int4) * pairs.size(), hipMemcpyHostToDevice, st));
			CLA_HIP(hipStreamSynchronize(st)); // `pairs` is a local: the copy must have read it
		}
		// blocks per pair: fill the machine about 8x over all pairs, but keep at least 64 tiles per block.
		// A target dictionary of a handful of tuples sums most rows of a block into the same few cells, one
		// after the other, and such a sum of like values drifts with its length (about n / 2 units in the last
		// place): those pairs get blocks of 8 tiles, whose partial results add up with independent roundings.
		const int64_t want = std::max<int64_t>(1, (int64_t) g_numCU * 8 / (int64_t) pairs.size());
		bool fewCells = false;
		for(auto& pr : pairs) fewCells |= b->groups[pr.x].d.nVals <= 8;
		int bpp = fewCells ? std::max(1, nTiles / 8) : (int) std::min<int64_t>(want, std::max(1, nTiles / 64));
		const int tpb = (nTiles + bpp - 1) / bpp;
		bpp = (nTiles + tpb - 1) / tpb;
		double codeBytes = 0;
		for(auto& pr : pairs) {
			const DGroup& T = b->groups[pr.x].d;
			const DGroup& S = b->groups[pr.y].d;
			codeBytes += (double) nRows * ((T.type == G_DDC ? T.codeWidth : 0) + (S.type == G_DDC ? S.codeWidth : 0));
		}
		{
			Prof pf(b, "k_tsmm_pair", (long) bpp * (long) pairs.size(), PAIR_THREADS, (long) ldsMax, codeBytes);
			CLA_HIP(allow_full_lds((const void*) k_tsmm_pair));
			hipLaunchKernelGGL(k_tsmm_pair, dim3(bpp, (unsigned) pairs.size()), dim3(PAIR_THREADS), ldsMax, st, b->dGroups,
				dPairs, nRows, tpb, dOut, nCols);
		}
	}
	{
		Prof pf(b, "k_tsmm_finish", 1, 256, 0, 0);
		hipLaunchKernelGGL(k_tsmm_finish, dim3(1), dim3(256), 0, st, dOut, nCols, b->dConstV, dColSum, (double) nRows,
			b->hasConst ? 1 : 0, dNnz);
	}
	CLA_HIP(hipGetLastError());
	return 0;
}

// ---------------------------------------------------------------------------
// Exact integer co-occurrence N[a, b] = #{r : code_A(r) = a, code_B(r) = b}.
// 64-bit bins in HBM updated with integer atomics; block-private 32-bit bins in
// LDS first when the whole table fits.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(TSMM_THREADS) void k_cooc(const DGroup* __restrict__ groups, int ga, int gb, int64_t nRows,
	int tilesPerBlock, int useLds, unsigned long long* __restrict__ N) {
	extern __shared__ unsigned int lbins[];
	__shared__ int32_t ca[TT], cb[TT];
	const DGroup A = dgroup(groups + (ga));
	const DGroup B = dgroup(groups + (gb));
	const int tid = threadIdx.x;
	const int nBins = A.nVals * B.nVals;
	if(useLds) {
		for(int i = tid; i < nBins; i += TSMM_THREADS) lbins[i] = 0;
		__syncthreads();
	}
	const int nTiles = (int) ((nRows + TT - 1) / TT);
	const int t0 = blockIdx.x * tilesPerBlock, t1 = min(t0 + tilesPerBlock, nTiles);
	for(int tile = t0; tile < t1; tile++) {
		tile_codes(A, tile, nRows, ca);
		tile_codes(B, tile, nRows, cb);
		for(int t = tid; t < TT; t += TSMM_THREADS) {
			const int a = ca[t], c = cb[t];
			if(a >= 0 && c >= 0) {
				if(useLds) atomicAdd(&lbins[a * B.nVals + c], 1u);
				else atomicAdd(&N[(size_t) a * B.nVals + c], 1ull);
			}
		}
		__syncthreads();
	}
	if(useLds)
		for(int i = tid; i < nBins; i += TSMM_THREADS)
			if(lbins[i]) atomicAdd(&N[i], (unsigned long long) lbins[i]);
}

int launch_cooc(cla_block* b, int gA, int gB, unsigned long long* dOut) {
	const DGroup& A = b->groups[gA].d;
	const DGroup& B = b->groups[gB].d;
	if(A.type == G_UNC || B.type == G_UNC) { set_error("cooc: uncompressed groups have no codes"); return -CLA_ERR_UNSUPPORTED; }
	clear_stats(b);
	const size_t nBins = (size_t) A.nVals * B.nVals;
	CLA_HIP(hipMemsetAsync(dOut, 0, nBins * sizeof(unsigned long long), b->stream));
	if(b->nRows == 0) return 0;
	const int nTiles = (int) ((b->nRows + TT - 1) / TT);
	const int useLds = nBins * 4 <= (size_t) 48 * 1024;
	int tpb = std::max(1, nTiles / (g_numCU * 4));
	const unsigned grid = (unsigned) ((nTiles + tpb - 1) / tpb);
	const size_t lds = useLds ? nBins * 4 : 0;
	Prof pf(b, "k_cooc", grid, TSMM_THREADS, (long) lds, 0);
	hipLaunchKernelGGL(k_cooc, dim3(grid), dim3(TSMM_THREADS), lds, b->stream, b->dGroups, gA, gB, b->nRows, tpb, useLds,
		dOut);
	CLA_HIP(hipGetLastError());
	return 0;
}

// ---------------------------------------------------------------------------
// Additive decompression: out[r, c] = constV[c] + sum over groups covering c.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_decompress_fill(double* __restrict__ out, int64_t n, int nCols,
	const double* __restrict__ constV) {
	for(int64_t i = (int64_t) blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t) gridDim.x * 256) out[i] = constV[i % nCols];
}

__global__ __launch_bounds__(256) void k_decompress_rows(const DGroup* __restrict__ groups, int g, int64_t r0, int64_t r1, int nCols,
	double* __restrict__ out) {
	const DGroup G = dgroup(groups + (g));
	const int64_t idx = (int64_t) blockIdx.x * 256 + threadIdx.x;
	if(idx >= (r1 - r0) * G.nColG) return;
	const int64_t rr = idx / G.nColG, r = r0 + rr;
	const int j = (int) (idx - rr * G.nColG);
	double v;
	if(G.type == G_UNC) v = G.dense[(size_t) r * G.nColG + j];
	else {
		const int code = G.type == G_DDC ? load_code(G.codes, G.codeWidth, r) : G.runCode[rle_find(G.runStart, G.nRuns, (int32_t) r)];
		if(code < 0) return;
		v = G.dict[(size_t) code * G.nColG + j];
	}
	unsafeAtomicAdd(&out[(size_t) rr * nCols + G.cols[j]], v);
}

// The constants and all groups but the offset lists, a tile of rows at a time through LDS: a block sets its tile to the
// constants, its waves add the values of (group, 64 rows) items (a lane reads its row's code once and walks the tuple;
// a dense group is read in the order it is stored), then the block writes whole rows. The adds are LDS atomics, since
// groups may share columns. The per-group form above writes one value per row with the row stride of the matrix
// between threads, through an atomic add in HBM: 0.18 ms per column of 4 M rows.
constexpr int DCT_THREADS = 512;
__global__ __launch_bounds__(DCT_THREADS) void k_decompress_tiles(const DGroup* __restrict__ groups, int nGroups, int64_t r0, int64_t r1, int nCols,
	const double* __restrict__ constV, int tileRows, double* __restrict__ out) {
	extern __shared__ __align__(16) double dtile[];
	const int tid = threadIdx.x, lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	for(int64_t t0 = r0 + (int64_t) blockIdx.x * tileRows; t0 < r1; t0 += (int64_t) gridDim.x * tileRows) {
		const int rows = (int) min((int64_t) tileRows, r1 - t0);
		const int cells = rows * nCols, nChunks = (rows + 63) >> 6;
		for(int i = tid; i < cells; i += DCT_THREADS) dtile[i] = constV[i % nCols];
		__syncthreads();
		for(int item = wave; item < nGroups * nChunks; item += DCT_THREADS / 64) {
			const int g = item / nChunks, c0 = (item - g * nChunks) << 6;
			const DGroup G = dgroup(groups + g);
			if(G.type == G_SDCZ) continue;
			if(G.type == G_UNC) {
				const int n = min(64, rows - c0) * G.nColG;
				const double* src = G.dense + (size_t) (t0 + c0) * G.nColG;
				for(int idx = lane; idx < n; idx += 64) {
					const int rr = idx / G.nColG, j = idx - rr * G.nColG;
					unsafeAtomicAdd(&dtile[(c0 + rr) * nCols + G.cols[j]], src[idx]);
				}
				continue;
			}
			const int rr = c0 + lane;
			if(G.nVals <= 0 || rr >= rows) continue;
			const int64_t r = t0 + rr;
			const int code = G.type == G_DDC ? load_code(G.codes, G.codeWidth, r) : G.runCode[rle_find(G.runStart, G.nRuns, (int32_t) r)];
			if(code < 0) continue;
			const double* tup = G.dict + (size_t) code * G.nColG;
			for(int j = 0; j < G.nColG; j++) unsafeAtomicAdd(&dtile[rr * nCols + G.cols[j]], tup[j]);
		}
		__syncthreads();
		double* o = out + (size_t) (t0 - r0) * nCols;
		if(((uintptr_t) o & 15) == 0) { // 16 bytes per lane
			typedef double dct_f64x2 __attribute__((ext_vector_type(2)));
			for(int i = tid; i < (cells >> 1); i += DCT_THREADS) ((dct_f64x2*) o)[i] = ((const dct_f64x2*) dtile)[i];
			if((cells & 1) && tid == 0) o[cells - 1] = dtile[cells - 1];
		}
		else
			for(int i = tid; i < cells; i += DCT_THREADS) o[i] = dtile[i];
		__syncthreads();
	}
}

// rows [r0, r1) of the group go to out rows 0 .. r1 - r0; a block of list entries whose rows all lie outside leaves early
template <int W>
__global__ __launch_bounds__(256) void k_decompress_sdc(const DGroup* __restrict__ groups, int64_t r0, int64_t r1, int nCols,
	double* __restrict__ out) {
	// one launch for all offset lists with entries of W bytes (a launch per list: 5 us of work behind 6 us of launch)
	const DGroup G = dgroup(groups + blockIdx.y);
	if(G.type != G_SDCZ || G.deltaWidth != W || G.nOffsets == 0) return;
	const int chunk = blockIdx.x, wave = threadIdx.x >> 6;
	if(chunk == 0 && threadIdx.x == 0 && G.nOffsets > 0 && G.first >= r0 && G.first < r1) {
		const int code = load_code(G.codes, G.codeWidth, 0);
		for(int j = 0; j < G.nColG; j++) unsafeAtomicAdd(&out[(size_t) (G.first - r0) * nCols + G.cols[j]], G.dict[(size_t) code * G.nColG + j]);
	}
	if(chunk >= G.nCkpt) return;
	const OffState st = G.ckpt[chunk];
	if(st.row >= r1 || G.ckpt[chunk + 1].row < r0) return; // rows only grow along the list; entry nCkpt is the final state
	int32_t row = st.row, emit = st.emit;
	int32_t rows[4], didx[4];
	unsigned mask;
	const int64_t base = (int64_t) chunk * SDC_CK;
	for(int w = 0; w < wave; w++) sdc_decode256<W>(G.deltas, G.nDeltas, base + w * 256, row, emit, rows, didx, mask);
	sdc_decode256<W>(G.deltas, G.nDeltas, base + wave * 256, row, emit, rows, didx, mask);
#pragma unroll
	for(int k = 0; k < 4; k++)
		if((mask & (1u << k)) && rows[k] >= r0 && rows[k] < r1) {
			const int code = load_code(G.codes, G.codeWidth, didx[k]);
			for(int j = 0; j < G.nColG; j++)
				unsafeAtomicAdd(&out[(size_t) (rows[k] - r0) * nCols + G.cols[j]], G.dict[(size_t) code * G.nColG + j]);
		}
}

// (16-byte loads, four in flight per thread)
__global__ __launch_bounds__(256) void k_count_nnz2(const double* __restrict__ x, int64_t n, unsigned long long* __restrict__ nnz) {
	typedef double cn_f64x2 __attribute__((ext_vector_type(2)));
	int cnt = 0;
	const int64_t n2 = ((uintptr_t) x & 15) == 0 ? n >> 1 : 0; // pairs
	const cn_f64x2* x2 = (const cn_f64x2*) x;
	const int64_t stride = (int64_t) gridDim.x * 256, first = (int64_t) blockIdx.x * 256 + threadIdx.x;
	int64_t i = first;
	for(; i + 3 * stride < n2; i += 4 * stride) {
		const cn_f64x2 a = x2[i], b = x2[i + stride], c = x2[i + 2 * stride], d = x2[i + 3 * stride];
		cnt += (a.x != 0.0) + (a.y != 0.0) + (b.x != 0.0) + (b.y != 0.0) + (c.x != 0.0) + (c.y != 0.0) + (d.x != 0.0) + (d.y != 0.0);
	}
	for(; i < n2; i += stride) {
		const cn_f64x2 a = x2[i];
		cnt += (a.x != 0.0) + (a.y != 0.0);
	}
	for(int64_t j = 2 * n2 + first; j < n; j += stride) cnt += x[j] != 0.0;
	// one atomic per block (65 k atomics on the one counter took 0.8 ms, whatever the size of x)
	__shared__ int part[4];
	cnt = wave_sum_i32(cnt);
	if((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = cnt;
	__syncthreads();
	if(threadIdx.x == 0) {
		const int s = part[0] + part[1] + part[2] + part[3];
		if(s) atomicAdd(nnz, (unsigned long long) s);
	}
}

// dOut[(r - r0) * nCols + c] = X[r, c] for r0 <= r < r1
int launch_decompress_rows(cla_block* b, int64_t r0, int64_t r1, double* dOut) {
	const int nG = (int) b->groups.size();
	const int64_t n = (r1 - r0) * b->nCols;
	hipStream_t st = b->stream;
	if(n <= 0) return 0;
	// tiles of rows through LDS: 32 KB (four or more blocks per CU, whose phases overlap: 4M x 60 1.24 against 1.38 ms
	// with 64 KB), 64 KB where fewer than 16 rows would fit; whole chunks of 64 rows where 64 rows fit, at least 8 rows;
	// blocks too wide for that: group by group
	int tileRows = (int) std::min<int64_t>(512, 4096 / std::max(b->nCols, 1));
	if(tileRows < 16) tileRows = 8192 / std::max(b->nCols, 1);
	if(tileRows >= 64) tileRows &= ~63;
	const bool tiled = tileRows >= 8;
	if(tiled) {
		const int64_t nTiles = (r1 - r0 + tileRows - 1) / tileRows;
		const unsigned tg = (unsigned) std::min<int64_t>(nTiles, (int64_t) g_numCU * 8);
		const size_t lds = (size_t) tileRows * b->nCols * 8;
		Prof pf(b, "k_decompress_tiles", tg, DCT_THREADS, (long) lds, (double) n * 8);
		CLA_HIP(allow_full_lds((const void*) k_decompress_tiles));
		hipLaunchKernelGGL(k_decompress_tiles, dim3(tg), dim3(DCT_THREADS), lds, st, b->dGroups, nG, r0, r1, b->nCols, b->dConstV, tileRows, dOut);
	}
	else {
		const unsigned fg = (unsigned) std::min<int64_t>((n + 255) / 256, (int64_t) g_numCU * 64);
		Prof pf(b, "k_decompress_fill", fg, 256, 0, 0);
		hipLaunchKernelGGL(k_decompress_fill, dim3(fg), dim3(256), 0, st, dOut, n, b->nCols, b->dConstV);
	}
	int maxCkpt[3] = {0, 0, 0}; // offset lists by entry width
	for(int g = 0; g < nG; g++) {
		const DGroup& G = b->groups[g].d;
		if(G.type != G_SDCZ && tiled) continue;
		if(G.type == G_SDCZ) {
			if(G.nOffsets > 0) maxCkpt[G.deltaWidth == 1 ? 1 : 2] = std::max(maxCkpt[G.deltaWidth == 1 ? 1 : 2], std::max(G.nCkpt, 1));
		}
		else {
			const int64_t m = (r1 - r0) * G.nColG;
			if(m == 0) continue;
			Prof pf(b, "k_decompress_rows", (long) ((m + 255) / 256), 256, 0, 0);
			hipLaunchKernelGGL(k_decompress_rows, dim3((unsigned) ((m + 255) / 256)), dim3(256), 0, st, b->dGroups, g, r0, r1,
				b->nCols, dOut);
		}
	}
	if(maxCkpt[1] > 0) {
		Prof pf(b, "k_decompress_sdc", (long) maxCkpt[1] * nG, 256, 0, 0);
		hipLaunchKernelGGL(k_decompress_sdc<1>, dim3((unsigned) maxCkpt[1], (unsigned) nG), dim3(256), 0, st, b->dGroups, r0, r1, b->nCols, dOut);
	}
	if(maxCkpt[2] > 0) {
		Prof pf(b, "k_decompress_sdc", (long) maxCkpt[2] * nG, 256, 0, 0);
		hipLaunchKernelGGL(k_decompress_sdc<2>, dim3((unsigned) maxCkpt[2], (unsigned) nG), dim3(256), 0, st, b->dGroups, r0, r1, b->nCols, dOut);
	}
	CLA_HIP(hipGetLastError());
	return 0;
}

// ---------------------------------------------------------------------------
// out[rows x qv] = D[rows x m] %*% B[m x qv] for a dense row-major D (decompressed rows) on v_mfma_f64_16x16x4_f64.
// A wave takes tiles of 16 rows: lane (k4, i16) reads the four values D[row i16, 16 kk + 4 k4 ..+3] in one piece
// (16 lanes = one or two whole lines of the row) and feeds them to four instructions, whose other operand is
// B[16 kk + 4 k4 + s, 16 jt + i16] from the block's LDS copy of B (row stride 16 NQ + 4 doubles: the four rows that a
// wave reads together fall into different halves of the banks). Register v of the result is cell (4 v + k4, i16).
// ---------------------------------------------------------------------------
typedef double dg_f64x4u __attribute__((ext_vector_type(4), aligned(8)));
template <int NQ>
__global__ __launch_bounds__(256) void k_dense_rmm(const double* __restrict__ D, int64_t nRows, int m, const double* __restrict__ B, int ldb,
	int qv, double* __restrict__ out, int ldo, unsigned long long* __restrict__ nnz) {
	extern __shared__ __align__(16) double dgB[];
	constexpr int LD = 16 * NQ + 4;
	const int mPad = (m + 15) & ~15;
	const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
	const int i16 = lane & 15, k4 = lane >> 4;
	for(int i = tid; i < mPad * 16 * NQ; i += 256) {
		const int k = i / (16 * NQ), j = i - k * (16 * NQ);
		dgB[k * LD + j] = k < m && j < qv ? B[(size_t) k * ldb + j] : 0.0;
	}
	__syncthreads();
	int cnt = 0;
	const int64_t nTiles = (nRows + 15) / 16;
	for(int64_t t = (int64_t) blockIdx.x * 4 + wave; t < nTiles; t += (int64_t) gridDim.x * 4) {
		const int64_t r0 = t * 16;
		const double* drow = D + (size_t) min(r0 + i16, nRows - 1) * m; // (rows past the end: computed, not stored)
		gd_f64x4 acc[NQ];
#pragma unroll
		for(int jt = 0; jt < NQ; jt++) acc[jt] = gd_f64x4{0.0, 0.0, 0.0, 0.0};
#pragma unroll 2
		for(int kk = 0; kk < mPad; kk += 16) {
			const int kb = kk + 4 * k4;
			double a[4];
			if(kb + 3 < m) {
				const dg_f64x4u v = *(const dg_f64x4u*) (drow + kb);
				a[0] = v.x; a[1] = v.y; a[2] = v.z; a[3] = v.w;
			}
			else {
#pragma unroll
				for(int s = 0; s < 4; s++) a[s] = kb + s < m ? drow[kb + s] : 0.0;
			}
#pragma unroll
			for(int s = 0; s < 4; s++)
#pragma unroll
				for(int jt = 0; jt < NQ; jt++)
					acc[jt] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[s], dgB[(kb + s) * LD + jt * 16 + i16], acc[jt], 0, 0, 0);
		}
#pragma unroll
		for(int jt = 0; jt < NQ; jt++)
#pragma unroll
			for(int v = 0; v < 4; v++) {
				const int64_t r = r0 + 4 * v + k4;
				const int c = jt * 16 + i16;
				if(r < nRows && c < qv) {
					out[(size_t) r * ldo + c] = acc[jt][v];
					cnt += acc[jt][v] != 0.0;
				}
			}
	}
	__shared__ int part[4];
	cnt = wave_sum_i32(cnt);
	if(lane == 0) part[wave] = cnt;
	__syncthreads();
	if(tid == 0) {
		const int s = part[0] + part[1] + part[2] + part[3];
		if(s) atomicAdd(nnz, (unsigned long long) s);
	}
}

// X %*% B through decompressed chunks of rows (at most 512 MiB in the block's scratch buffer) for blocks that only the
// gather kernels per row and group would take, where B is wide: those move a table row of q values per group and row
// (or list entry) through L2, this a dense row per row. dOut (nRows x q) and *dNnz (cleared by the caller) are
// written. Returns 1 when the gather kernels are expected to be faster or the block is too wide for B in LDS.
int launch_rmm_decompressed(cla_block* b, const double* dB, int q, double* dOut, unsigned long long* dNnz) {
	const int m = b->nCols;
	const int64_t nRows = b->nRows;
	if(m > 256 || q < 16 || nRows == 0) return 1;
	int64_t rowsPerChunk = std::max<int64_t>((int64_t) 512 * 1024 * 1024 / ((int64_t) m * 8) / 1024 * 1024, 1024);
	rowsPerChunk = std::min(rowsPerChunk, (nRows + 1023) / 1024 * 1024);
	const int64_t nChunks = (nRows + rowsPerChunk - 1) / rowsPerChunk;
	{
		// gather kernels: (list entries + rows x other groups) table rows of q values at about 1.5 TB/s (measured 1.45 -
		// 2.2); here the dense rows written, read for the lists and read again at about 1 TB/s together (0.9 - 1.3)
		double entries = 0.0, lists = 0.0;
		for(auto& g : b->groups) {
			if(g.d.type == G_SDCZ) { entries += (double) g.d.nOffsets; lists += g.d.nOffsets > 0; }
			else entries += (double) nRows;
		}
		const double gather = entries * q * 8 / 1.5e12;
		const double dense = (double) nRows * m * 8 / 1.0e12 + (double) nRows * q * 8 / 4e12 + (20e-6 + lists * 1e-6) * (double) nChunks;
		if(gather <= dense) return 1;
	}
	int rc = ensure_scratch(b, sizeof(double) * (size_t) rowsPerChunk * m);
	if(rc) return rc;
	double* dense = (double*) b->dScratch;
	hipStream_t st = b->stream;
	const int mPad = (m + 15) & ~15;
	for(int64_t r0 = 0; r0 < nRows; r0 += rowsPerChunk) {
		const int64_t rows = std::min(rowsPerChunk, nRows - r0);
		if((rc = launch_decompress_rows(b, r0, r0 + rows, dense))) return rc;
		const unsigned grid = (unsigned) std::min<int64_t>(((rows + 15) / 16 + 3) / 4, (int64_t) g_numCU * 8);
		for(int c0 = 0; c0 < q; c0 += 64) {
			const int qv = std::min(64, q - c0), nq = (qv + 15) / 16;
			const size_t lds = (size_t) mPad * (16 * nq + 4) * 8;
			Prof pf(b, "k_dense_rmm", grid, 256, (long) lds, (double) rows * (m + qv) * 8);
#define DG_LAUNCH(NQV)                                                                                          \
	do {                                                                                                        \
		CLA_HIP(allow_full_lds((const void*) k_dense_rmm<NQV>));                                                \
		hipLaunchKernelGGL(k_dense_rmm<NQV>, dim3(grid), dim3(256), lds, st, dense, rows, m, dB + c0, q, qv,    \
			dOut + (size_t) r0 * q + c0, q, dNnz);                                                              \
	} while(0)
			if(nq == 1) DG_LAUNCH(1); else if(nq == 2) DG_LAUNCH(2); else if(nq == 3) DG_LAUNCH(3); else DG_LAUNCH(4);
#undef DG_LAUNCH
		}
	}
	CLA_HIP(hipGetLastError());
	return 0;
}

int launch_decompress(cla_block* b, double* dOut, unsigned long long* dNnz) {
	const int64_t nRows = b->nRows, n = nRows * b->nCols;
	hipStream_t st = b->stream;
	clear_stats(b);
	CLA_HIP(hipMemsetAsync(dNnz, 0, sizeof(unsigned long long), st));
	if(n == 0) return 0;
	const int rc = launch_decompress_rows(b, 0, nRows, dOut);
	if(rc) return rc;
	const unsigned fg = (unsigned) std::min<int64_t>((n + 255) / 256, (int64_t) g_numCU * 8);
	{
		Prof pf(b, "k_count_nnz", fg, 256, 0, (double) n * 8);
		hipLaunchKernelGGL(k_count_nnz2, dim3(fg), dim3(256), 0, st, dOut, n, dNnz);
	}
	CLA_HIP(hipGetLastError());
	return 0;
}

} // namespace cla
