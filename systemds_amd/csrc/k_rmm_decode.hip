// Right multiply X %*% B for narrow B (2 <= q <= 16) on blocks of any group mix.
// A block owns a contiguous range of 1024-row tiles. Per tile every dictionary
// coded group gets its codes expanded into an LDS code tile (DDC: straight copy,
// prefetched one tile ahead in registers; SDCZeros: wave-wide offset decode from
// the tile index; RLE: run expansion with the run cursor carried from tile to
// tile). Each thread then decodes two rows group by group from dictionary copies
// in LDS and accumulates value x B[col, :]; B is kept in LDS in decoded column
// order. The output tile is staged in LDS and written with full-line stores.
// (Wide B on all-DDC blocks uses k_rmm_mfma instead.)
#include "../../include/cla_hip.h"
#include "cla_device.hpp"
#include <algorithm>

namespace cla {

constexpr int DEC_THREADS = 512;       // one thread per row of a half tile
constexpr int DEC_TILE = SDC_TILE;     // rows per tile = granularity of the offset tile index
constexpr int DEC_QMAX = 16;
constexpr int DEC_PF = 4;              // 16-byte code chunks a thread holds for the next tile

struct DecGroup {
	int32_t type;
	int32_t nC;
	int32_t dictOff;   // doubles, into the LDS dictionary copy (-1: dense group)
	int32_t slotOff;   // bytes, into the LDS code tiles (-1: dense group)
	int32_t slotW;     // 1 or 2 bytes per code in the tile; all ones = row has no value
	int32_t kOff;      // first decoded column of the group (row of the LDS copy of B)
	int32_t copyIdx;   // DDC with codeWidth == slotW: index in the chunk copy list, else -1
	int32_t pad;       // t(X) %*% X mode, dense group: offset of its LDS tile (doubles)
};

// Chunk copy list: DDC groups whose code tile is a plain copy of 1024 codes.
struct DecCopy {
	int32_t group;
	int32_t chunk0;    // first 16-byte chunk of this group in the flattened chunk numbering
};

// t(X) %*% X mode: where lane l of a wave finds column 16 * cb + l % 16 of a decoded row
struct DecCol {
	int32_t kind;      // 0: no such column, 1: dictionary coded group, 2: dense group, 3: constant only
	int32_t slotOff;   // kind 1: code tile (bytes); kind 2: offset of the group's dense tile (doubles)
	int32_t slotW;
	int32_t dictOff;   // kind 1: dictionary copy (doubles)
	int32_t nC, h;     // columns of the group, this column's place among them
	double constV;     // constant part of the column (SDC defaults, const groups)
};

struct DecArgs {
	const DGroup* groups;
	const DecGroup* plan;
	const DecCopy* copies;
	int nGroups, nCopies, nChunks;     // nChunks: 16-byte chunks per tile over all copy-list groups
	int dictDoubles, slotBytes, K;     // LDS sizes: dictionaries, code tiles, decoded columns
	int auxDoubles, tileDoubles;       // LDS: B copy / dense tiles, output tile / Gram tile
	const double* B;
	int q;
	const double* constRow;
	double* out;
	int64_t nRows;
	unsigned long long* nnz;
	const DecCol* cols;                // t(X) %*% X mode: 16 * NB entries
	int nCols;
};

typedef double f64x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void dec_store_code(uint8_t* slot, int w, int i, int code) {
	if(w == 1) slot[i] = (uint8_t) code;
	else ((uint16_t*) slot)[i] = (uint16_t) code;
}

// GRAM == 0: out = X %*% B. GRAM == 1: out += upper triangle of t(X) %*% X (constants
// included) for blocks of at most 16 * NB columns; the fill phase is the same, then every
// wave feeds 4 decoded rows at a time to v_mfma_f64_16x16x4_f64 (lane l: row l / 16, column
// 16 * cb + l % 16 is both the A and the B operand) and keeps the NB (NB + 1) / 2 upper tiles
// of the Gram matrix in registers until the block has walked all its row tiles.
template <int Q, int GRAM = 0, int NB = 1>
__global__ __launch_bounds__(DEC_THREADS) void k_rmm_decode(const DecArgs A) {
	extern __shared__ __align__(16) double smem[];
	constexpr int OS = Q + 1; // LDS row stride of the output tile (odd: conflict-free column access)
	double* dictS = smem;                                         // dictDoubles
	double* Bs = dictS + A.dictDoubles;                           // auxDoubles: K * Q zero padded columns of B / dense tiles
	double* otile = Bs + A.auxDoubles;                            // tileDoubles: DEC_THREADS * OS / Gram tile
	uint8_t* slots = (uint8_t*) (smem + (((size_t) A.dictDoubles + (size_t) A.auxDoubles + (size_t) A.tileDoubles + 1) & ~(size_t) 1)); // slotBytes, 16-byte aligned
	DecGroup* planS = (DecGroup*) (slots + A.slotBytes);          // nGroups
	int32_t* runBase = (int32_t*) (planS + A.nGroups);            // nGroups
	DecCopy* copyS = (DecCopy*) (runBase + A.nGroups);            // nCopies
	const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
	const DGroup* __restrict__ groups = A.groups;
	const int nGroups = A.nGroups;
	const int64_t nRows = A.nRows;

	const int nTiles = (int) ((nRows + DEC_TILE - 1) / DEC_TILE);
	const int tileBeg = (int) ((int64_t) nTiles * blockIdx.x / gridDim.x);
	const int tileEnd = (int) ((int64_t) nTiles * (blockIdx.x + 1) / gridDim.x);
	if(tileBeg >= tileEnd) return;

	// ---- once per block: plan, dictionaries, B in decoded column order, run cursors
	for(int g = tid; g < nGroups; g += DEC_THREADS) {
		planS[g] = A.plan[g];
		runBase[g] = groups[g].type == G_RLE ? rle_find(groups[g].runStart, groups[g].nRuns, (int32_t) ((int64_t) tileBeg * DEC_TILE)) : 0;
	}
	for(int i = tid; i < A.nCopies; i += DEC_THREADS) copyS[i] = A.copies[i];
	for(int i = tid; i < A.dictDoubles; i += DEC_THREADS) dictS[i] = 0.0;
	__syncthreads();
	for(int g = 0; g < nGroups; g++) {
		const DecGroup P = planS[g];
		const DGroup& G = groups[g];
		if(P.dictOff >= 0) {
			const int n = G.nVals * G.nColG;
			for(int i = tid; i < n; i += DEC_THREADS) dictS[P.dictOff + i] = G.dict[i];
		}
		if(GRAM == 0)
			for(int i = tid; i < P.nC * Q; i += DEC_THREADS) {
				const int h = i / Q, c = i - h * Q;
				Bs[(size_t) (P.kOff + h) * Q + c] = c < A.q ? A.B[(size_t) G.cols[h] * A.q + c] : 0.0;
			}
	}
	double cadd[Q];
#pragma unroll
	for(int c = 0; c < Q; c++) cadd[c] = (GRAM == 0 && A.constRow != nullptr && c < A.q) ? A.constRow[c] : 0.0;
	// Gram mode: this lane's columns and the accumulator tiles (ib <= jb, row major)
	DecCol myCol[NB];
	f64x4 gram[NB * (NB + 1) / 2];
	if(GRAM) {
#pragma unroll
		for(int cb = 0; cb < NB; cb++) myCol[cb] = A.cols[cb * 16 + (lane & 15)];
#pragma unroll
		for(int t = 0; t < NB * (NB + 1) / 2; t++) gram[t] = f64x4{0.0, 0.0, 0.0, 0.0};
	}

	// DDC code chunks of one tile, flattened over the copy list: chunk i of a thread is
	// tid + k * DEC_THREADS, so its group and place in the tile never change. Whole
	// chunks are loaded as 16 bytes one tile ahead; the ragged end of the last tile is
	// copied element-wise.
	auto chunk_place = [&](int i, const uint8_t*& src, int& dstOff, int& w, int& row) {
		int lo = 0, hi = A.nCopies - 1;
		while(lo < hi) {
			const int mid = (lo + hi + 1) >> 1;
			if(copyS[mid].chunk0 <= i) lo = mid; else hi = mid - 1;
		}
		const DecCopy C = copyS[lo];
		const DecGroup P = planS[C.group];
		w = P.slotW;
		const int ci = i - C.chunk0;
		row = ci * (16 / w);
		src = (const uint8_t*) groups[C.group].codes + (size_t) ci * 16;
		dstOff = P.slotOff + ci * 16;
	};
	auto copy_ragged = [&](const uint8_t* src, int dstOff, int w, int64_t row0) {
		for(int e = 0; e < 16 / w; e++)
			if(row0 + e < nRows) {
				if(w == 1) slots[dstOff + e] = src[e];
				else ((uint16_t*) (slots + dstOff))[e] = ((const uint16_t*) src)[e];
			}
	};
	const uint8_t* pfSrc[DEC_PF];
	int pfDst[DEC_PF], pfW[DEC_PF], pfRow[DEC_PF];
	u32x4 pf[DEC_PF];
#pragma unroll
	for(int k = 0; k < DEC_PF; k++) {
		pfSrc[k] = nullptr; pfDst[k] = 0; pfW[k] = 1; pfRow[k] = 0;
		if(tid + k * DEC_THREADS < A.nChunks) chunk_place(tid + k * DEC_THREADS, pfSrc[k], pfDst[k], pfW[k], pfRow[k]);
	}
	auto prefetch = [&](int tile) {
		const int64_t t0 = (int64_t) tile * DEC_TILE;
#pragma unroll
		for(int k = 0; k < DEC_PF; k++) {
			pf[k] = u32x4{0, 0, 0, 0};
			if(pfSrc[k] != nullptr && t0 + pfRow[k] + 16 / pfW[k] <= nRows)
				pf[k] = __builtin_nontemporal_load((const u32x4*) (pfSrc[k] + t0 * pfW[k]));
		}
	};
	prefetch(tileBeg);

	int cnt = 0;
	for(int tile = tileBeg; tile < tileEnd; tile++) {
		const int64_t t0 = (int64_t) tile * DEC_TILE;
		const int64_t rEnd = t0 + DEC_TILE;
		__syncthreads(); // previous tile's readers are done with the code tiles
		// ---- DDC tiles: prefetched chunks, then what did not fit the prefetch registers
#pragma unroll
		for(int k = 0; k < DEC_PF; k++) {
			if(pfSrc[k] == nullptr) continue;
			if(t0 + pfRow[k] + 16 / pfW[k] <= nRows) *(u32x4*) (slots + pfDst[k]) = pf[k];
			else copy_ragged(pfSrc[k] + t0 * pfW[k], pfDst[k], pfW[k], t0 + pfRow[k]);
		}
		for(int i = tid + DEC_PF * DEC_THREADS; i < A.nChunks; i += DEC_THREADS) {
			const uint8_t* src; int dstOff, w, row;
			chunk_place(i, src, dstOff, w, row);
			if(t0 + row + 16 / w <= nRows) *(u32x4*) (slots + dstOff) = __builtin_nontemporal_load((const u32x4*) (src + t0 * w));
			else copy_ragged(src + t0 * w, dstOff, w, t0 + row);
		}
		if(tile + 1 < tileEnd) prefetch(tile + 1);

		// ---- other dictionary coded groups, one wave per group
		for(int g = wave; g < nGroups; g += DEC_THREADS / 64) {
			const DecGroup P = planS[g];
			if(P.slotOff < 0 || P.copyIdx >= 0) continue;
			const DGroup& G = groups[g];
			uint8_t* slot = slots + P.slotOff;
			const int w = P.slotW;
			if(P.type == G_DDC) { // code width differs from the tile's: convert
				for(int i = lane; i < DEC_TILE; i += 64)
					if(t0 + i < nRows) dec_store_code(slot, w, i, load_code(G.codes, G.codeWidth, t0 + i));
			}
			else if(P.type == G_RLE) {
				int j = runBase[g];
				while(true) {
					const int jj = j + lane;
					const bool inTable = jj < G.nRuns;
					const int32_t s = inTable ? G.runStart[jj] : 0x7fffffff;
					const int32_t e = inTable ? G.runStart[jj + 1] : 0x7fffffff;
					const int32_t code = inTable ? G.runCode[jj] : -1;
					const unsigned long long valid = __ballot(inTable && s < rEnd);
					const int nv = __popcll(valid);
					if(nv <= 8) { // long runs: all lanes write each run
						for(int k = 0; k < nv; k++) {
							const int sk = max((int) (__shfl(s, k, 64) - t0), 0);
							const int ek = (int) (min((int64_t) __shfl(e, k, 64), rEnd) - t0);
							const int ck = __shfl(code, k, 64);
							for(int i = sk + lane; i < ek; i += 64) dec_store_code(slot, w, i, ck);
						}
					}
					else if(inTable && s < rEnd) { // short runs: one run per lane
						const int sk = max((int) (s - t0), 0);
						const int ek = (int) (min((int64_t) e, rEnd) - t0);
						for(int i = sk; i < ek; i++) dec_store_code(slot, w, i, code);
					}
					if(nv < 64) { j += max(nv - 1, 0); break; }      // base: last run starting before the tile end
					if(__shfl(e, 63, 64) >= rEnd) { j += 63; break; }
					j += 64;
				}
				j = min(j, G.nRuns - 1);
				if(lane == 0) runBase[g] = j;
			}
			else { // SDCZeros: rows without an entry hold the no-value code
				for(int i = lane; i < DEC_TILE; i += 64) dec_store_code(slot, w, i, 0xffff);
				if(G.nOffsets <= 0) continue;
				// same-wave LDS writes are ordered, no barrier needed between fill and scatter
				if(lane == 0 && G.first >= t0 && G.first < rEnd) dec_store_code(slot, w, (int) (G.first - t0), load_code(G.codes, G.codeWidth, 0));
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
							if((mask & (1u << k)) && rows[k] < rEnd)
								dec_store_code(slot, w, (int) (rows[k] - t0), load_code(G.codes, G.codeWidth, didx[k]));
						i0 += 256;
					}
				}
			}
		}
		if(GRAM) { // dense groups: their rows of the tile, row major per group, zero beyond the matrix
			for(int g = 0; g < nGroups; g++) {
				const DecGroup P = planS[g];
				if(P.type != G_UNC) continue;
				const double* src = groups[g].dense + (size_t) t0 * P.nC;
				const int64_t nIn = (min(nRows, rEnd) - t0) * P.nC;
				for(int i = tid; i < DEC_TILE * P.nC; i += DEC_THREADS) Bs[P.pad + i] = i < nIn ? src[i] : 0.0;
			}
		}
		__syncthreads();

		if(GRAM) {
			// wave w: rows w * 128 .. + 127 of the tile, four at a time
			const int kRow = lane >> 4;
#pragma unroll 2
			for(int st = 0; st < DEC_TILE / (DEC_THREADS / 64) / 4; st++) {
				const int rt = wave * (DEC_TILE / (DEC_THREADS / 64)) + st * 4 + kRow;
				const bool in = t0 + rt < nRows;
				double x[NB];
#pragma unroll
				for(int cb = 0; cb < NB; cb++) {
					const DecCol C = myCol[cb];
					double v = 0.0;
					if(C.kind == 1) {
						const int code = C.slotW == 1 ? (int) slots[C.slotOff + rt] : (int) ((const uint16_t*) (slots + C.slotOff))[rt];
						const bool has = in && code != (C.slotW == 1 ? 0xff : 0xffff);
						v = C.constV + (has ? dictS[C.dictOff + code * C.nC + C.h] : 0.0);
					}
					else if(C.kind == 2)
						v = C.constV + Bs[C.slotOff + rt * C.nC + C.h];
					else if(C.kind == 3)
						v = C.constV;
					x[cb] = in ? v : 0.0;
				}
				int t = 0;
#pragma unroll
				for(int ib = 0; ib < NB; ib++)
#pragma unroll
					for(int jb = ib; jb < NB; jb++, t++) gram[t] = __builtin_amdgcn_mfma_f64_16x16x4f64(x[ib], x[jb], gram[t], 0, 0, 0);
			}
			continue;
		}

		// ---- decode two rows per thread
		double acc0[Q], acc1[Q];
#pragma unroll
		for(int c = 0; c < Q; c++) { acc0[c] = 0.0; acc1[c] = 0.0; }
		const int rt0 = tid, rt1 = tid + DEC_THREADS;
		const int64_t r0 = t0 + rt0, r1 = t0 + rt1;
		const bool in0 = r0 < nRows, in1 = r1 < nRows;
		for(int g = 0; g < nGroups; g++) {
			const DecGroup P = planS[g];
			const int nC = P.nC;
			if(P.slotOff < 0) { // dense columns
				const double* dense = groups[g].dense;
				for(int h = 0; h < nC; h++) {
					const double a0 = in0 ? dense[(size_t) r0 * nC + h] : 0.0;
					const double a1 = in1 ? dense[(size_t) r1 * nC + h] : 0.0;
					const double* bq = Bs + (size_t) (P.kOff + h) * Q;
#pragma unroll
					for(int c = 0; c < Q; c++) { const double bv = bq[c]; acc0[c] += a0 * bv; acc1[c] += a1 * bv; }
				}
				continue;
			}
			int c0, c1;
			bool v0, v1;
			if(P.slotW == 1) {
				c0 = slots[P.slotOff + rt0]; c1 = slots[P.slotOff + rt1];
				v0 = in0 && c0 != 0xff; v1 = in1 && c1 != 0xff;
			}
			else {
				c0 = ((const uint16_t*) (slots + P.slotOff))[rt0]; c1 = ((const uint16_t*) (slots + P.slotOff))[rt1];
				v0 = in0 && c0 != 0xffff; v1 = in1 && c1 != 0xffff;
			}
			const double* p0 = dictS + P.dictOff + (v0 ? c0 * nC : 0);
			const double* p1 = dictS + P.dictOff + (v1 ? c1 * nC : 0);
			for(int h = 0; h < nC; h++) {
				const double a0 = p0[h], a1 = p1[h];
				const double* bq = Bs + (size_t) (P.kOff + h) * Q;
				double bv[Q];
#pragma unroll
				for(int c = 0; c < Q; c++) bv[c] = bq[c];
				if(v0) {
#pragma unroll
					for(int c = 0; c < Q; c++) acc0[c] += a0 * bv[c];
				}
				if(v1) {
#pragma unroll
					for(int c = 0; c < Q; c++) acc1[c] += a1 * bv[c];
				}
			}
		}

		// ---- output: two half tiles through LDS, full-line stores
		const int q = A.q;
#pragma unroll
		for(int half = 0; half < 2; half++) {
			if(half == 1) __syncthreads(); // the first half has been read
#pragma unroll
			for(int c = 0; c < Q; c++) otile[tid * OS + c] = (half == 0 ? acc0[c] : acc1[c]) + cadd[c];
			__syncthreads();
			const int64_t rowBase = t0 + (int64_t) half * DEC_THREADS;
			const int nr = (int) max((int64_t) 0, min((int64_t) DEC_THREADS, nRows - rowBase));
			for(int i = tid; i < nr * q; i += DEC_THREADS) {
				const int rr = i / q, c = i - rr * q;
				const double v = otile[rr * OS + c];
				cnt += v != 0.0;
				__builtin_nontemporal_store(v, A.out + (size_t) rowBase * q + i);
			}
		}
	}
	if(GRAM) {
		// Gram tiles of the block's waves summed in LDS, then one global add per cell of the
		// upper triangle. Accumulator register v of lane l is cell (4 v + l / 16, l % 16) of its tile.
		constexpr int NP = NB * 16;
		__syncthreads();
		for(int i = tid; i < NP * NP; i += DEC_THREADS) otile[i] = 0.0;
		__syncthreads();
		int t = 0;
#pragma unroll
		for(int ib = 0; ib < NB; ib++)
#pragma unroll
			for(int jb = ib; jb < NB; jb++, t++)
#pragma unroll
				for(int v = 0; v < 4; v++)
					unsafeAtomicAdd(&otile[(ib * 16 + 4 * v + (lane >> 4)) * NP + jb * 16 + (lane & 15)], gram[t][v]);
		__syncthreads();
		for(int i = tid; i < NP * NP; i += DEC_THREADS) {
			const int r = i / NP, c = i - r * NP;
			if(r <= c && c < A.nCols && otile[i] != 0.0) unsafeAtomicAdd(&A.out[(size_t) r * A.nCols + c], otile[i]);
		}
		return;
	}
	count_add(A.nnz, cnt);
}

// LDS plan shared by both modes. gram: dense groups get an LDS tile (offset in DecGroup::pad,
// doubles from the start of the aux region) instead of a share of the B copy, and groups
// without row data (const, empty) get no code tile. Returns 1 when the block does not fit.
static int dec_plan(cla_block* b, bool gram, int Q, DecArgs& A, size_t& lds, std::vector<DecGroup>& plan,
	std::vector<DecCopy>& copies) {
	const int nG = (int) b->groups.size();
	plan.assign((size_t) nG, DecGroup{});
	copies.clear();
	size_t dictD = 0, slotB = 0, denseD = 0;
	int K = 0, nChunks = 0;
	for(int g = 0; g < nG; g++) {
		const DGroup& G = b->groups[g].d;
		DecGroup& P = plan[g];
		P.type = G.type; P.nC = G.nColG; P.dictOff = -1; P.slotOff = -1; P.slotW = 0; P.copyIdx = -1; P.pad = 0;
		P.kOff = K;
		K += G.nColG;
		if(G.type == G_UNC) {
			P.pad = (int32_t) denseD;
			denseD += (size_t) DEC_TILE * G.nColG;
			continue;
		}
		if(gram && G.type != G_DDC && G.type != G_RLE && !(G.type == G_SDCZ && G.nOffsets > 0)) continue;
		if(G.nVals > 65535) return 1;
		P.dictOff = (int32_t) dictD;
		dictD += (size_t) G.nVals * G.nColG;
		P.slotW = G.nVals <= 255 ? 1 : 2;
		P.slotOff = (int32_t) slotB;
		slotB += (size_t) DEC_TILE * P.slotW;
		if(G.type == G_DDC && G.codeWidth == P.slotW && ((uintptr_t) G.codes & 15) == 0) {
			P.copyIdx = (int32_t) copies.size();
			copies.push_back(DecCopy{g, nChunks});
			nChunks += DEC_TILE * P.slotW / 16;
		}
	}
	if(dictD == 0) dictD = 1;
	const size_t aux = gram ? denseD : (size_t) K * Q;
	const size_t tileD = gram ? (size_t) Q * Q : (size_t) DEC_THREADS * (Q + 1);
	lds = (dictD + aux + tileD) * 8 + slotB + (size_t) nG * (sizeof(DecGroup) + 4) + copies.size() * sizeof(DecCopy) + 96;
	if(lds > (size_t) std::min(g_ldsPerBlock, 160 * 1024) - 1024) return 1;
	A.nGroups = nG; A.nCopies = (int) copies.size(); A.nChunks = nChunks;
	A.dictDoubles = (int) dictD; A.slotBytes = (int) ((slotB + 15) & ~(size_t) 15); A.K = K;
	A.auxDoubles = (int) aux; A.tileDoubles = (int) tileD;
	A.groups = b->dGroups; A.nRows = b->nRows;
	A.B = nullptr; A.q = 0; A.constRow = nullptr; A.out = nullptr; A.nnz = nullptr; A.cols = nullptr; A.nCols = b->nCols;
	return 0;
}

// Returns 1 when the block/shape is not eligible (caller uses the generic path).
int launch_rmm_decode(cla_block* b, const double* dB, int q, const double* dConstRow, double* dOut,
	unsigned long long* dNnz) {
	const int nG = (int) b->groups.size();
	if(nG == 0 || b->nRows == 0 || q < 2 || q > DEC_QMAX) return 1;
	const int Q = q <= 4 ? 4 : q <= 8 ? 8 : q <= 12 ? 12 : 16;
	std::vector<DecGroup> plan;
	std::vector<DecCopy> copies;
	DecArgs A;
	size_t lds;
	if(dec_plan(b, false, Q, A, lds, plan, copies)) return 1;
	const size_t planBytes = plan.size() * sizeof(DecGroup), copyBytes = copies.size() * sizeof(DecCopy);
	int rc = ensure_scratch(b, planBytes + copyBytes + 64);
	if(rc) return rc;
	DecGroup* dPlan = (DecGroup*) b->dScratch;
	DecCopy* dCopies = (DecCopy*) ((uint8_t*) b->dScratch + planBytes);
	CLA_HIP(hipMemcpyAsync(dPlan, plan.data(), planBytes, hipMemcpyHostToDevice, b->stream));
	if(copyBytes) CLA_HIP(hipMemcpyAsync(dCopies, copies.data(), copyBytes, hipMemcpyHostToDevice, b->stream));
	CLA_HIP(hipStreamSynchronize(b->stream));
	const int nTiles = (int) ((b->nRows + DEC_TILE - 1) / DEC_TILE);
	const int blocksPerCU = lds <= 76 * 1024 ? 2 : 1;
	const unsigned grid = (unsigned) std::min(nTiles, g_numCU * blocksPerCU);
	A.plan = dPlan; A.copies = dCopies;
	A.B = dB; A.q = q; A.constRow = dConstRow; A.out = dOut; A.nnz = dNnz;
	double algo = (double) b->device_bytes_cached + (double) b->nRows * q * 8;
	Prof pf(b, "k_rmm_decode", grid, DEC_THREADS, (long) lds, algo);
#define DEC_LAUNCH(QV)                                                                                          \
	do {                                                                                                        \
		CLA_HIP(hipFuncSetAttribute((const void*) k_rmm_decode<QV>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds)); \
		hipLaunchKernelGGL(k_rmm_decode<QV>, dim3(grid), dim3(DEC_THREADS), lds, b->stream, A);                 \
	} while(0)
	if(Q == 4) DEC_LAUNCH(4);
	else if(Q == 8) DEC_LAUNCH(8);
	else if(Q == 12) DEC_LAUNCH(12);
	else DEC_LAUNCH(16);
#undef DEC_LAUNCH
	CLA_HIP(hipGetLastError());
	return 0;
}

// dOut (nCols x nCols, zeroed) += upper triangle of t(D) %*% D of the decoded rows, constants
// included. Returns 1 when the block is not eligible (more than 64 columns, LDS plan too large).
int launch_tsmm_decode(cla_block* b, double* dOut) {
	const int nG = (int) b->groups.size();
	const int nCols = b->nCols;
	if(nG == 0 || b->nRows == 0 || nCols > 64) return 1;
	const int NB = (nCols + 15) / 16;
	std::vector<DecGroup> plan;
	std::vector<DecCopy> copies;
	DecArgs A;
	size_t lds;
	if(dec_plan(b, true, NB * 16, A, lds, plan, copies)) return 1;
	std::vector<DecCol> cols((size_t) NB * 16);
	for(auto& c : cols) { c.kind = 0; c.slotOff = 0; c.slotW = 1; c.dictOff = 0; c.nC = 1; c.h = 0; c.constV = 0.0; }
	for(int c = 0; c < nCols; c++) { cols[c].kind = 3; cols[c].constV = b->constV[c]; }
	for(int g = 0; g < nG; g++) {
		const DecGroup& P = plan[g];
		const auto& hc = b->groups[g].cols;
		for(int h = 0; h < P.nC; h++) {
			DecCol& C = cols[hc[h]];
			if(C.kind != 3) return 1; // overlapping groups
			C.nC = P.nC; C.h = h;
			if(P.type == G_UNC) { C.kind = 2; C.slotOff = P.pad; }
			else if(P.slotOff >= 0) { C.kind = 1; C.slotOff = P.slotOff; C.slotW = P.slotW; C.dictOff = P.dictOff; }
		}
	}
	const size_t planBytes = plan.size() * sizeof(DecGroup), copyBytes = copies.size() * sizeof(DecCopy);
	const size_t colOff = (planBytes + copyBytes + 15) & ~(size_t) 15, colBytes = cols.size() * sizeof(DecCol);
	int rc = ensure_scratch(b, colOff + colBytes + 64);
	if(rc) return rc;
	DecGroup* dPlan = (DecGroup*) b->dScratch;
	DecCopy* dCopies = (DecCopy*) ((uint8_t*) b->dScratch + planBytes);
	DecCol* dCols = (DecCol*) ((uint8_t*) b->dScratch + colOff);
	CLA_HIP(hipMemcpyAsync(dPlan, plan.data(), planBytes, hipMemcpyHostToDevice, b->stream));
	if(copyBytes) CLA_HIP(hipMemcpyAsync(dCopies, copies.data(), copyBytes, hipMemcpyHostToDevice, b->stream));
	CLA_HIP(hipMemcpyAsync(dCols, cols.data(), colBytes, hipMemcpyHostToDevice, b->stream));
	CLA_HIP(hipStreamSynchronize(b->stream));
	const int nTiles = (int) ((b->nRows + DEC_TILE - 1) / DEC_TILE);
	const int blocksPerCU = lds <= 76 * 1024 ? 2 : 1;
	const unsigned grid = (unsigned) std::min(nTiles, g_numCU * blocksPerCU);
	A.plan = dPlan; A.copies = dCopies; A.cols = dCols; A.out = dOut;
	Prof pf(b, "k_tsmm_decode", grid, DEC_THREADS, (long) lds, (double) b->device_bytes_cached);
#define GRAM_LAUNCH(NBV)                                                                                        \
	do {                                                                                                        \
		CLA_HIP(hipFuncSetAttribute((const void*) k_rmm_decode<NBV * 16, 1, NBV>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds)); \
		hipLaunchKernelGGL((k_rmm_decode<NBV * 16, 1, NBV>), dim3(grid), dim3(DEC_THREADS), lds, b->stream, A); \
	} while(0)
	if(NB == 1) GRAM_LAUNCH(1);
	else if(NB == 2) GRAM_LAUNCH(2);
	else if(NB == 3) GRAM_LAUNCH(3);
	else GRAM_LAUNCH(4);
#undef GRAM_LAUNCH
	CLA_HIP(hipGetLastError());
	return 0;
}

} // namespace cla
