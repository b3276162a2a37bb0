// Right multiply X %*% B for wide B: fused decode + fp64 MFMA (gfx950).
//
// The pre-aggregate-then-gather scheme would move nRows x nGroups x q table
// entries through LDS; for wide B the product is a real dense contraction
// (K = number of columns of X), so rows of X are decoded on the fly
// (value = dict[code]) straight into MFMA A-operands and multiplied with B held
// in LDS. Codes are read once, the output tile is written once.
//
// v_mfma_f64_16x16x4_f64 operand layout (wave64, lane l):
//   A[i][k]: i = l % 16, k = l / 16        (one double per lane)
//   B[k][j]: k = l / 16, j = l % 16        (one double per lane)
//   D[i][j]: i = 4 * v + l / 16, j = l % 16 for accumulator register v = 0..3
// (checked on the device against a CPU product by the parity tests)
#include "../../include/cla_hip.h"
#include "cla_device.hpp"
#include <algorithm>
#include <cstring>

namespace cla {

typedef double f64x4 __attribute__((ext_vector_type(4)));

constexpr int MF_MT = 2;                     // 16-row tiles per wave
constexpr int MF_NT = 4;                     // 16-column tiles per pass (64 output columns)
constexpr int MF_BS = 80;                    // LDS row stride of the B slab in doubles: rows 32 banks apart

// decoded column c of a slab: where its values come from
struct MfCol {
	int32_t dictOff;   // offset (doubles) of the group's dictionary copy in the LDS slab, + j
	int32_t nColG;     // tuple width of the group
	int32_t group;     // group index
	int32_t pad;
};

// per decoded column, resolved for the current block (lives in LDS during a slab)
struct MfSrc {
	const uint8_t* codes; // the group's codes at the block's first row
	int32_t dictOff;
	int16_t nColG, width;
};

// slab descriptor: groups [g0,g1), decoded columns [c0, c0+nc)
struct MfSlab {
	int32_t g0, g1, c0, nc;
	int32_t dictDoubles, pad0, pad1, pad2;
};

// LDS layout of a slab:
//   dictS  the slab's dictionaries back to back behind one zero double
//   Bs     B rows of the slab's decoded columns, row stride MF_BS doubles
//   offS   per decoded column an "offset tile": for each of the block's rows the
//          position in dictS of that row's value (dictOff + code * nColG + j), as
//          uint16 — the whole decode of an A operand is then two dependent LDS
//          reads (offset, value) and no arithmetic. Padding columns and rows
//          beyond the block's end point at the zero double.
template <int MF_WAVES>
__global__ __launch_bounds__(MF_WAVES * 64) void k_rmm_mfma(const DGroup* __restrict__ groups,
	const MfSlab* __restrict__ slabs, int nSlabs, const MfCol* __restrict__ cols, const int32_t* __restrict__ colGlobal,
	const double* __restrict__ B, int q, int n0, const double* __restrict__ constRow, double* __restrict__ out,
	int64_t nRows, int ldsDictDoubles, int ldsKc, unsigned long long* __restrict__ nnz) {
	constexpr int MF_THREADS = MF_WAVES * 64;
	constexpr int MF_ROWS = MF_WAVES * MF_MT * 16; // rows per block
	extern __shared__ double smem[];
	double* dictS = smem;                                   // ldsDictDoubles
	double* Bs = dictS + ldsDictDoubles;                    // ldsKc rows of MF_BS doubles
	MfSrc* srcS = (MfSrc*) (Bs + (size_t) ldsKc * MF_BS);    // ldsKc
	uint16_t* offS = (uint16_t*) (srcS + ldsKc);            // ldsKc tiles of MF_ROWS offsets

	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const int64_t blockRow0 = (int64_t) blockIdx.x * MF_ROWS;
	const int rowsHere = (int) min((int64_t) MF_ROWS, nRows - blockRow0);
	const int li = lane & 15, lk = lane >> 4;

	f64x4 acc[MF_MT][MF_NT];
#pragma unroll
	for(int m = 0; m < MF_MT; m++)
#pragma unroll
		for(int n = 0; n < MF_NT; n++) acc[m][n] = (f64x4){0.0, 0.0, 0.0, 0.0};

	for(int s = 0; s < nSlabs; s++) {
		const MfSlab sl = slabs[s];
		__syncthreads();
		if(tid == 0) dictS[0] = 0.0;
		{
			const double* src = as_global(groups[sl.g0].dict);
			const int n = sl.dictDoubles - 1;
			for(int i = tid; i < n; i += MF_THREADS) dictS[1 + i] = src[i];
		}
		const int kc = (sl.nc + 7) & ~7; // two k-steps per loop iteration below
		for(int i = tid; i < kc * 64; i += MF_THREADS) {
			const int k = i >> 6, j = i & 63;
			double v = 0.0;
			if(k < sl.nc && n0 + j < q) v = B[(size_t) colGlobal[sl.c0 + k] * q + n0 + j];
			Bs[k * MF_BS + j] = v;
		}
		// per-column source description into LDS first, so that the tile fill below
		// issues exactly one independent global load per step
		for(int c = tid; c < kc; c += MF_THREADS) {
			MfSrc src;
			src.codes = nullptr; src.dictOff = 0; src.nColG = 0; src.width = 0;
			if(c < sl.nc) {
				const MfCol mc = cols[sl.c0 + c];
				const DGroup G = dgroup(groups + (mc.group));
				src.codes = (const uint8_t*) G.codes + (size_t) blockRow0 * G.codeWidth;
				src.dictOff = mc.dictOff; src.nColG = mc.nColG; src.width = G.codeWidth;
			}
			srcS[c] = src;
		}
		__syncthreads();
		// offset tiles, four rows per step
		{
			const int nQuads = kc * (MF_ROWS / 4);
#pragma unroll 4
			for(int i = tid; i < nQuads; i += MF_THREADS) {
				const int c = i / (MF_ROWS / 4), r4 = (i - c * (MF_ROWS / 4)) * 4;
				MfSrc src = srcS[c];
				src.codes = as_global(src.codes);
				uint32_t o[4] = {0, 0, 0, 0};
				if(src.width != 0) {
					int c4[4];
					if(src.width == 1 && r4 + 3 < rowsHere) {
						const uint32_t w = *(const uint32_t*) (src.codes + r4);
#pragma unroll
						for(int t = 0; t < 4; t++) c4[t] = (w >> (8 * t)) & 0xff;
					}
					else if(src.width == 2 && r4 + 3 < rowsHere) {
						const uint2 w = *(const uint2*) (src.codes + 2 * r4);
						c4[0] = w.x & 0xffff; c4[1] = w.x >> 16; c4[2] = w.y & 0xffff; c4[3] = w.y >> 16;
					}
					else {
#pragma unroll
						for(int t = 0; t < 4; t++) c4[t] = r4 + t < rowsHere ? load_code(src.codes, src.width, r4 + t) : -1;
					}
#pragma unroll
					for(int t = 0; t < 4; t++)
						o[t] = (r4 + t < rowsHere && c4[t] >= 0) ? (uint32_t) (src.dictOff + c4[t] * src.nColG) : 0u;
				}
				uint2 packed;
				packed.x = o[0] | (o[1] << 16);
				packed.y = o[2] | (o[3] << 16);
				*(uint2*) (offS + (size_t) c * MF_ROWS + r4) = packed;
			}
		}
		__syncthreads();

		// software pipeline over k-steps of 4 decoded columns: offsets two steps ahead,
		// values and B fragments one step ahead of the MFMAs
		const uint16_t* myOff = offS + (size_t) lk * MF_ROWS + wave * (MF_MT * 16) + li;
		const double* myB = Bs + (size_t) lk * MF_BS + li;
		uint16_t o1[MF_MT], o2[MF_MT];
		double a1[MF_MT], b1[MF_NT];
#pragma unroll
		for(int m = 0; m < MF_MT; m++) o1[m] = myOff[m * 16];
#pragma unroll
		for(int m = 0; m < MF_MT; m++) o2[m] = kc > 4 ? myOff[(size_t) 4 * MF_ROWS + m * 16] : (uint16_t) 0;
#pragma unroll
		for(int m = 0; m < MF_MT; m++) a1[m] = dictS[o1[m]];
#pragma unroll
		for(int n = 0; n < MF_NT; n++) b1[n] = myB[n * 16];
		for(int kt = 0; kt < kc; kt += 4) {
			double a0[MF_MT], b0[MF_NT];
#pragma unroll
			for(int m = 0; m < MF_MT; m++) { a0[m] = a1[m]; o1[m] = o2[m]; }
#pragma unroll
			for(int n = 0; n < MF_NT; n++) b0[n] = b1[n];
			// step kt+2 offsets, step kt+1 values and B (clamped reads at the end are unused)
			const int k2 = min(kt + 8, kc - 4), k1 = min(kt + 4, kc - 4);
#pragma unroll
			for(int m = 0; m < MF_MT; m++) o2[m] = myOff[(size_t) k2 * MF_ROWS + m * 16];
#pragma unroll
			for(int m = 0; m < MF_MT; m++) a1[m] = dictS[o1[m]];
#pragma unroll
			for(int n = 0; n < MF_NT; n++) b1[n] = myB[(size_t) k1 * MF_BS + n * 16];
#pragma unroll
			for(int m = 0; m < MF_MT; m++)
#pragma unroll
				for(int n = 0; n < MF_NT; n++)
					acc[m][n] = __builtin_amdgcn_mfma_f64_16x16x4f64(a0[m], b0[n], acc[m][n], 0, 0, 0);
		}
	}

	// epilogue: + constV x B, count non-zeros, store
	int cnt = 0;
	double cadd[MF_NT];
#pragma unroll
	for(int n = 0; n < MF_NT; n++) {
		const int col = n0 + n * 16 + li;
		cadd[n] = (constRow != nullptr && col < q) ? constRow[col] : 0.0;
	}
#pragma unroll
	for(int m = 0; m < MF_MT; m++) {
#pragma unroll
		for(int v = 0; v < 4; v++) {
			const int64_t row = blockRow0 + wave * (MF_MT * 16) + m * 16 + v * 4 + lk;
#pragma unroll
			for(int n = 0; n < MF_NT; n++) {
				const int col = n0 + n * 16 + li;
				if(row < nRows && col < q) {
					const double val = acc[m][n][v] + cadd[n];
					cnt += val != 0.0;
					__builtin_nontemporal_store(val, &out[(size_t) row * q + col]);
				}
			}
		}
	}
	count_add(nnz, cnt);
}

// Host-side plan + launch. Returns 1 when the block/shape is not eligible (caller
// uses the gather path), 0 on success, negative on error.
int launch_rmm_mfma(cla_block* b, const double* dB, int q, const double* dConstRow, double* dOut,
	unsigned long long* dNnz) {
	const int nG = (int) b->groups.size();
	if(nG == 0 || b->nRows == 0) return 1;
	for(auto& g : b->groups)
		if(g.d.type != G_DDC) return 1;
	// LDS budget per slab: dictionaries + B slab + column sources + offset tiles
	// (16 waves / 100 KiB measured best on the 10M x 100 DDC block)
	int waves = 16, budgetKb = 100;
	if(const char* e = getenv("CLA_MFMA_WAVES")) waves = atoi(e) == 16 ? 16 : 8;
	if(const char* e = getenv("CLA_MFMA_LDS_KB")) budgetKb = atoi(e);
	const int MF_ROWS = waves * MF_MT * 16;
	const int MF_THREADS = waves * 64;
	const size_t budget = (size_t) std::min(g_ldsPerBlock - 1024, budgetKb * 1024);
	std::vector<MfSlab> slabs;
	std::vector<MfCol> cols;
	std::vector<int32_t> colGlobal;
	size_t maxDict = 0;
	int maxKc = 0;
	int g = 0;
	while(g < nG) {
		MfSlab sl;
		memset(&sl, 0, sizeof(sl));
		sl.g0 = g; sl.c0 = (int) cols.size();
		size_t dictD = 1; // the leading zero double
		int nc = 0;
		while(g < nG) {
			const DGroup& G = b->groups[g].d;
			const size_t d2 = dictD + (size_t) G.nVals * G.nColG;
			const int nc2 = nc + G.nColG;
			const int kc2 = (nc2 + 7) & ~7;
			const size_t need = d2 * 8 + (size_t) kc2 * MF_BS * 8 + (size_t) kc2 * sizeof(MfSrc) + (size_t) kc2 * MF_ROWS * 2;
			if(need > budget || d2 > 65535) break; // offsets are 16 bit
			for(int j = 0; j < G.nColG; j++) {
				MfCol c;
				c.dictOff = (int32_t) dictD + j; c.nColG = G.nColG; c.group = g; c.pad = 0;
				cols.push_back(c);
				colGlobal.push_back(b->groups[g].cols[j]);
			}
			dictD = d2; nc = nc2;
			g++;
		}
		if(g == sl.g0) return 1; // a single group does not fit LDS
		sl.g1 = g; sl.nc = nc; sl.dictDoubles = (int32_t) dictD;
		maxDict = std::max(maxDict, dictD);
		maxKc = std::max(maxKc, (nc + 7) & ~7);
		slabs.push_back(sl);
	}
	// even out the slabs (same count, groups spread evenly) when that still fits
	hipStream_t st = b->stream;
	const size_t metaBytes = slabs.size() * sizeof(MfSlab) + cols.size() * sizeof(MfCol) + colGlobal.size() * 4;
	int rc = ensure_scratch(b, metaBytes + 256);
	if(rc) return rc;
	char* base = (char*) b->dScratch;
	MfSlab* dSlabs = (MfSlab*) base;
	MfCol* dCols = (MfCol*) (base + slabs.size() * sizeof(MfSlab));
	int32_t* dColGlobal = (int32_t*) ((char*) dCols + cols.size() * sizeof(MfCol));
	CLA_HIP(hipMemcpyAsync(dSlabs, slabs.data(), slabs.size() * sizeof(MfSlab), hipMemcpyHostToDevice, st));
	CLA_HIP(hipMemcpyAsync(dCols, cols.data(), cols.size() * sizeof(MfCol), hipMemcpyHostToDevice, st));
	CLA_HIP(hipMemcpyAsync(dColGlobal, colGlobal.data(), colGlobal.size() * 4, hipMemcpyHostToDevice, st));
	CLA_HIP(hipStreamSynchronize(st)); // the host vectors go out of scope

	const size_t lds = maxDict * 8 + (size_t) maxKc * MF_BS * 8 + (size_t) maxKc * sizeof(MfSrc) + (size_t) maxKc * MF_ROWS * 2;
	CLA_HIP(hipFuncSetAttribute((const void*) k_rmm_mfma<8>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds));
	CLA_HIP(hipFuncSetAttribute((const void*) k_rmm_mfma<16>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds));
	const unsigned grid = (unsigned) ((b->nRows + MF_ROWS - 1) / MF_ROWS);
	double codeBytes = 0;
	for(auto& gr : b->groups) codeBytes += (double) b->nRows * gr.d.codeWidth;
	for(int n0 = 0; n0 < q; n0 += 64) {
		const int qq = std::min(64, q - n0);
		Prof pf(b, "k_rmm_mfma", grid, MF_THREADS, (long) lds, codeBytes + (double) b->nRows * qq * 8);
#define MF_LAUNCH(W)                                                                                             \
	hipLaunchKernelGGL((k_rmm_mfma<W>), dim3(grid), dim3(MF_THREADS), lds, st, b->dGroups, dSlabs,                 \
		(int) slabs.size(), dCols, dColGlobal, dB, q, n0, dConstRow, dOut, b->nRows, (int) maxDict, maxKc, dNnz)
		if(waves == 16) MF_LAUNCH(16); else MF_LAUNCH(8);
#undef MF_LAUNCH
	}
	CLA_HIP(hipGetLastError());
	return 0;
}

} // namespace cla
