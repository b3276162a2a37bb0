// Right multiply X %*% B for wide B: fused decode + fp64 MFMA (gfx950).
//
// The pre-aggregate-then-gather scheme would move nRows x nGroups x q table
// entries through LDS; for wide B the product is a real dense contraction
// (K = number of columns of X), so rows of X are decoded on the fly
// (value = dict[code]) straight into MFMA A-operands and multiplied with B held
// in LDS. Codes are read once, the output tile is written once.
//
// v_mfma_f64_4x4x4_f64 (four independent 4 x 4 x 4 products per instruction; on this device it
// sustains 74-77 TFLOP/s against 48 of the 16 x 16 x 4 form). Operand layout, wave64, lane l,
// block b = (l / 4) % 4:
//   A_b[i][k]: i = l % 4, k = l / 16       (one double per lane)
//   B_b[k][j]: j = l % 4, k = l / 16       (one double per lane)
//   D_b[i][j]: i = l / 16, j = l % 4       (one double per lane)
// (probed on the device with one-hot operands; checked against a CPU product by the parity tests)
// Here the four blocks are four groups of four rows (A lane l holds row l % 16 of a 16-row tile,
// decoded column k) and B_b is the same for all blocks: B[column k][4 jg + j] of output group jg.
#include "../../include/cla_hip.h"
#include "cla_device.hpp"
#include <algorithm>
#include <cstring>

namespace cla {

constexpr int MF_MT = 4;                     // 16-row tiles per wave
constexpr int MF_NJ = 16;                    // groups of 4 output columns per pass (64 output columns)
// B slab in LDS: row k at k * MF_BK, inside it the 16 values of output columns 4 jg + j (jg = 0..15)
// of lane column j at j * MF_BJ: the 16 distinct 16-byte pieces of a wave's read fall on 16 distinct
// bank quads (row stride 16 banks, j stride 36 banks)
constexpr int MF_BJ = 18;
constexpr int MF_BK = 4 * MF_BJ;
constexpr int MF_SS = 68;                    // row stride (doubles) of the output staging: 8 rows on distinct banks

// decoded column c of a slab: where its values come from
struct MfCol {
	int32_t dictOff;   // offset (doubles) of the group's dictionary copy in the LDS slab, + j
	int32_t nColG;     // tuple width of the group
	int32_t group;     // group index
	int32_t pad;
};

// code stream of a decoded column (device array: at row 0; LDS copy: at the block's first row)
struct MfSrc {
	const uint8_t* codes;
	int32_t width, pad;
};

// slab descriptor: groups [g0,g1), decoded columns [c0, c0+nc)
struct MfSlab {
	int32_t g0, g1, c0, nc;
	int32_t dictDoubles;   // two zero doubles + the dictionaries of the slab's groups
	int32_t width;         // bytes per element of the slab's code tiles (1 or 2)
	int32_t kOff;          // first row of the slab in the re-laid B
	int32_t pad;
	const double* dictSrc; // the slab's dictionaries, back to back
};

// B in the slab layout: row r of the list (decoded column rowCol[r], -1 = padding) at r * MF_BK,
// output column n0 + 4 jg + j at j * MF_BJ + jg
__global__ __launch_bounds__(128) void k_mfma_blayout(const double* __restrict__ B, int q, int n0, const int32_t* __restrict__ rowCol,
	double* __restrict__ Bl) {
	const int r = blockIdx.x, t = threadIdx.x;
	if(t >= MF_BK) return;
	const int j = t / MF_BJ, jg = t - j * MF_BJ, col = n0 + 4 * jg + j, gc = rowCol[r];
	Bl[(size_t) r * MF_BK + t] = (jg < 16 && gc >= 0 && col < q) ? B[(size_t) gc * q + col] : 0.0;
}

// LDS layout:
//   dictS   the slab's dictionaries back to back behind two zero doubles
//   Bs      B rows of the slab's decoded columns (layout above)
//   infoS   per decoded column of the slab dictOff | nColG << 16 (0 for padding columns: they read a zero)
//   srcS    code streams of all decoded columns (row 0), slabS the slab descriptors: read once per block
//   codeS   per decoded column of the slab the codes of the tile's rows, W bytes each: plain copies of
//           the code streams (narrower codes are widened); rows behind the end hold 0
// A block is persistent and walks (row tile, slab) pairs. The global loads of the next pair's fill (its
// first pieces per thread; all addresses come from LDS or kernel arguments) are issued before the
// multiply loop of the current pair and stored to LDS behind it, so the memory latency of a fill is
// hidden under the matrix instructions. The decode of an A operand is two dependent LDS reads (code,
// value) and one multiply-add, also under the matrix instructions.
template <int WAVES, int W>
__global__ __launch_bounds__(WAVES * 64) void k_rmm_mfma(const MfSlab* __restrict__ slabs, int nSlabs,
	const MfCol* __restrict__ cols, const MfSrc* __restrict__ colSrc, int nColsAll, const double* __restrict__ Bl, int q, int n0,
	const double* __restrict__ constRow, double* __restrict__ out, int64_t nRows, int ldsDictDoubles, int ldsKc,
	unsigned long long* __restrict__ nnz, int stagger) {
	constexpr int THREADS = WAVES * 64;
	constexpr int ROWS = WAVES * MF_MT * 16; // rows per tile
	extern __shared__ __align__(16) double smem[];
	double* dictS = smem;                                   // ldsDictDoubles (even)
	double* Bs = dictS + ldsDictDoubles;                    // ldsKc rows of MF_BK doubles
	uint32_t* infoS = (uint32_t*) (Bs + (size_t) ldsKc * MF_BK); // ldsKc (multiple of 4)
	MfSrc* srcS = (MfSrc*) (infoS + ldsKc);                 // nColsAll
	MfSlab* slabS = (MfSlab*) (srcS + nColsAll);            // nSlabs
	uint8_t* codeS = (uint8_t*) (slabS + ((nSlabs + 1) & ~1)); // ldsKc tiles of ROWS codes (an even count keeps them 16-byte aligned)
	double* stageS = smem;                                  // epilogue: WAVES x 8 rows x MF_SS, over the slab

	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const int li = lane & 15, lk = lane >> 4, lj = lane & 3, lb = (lane >> 2) & 3;
	const int nTiles = (int) ((nRows + ROWS - 1) / ROWS);

	for(int c = tid; c < nColsAll; c += THREADS) srcS[c] = colSrc[c];
	for(int i = tid; i < nSlabs; i += THREADS) slabS[i] = slabs[i];
	int cnt = 0;
	// The blocks all have the same work per tile and would write their output tiles at the same moments;
	// a start delay of 0-3 quarters of a tile's time spreads the output bursts over the other blocks'
	// multiply phases.
	if(stagger > 0 && nTiles > 4 * (int) gridDim.x) {
		const long long until = __builtin_readcyclecounter() + (long long) (blockIdx.x & 3) * stagger;
		while((long long) __builtin_readcyclecounter() < until) __builtin_amdgcn_s_sleep(32);
	}
	__syncthreads();

	// ---- fill of (tile, slab): issue() loads the first pieces per thread into registers, commit() stores
	// them and copies what did not fit (large slabs) directly
	constexpr int NC_ = 2, NB_ = 3, ND_ = WAVES == 8 ? 3 : 8; // 16-byte pieces per thread in flight: codes, B, dictionaries
	constexpr int perCol = ROWS * W / 16;
	u32x4 tC[NC_];
	f64x2 tB[NB_], tD[ND_];
	uint32_t tI = 0;
	// piece i of the code tiles: bytes [off, off + 16) of column c's tile
	auto code_piece = [&](const MfSlab& sl, int64_t row0, int rowsHere, int i, bool& fast, const uint8_t*& src, int& gw, int& r0, int& dst) {
		const int c = i / perCol, off = (i - c * perCol) * 16;
		const MfSrc ms = srcS[sl.c0 + c];
		gw = ms.width;
		src = as_global(ms.codes) + (size_t) row0 * gw;
		r0 = off / W;
		dst = c * ROWS * W + off;
		fast = gw == W && r0 + 16 / W <= rowsHere;
		if(fast) src += off;
	};
	auto code_slow = [&](const uint8_t* src, int gw, int r0, int rowsHere) { // widened or ragged piece
		uint32_t e[4] = {0, 0, 0, 0};
		for(int t = 0; t < 16 / W; t++) {
			const uint32_t code = r0 + t < rowsHere ? (uint32_t) load_code(src, gw, r0 + t) : 0u;
			e[(t * W) >> 2] |= code << (8 * ((t * W) & 3));
		}
		return u32x4{e[0], e[1], e[2], e[3]};
	};
	auto issue = [&](int tile, int s) {
		const MfSlab sl = slabS[s];
		const int64_t row0 = (int64_t) tile * ROWS;
		const int rowsHere = (int) min((int64_t) ROWS, nRows - row0);
		const int kc = (sl.nc + 3) & ~3;
		tI = 0;
		if(tid < sl.nc) {
			const MfCol mc = cols[sl.c0 + tid];
			tI = (uint32_t) mc.dictOff | ((uint32_t) mc.nColG << 16);
		}
#pragma unroll
		for(int k = 0; k < NC_; k++) {
			const int i = tid + k * THREADS;
			if(i < sl.nc * perCol) {
				bool fast; const uint8_t* src; int gw, r0, dst;
				code_piece(sl, row0, rowsHere, i, fast, src, gw, r0, dst);
				tC[k] = fast ? __builtin_nontemporal_load((const u32x4*) src) : code_slow(src, gw, r0, rowsHere);
			}
		}
		const f64x2* srcB = (const f64x2*) (Bl + (size_t) sl.kOff * MF_BK);
#pragma unroll
		for(int k = 0; k < NB_; k++)
			if(tid + k * THREADS < kc * (MF_BK / 2)) tB[k] = srcB[tid + k * THREADS];
		const double* srcD = as_global(sl.dictSrc);
		const int nD = sl.dictDoubles - 2;
#pragma unroll
		for(int k = 0; k < ND_; k++) {
			const int i = tid + k * THREADS;
			if(2 * i + 1 < nD) tD[k] = *(const f64x2*) (srcD + 2 * i);
			else if(2 * i < nD) tD[k] = f64x2{srcD[2 * i], 0.0};
		}
	};
	auto commit = [&](int tile, int s) {
		const MfSlab sl = slabS[s];
		const int64_t row0 = (int64_t) tile * ROWS;
		const int rowsHere = (int) min((int64_t) ROWS, nRows - row0);
		const int kc = (sl.nc + 3) & ~3;
		const int nChunksC = sl.nc * perCol, nChunksB = kc * (MF_BK / 2), nD = sl.dictDoubles - 2;
		if(tid < 2) dictS[tid] = 0.0; // (the epilogue's staging lies over it)
		if(tid < kc) infoS[tid] = tI;
		for(int c = tid + THREADS; c < kc; c += THREADS) { // (more columns in a slab than threads: never with these tiles)
			uint32_t info = 0;
			if(c < sl.nc) info = (uint32_t) cols[sl.c0 + c].dictOff | ((uint32_t) cols[sl.c0 + c].nColG << 16);
			infoS[c] = info;
		}
#pragma unroll
		for(int k = 0; k < NC_; k++) {
			const int i = tid + k * THREADS;
			if(i < nChunksC) {
				const int c = i / perCol, off = (i - c * perCol) * 16;
				*(u32x4*) (codeS + c * ROWS * W + off) = tC[k];
			}
		}
#pragma unroll
		for(int k = 0; k < NB_; k++)
			if(tid + k * THREADS < nChunksB) ((f64x2*) Bs)[tid + k * THREADS] = tB[k];
#pragma unroll
		for(int k = 0; k < ND_; k++) {
			const int i = tid + k * THREADS;
			if(2 * i < nD) *(f64x2*) (dictS + 2 + 2 * i) = tD[k]; // (an odd end writes one zero behind the dictionaries)
		}
		for(int i = tid + NC_ * THREADS; i < nChunksC; i += THREADS) {
			bool fast; const uint8_t* src; int gw, r0, dst;
			code_piece(sl, row0, rowsHere, i, fast, src, gw, r0, dst);
			*(u32x4*) (codeS + dst) = fast ? __builtin_nontemporal_load((const u32x4*) src) : code_slow(src, gw, r0, rowsHere);
		}
		const f64x2* srcB = (const f64x2*) (Bl + (size_t) sl.kOff * MF_BK);
		for(int i = tid + NB_ * THREADS; i < nChunksB; i += THREADS) ((f64x2*) Bs)[i] = srcB[i];
		const double* srcD = as_global(sl.dictSrc);
		for(int i = tid + ND_ * THREADS; 2 * i < nD; i += THREADS) {
			if(2 * i + 1 < nD) *(f64x2*) (dictS + 2 + 2 * i) = *(const f64x2*) (srcD + 2 * i);
			else dictS[2 + 2 * i] = srcD[2 * i];
		}
	};

	// persistent block: row tiles blockIdx.x, + gridDim.x, ...
	if((int) blockIdx.x < nTiles) issue(blockIdx.x, 0);
	for(int tile = blockIdx.x; tile < nTiles; tile += gridDim.x) {
		const int64_t blockRow0 = (int64_t) tile * ROWS;
		double acc[MF_MT][MF_NJ];
#pragma unroll
		for(int m = 0; m < MF_MT; m++)
#pragma unroll
			for(int n = 0; n < MF_NJ; n++) acc[m][n] = 0.0;

		for(int s = 0; s < nSlabs; s++) {
			const int kc = (slabS[s].nc + 3) & ~3;
			__syncthreads(); // the previous pair's readers (multiply loop, epilogue) are done
			commit(tile, s);
			__syncthreads();
			if(s + 1 < nSlabs) issue(tile, s + 1);
			else if(tile + (int) gridDim.x < nTiles) issue(tile + gridDim.x, 0);

			// software pipeline over k-steps of 4 decoded columns: codes and column info two steps ahead,
			// values one step ahead; the B fragments in two halves, each loaded while the other is multiplied
			const uint8_t* myCode = codeS + ((size_t) lk * ROWS + wave * (MF_MT * 16) + li) * W;
			constexpr size_t codeStep = (size_t) 4 * ROWS * W;
			const double* myB = Bs + (size_t) lk * MF_BK + lj * MF_BJ;
			auto codes_at = [&](int kt, int (&c)[MF_MT], uint32_t& info) {
				const uint8_t* p = myCode + (size_t) (kt >> 2) * codeStep;
				info = infoS[kt + lk];
#pragma unroll
				for(int m = 0; m < MF_MT; m++) c[m] = W == 1 ? (int) p[m * 16] : (int) *(const uint16_t*) (p + m * 32);
			};
			auto values_at = [&](const int (&c)[MF_MT], uint32_t info, double (&a)[MF_MT]) {
				const int dOff = (int) (info & 0xffff), nC = (int) (info >> 16);
#pragma unroll
				for(int m = 0; m < MF_MT; m++) a[m] = dictS[dOff + c[m] * nC];
			};
			// a quarter of the B fragments of step kt: output groups 4 quarter .. 4 quarter + 3
			auto b_quarter = [&](int kt, int quarter, double (&b)[4]) {
				const f64x2* p = (const f64x2*) (myB + (size_t) kt * MF_BK) + quarter * 2;
				const f64x2 v0 = p[0], v1 = p[1];
				b[0] = v0[0]; b[1] = v0[1]; b[2] = v1[0]; b[3] = v1[1];
			};
			int c1[MF_MT], c2[MF_MT];
			uint32_t i1, i2;
			double a1[MF_MT], bA[4], bB[4];
			codes_at(0, c1, i1);
			codes_at(min(4, kc - 4), c2, i2);
			values_at(c1, i1, a1);
			b_quarter(0, 0, bA);
			for(int kt = 0; kt < kc; kt += 4) {
				double a0[MF_MT];
#pragma unroll
				for(int m = 0; m < MF_MT; m++) { a0[m] = a1[m]; c1[m] = c2[m]; }
				i1 = i2;
				// step kt+2 codes, step kt+1 values (clamped reads at the end are unused)
				const int k2 = min(kt + 8, kc - 4), k1 = min(kt + 4, kc - 4);
				codes_at(k2, c2, i2);
				values_at(c1, i1, a1);
				// the B fragments in quarters, each loaded while the one before is multiplied
#define MF_QUARTER(QI, CUR, NXT, NKT, NQ)                                                                          \
				b_quarter(NKT, NQ, NXT);                                                                             \
				_Pragma("unroll") for(int m = 0; m < MF_MT; m++)                                                      \
					_Pragma("unroll") for(int n = 0; n < 4; n++)                                                      \
						acc[m][4 * QI + n] = __builtin_amdgcn_mfma_f64_4x4x4f64(a0[m], CUR[n], acc[m][4 * QI + n], 0, 0, 0);
				MF_QUARTER(0, bA, bB, kt, 1)
				MF_QUARTER(1, bB, bA, kt, 2)
				MF_QUARTER(2, bA, bB, kt, 3)
				MF_QUARTER(3, bB, bA, k1, 0)
#undef MF_QUARTER
			}
		}

		// epilogue: eight rows of a 16-row tile at a time through LDS, so that every store instruction
		// writes one whole output row; + constV x B, count non-zeros.
		// acc[m][n] of lane l is output row 16 m + 4 b + i (b = (l / 4) % 4, i = l / 16), column 4 n + l % 4.
		__syncthreads();
		// (two columns per lane and two rows per store instruction: 1 KB per instruction)
		const int col = n0 + 2 * (lane & 31), rsel = lane >> 5;
		const double cadd0 = (constRow != nullptr && col < q) ? constRow[col] : 0.0;
		const double cadd1 = (constRow != nullptr && col + 1 < q) ? constRow[col + 1] : 0.0;
		double* st = stageS + (size_t) wave * 8 * MF_SS;
#pragma unroll
		for(int m = 0; m < MF_MT; m++) {
#pragma unroll
			for(int h = 0; h < 2; h++) {
				if((lb >> 1) == h) {
					double* p = st + (size_t) ((lb & 1) * 4 + lk) * MF_SS + lj;
#pragma unroll
					for(int n = 0; n < MF_NJ; n++) p[4 * n] = acc[m][n];
				}
				__builtin_amdgcn_wave_barrier(); // same-wave LDS accesses complete in order
				const int64_t row0 = blockRow0 + wave * (MF_MT * 16) + m * 16 + h * 8 + rsel;
#pragma unroll
				for(int r = 0; r < 8; r += 2) {
					f64x2 v = *(const f64x2*) (st + (size_t) (r + rsel) * MF_SS + 2 * (lane & 31));
					v[0] += cadd0; v[1] += cadd1;
					if(row0 + r < nRows) {
						double* o = &out[(size_t) (row0 + r) * q + col];
						if(col + 1 < q) {
							cnt += (v[0] != 0.0) + (v[1] != 0.0);
							__builtin_nontemporal_store(v, (f64x2*) o);
						}
						else if(col < q) {
							cnt += v[0] != 0.0;
							__builtin_nontemporal_store(v[0], o);
						}
					}
				}
				__builtin_amdgcn_wave_barrier();
			}
		}
	} // tiles
	count_add(nnz, cnt);
}

// LDS bytes: dictionaries (even count, so that the B slab is 16-byte aligned), B slab, column info,
// code streams of all columns, code tiles
static size_t mf_lds_bytes(size_t dictDoubles, int kc, int width, int rows, int nColsAll, int nSlabs) {
	// (kc is a multiple of 4, the column sources are 16 bytes each, the slab descriptors 40: room for an even
	// number of them keeps the code tiles 16-byte aligned)
	return ((dictDoubles + 1) & ~(size_t) 1) * 8 + (size_t) kc * MF_BK * 8 + (size_t) kc * 4 + (size_t) nColsAll * sizeof(MfSrc) +
		(size_t) ((nSlabs + 1) & ~1) * sizeof(MfSlab) + (size_t) kc * rows * width;
}

// Host-side plan + launch. Returns 1 when the block/shape is not eligible (caller
// uses the gather path), 0 on success, negative on error.
int launch_rmm_mfma(cla_block* b, const double* dB, int q, const double* dConstRow, double* dOut,
	unsigned long long* dNnz) {
	const int nG = (int) b->groups.size();
	if(nG == 0 || b->nRows == 0) return 1;
	int nColsAll = 0, blockWidth = 1; // bytes per element of the code tiles: the widest code of the block
	for(auto& g : b->groups) {
		if(g.d.type != G_DDC || g.d.codeWidth > 2) return 1; // (a dictionary behind 4-byte codes does not fit LDS)
		nColsAll += g.d.nColG;
		blockWidth = std::max(blockWidth, g.d.codeWidth);
	}
	// waves per block and LDS budget per slab: 8 waves (512-row tiles, two waves per SIMD) with 100 KiB measured
	// best on the 10M x 100 DDC block (3.4 ms against 5.7 ms with 4 waves and two blocks per CU)
	int waves = 8, budgetKb = 100;
	if(const char* e = getenv("CLA_MFMA_WAVES")) waves = atoi(e) == 4 ? 4 : 8;
	if(waves == 4) budgetKb = 76;
	if(const char* e = getenv("CLA_MFMA_LDS_KB")) budgetKb = atoi(e);
	const int rows = waves * MF_MT * 16;
	const size_t budget = (size_t) std::min(g_ldsPerBlock - 1024, budgetKb * 1024);
	std::vector<MfSlab> slabs;
	std::vector<MfCol> cols;
	std::vector<MfSrc> colSrc;
	std::vector<int32_t> rowCol; // B row list: global column per slab row, -1 = padding
	size_t maxDict = 0;
	int maxKc = 0, maxWidth = 1;
	int g = 0;
	while(g < nG) {
		MfSlab sl;
		memset(&sl, 0, sizeof(sl));
		sl.g0 = g; sl.c0 = (int) cols.size(); sl.kOff = (int) rowCol.size();
		sl.dictSrc = b->groups[g].d.dict; // the block's dictionaries lie back to back in group order
		size_t dictD = 2, goodDict = 2; // the leading zero doubles
		int nc = 0, width = blockWidth, goodG = g, goodNc = 0, goodWidth = blockWidth;
		while(g < nG) {
			const DGroup& G = b->groups[g].d;
			const size_t d2 = dictD + (size_t) G.nVals * G.nColG;
			const int nc2 = nc + G.nColG;
			const int kc2 = (nc2 + 3) & ~3;
			const int w2 = blockWidth;
			const size_t need = mf_lds_bytes(d2, kc2, w2, rows, nColsAll, 32);
			if(need > budget || d2 > 65535 || G.nColG > 0x7fff) break; // dictionary offsets are 16 bit
			for(int j = 0; j < G.nColG; j++) {
				MfCol c;
				c.dictOff = (int32_t) dictD + j; c.nColG = G.nColG; c.group = g; c.pad = 0;
				cols.push_back(c);
				MfSrc src;
				src.codes = (const uint8_t*) G.codes; src.width = G.codeWidth; src.pad = 0;
				colSrc.push_back(src);
				rowCol.push_back(b->groups[g].cols[j]);
			}
			dictD = d2; nc = nc2; width = w2;
			g++;
			if(nc % 4 == 0) { goodG = g; goodNc = nc; goodDict = dictD; goodWidth = width; }
		}
		if(g == sl.g0) return 1; // a single group does not fit LDS
		// k-steps take four decoded columns: a slab that is not the last ends on a multiple of four if it can
		if(g < nG && nc % 4 != 0 && goodG > sl.g0) {
			cols.resize(cols.size() - (size_t) (nc - goodNc));
			colSrc.resize(colSrc.size() - (size_t) (nc - goodNc));
			rowCol.resize(rowCol.size() - (size_t) (nc - goodNc));
			g = goodG; nc = goodNc; dictD = goodDict; width = goodWidth;
		}
		sl.g1 = g; sl.nc = nc; sl.dictDoubles = (int32_t) dictD; sl.width = width;
		while(rowCol.size() % 4) rowCol.push_back(-1);
		maxDict = std::max(maxDict, (dictD + 1) & ~(size_t) 1);
		maxKc = std::max(maxKc, (nc + 3) & ~3);
		maxWidth = std::max(maxWidth, width);
		slabs.push_back(sl);
	}
	hipStream_t st = b->stream;
	auto up16 = [](size_t n) { return (n + 15) & ~(size_t) 15; };
	const size_t oSlabs = 0, oCols = up16(oSlabs + slabs.size() * sizeof(MfSlab)), oSrc = up16(oCols + cols.size() * sizeof(MfCol)),
		oRowCol = up16(oSrc + colSrc.size() * sizeof(MfSrc)), oBl = up16(oRowCol + rowCol.size() * 4),
		total = oBl + rowCol.size() * MF_BK * 8;
	int rc = ensure_scratch(b, total + 256);
	if(rc) return rc;
	char* base = (char*) b->dScratch;
	MfSlab* dSlabs = (MfSlab*) (base + oSlabs);
	MfCol* dCols = (MfCol*) (base + oCols);
	MfSrc* dSrc = (MfSrc*) (base + oSrc);
	int32_t* dRowCol = (int32_t*) (base + oRowCol);
	double* dBl = (double*) (base + oBl);
	CLA_HIP(hipMemcpyAsync(dSlabs, slabs.data(), slabs.size() * sizeof(MfSlab), hipMemcpyHostToDevice, st));
	CLA_HIP(hipMemcpyAsync(dCols, cols.data(), cols.size() * sizeof(MfCol), hipMemcpyHostToDevice, st));
	CLA_HIP(hipMemcpyAsync(dSrc, colSrc.data(), colSrc.size() * sizeof(MfSrc), hipMemcpyHostToDevice, st));
	CLA_HIP(hipMemcpyAsync(dRowCol, rowCol.data(), rowCol.size() * 4, hipMemcpyHostToDevice, st));
	CLA_HIP(hipStreamSynchronize(st)); // the host vectors go out of scope

	if(slabs.size() > 32) return 1; // (the plan above reserves LDS for 32 descriptors)
	const size_t lds = std::max(mf_lds_bytes(maxDict, maxKc, maxWidth, rows, nColsAll, (int) slabs.size()), (size_t) waves * 8 * MF_SS * 8);
	CLA_HIP(hipFuncSetAttribute((const void*) k_rmm_mfma<4, 1>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds));
	CLA_HIP(hipFuncSetAttribute((const void*) k_rmm_mfma<8, 1>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds));
	CLA_HIP(hipFuncSetAttribute((const void*) k_rmm_mfma<4, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds));
	CLA_HIP(hipFuncSetAttribute((const void*) k_rmm_mfma<8, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds));
	// persistent blocks: as many as fit the device at once (LDS bound), each walks its row tiles
	const int perCU = std::max(1, std::min(2, (int) ((size_t) 160 * 1024 / (lds + 512))));
	const unsigned grid = (unsigned) std::min<int64_t>((b->nRows + rows - 1) / rows, (int64_t) g_numCU * perCU);
	double codeBytes = 0;
	for(auto& gr : b->groups) codeBytes += (double) b->nRows * gr.d.codeWidth;
	// cycles between the starts of blocks: a quarter of a tile's multiply time (64 matrix instructions of about
	// 17 cycles per k-step and wave, two waves per SIMD)
	int stagger = (int) (rowCol.size() / 4) * 64 * 17 * 2 / 4;
	if(const char* e = getenv("CLA_MFMA_STAGGER")) stagger = atoi(e);
	for(int n0 = 0; n0 < q; n0 += 64) {
		const int qq = std::min(64, q - n0);
		{
			Prof pf(b, "k_mfma_blayout", (long) rowCol.size(), 128, 0, 0);
			hipLaunchKernelGGL(k_mfma_blayout, dim3((unsigned) rowCol.size()), dim3(128), 0, st, dB, q, n0, dRowCol, dBl);
		}
		Prof pf(b, "k_rmm_mfma", grid, waves * 64, (long) lds, codeBytes + (double) b->nRows * qq * 8);
#define MF_LAUNCH(WV, CW)                                                                                            \
	hipLaunchKernelGGL((k_rmm_mfma<WV, CW>), dim3(grid), dim3(WV * 64), lds, st, dSlabs, (int) slabs.size(), dCols, dSrc, \
		nColsAll, dBl, q, n0, dConstRow, dOut, b->nRows, (int) maxDict, maxKc, dNnz, stagger)
		if(waves == 8) { if(blockWidth == 1) MF_LAUNCH(8, 1); else MF_LAUNCH(8, 2); }
		else { if(blockWidth == 1) MF_LAUNCH(4, 1); else MF_LAUNCH(4, 2); }
#undef MF_LAUNCH
	}
	CLA_HIP(hipGetLastError());
	return 0;
}

} // namespace cla
