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
// decoded column k) and B_b is the same for all blocks: B[column k][8 (jg / 2) + 2 j + jg % 2] for the jg-th of a
// lane's 16 accumulators, so that the four lanes of a row hold eight consecutive output columns in each pair of
// accumulators: 64 contiguous bytes per row and store instruction.
#include "../../include/cla_hip.h"
#include "cla_device.hpp"
#include <algorithm>
#include <cstring>
#include <type_traits>

namespace cla {

constexpr int MF_WAVES = 8;                  // waves per block (two per SIMD): 512-row tiles
constexpr int MF_MT = 4;                     // 16-row tiles per wave
// B slab in LDS: row k at k * MF_BK, inside it the 16 values of lane column j (accumulators jg = 0..15)
// at j * MF_BJ: the 16 distinct 16-byte pieces of a wave's read fall on 16 distinct
// bank quads (row stride 16 banks, j stride 36 banks)
constexpr int MF_BJ = 18;
constexpr int MF_BK = 4 * MF_BJ;
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
	int32_t pad;           // 1: a code stream of the slab is narrower than the tiles' width
	const double* dictSrc; // the slab's dictionaries, back to back
};

// B in the slab layout: row r of the list (decoded column rowCol[r], -1 = padding) at r * MF_BK,
// output column n0 + 8 (jg / 2) + 2 j + jg % 2 at j * MF_BJ + jg
__global__ __launch_bounds__(128) void k_mfma_blayout(const double* __restrict__ B, int q, int n0, const int32_t* __restrict__ rowCol,
	double* __restrict__ Bl) {
	const int r = blockIdx.x, t = threadIdx.x;
	if(t >= MF_BK) return;
	const int j = t / MF_BJ, jg = t - j * MF_BJ, col = n0 + 8 * (jg >> 1) + 2 * j + (jg & 1), gc = rowCol[r];
	Bl[(size_t) r * MF_BK + t] = (jg < 16 && gc >= 0 && col < q) ? B[(size_t) gc * q + col] : 0.0;
}

// LDS layout: two slab buffers, then the code streams of all decoded columns (srcS) and the slab
// descriptors (slabS), read once per block. A slab buffer holds
//   dict    the slab's dictionaries back to back behind two zero doubles
//   Bs      B rows of the slab's decoded columns (layout above)
//   info    per decoded column of the slab dictOff | nColG << 16 (0 for padding columns: they read a zero)
//   codes   per decoded column of the slab the codes of the tile's rows, W bytes each: plain copies of
//           the code streams (narrower codes are widened); rows behind the end hold 0
// A block is persistent and walks (row tile, slab) pairs, pair p in buffer p % 2. The fill of pair p + 1
// is issued in front of the multiply loop of pair p as global -> LDS loads that bypass the registers
// (global_load_lds_dwordx4: every lane fetches 16 bytes from its own address, the wave's 1 KB lands
// contiguously in LDS), in pieces of 1 KB spread over the waves; one barrier per pair. The memory latency
// of a fill is hidden under the matrix instructions, and so is the decode of an A operand (two dependent
// LDS reads: code, value; one multiply-add).
#define MF_GPTR(p) ((const __attribute__((address_space(1))) void*) (p))
#define MF_LPTR(p) ((__attribute__((address_space(3))) void*) (p))

// Code tiles of a slab through registers: a ragged last tile (rows behind the end of the matrix hold code 0) or
// code streams narrower than the tile's width (widened). Piece = 16 bytes of one column's tile per lane.
template <int W>
__device__ __attribute__((noinline)) void mf_fill_codes_slow(const MfSrc* __restrict__ src, int nc, int64_t row0, int rowsHere, int rows,
	uint8_t* __restrict__ dst, int wave, int waves, int lane) {
	const int tileBytes = rows * W, total = nc * tileBytes;
	for(int byte = (wave * 64 + lane) * 16; byte < total; byte += waves * 1024) {
		const int c = byte / tileBytes, off = byte - c * tileBytes;
		const MfSrc ms = src[c];
		const uint8_t* codes = as_global(ms.codes) + (size_t) row0 * ms.width;
		const int r0 = off / W;
		uint32_t e[4] = {0, 0, 0, 0};
		for(int t = 0; t < 16 / W; t++) {
			const uint32_t code = r0 + t < rowsHere ? (uint32_t) load_code(codes, ms.width, r0 + t) : 0u;
			e[(t * W) >> 2] |= code << (8 * ((t * W) & 3));
		}
		*(u32x4*) (dst + byte) = u32x4{e[0], e[1], e[2], e[3]};
	}
}

// keep: lanes outside the banks of BANK (bit k = lanes 4 k .. 4 k + 3 of every row of 16 lanes) keep their own
// `keep`, the others take `from` of the lane that CTRL names
template <int CTRL, int BANK>
__device__ __forceinline__ double mf_dpp_merge(double keep, double from) {
	int k[2], f[2];
	__builtin_memcpy(k, &keep, 8);
	__builtin_memcpy(f, &from, 8);
	k[0] = __builtin_amdgcn_update_dpp(k[0], f[0], CTRL, 0xf, BANK, false);
	k[1] = __builtin_amdgcn_update_dpp(k[1], f[1], CTRL, 0xf, BANK, false);
	double r;
	__builtin_memcpy(&r, k, 8);
	return r;
}

// NQ: quarters of the 64 output columns of a pass that B has (16 columns each): the others are neither multiplied nor
// stored (a pass costs 0.7 ms of fill, decode and output + 0.5 ms per quarter on C2)
template <int WAVES, int W, int NQ = 4>
__global__ __launch_bounds__(WAVES * 64) void k_rmm_mfma(const MfSlab* __restrict__ slabs, int nSlabs,
	const uint32_t* __restrict__ infoG, const MfSrc* __restrict__ colSrc, int nColsAll, const double* __restrict__ Bl, int q, int n0,
	const double* __restrict__ constRow, double* __restrict__ out, int64_t nRows, int ldsDictDoubles, int ldsKc, int bufBytes,
	unsigned long long* __restrict__ nnz) {
	constexpr int THREADS = WAVES * 64;
	constexpr int ROWS = WAVES * MF_MT * 16; // rows per tile
	extern __shared__ __align__(16) double smem[];
	uint8_t* const lds = (uint8_t*) smem;
	// offsets inside a slab buffer
	const int oB = ldsDictDoubles * 8, oInfo = oB + ldsKc * MF_BK * 8, oCodes = oInfo + ldsKc * 4;
	MfSrc* srcS = (MfSrc*) (lds + 2 * (size_t) bufBytes);   // nColsAll
	MfSlab* slabS = (MfSlab*) (srcS + nColsAll);            // nSlabs

	const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int li = lane & 15, lk = lane >> 4, lj = lane & 3, lb = (lane >> 2) & 3;
	const int nTiles = (int) ((nRows + ROWS - 1) / ROWS);

	for(int c = tid; c < nColsAll; c += THREADS) srcS[c] = colSrc[c];
	for(int i = tid; i < nSlabs; i += THREADS) slabS[i] = slabs[i];
	if(tid < 4) *(double*) (lds + (size_t) (tid >> 1) * bufBytes + (tid & 1) * 8) = 0.0; // the zero doubles of both buffers
	int cnt = 0;
	__syncthreads();

	// ---- fill of (tile, slab) into buffer `buf`: pieces of 1 KB spread over the waves. The three contiguous
	// regions (dictionaries, rows of B, column info) and the code tiles of a full tile whose code streams have
	// the tile's width are straight global -> LDS copies with a handful of instructions per piece (the loops are
	// kept rolled: unrolled with the ragged path inlined, the fill was 3000 instructions per pair and took a
	// seventh of the kernel's time); a ragged last tile or narrower codes go through mf_fill_codes_slow.
	// (Letting only one of the two waves of a SIMD issue a fill, so that the other keeps the matrix pipe busy
	// meanwhile, was measured slower with either assignment of waves: 2.84 / 2.91 ms against 2.79; so were two
	// single-buffered blocks of four waves per CU, one filling while the other multiplies: 3.25 ms, and two
	// double-buffered ones on half-size slabs (256-row tiles, twice the dictionary traffic from L2): 3.18 ms.)
	constexpr int FW = WAVES;
	auto copy_region = [&](const uint8_t* src, uint8_t* dst, int bytes, int fw, int rot) {
		const int ew = (fw + rot) & (FW - 1);
#pragma unroll 1
		for(int off0 = ew * 1024; off0 < bytes; off0 += FW * 1024) {
			const int off = off0 + lane * 16;
			if(off < bytes) __builtin_amdgcn_global_load_lds(MF_GPTR(as_global(src) + off), MF_LPTR(dst + off0), 16, 0, 0);
		}
	};
	auto fill = [&](int tile, int s, int buf) {
		const int fw = wave;
		const MfSlab sl = slabS[s];
		const int64_t row0 = (int64_t) tile * ROWS;
		const int rowsHere = (int) min((int64_t) ROWS, nRows - row0);
		const int kc = (sl.nc + 3) & ~3;
		uint8_t* const base = lds + (size_t) buf * bufBytes;
		// (an odd number of dictionary doubles: the last lane reads 8 bytes more; the allocation is padded)
		copy_region((const uint8_t*) sl.dictSrc, base + 16, (sl.dictDoubles - 2) * 8, fw, 0);
		copy_region((const uint8_t*) (Bl + (size_t) sl.kOff * MF_BK), base + oB, kc * MF_BK * 8, fw, 1);
		copy_region((const uint8_t*) (infoG + sl.kOff), base + oInfo, kc * 4, fw, 3);
		constexpr int TILE_BYTES = ROWS * W; // 512 or 1024 (W = 1, 2; 8 waves) / 256 or 512 (4 waves): a power of two up to 1 KB
		static_assert((TILE_BYTES & (TILE_BYTES - 1)) == 0 && TILE_BYTES <= 1024, "code tiles divide a 1 KB piece");
		const int codeBytes = sl.nc * TILE_BYTES;
		if(rowsHere == ROWS && sl.pad == 0) { // full tile, every code stream of the slab has the tile's width
			const int ew = (fw + 2) & (FW - 1);
#pragma unroll 1
			for(int off0 = ew * 1024; off0 < codeBytes; off0 += FW * 1024) {
				const int byte = off0 + lane * 16;
				const int c = byte / TILE_BYTES, off = byte & (TILE_BYTES - 1);
				if(byte < codeBytes) {
					const uint8_t* src = as_global(srcS[sl.c0 + c].codes) + (size_t) row0 * W + off;
					__builtin_amdgcn_global_load_lds(MF_GPTR(src), MF_LPTR(base + oCodes + off0), 16, 0, 0);
				}
			}
		}
		else mf_fill_codes_slow<W>(srcS + sl.c0, sl.nc, row0, rowsHere, ROWS, base + oCodes, fw, FW, lane);
	};

	// persistent block: row tiles blockIdx.x, + gridDim.x, ...
	int buf = 0;
	if((int) blockIdx.x < nTiles) fill(blockIdx.x, 0, 0);
	for(int tile = blockIdx.x; tile < nTiles; tile += gridDim.x) {
		const int64_t blockRow0 = (int64_t) tile * ROWS;
		double acc[MF_MT][4 * NQ];
#pragma unroll
		for(int m = 0; m < MF_MT; m++)
#pragma unroll
			for(int n = 0; n < 4 * NQ; n++) acc[m][n] = 0.0;

		for(int s = 0; s < nSlabs; s++, buf ^= 1) {
			const int kc = (slabS[s].nc + 3) & ~3;
			// this wave's pieces of the pair's fill have landed; behind the barrier all of them have, and
			// the other buffer's readers (the pair before) are done
			__builtin_amdgcn_s_waitcnt(0x0f70); // vmcnt(0)
			__syncthreads();
			if(s + 1 < nSlabs) fill(tile, s + 1, buf ^ 1);
			else if(tile + (int) gridDim.x < nTiles) fill(tile + gridDim.x, 0, buf ^ 1);

			const uint8_t* const base = lds + (size_t) buf * bufBytes;
			const double* dictS = (const double*) base;
			const uint32_t* infoS = (const uint32_t*) (base + oInfo);
			// software pipeline over k-steps of 4 decoded columns: codes and column info two steps ahead,
			// values one step ahead; the B fragments in quarters, each loaded while the one before is multiplied
			const uint8_t* myCode = base + oCodes + ((size_t) lk * ROWS + wave * (MF_MT * 16) + li) * W;
			constexpr size_t codeStep = (size_t) 4 * ROWS * W;
			const double* myB = (const double*) (base + oB) + (size_t) lk * MF_BK + lj * MF_BJ;
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
#define MF_QUARTER(QI, CUR, NXT, NKT, NQI)                                                                         \
				b_quarter(NKT, NQI, NXT);                                                                            \
				_Pragma("unroll") for(int m = 0; m < MF_MT; m++)                                                      \
					_Pragma("unroll") for(int n = 0; n < 4; n++)                                                      \
						acc[m][4 * QI + n] = __builtin_amdgcn_mfma_f64_4x4x4f64(a0[m], CUR[n], acc[m][4 * QI + n], 0, 0, 0);
				if constexpr(NQ == 4) {
					MF_QUARTER(0, bA, bB, kt, 1)
					MF_QUARTER(1, bB, bA, kt, 2)
					MF_QUARTER(2, bA, bB, kt, 3)
					MF_QUARTER(3, bB, bA, k1, 0)
				}
				else if constexpr(NQ == 3) {
					MF_QUARTER(0, bA, bB, kt, 1)
					MF_QUARTER(1, bB, bA, kt, 2)
					MF_QUARTER(2, bA, bB, k1, 0)
#pragma unroll
					for(int n = 0; n < 4; n++) bA[n] = bB[n];
				}
				else if constexpr(NQ == 2) {
					MF_QUARTER(0, bA, bB, kt, 1)
					MF_QUARTER(1, bB, bA, k1, 0)
				}
				else {
					MF_QUARTER(0, bA, bB, k1, 0)
#pragma unroll
					for(int n = 0; n < 4; n++) bA[n] = bB[n];
				}
#undef MF_QUARTER
			}
		}

		// epilogue: straight from the accumulators (+ constV x B, count non-zeros), without staging in LDS and
		// without a barrier. acc[m][n] of lane l is output row 16 m + 4 b + i (b = (l / 4) % 4, i = l / 16), column
		// 8 (n / 2) + 2 (l % 4) + n % 2: the four lanes of a quad hold 64 contiguous bytes of a row in each pair of
		// accumulators. Two neighbouring quads (rows r and r + 4) swap pieces through the cross-lane data path so
		// that eight lanes hold a whole 128-byte line of one row: a store instruction then writes eight full
		// lines (stores of half lines reach memory at half the rate on this device).
		//   first store:  row r,     even quad keeps its first half line, odd quad takes the even quad's second half
		//   second store: row r + 4, even quad takes the odd quad's first half, odd quad keeps its second half
		const int odd = lb & 1;
		const int64_t rowBase = blockRow0 + wave * (MF_MT * 16) + (lb & 2) * 4 + lk;
		// (the two forms are separate code: a load of constRow under a branch would put a wait for all outstanding
		// memory operations, the stores before it included, behind every store)
		auto store_rows = [&](auto withConst) {
			auto put = [&](int64_t row, int col, f64x2 v) {
				if(row >= nRows) return;
				double* const o = out + (size_t) row * q + col;
				if constexpr(decltype(withConst)::value) {
					v[0] += constRow[min(col, q - 1)];
					v[1] += constRow[min(col + 1, q - 1)];
				}
				if(col + 1 < q) {
					cnt += (v[0] != 0.0) + (v[1] != 0.0);
					__builtin_nontemporal_store(v, (f64x2*) o);
				}
				else if(col < q) {
					cnt += v[0] != 0.0;
					__builtin_nontemporal_store(v[0], o);
				}
			};
#pragma unroll
			for(int m = 0; m < MF_MT; m++) {
				const int64_t row = rowBase + 16 * m;
#pragma unroll
				for(int L = 0; L < NQ; L++) {
					const int col = n0 + 16 * L + 8 * odd + 2 * lj;
					f64x2 first, second;
					// odd quads: the second half line of the even quad four lanes below (row_shr:4 = 0x114, banks 1 and 3)
					first[0] = mf_dpp_merge<0x114, 0xa>(acc[m][4 * L], acc[m][4 * L + 2]);
					first[1] = mf_dpp_merge<0x114, 0xa>(acc[m][4 * L + 1], acc[m][4 * L + 3]);
					// even quads: the first half line of the odd quad four lanes above (row_shl:4 = 0x104, banks 0 and 2)
					second[0] = mf_dpp_merge<0x104, 0x5>(acc[m][4 * L + 2], acc[m][4 * L]);
					second[1] = mf_dpp_merge<0x104, 0x5>(acc[m][4 * L + 3], acc[m][4 * L + 1]);
					put(row, col, first);
					put(row + 4, col, second);
				}
			}
		};
		if(constRow == nullptr) store_rows(std::false_type());
		else store_rows(std::true_type());
	} // tiles
	count_add(nnz, cnt);
}

// bytes of a slab buffer: dictionaries (even count, so that the B slab is 16-byte aligned), B slab, column
// info (kc is a multiple of 4), code tiles
static size_t mf_buf_bytes(size_t dictDoubles, int kc, int width, int rows) {
	return ((dictDoubles + 1) & ~(size_t) 1) * 8 + (size_t) kc * MF_BK * 8 + (size_t) kc * 4 + (size_t) kc * rows * width;
}

// The plan of a block: slabs of groups whose dictionaries, rows of B and code tiles fit a buffer, built at the
// first call and kept on the device. Returns 1 when the block is not eligible.
static int mf_plan(cla_block* b) {
	if(b->mfState != 0) return b->mfState < 0 ? 1 : 0;
	b->mfState = -1;
	const int nG = (int) b->groups.size();
	if(nG == 0 || b->nRows == 0) return 1;
	int nColsAll = 0, blockWidth = 1; // bytes per element of the code tiles: the widest code of the block
	for(auto& g : b->groups) {
		if(g.d.type != G_DDC || g.d.codeWidth > 2) return 1; // (a dictionary behind 4-byte codes does not fit LDS)
		nColsAll += g.d.nColG;
		blockWidth = std::max(blockWidth, g.d.codeWidth);
	}
	// 8 waves per block (512-row tiles, two waves per SIMD), one block per CU with two slab buffers
	const int rows = MF_WAVES * MF_MT * 16;
	const int ldsKb = 156;
	const size_t fixedBytes = (size_t) nColsAll * sizeof(MfSrc) + 32 * sizeof(MfSlab);
	const size_t ldsTotal = (size_t) std::min(g_ldsPerBlock - 1024, ldsKb * 1024);
	if(ldsTotal < fixedBytes + 4096) return 1;
	size_t budget = (ldsTotal - fixedBytes) / 2 & ~(size_t) 15; // per slab buffer
	auto up16 = [](size_t n) { return (n + 15) & ~(size_t) 15; };

	std::vector<MfSlab> slabs;
	std::vector<uint32_t> info;  // per slab row dictOff | nColG << 16, 0 = padding
	std::vector<MfSrc> colSrc;
	std::vector<int32_t> rowCol; // B row list: global column per slab row, -1 = padding
	size_t maxDict = 0;
	int maxKc = 0;
	// first pass: how many slabs the budget needs; second pass: the columns spread evenly over them
	// (in multiples of four, the k-step), so that every fill has a whole multiply loop to hide under
	// The kernel lays a buffer out for the largest dictionary range and the largest column count of any slab,
	// which need not be the same slab: when two such buffers exceed LDS, the plan is redone on a smaller budget.
	for(int attempt = 0;; attempt++) {
		int colCap = 1 << 30;
		for(int pass = 0; pass < 2; pass++) {
			slabs.clear(); info.clear(); colSrc.clear(); rowCol.clear();
			maxDict = 0; maxKc = 0;
			int g = 0;
			while(g < nG) {
				MfSlab sl;
				memset(&sl, 0, sizeof(sl));
				sl.g0 = g; sl.c0 = (int) colSrc.size(); sl.kOff = (int) rowCol.size();
				sl.dictSrc = b->groups[g].d.dict; // the block's dictionaries lie back to back in group order
				size_t dictD = 2, goodDict = 2; // the leading zero doubles
				int nc = 0, goodG = g, goodNc = 0;
				while(g < nG) {
					const DGroup& G = b->groups[g].d;
					const size_t d2 = dictD + (size_t) G.nVals * G.nColG;
					const int nc2 = nc + G.nColG;
					const size_t need = mf_buf_bytes(d2, (nc2 + 3) & ~3, blockWidth, rows);
					if(need > budget || d2 > 65535 || G.nColG > 0x7fff) break; // dictionary offsets are 16 bit
					if(nc > 0 && nc2 > colCap) break;
					for(int j = 0; j < G.nColG; j++) {
						info.push_back((uint32_t) (dictD + j) | ((uint32_t) G.nColG << 16));
						MfSrc src;
						src.codes = (const uint8_t*) G.codes; src.width = G.codeWidth; src.pad = 0;
						colSrc.push_back(src);
						rowCol.push_back(b->groups[g].cols[j]);
					}
					dictD = d2; nc = nc2;
					g++;
					if(nc % 4 == 0) { goodG = g; goodNc = nc; goodDict = dictD; }
				}
				if(g == sl.g0) return 1; // a single group does not fit LDS
				// a slab that is not the last ends on a multiple of four columns if it can
				if(g < nG && nc % 4 != 0 && goodG > sl.g0) {
					info.resize(info.size() - (size_t) (nc - goodNc));
					colSrc.resize(colSrc.size() - (size_t) (nc - goodNc));
					rowCol.resize(rowCol.size() - (size_t) (nc - goodNc));
					g = goodG; nc = goodNc; dictD = goodDict;
				}
				sl.g1 = g; sl.nc = nc; sl.dictDoubles = (int32_t) dictD; sl.width = blockWidth;
				sl.pad = 0; // 1: some code stream of the slab is narrower than the tiles (no plain copy)
				for(int gg = sl.g0; gg < g; gg++)
					if(b->groups[gg].d.codeWidth != blockWidth) sl.pad = 1;
				while(rowCol.size() % 4) { rowCol.push_back(-1); info.push_back(0); }
				maxDict = std::max(maxDict, (dictD + 1) & ~(size_t) 1);
				maxKc = std::max(maxKc, (nc + 3) & ~3);
				slabs.push_back(sl);
			}
			if(slabs.size() > 32) return 1;
			if(pass == 0) colCap = std::max(4, (int) ((nColsAll + slabs.size() - 1) / slabs.size() + 3) / 4 * 4);
		}
		if(2 * up16(mf_buf_bytes(maxDict, maxKc, blockWidth, rows)) + fixedBytes <= ldsTotal) break;
		if(attempt == 8) return 1;
		budget = (budget * 3 / 4) & ~(size_t) 15;
	}
	// (colSrc is indexed by decoded column, info and rowCol by slab row: they differ by the padding rows)
	const size_t oSlabs = 0, oInfo = up16(oSlabs + slabs.size() * sizeof(MfSlab)), oSrc = up16(oInfo + info.size() * 4 + 16),
		oRowCol = up16(oSrc + colSrc.size() * sizeof(MfSrc)), total = up16(oRowCol + rowCol.size() * 4);
	char* base = nullptr;
	CLA_HIP(hipMalloc((void**) &base, total + 256));
	b->dMfPlan = base;
	b->derivedBytes += (int64_t) total + 256;
	CLA_HIP(hipMemcpy(base + oSlabs, slabs.data(), slabs.size() * sizeof(MfSlab), hipMemcpyHostToDevice));
	CLA_HIP(hipMemcpy(base + oInfo, info.data(), info.size() * 4, hipMemcpyHostToDevice));
	CLA_HIP(hipMemcpy(base + oSrc, colSrc.data(), colSrc.size() * sizeof(MfSrc), hipMemcpyHostToDevice));
	CLA_HIP(hipMemcpy(base + oRowCol, rowCol.data(), rowCol.size() * 4, hipMemcpyHostToDevice));
	b->mfOff[0] = oSlabs; b->mfOff[1] = oInfo; b->mfOff[2] = oSrc; b->mfOff[3] = oRowCol;
	b->mfNSlabs = (int) slabs.size(); b->mfNColsAll = nColsAll; b->mfWidth = blockWidth; b->mfMaxKc = maxKc;
	b->mfNRowCol = (int) rowCol.size(); b->mfMaxDict = (int) maxDict;
	b->mfBufBytes = up16(mf_buf_bytes(maxDict, maxKc, blockWidth, rows));
	b->mfState = 1;
	return 0;
}

// Plan (once per block) + launch. Returns 1 when the block/shape is not eligible (caller
// uses the gather path), 0 on success, negative on error.
int launch_rmm_mfma(cla_block* b, const double* dB, int q, const double* dConstRow, double* dOut,
	unsigned long long* dNnz) {
	int rc = mf_plan(b);
	if(rc) return rc;
	hipStream_t st = b->stream;
	const int rows = MF_WAVES * MF_MT * 16;
	if((rc = ensure_scratch(b, (size_t) b->mfNRowCol * MF_BK * 8 + 256))) return rc;
	double* dBl = (double*) b->dScratch;
	char* base = (char*) b->dMfPlan;
	const MfSlab* dSlabs = (const MfSlab*) (base + b->mfOff[0]);
	const uint32_t* dInfo = (const uint32_t*) (base + b->mfOff[1]);
	const MfSrc* dSrc = (const MfSrc*) (base + b->mfOff[2]);
	const int32_t* dRowCol = (const int32_t*) (base + b->mfOff[3]);
	const size_t lds = 2 * b->mfBufBytes + (size_t) b->mfNColsAll * sizeof(MfSrc) + (size_t) b->mfNSlabs * sizeof(MfSlab);
	if(lds > (size_t) g_ldsPerBlock) return 1;
	// persistent blocks: one per CU, each walks its row tiles
	const unsigned grid = (unsigned) std::min<int64_t>((b->nRows + rows - 1) / rows, (int64_t) g_numCU);
	double codeBytes = 0;
	for(auto& gr : b->groups) codeBytes += (double) b->nRows * gr.d.codeWidth;
	for(int n0 = 0; n0 < q; n0 += 64) {
		const int qq = std::min(64, q - n0);
		{
			Prof pf(b, "k_mfma_blayout", (long) b->mfNRowCol, 128, 0, 0);
			hipLaunchKernelGGL(k_mfma_blayout, dim3((unsigned) b->mfNRowCol), dim3(128), 0, st, dB, q, n0, dRowCol, dBl);
		}
		Prof pf(b, "k_rmm_mfma", grid, MF_WAVES * 64, (long) lds, codeBytes + (double) b->nRows * qq * 8);
		const int nq = (qq + 15) / 16; // quarters of the pass's 64 columns that B has
#define MF_LAUNCH(CW, NQV)                                                                                                     \
	do {                                                                                                                       \
		CLA_HIP(allow_full_lds((const void*) k_rmm_mfma<MF_WAVES, CW, NQV>));                                                  \
		hipLaunchKernelGGL((k_rmm_mfma<MF_WAVES, CW, NQV>), dim3(grid), dim3(MF_WAVES * 64), lds, st, dSlabs, b->mfNSlabs, dInfo, dSrc, \
			b->mfNColsAll, dBl, q, n0, dConstRow, dOut, b->nRows, b->mfMaxDict, b->mfMaxKc, (int) b->mfBufBytes, dNnz);               \
	} while(0)
#define MF_WIDTH(NQV)                                                   \
	do {                                                                \
		if(b->mfWidth == 1) MF_LAUNCH(1, NQV); else MF_LAUNCH(2, NQV); \
	} while(0)
		if(nq == 1) MF_WIDTH(1); else if(nq == 2) MF_WIDTH(2); else if(nq == 3) MF_WIDTH(3); else MF_WIDTH(4);
#undef MF_WIDTH
#undef MF_LAUNCH
	}
	CLA_HIP(hipGetLastError());
	return 0;
}

} // namespace cla
