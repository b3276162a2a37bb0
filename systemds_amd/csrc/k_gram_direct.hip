// t(X) %*% X of blocks that are a few "varying" columns next to run-length columns, on the vector unit
// (the reference decompresses such blocks and multiplies the rows, CLALibTSMM.java:73-77; the run-length
// side replaces the per-row loop of ColGroupRLE.java:104-141 by work per run).
//
// Varying columns (NV <= 12): one value per row behind a plain stream - DDC codes of one or two bytes, the
// one-code-per-row copy of an SDCZeros group (0xff = the row has no entry), a column of an uncompressed
// group. Run-length columns (nR <= 8): columns of RLE groups, followed by run cursors (cla_runs.hpp).
//
// A wave owns a contiguous range of rows and walks it 64 rows (lane = row) at a time:
//   V x V   lane-private sums acc[i][j] += x_i x_j (NV (NV + 1) / 2 multiply-adds per row on the vector unit,
//           whose fp64 rate equals the matrix unit's and which computes neither padding nor the lower triangle),
//           reduced over the lanes once at the end of the range;
//   R x V   a run-length column is constant between two run ends; by summation by parts
//             sum_r v_a x_c = v_a(now) U_c(now) + sum over a's run ends of (v_a before - v_a behind) U_c(at that row)
//           with U_c the running sum of x_c: lanes keep U_c of their own rows, and where column a's run ends only
//           that column's sums take U_c times the step of v_a (the lanes fold their twelve U_c eight to one first,
//           so that the sums are two registers per run-length column, kept in accumulation registers); no sum over
//           the wave's lanes before the end of its range;
//   R x R   likewise with the row count in place of U_c.
// No value of a run-length column is ever looked up per row, and no one-code-per-row copy of it is read.
//
// The streams reach the wave through a ring of three chunks of 128 rows in LDS, filled by global -> LDS loads
// that bypass the registers (two chunks in flight while one is read): a wave is alone on its SIMD (the sums
// take most of the register file), so nothing else would hide the memory latency.
#include "../../include/cla_hip.h"
#include "cla_runs.hpp"
#include <algorithm>
#include <cmath>
#include <cstring>
#include <vector>

namespace cla {

constexpr int GDR_THREADS = 256;
constexpr int GDR_WAVES = GDR_THREADS / 64;
constexpr int GDR_VMAX = 12;                 // varying columns
constexpr int GDR_NP = 16 + RC_MAX;          // block tile: index < 16 varying column, 16 + a run-length column a
constexpr int GDR_WDOUBLES = 64 + 32 + RC_MAX * RC_MAX; // per wave: window values, window ends, the R x R sums
constexpr int GDR_CH = 128;                  // rows per chunk of the wave's stream ring (2 slices of 64 rows)
constexpr int GDR_NBUF = 4;                  // ring buffers per wave: one being read, three in flight
constexpr int GDR_REBASE = 128;             // chunks between two rebases of the run-length columns' running sums (a power of two)
constexpr int GDR_NI = 8;                    // at most this many 1 KB pieces per chunk and wave (8 KB per ring buffer)

struct GdrCol {            // 24 bytes
	int32_t ringOff;       // bytes from the start of a ring buffer: the column's code / value of the chunk's first row
	int32_t base8;         // bytes from the LDS base: the column's values by tuple
	int32_t stride;        // bytes per row of the stream in the ring
	int32_t col;           // column of the matrix
	int32_t pad[2];
};
struct GdrStream {         // what the ring holds per chunk: bpr * GDR_CH consecutive bytes of each stream
	const uint8_t* src;
	int32_t bpr;           // bytes per row
	int32_t piece0;        // first 16-byte piece of the stream in a ring buffer
};
struct GdrDict {           // values of one varying column by tuple: add + src[t * nC + h] for t < n, add up to fill
	const double* src;
	double add;
	int32_t n, nC, h, off, fill, pad;
};
struct GdrArgs {
	const GdrCol* cols;
	const GdrDict* dicts;
	const RunCol* runs;
	const GdrStream* streams;
	int nDicts, nV, n2, n12, nR, nStreams; // columns [0, n2) two-byte codes, [n2, n12) one-byte codes, [n12, nV) dense
	int packed;            // every code column has a stream of its own and the dense columns are one uncompressed group: the ring is columns in order
	int valDoubles;        // values by tuple
	int ringBytes;         // one ring buffer
	int64_t nRows;
	double* out;
	int nCols;
	double* acc;               // the call's only kernel: the blocks add here and the last one writes out (gram_tail)
	unsigned* done;            // its ticket counter (nullptr: the blocks add into out, the caller fills and finishes)
	unsigned long long* nnz;
};

struct GdrPlan {
	int rc = 1;            // 0 usable, 1 the block does not qualify
	void* dImg = nullptr;
	int64_t bytes = 0;
	size_t lds = 0;
	GdrArgs A;
};

// One piece of up to 1 KB global -> LDS without registers: lane l fetches 16 bytes from its own address, they land at
// the (wave-uniform) LDS address + 16 l. Written as assembly on purpose: the compiler then does not know of the LDS
// write and puts no wait for all outstanding memory operations in front of every later LDS read; the kernel waits
// itself (gdr_dma_wait) before it reads a ring buffer.
__device__ __forceinline__ void gdr_dma16(uint64_t gsrc, uint32_t ldsAddr) {
	asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(ldsAddr), "v"(gsrc) : "memory");
}
// Waits until at most `keep` of the wave's memory operations are outstanding (they complete in order: everything
// but the newest `keep` has landed).
__device__ __forceinline__ void gdr_dma_wait(int keep) {
	switch(keep) {
		case 0: asm volatile("s_waitcnt vmcnt(0)" : : : "memory"); break;
		case 1: asm volatile("s_waitcnt vmcnt(1)" : : : "memory"); break;
		case 2: asm volatile("s_waitcnt vmcnt(2)" : : : "memory"); break;
		case 3: asm volatile("s_waitcnt vmcnt(3)" : : : "memory"); break;
		case 4: asm volatile("s_waitcnt vmcnt(4)" : : : "memory"); break;
		case 5: asm volatile("s_waitcnt vmcnt(5)" : : : "memory"); break;
		case 6: asm volatile("s_waitcnt vmcnt(6)" : : : "memory"); break;
		case 7: asm volatile("s_waitcnt vmcnt(7)" : : : "memory"); break;
		default: asm volatile("s_waitcnt vmcnt(8)" : : : "memory"); break;
	}
}

typedef const __attribute__((address_space(3))) uint8_t* gdr_lp8;
typedef const __attribute__((address_space(3))) uint16_t* gdr_lp16;
typedef const __attribute__((address_space(3))) double* gdr_lpd;

// N2 columns of two-byte codes, N1 columns of one-byte codes, ND dense columns.
// SPEC: the ring holds the columns in this order, one stream per code column and the dense columns as one
// uncompressed group, so every place in it is an immediate offset. Without SPEC the code width of a column is not
// known to the compiler (N1 is 0, N2 counts all code columns): a column's place in the ring and the width of its
// code are run-time values (a 16-bit read and a mask).
template <int N2, int N1, int ND, bool SPEC, bool HASR>
__global__ __launch_bounds__(GDR_THREADS) void k_tsmm_direct(const GdrArgs A) {
	extern __shared__ __align__(16) double smem[];
	constexpr int NC = N2 + N1, NV = NC + ND;
	constexpr int NACC = NV * (NV + 1) / 2;
	// pieces of 1 KB per chunk: known with SPEC
	constexpr int NIT = SPEC ? (GDR_CH * (N2 * 2 + N1 + ND * 8) + 1023) / 1024 : GDR_NI;
	static_assert(NIT <= GDR_NI, "ring buffer of at most 8 KB");
	const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const uint8_t* const ldsBytes = (const uint8_t*) smem;
	double* const gramS = smem + A.valDoubles;
	double* const wbase = gramS + GDR_NP * GDR_NP + wave * GDR_WDOUBLES;
	double* const winVal = wbase;
	int32_t* const winEnd = (int32_t*) (wbase + 64);
	double* const rrS = wbase + 96;                 // RC_MAX x RC_MAX: where the cursor lanes put their R x R sums at the end (cell (a, b) by cursor lane b)
	// the wave's ring: GDR_NBUF buffers of ringBytes behind everything else
	const uint32_t ringBytes = (uint32_t) A.ringBytes;
	const uint32_t ring0 = (uint32_t) ((A.valDoubles + GDR_NP * GDR_NP + GDR_WAVES * GDR_WDOUBLES) * 8) + (uint32_t) wave * GDR_NBUF * ringBytes;

	for(int d = 0; d < A.nDicts; d++) {
		const GdrDict D = A.dicts[d];
		const double* __restrict__ src = as_global(D.src);
#pragma unroll 8
		for(int t = tid; t < D.fill; t += GDR_THREADS) smem[D.off + t] = D.add + (t < D.n ? src[(size_t) t * D.nC + D.h] : 0.0);
	}
	for(int i = tid; i < GDR_NP * GDR_NP; i += GDR_THREADS) gramS[i] = 0.0;
	__syncthreads();

	const int32_t nRows = (int32_t) A.nRows;
	const int nChunks = (nRows + GDR_CH - 1) / GDR_CH;
	const int nW = gridDim.x * GDR_WAVES, gw = blockIdx.x * GDR_WAVES + wave;
	const int ch0 = (int) ((int64_t) nChunks * gw / nW), ch1 = (int) ((int64_t) nChunks * (gw + 1) / nW);
	const int nR = HASR ? A.nR : 0;
	const int nI = SPEC ? NIT : (int) ((ringBytes + 1023) >> 10);

	if(ch0 < ch1) {
		// the pieces this lane fetches per chunk: global address of the next one and the bytes a chunk moves it
		// (0: the lane has no piece in that kilobyte of the ring)
		uint64_t gptr[NIT];
		int32_t gstep[NIT];
		// stream and place in it of piece p of a chunk
		auto piece_of = [&](int p, GdrStream& S, int& inStream) {
			int sIdx = 0;
			for(int t = 1; t < A.nStreams; t++)
				if(A.streams[t].piece0 <= p) sIdx = t;
			S = A.streams[sIdx];
			inStream = p - S.piece0;
			return inStream < GDR_CH * S.bpr / 16; // (false behind the last stream)
		};
#pragma unroll
		for(int k = 0; k < NIT; k++) {
			gptr[k] = 0; gstep[k] = 0;
			if(k < nI) {
				GdrStream S;
				int inS;
				if(piece_of(k * 64 + lane, S, inS)) {
					gptr[k] = (uint64_t) S.src + (uint64_t) ((int64_t) ch0 * GDR_CH * S.bpr + (int64_t) inS * 16);
					gstep[k] = GDR_CH * S.bpr;
				}
			}
		}
		// the next chunk (number ch) into ring buffer buf; returns the number of load instructions issued
		auto dma = [&](int ch, int buf) {
			int n = 0;
			const bool ragged = (ch + 1) * GDR_CH > nRows; // (uniform) the last chunk of the matrix: no piece that starts behind the end of its stream
#pragma unroll
			for(int k = 0; k < NIT; k++) {
				if(k < nI) {
					bool go = gstep[k] != 0;
					if(ragged && go) {
						GdrStream S;
						int inS;
						piece_of(k * 64 + lane, S, inS);
						go = (int64_t) ch * GDR_CH * S.bpr + (int64_t) inS * 16 < (int64_t) nRows * S.bpr;
					}
					n += __ballot(go) != 0 ? 1 : 0;
					if(go) gdr_dma16(gptr[k], ring0 + (uint32_t) buf * ringBytes + (uint32_t) k * 1024u);
					gptr[k] += (uint64_t) (uint32_t) gstep[k];
				}
			}
			return n;
		};

		// where the lane reads its row of the chunk's first slice in ring buffer 0: per class with SPEC, per column without
		const uint32_t la2 = ring0 + (uint32_t) lane * 2u, la1 = ring0 + (uint32_t) (N2 * GDR_CH * 2) + (uint32_t) lane;
		const uint32_t lad = ring0 + (uint32_t) (N2 * GDR_CH * 2 + N1 * GDR_CH) + (uint32_t) lane * (uint32_t) (ND * 8);
		uint32_t la[SPEC ? 1 : NV];
		int cstep[SPEC ? 1 : NV];
		uint32_t cmask[SPEC || NC == 0 ? 1 : NC];
		int base8[NC > 0 ? NC : 1];
#pragma unroll
		for(int i = 0; i < NV; i++) {
			const GdrCol C = A.cols[i];
			if(i < NC) base8[i] = C.base8;
			if(!SPEC) {
				la[i] = ring0 + (uint32_t) C.ringOff + (uint32_t) (lane * C.stride);
				cstep[i] = 64 * C.stride;
				if(i < NC) cmask[i] = C.col < 0 ? 0u : C.stride == 1 ? 0xffu : 0xffffu; // (a filler column: code 0 whatever it reads, which looks a zero up)
			}
		}
		double acc[NACC], T[NV];
#pragma unroll
		for(int t = 0; t < NACC; t++) acc[t] = 0.0;
#pragma unroll
		for(int c = 0; c < NV; c++) T[c] = 0.0;

		RunCursors rc;
		rc.start(A.runs, nR, winEnd, winVal, ch0 * GDR_CH, lane);
		int32_t eNext = HASR ? rc.next_end() : RC_NEVER;

		// Run-length columns by summation by parts. With U_c(l) the sum of x_c over lane l's rows since the last rebase
		// and v_a constant between two run ends,  sum_rows v_a x_c = v_a(now) U_c(now) + sum over a's run ends of
		// (v_a before - v_a behind) U_c(at the end):  where column a's run ends the lanes add U_c times the step of v_a
		// into sums H[a][c] of their own, which are summed over the lanes once, at the end of the wave's range. R x R
		// likewise with the row count in place of U_c (products v_a v_b: cursor lane b keeps cell (a, b), the steps at
		// a's run ends). A rebase
		// (every GDR_REBASE chunks and at the end) adds v_a(now) U_c and restarts U and the row count, so that the
		// terms stay of the size of a few hundred rows' sums.
		// H is kept folded: where a run ends the lanes of every group of eight fold their twelve U_c into one value per
		// lane (lane k of the group ends up with the group's sum of column k in fold0 and of column 8 + k % 4 in fold1:
		// three exchange steps that halve the number of values a lane holds), so H is two values per run-length column
		// and lane instead of twelve; the groups of eight are summed once, at the end of the wave's range.
		static_assert(NV <= 12, "two folded registers hold twelve columns");
		// H is touched where a run ends and nowhere else: it is pinned to accumulation registers (a lone wave per SIMD
		// has 256 of them next to its vector registers, and this kernel runs no matrix instruction) and moved to a
		// vector register and back around each multiply-add, so that it never competes with the row loop's sums.
		int Hr[HASR ? RC_MAX : 1][6]; // H0 low, H0 high, H1 low, H1 high; cursor lane b: the R x R cell (a, b) low, high
#pragma unroll
		for(int a = 0; a < (HASR ? RC_MAX : 1); a++)
#pragma unroll
			for(int k = 0; k < 6; k++) asm volatile("v_accvgpr_write_b32 %0, 0" : "=a"(Hr[a][k]));
		auto h_get = [&](int lo, int hi) __attribute__((always_inline)) {
			int p[2];
			asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(p[0]) : "a"(lo));
			asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(p[1]) : "a"(hi));
			double r;
			__builtin_memcpy(&r, p, 8);
			return r;
		};
		auto h_put = [&](int& lo, int& hi, double v) __attribute__((always_inline)) {
			int p[2];
			__builtin_memcpy(p, &v, 8);
			asm volatile("v_accvgpr_write_b32 %0, %1" : "=a"(lo) : "v"(p[0]));
			asm volatile("v_accvgpr_write_b32 %0, %1" : "=a"(hi) : "v"(p[1]));
		};
		const bool fb0 = (lane & 1) != 0, fb1 = (lane & 2) != 0, fb2 = (lane & 4) != 0;
		auto dpp_f64 = [](double v, auto ctrlTag) __attribute__((always_inline)) {
			constexpr int ctrl = decltype(ctrlTag)::value;
			int p[2];
			__builtin_memcpy(p, &v, 8);
			p[0] = __builtin_amdgcn_update_dpp(0, p[0], ctrl, 0xf, 0xf, false);
			p[1] = __builtin_amdgcn_update_dpp(0, p[1], ctrl, 0xf, 0xf, false);
			double r;
			__builtin_memcpy(&r, p, 8);
			return r;
		};
		auto xchg1 = [&](double v) __attribute__((always_inline)) { return dpp_f64(v, std::integral_constant<int, 0xB1>()); }; // lane ^ 1
		auto xchg2 = [&](double v) __attribute__((always_inline)) { return dpp_f64(v, std::integral_constant<int, 0x4E>()); }; // lane ^ 2
		auto xchg4 = [&](double v) __attribute__((always_inline)) { // lane ^ 4: banks 0 and 2 from the bank above, 1 and 3 from the bank below
			int p[2];
			__builtin_memcpy(p, &v, 8);
#pragma unroll
			for(int h = 0; h < 2; h++) {
				int r = __builtin_amdgcn_update_dpp(0, p[h], 0x104, 0xf, 0x5, false); // row_shl:4
				p[h] = __builtin_amdgcn_update_dpp(r, p[h], 0x114, 0xf, 0xA, false);   // row_shr:4
			}
			double r;
			__builtin_memcpy(&r, p, 8);
			return r;
		};
		// fold0 / fold1 of the running sums el(c), c < NV
		auto fold = [&](double& f0, double& f1, auto el) __attribute__((always_inline)) {
			double w[4], u[2];
#pragma unroll
			for(int j = 0; j < 4; j++) {
				const double lo = 2 * j < NV ? el(2 * j < NV ? 2 * j : 0) : 0.0, hi = 2 * j + 1 < NV ? el(2 * j + 1 < NV ? 2 * j + 1 : 0) : 0.0;
				w[j] = (fb0 ? hi : lo) + xchg1(fb0 ? lo : hi);
			}
#pragma unroll
			for(int i = 0; i < 2; i++) u[i] = (fb1 ? w[2 * i + 1] : w[2 * i]) + xchg2(fb1 ? w[2 * i] : w[2 * i + 1]);
			f0 = (fb2 ? u[1] : u[0]) + xchg4(fb2 ? u[0] : u[1]);
			f1 = 0.0;
			if(NV > 8) {
				double w1[2];
#pragma unroll
				for(int j = 0; j < 2; j++) {
					const double lo = 8 + 2 * j < NV ? el(8 + 2 * j < NV ? 8 + 2 * j : 0) : 0.0, hi = 9 + 2 * j < NV ? el(9 + 2 * j < NV ? 9 + 2 * j : 0) : 0.0;
					w1[j] = (fb0 ? hi : lo) + xchg1(fb0 ? lo : hi);
				}
				const double u1 = (fb1 ? w1[1] : w1[0]) + xchg2(fb1 ? w1[0] : w1[1]);
				const double t1 = u1 + xchg4(u1); // (lanes k and k ^ 4 hold the same column: one of them keeps it)
				f1 = fb2 ? 0.0 : t1;
			}
		};
		int32_t base = ch0 * GDR_CH;
		auto bcast_f64 = [](double v, int src) {
			int p[2];
			__builtin_memcpy(p, &v, 8);
			p[0] = __builtin_amdgcn_readlane(p[0], src);
			p[1] = __builtin_amdgcn_readlane(p[1], src);
			double r;
			__builtin_memcpy(&r, p, 8);
			return r;
		};
		auto add_h = [&](auto aTag, double f0, double f1, double f, double rr) __attribute__((always_inline)) {
			constexpr int a = decltype(aTag)::value;
			if(a < (HASR ? RC_MAX : 1)) {
				h_put(Hr[a][0], Hr[a][1], __builtin_fma(f0, f, h_get(Hr[a][0], Hr[a][1])));
				if(NV > 8) h_put(Hr[a][2], Hr[a][3], __builtin_fma(f1, f, h_get(Hr[a][2], Hr[a][3])));
				h_put(Hr[a][4], Hr[a][5], h_get(Hr[a][4], Hr[a][5]) + rr);
			}
		};
		// the runs that end at row e (el(c): the running sums with the rows in front of e): their columns move on, H and the
		// R x R cells take the steps
		auto event = [&](int32_t e, auto el) __attribute__((always_inline)) {
			const double vOldL = rc.val;
			const unsigned long long mine = __ballot(rc.end == e); // (cursor lanes only)
			rc.advance(e, lane);
			const double vNewL = rc.val;
			const double dvl = vOldL - vNewL, svl = vOldL + vNewL;
			const double nrel = (double) (e - base);
			const int bL = lane - RC_LANE0;
			const bool mineL = ((mine >> lane) & 1ull) != 0;
			unsigned mm = (unsigned) (mine >> RC_LANE0) & ((1u << RC_MAX) - 1u);
			double f0, f1;
			fold(f0, f1, el);
			while(mm != 0) {
				const int a = __builtin_ctz(mm);
				mm &= mm - 1;
				const double dv = bcast_f64(dvl, RC_LANE0 + a);
				// v_a v_b steps by (v_a - v_a') v_b, with v_b already moved on where b < a ends here too; b = a: v_a^2 - v_a'^2
				const double fr = bL == a ? svl : (mineL && bL < a ? vNewL : vOldL);
				const double rr = bL >= 0 && bL < nR ? nrel * dv * fr : 0.0;
				switch(a) {
					case 0: add_h(std::integral_constant<int, 0>(), f0, f1, dv, rr); break;
					case 1: add_h(std::integral_constant<int, 1>(), f0, f1, dv, rr); break;
					case 2: add_h(std::integral_constant<int, 2>(), f0, f1, dv, rr); break;
					case 3: add_h(std::integral_constant<int, 3>(), f0, f1, dv, rr); break;
					case 4: add_h(std::integral_constant<int, 4>(), f0, f1, dv, rr); break;
					case 5: add_h(std::integral_constant<int, 5>(), f0, f1, dv, rr); break;
					case 6: add_h(std::integral_constant<int, 6>(), f0, f1, dv, rr); break;
					default: add_h(std::integral_constant<int, 7>(), f0, f1, dv, rr); break;
				}
			}
		};
		auto rebase = [&](int32_t upTo) __attribute__((always_inline)) {
			const double nrel = (double) (upTo - base);
			base = upTo;
			const int bL = lane - RC_LANE0;
			double f0, f1;
			fold(f0, f1, [&](int c) __attribute__((always_inline)) { return T[c]; });
			auto one = [&](auto aTag) __attribute__((always_inline)) {
				constexpr int a = decltype(aTag)::value;
				if(a < nR) { // (uniform)
					const double va = rc.value(a);
					add_h(aTag, f0, f1, va, bL >= a && bL < nR ? nrel * va * rc.val : 0.0); // (every pair a <= b once)
				}
			};
			one(std::integral_constant<int, 0>()); one(std::integral_constant<int, 1>());
			one(std::integral_constant<int, 2>()); one(std::integral_constant<int, 3>());
			one(std::integral_constant<int, 4>()); one(std::integral_constant<int, 5>());
			one(std::integral_constant<int, 6>()); one(std::integral_constant<int, 7>());
#pragma unroll
			for(int c = 0; c < NV; c++) T[c] = 0.0;
		};

		uint32_t raw[NC > 0 ? NC : 1];
		double rawd[ND > 0 ? ND : 1];
		// codes / dense values of slice k of the chunk in the ring buffer at `boff` bytes, one row per lane
		auto codes = [&](auto kTag, uint32_t boff) {
			constexpr int k = decltype(kTag)::value;
#pragma unroll
			for(int i = 0; i < NV; i++) {
				if(SPEC) {
					if(i < N2) raw[i] = *(gdr_lp16) ((gdr_lp8) (size_t) (la2 + boff) + (i * GDR_CH * 2 + k * 128));
					else if(i < NC) raw[i] = *((gdr_lp8) (size_t) (la1 + boff) + ((i - N2) * GDR_CH + k * 64));
					else rawd[i - NC] = *(gdr_lpd) ((gdr_lp8) (size_t) (lad + boff) + ((i - NC) * 8 + k * 64 * ND * 8));
				}
				else if(i < NC) raw[i] = *(gdr_lp16) (gdr_lp8) (size_t) (la[i] + boff + (uint32_t) (k * cstep[i])) & cmask[i];
				else rawd[i - NC] = *(gdr_lpd) (gdr_lp8) (size_t) (la[i] + boff + (uint32_t) (k * cstep[i]));
			}
		};

		// one slice: s0 its first row, kTag its place in the chunk, guard: rows behind the end of the matrix count as zeros
		auto slice = [&](auto kTag, int32_t s0, uint32_t boff, bool guard) __attribute__((always_inline)) {
			constexpr int k = decltype(kTag)::value;
			const int32_t row = s0 + lane;
			__builtin_amdgcn_sched_barrier(0); // (slices one after the other: interleaved, their values do not fit the registers next to the sums)
			if(guard) { // (uniform) stale codes behind the end of the matrix: never an index
				const bool in = row < nRows;
#pragma unroll
				for(int i = 0; i < NC; i++) raw[i] = in ? raw[i] : 0u;
			}
			double x[NV];
#pragma unroll
			for(int i = 0; i < NC; i++) x[i] = *(const double*) (ldsBytes + (base8[i] + (raw[i] << 3)));
#pragma unroll
			for(int j = 0; j < ND; j++) x[NC + j] = rawd[j];
			if(k + 1 < GDR_CH / 64) codes(std::integral_constant<int, (k + 1) % (GDR_CH / 64)>(), boff);
			if(guard) {
				const bool in = row < nRows;
#pragma unroll
				for(int i = 0; i < NV; i++) x[i] = in ? x[i] : 0.0;
			}
			int t = 0;
#pragma unroll
			for(int i = 0; i < NV; i++)
#pragma unroll
				for(int j = i; j < NV; j++, t++) acc[t] = __builtin_fma(x[i], x[j], acc[t]);
			if(!HASR) {}
			else if(__builtin_expect(eNext >= s0 + 64, 1)) {
#pragma unroll
				for(int c = 0; c < NV; c++) T[c] += x[c];
			}
			else {
				// runs end inside the slice: a run end sees the running sums with the slice's rows in front of it
				while(eNext < s0 + 64) {
					const bool m = row < eNext;
					event(eNext, [&](int c) __attribute__((always_inline)) { return T[c] + (m ? x[c] : 0.0); });
					eNext = rc.next_end();
				}
#pragma unroll
				for(int c = 0; c < NV; c++) T[c] += x[c];
			}
		};

		// ring: chunk ch sits in buffer (ch - ch0) % GDR_NBUF; while it is read the next GDR_NBUF - 1 are in flight
		// (at the top of a round chunks ch .. ch + GDR_NBUF - 2 have been requested, in this order, and complete in this order)
		int inF[GDR_NBUF - 2]; // loads requested for chunks ch + 1 .. ch + GDR_NBUF - 2
		dma(ch0, 0);
#pragma unroll
		for(int d = 1; d < GDR_NBUF - 1; d++) inF[d - 1] = ch0 + d < ch1 ? dma(ch0 + d, d) : 0;
		int buf = 0;
		const int chFull = min(ch1, nRows / GDR_CH); // (only the matrix's last chunk can be partly filled: a loop of its own keeps this one free of branches)
		// (the rebase sits between two runs of the chunk loop, not inside it: code at the loop's own depth, however rarely
		// taken, costs the loop registers)
		for(int chB = ch0; chB < chFull; chB += GDR_REBASE) {
		const int chE = min(chB + GDR_REBASE, chFull);
		for(int ch = chB; ch < chE; ch++) {
			const uint32_t boff = (uint32_t) buf * ringBytes;
			const int32_t c0 = ch * GDR_CH;
			int keep = 0;
#pragma unroll
			for(int d = 0; d < GDR_NBUF - 2; d++) keep += inF[d];
			gdr_dma_wait(keep); // this chunk has landed: only later chunks' pieces may still be on their way
			// the chunk GDR_NBUF - 1 behind this one into the buffer of the chunk before this one, whose readers are done
#pragma unroll
			for(int d = 0; d + 1 < GDR_NBUF - 2; d++) inF[d] = inF[d + 1];
			inF[GDR_NBUF - 3] = ch + GDR_NBUF - 1 < ch1 ? dma(ch + GDR_NBUF - 1, buf == 0 ? GDR_NBUF - 1 : buf - 1) : 0;
			codes(std::integral_constant<int, 0>(), boff);
			slice(std::integral_constant<int, 0>(), c0, boff, false);
			slice(std::integral_constant<int, 1>(), c0 + 64, boff, false);
			buf = buf + 1 == GDR_NBUF ? 0 : buf + 1;
		}
		if(HASR) rebase(chE * GDR_CH);
		}
		if(chFull < ch1) { // the last, partly filled chunk of the matrix
			const uint32_t boff = (uint32_t) buf * ringBytes;
			const int32_t c0 = chFull * GDR_CH;
			gdr_dma_wait(0);
			codes(std::integral_constant<int, 0>(), boff);
			slice(std::integral_constant<int, 0>(), c0, boff, true);
			if(c0 + 64 < nRows) slice(std::integral_constant<int, 1>(), c0 + 64, boff, true);
		}
		if(HASR) rebase(min(ch1 * GDR_CH, nRows));

		// the wave's sums into the block's tile
		{
			int t = 0;
#pragma unroll
			for(int i = 0; i < NV; i++)
#pragma unroll
				for(int j = i; j < NV; j++, t++) {
					const double s = wave_sum_f64_all(acc[t]);
					if(lane == 0 && s != 0.0) unsafeAtomicAdd(&gramS[i * GDR_NP + j], s);
				}
			if(HASR) {
				// lane k of every group of eight: its group's share of column k (and of column 8 + k % 4 where k < 4)
#pragma unroll
				for(int a = 0; a < RC_MAX; a++) {
					if(a >= nR) continue; // (uniform)
					const int c0 = lane & 7, c1 = 8 + (lane & 3);
					const double h0 = h_get(Hr[a][0], Hr[a][1]), h1 = h_get(Hr[a][2], Hr[a][3]);
					if(c0 < NV && h0 != 0.0) unsafeAtomicAdd(&gramS[c0 * GDR_NP + 16 + a], h0);
					if((lane & 4) == 0 && c1 < NV && h1 != 0.0) unsafeAtomicAdd(&gramS[c1 * GDR_NP + 16 + a], h1);
				}
				// lane 8 a + b2: cell (a, b2) of the upper triangle = the steps at a's run ends + those at b2's
				{
					const int bL = lane - RC_LANE0;
#pragma unroll
					for(int a = 0; a < RC_MAX; a++) {
						const double r = h_get(Hr[a][4], Hr[a][5]);
						if(bL >= 0 && bL < RC_MAX) rrS[a * RC_MAX + bL] = r;
					}
				}
				wave_lds_sync();
				const int a = lane >> 3, b2 = lane & 7;
				if(a <= b2 && b2 < nR) {
					const double sr = a == b2 ? rrS[a * RC_MAX + a] : rrS[a * RC_MAX + b2] + rrS[b2 * RC_MAX + a];
					if(sr != 0.0) unsafeAtomicAdd(&gramS[(16 + a) * GDR_NP + 16 + b2], sr);
				}
			}
		}
	}
	__syncthreads();
	for(int idx = tid; idx < GDR_NP * GDR_NP; idx += GDR_THREADS) {
		const double s = gramS[idx];
		if(s == 0.0) continue;
		const int i = idx / GDR_NP, j = idx - i * GDR_NP;
		const int ci = i < 16 ? (i < A.nV ? A.cols[i].col : -1) : (i - 16 < nR ? A.runs[i - 16].col : -1);
		const int cj = j < 16 ? (j < A.nV ? A.cols[j].col : -1) : (j - 16 < nR ? A.runs[j - 16].col : -1);
		if(ci < 0 || cj < 0) continue;
		unsafeAtomicAdd(&(A.done != nullptr ? A.acc : A.out)[(size_t) min(ci, cj) * A.nCols + max(ci, cj)], s);
	}
	if(A.done != nullptr) gram_tail(A.done, gridDim.x, A.acc, A.out, A.nCols, A.nnz, (unsigned*) gramS);
}

// Which columns of the block are streams, which are followed by run cursors; 1 when the block is not of this shape.
static int gdr_build_plan(cla_block* b, GdrPlan& P) {
	P.rc = 1;
	const int nG = (int) b->groups.size();
	if(b->nRows <= 0 || b->nRows >= ((int64_t) 1 << 31) - 2 * GDR_CH || b->nCols > 64) return 0;
	struct Src { const uint8_t* src; int bpr; std::vector<GdrCol> cols; };
	std::vector<Src> srcs[3]; // streams by class: two-byte codes, one-byte codes, dense rows
	std::vector<GdrDict> dicts;
	std::vector<RunCol> runs;
	std::vector<char> seen((size_t) b->nCols, 0);
	size_t valD = 0;
	int covered = 0;
	for(int g = 0; g < nG; g++) {
		const DGroup& G = b->groups[g].d;
		const auto& hc = b->groups[g].cols;
		for(int c : hc) {
			if(seen[c]) return 0; // overlapping groups
			seen[c] = 1;
		}
		if(G.type == G_UNC) {
			if(((uintptr_t) G.dense & 15) != 0 || G.nColG > 8) return 0;
			Src S{(const uint8_t*) G.dense, G.nColG * 8, {}};
			for(int h = 0; h < G.nColG; h++) {
				if(b->constV[hc[h]] != 0.0) return 0; // (a dense column next to a constant: the tile kernel adds it)
				S.cols.push_back(GdrCol{h * 8, 0, G.nColG * 8, hc[h], {0, 0}});
			}
			srcs[2].push_back(S);
			covered += G.nColG;
			continue;
		}
		if(G.type != G_DDC && G.type != G_RLE && !(G.type == G_SDCZ && G.nOffsets > 0)) continue; // no row data
		const bool haveStream = g < (int) b->expCodes.size() && b->expCodes[g] != nullptr;
		if(G.type == G_RLE && !haveStream) {
			for(int h = 0; h < G.nColG; h++) runs.push_back(RunCol{G.runStart, G.runCode, G.dict, b->constV[hc[h]], G.nRuns, G.nColG, h, hc[h]});
			covered += G.nColG;
			continue;
		}
		const uint8_t* src;
		int cls, fill;
		if(G.type == G_DDC) {
			if(G.codeWidth > 2) return 0;
			src = (const uint8_t*) G.codes;
			cls = G.codeWidth == 2 ? 0 : 1;
			fill = G.nVals;
		}
		else {
			if(!haveStream) return 0;
			src = b->expCodes[g];
			cls = 1;
			fill = 256; // code 0xff: no value on the row
		}
		if(((uintptr_t) src & 15) != 0) return 0;
		Src S{src, cls == 0 ? 2 : 1, {}};
		for(int h = 0; h < G.nColG; h++) {
			dicts.push_back(GdrDict{G.dict, b->constV[hc[h]], G.nVals, G.nColG, h, (int32_t) valD, fill, 0});
			S.cols.push_back(GdrCol{0, (int32_t) (8 * valD), S.bpr, hc[h], {0, 0}});
			valD += (size_t) fill;
		}
		srcs[cls].push_back(S);
		covered += G.nColG;
	}
	// (columns that no group holds row data for are constants: the tile kernel and the pair kernels serve them)
	if(covered != b->nCols) return 0;
	// Summation by parts multiplies sums of earlier rows by the step of a run-length value: with an infinite or NaN value
	// among the dictionaries that is no longer the product of the rows' own cells (0 x inf where every row's product is
	// finite). Such blocks take the tile kernel, which forms every row's cells.
	bool nonFinite = b->dictNonFinite;
	for(const RunCol& R : runs) nonFinite |= !std::isfinite(R.add);
	if(nonFinite && !runs.empty()) return 0;
	std::vector<GdrCol> all;
	std::vector<GdrStream> streams;
	int pieces = 0;
	bool packed = srcs[2].size() <= 1;
	for(int k = 0; k < 3; k++)
		for(const Src& S : srcs[k]) {
			streams.push_back(GdrStream{S.src, S.bpr, pieces});
			if(k < 2 && S.cols.size() != 1) packed = false;
			for(GdrCol C : S.cols) {
				C.ringOff += pieces * 16;
				all.push_back(C);
			}
			pieces += GDR_CH * S.bpr / 16;
		}
	int nCode = 0;
	for(const Src& S : srcs[0]) nCode += (int) S.cols.size();
	for(const Src& S : srcs[1]) nCode += (int) S.cols.size();
	const int nR = (int) runs.size();
	// the kernel without compile-time code widths exists for even numbers of code columns: a filler column reads
	// the ring's first two bytes, masks them away and looks a zero up
	const size_t zeroAt = valD;
	valD += 2;
	dicts.push_back(GdrDict{nullptr, 0.0, 0, 1, 0, (int32_t) zeroAt, 2, 0}); // two zeros
	int nFill = 0;
	if(nCode >= 1 && (nCode & 1)) {
		all.insert(all.begin() + nCode, GdrCol{0, (int32_t) (8 * zeroAt), 2, -1, {0, 0}});
		nFill = 1;
	}
	const int nV = (int) all.size();
	if(nCode < 1 || nV > GDR_VMAX || nR > RC_MAX || pieces > GDR_NI * 64) return 0;
	valD = (valD + 1) & ~(size_t) 1;
	const int ringBytes = pieces * 16;
	P.lds = (valD + GDR_NP * GDR_NP + (size_t) GDR_WAVES * GDR_WDOUBLES) * 8 + (size_t) GDR_WAVES * GDR_NBUF * ringBytes;
	if(P.lds > (size_t) std::min(g_ldsPerBlock, 160 * 1024) - 1024) return 0;
	const size_t colBytes = all.size() * sizeof(GdrCol), dictBytes = dicts.size() * sizeof(GdrDict), runBytes = runs.size() * sizeof(RunCol);
	const size_t streamBytes = streams.size() * sizeof(GdrStream);
	std::vector<uint8_t> img(dictBytes + runBytes + streamBytes + colBytes + 16, 0); // (structs with pointers first: 8-byte aligned)
	if(dictBytes) std::memcpy(img.data(), dicts.data(), dictBytes);
	if(runBytes) std::memcpy(img.data() + dictBytes, runs.data(), runBytes);
	std::memcpy(img.data() + dictBytes + runBytes, streams.data(), streamBytes);
	std::memcpy(img.data() + dictBytes + runBytes + streamBytes, all.data(), colBytes);
	uint8_t* d = nullptr;
	CLA_HIP(hipMalloc((void**) &d, img.size() + 64));
	P.dImg = d;
	P.bytes = (int64_t) img.size() + 64;
	CLA_HIP(hipMemcpy(d, img.data(), img.size(), hipMemcpyHostToDevice));
	P.A.dicts = (const GdrDict*) d;
	P.A.runs = (const RunCol*) (d + dictBytes);
	P.A.streams = (const GdrStream*) (d + dictBytes + runBytes);
	P.A.cols = (const GdrCol*) (d + dictBytes + runBytes + streamBytes);
	P.A.nDicts = (int) dicts.size();
	P.A.nStreams = (int) streams.size();
	P.A.nV = nV; P.A.nR = nR;
	P.A.n2 = 0; P.A.n12 = 0;
	for(const Src& S : srcs[0]) { P.A.n2 += (int) S.cols.size(); P.A.n12 += (int) S.cols.size(); }
	for(const Src& S : srcs[1]) P.A.n12 += (int) S.cols.size();
	P.A.n12 += nFill;
	P.A.packed = packed && nFill == 0 ? 1 : 0;
	P.A.valDoubles = (int) valD;
	P.A.ringBytes = ringBytes;
	P.A.nRows = b->nRows;
	P.A.nCols = b->nCols;
	P.rc = 0;
	return 0;
}

void gdr_plan_drop(cla_block* b) {
	if(b->gdrPlan == nullptr) return;
	if(b->gdrPlan->dImg) { (void) hipFree(b->gdrPlan->dImg); b->derivedBytes -= b->gdrPlan->bytes; }
	delete b->gdrPlan;
	b->gdrPlan = nullptr;
}

// dOut (nCols x nCols, zeroed) += upper triangle of t(D) %*% D of the decoded rows, constants included. Returns 1
// when the block is not of this kernel's shape (the caller takes the tile kernel on the matrix cores).
int launch_tsmm_direct(cla_block* b, double* dOut, unsigned long long* dNnz) {
	if(!b->opt.tsmmDirect || b->crossSplit > 0 || b->crossBlocks > 0) return 1;
	if(b->gdrPlan == nullptr) {
		int rc = ensure_expanded(b);
		if(rc) return rc;
		b->gdrPlan = new GdrPlan();
		rc = gdr_build_plan(b, *b->gdrPlan);
		if(rc < 0) { gdr_plan_drop(b); return rc; }
		if(b->gdrPlan->dImg) b->derivedBytes += b->gdrPlan->bytes;
	}
	if(b->gdrPlan->rc) return b->gdrPlan->rc;
	GdrArgs A = b->gdrPlan->A;
	A.out = dOut;
	A.acc = nullptr; A.done = nullptr; A.nnz = nullptr;
	if(dNnz != nullptr) {
		const int rc = ensure_gram_acc(b);
		if(rc) return rc;
		A.acc = b->dGramAcc; A.done = (unsigned*) (b->dCounters + 7); A.nnz = dNnz;
	}
	const size_t lds = b->gdrPlan->lds;
	const int nChunks = (int) ((b->nRows + GDR_CH - 1) / GDR_CH);
	const unsigned grid = (unsigned) std::max(1, std::min((nChunks + GDR_WAVES - 1) / GDR_WAVES, g_numCU * (lds <= 76 * 1024 ? 2 : 1)));
	Prof pf(b, "k_tsmm_direct", grid, GDR_THREADS, (long) lds, (double) b->device_bytes_cached);
	const int n2 = A.n2, n1 = A.n12 - A.n2, nd = A.nV - A.n12;
	bool launched = false;
#define GDR_CASE(N2V, N1V, NDV, SPECV, HASRV)                                                                                 \
	if(!launched && (SPECV ? A.packed && n2 == N2V && n1 == N1V : n2 + n1 == N2V) && nd == NDV && (HASRV || A.nR == 0) && (SPECV || HASRV)) {          \
		CLA_HIP(allow_full_lds((const void*) k_tsmm_direct<N2V, N1V, NDV, SPECV, HASRV>));                                        \
		hipLaunchKernelGGL((k_tsmm_direct<N2V, N1V, NDV, SPECV, HASRV>), dim3(grid), dim3(GDR_THREADS), lds, b->stream, A);       \
		launched = true;                                                                                                          \
	}
	GDR_CASE(8, 2, 2, true, false)
	GDR_CASE(8, 2, 2, true, true)
	GDR_CASE(2, 0, 0, false, true) GDR_CASE(4, 0, 0, false, true) GDR_CASE(6, 0, 0, false, true)
	GDR_CASE(8, 0, 0, false, true) GDR_CASE(10, 0, 0, false, true) GDR_CASE(12, 0, 0, false, true)
	GDR_CASE(2, 0, 1, false, true) GDR_CASE(4, 0, 1, false, true) GDR_CASE(6, 0, 1, false, true)
	GDR_CASE(8, 0, 1, false, true) GDR_CASE(10, 0, 1, false, true)
	GDR_CASE(2, 0, 2, false, true) GDR_CASE(4, 0, 2, false, true) GDR_CASE(6, 0, 2, false, true)
	GDR_CASE(8, 0, 2, false, true) GDR_CASE(10, 0, 2, false, true)
	GDR_CASE(2, 0, 4, false, true) GDR_CASE(4, 0, 4, false, true) GDR_CASE(6, 0, 4, false, true)
	GDR_CASE(8, 0, 4, false, true)
#undef GDR_CASE
	if(!launched) return 1;
	CLA_HIP(hipGetLastError());
	return 0;
}

} // namespace cla
