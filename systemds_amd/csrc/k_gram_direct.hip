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
//   R x V   a run-length column is constant between two run ends, so  sum_r v_a x_c = sum_segments v_a(seg) T_c(seg)
//           with T_c the sum of x_c over a segment: lanes keep T_c, and where some column's run ends the
//           wave reduces T over its lanes (through LDS), adds v_a T_c for every run-length column a and
//           starts a new segment;
//   R x R   likewise with the segment's row count in place of T_c.
// No value of a run-length column is ever looked up per row, and no one-code-per-row copy of it is read.
//
// The streams reach the wave through a ring of three chunks of 128 rows in LDS, filled by global -> LDS loads
// that bypass the registers (two chunks in flight while one is read): a wave is alone on its SIMD (the sums
// take most of the register file), so nothing else would hide the memory latency.
#include "../../include/cla_hip.h"
#include "cla_runs.hpp"
#include <algorithm>
#include <cstring>
#include <vector>

namespace cla {

constexpr int GDR_THREADS = 256;
constexpr int GDR_WAVES = GDR_THREADS / 64;
constexpr int GDR_VMAX = 12;                 // varying columns
constexpr int GDR_NP = 16 + RC_MAX;          // block tile: index < 16 varying column, 16 + a run-length column a
constexpr int GDR_RED = 65;                  // doubles per column in the lane transposition (odd: few bank conflicts on the way back)
constexpr int GDR_REDC = 6;                  // columns per pass of the transposition
constexpr int GDR_SV = GDR_VMAX + RC_MAX;    // entries of a segment's vector: T of the varying columns, then value x rows of the run-length columns
constexpr int GDR_WDOUBLES = 64 + 32 + GDR_REDC * GDR_RED + 24 + RC_MAX; // per wave: window values, window ends, transposition, segment vector, run-length values
constexpr int GDR_CH = 128;                  // rows per chunk of the wave's stream ring (2 slices of 64 rows)
constexpr int GDR_NBUF = 4;                  // ring buffers per wave: one being read, three in flight
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
	double* const red = wbase + 96;
	double* const svS = red + GDR_REDC * GDR_RED;   // GDR_SV (24 reserved): the closing segment's vector
	double* const vvS = svS + 24;                   // RC_MAX: the run-length columns' values on the closing segment
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
	if(lane < 24 + RC_MAX) svS[lane] = 0.0; // (entries of columns the block does not have stay zero)
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
		int32_t segStart = ch0 * GDR_CH;
		int32_t eNext = HASR ? rc.next_end() : RC_NEVER;

		// Where a run ends: T of all lanes summed per column, through LDS, GDR_REDC columns per pass: the eight lanes of
		// group g = lane / 8 (groups 0, 1, 3 .. 6; group 2 is the cursor lanes) sum eight lanes' values each and meet
		// through three moves inside their half row. The sums go to LDS as the segment's vector s next to the
		// run-length columns' values v; then lane (a, cs) adds v_a s_c for its columns c = cs, cs + 8, cs + 16 into
		// registers. T restarts.
		double G[3] = {0.0, 0.0, 0.0};
		auto dpp_f64 = [](double v, auto ctrlTag) {
			constexpr int ctrl = decltype(ctrlTag)::value;
			int p[2];
			__builtin_memcpy(p, &v, 8);
			p[0] = __builtin_amdgcn_update_dpp(0, p[0], ctrl, 0xf, 0xf, false);
			p[1] = __builtin_amdgcn_update_dpp(0, p[1], ctrl, 0xf, 0xf, false);
			double r;
			__builtin_memcpy(&r, p, 8);
			return r;
		};
		auto flush = [&](int32_t upTo) {
			const double nseg = (double) (upTo - segStart);
			segStart = upTo;
			const int g = lane >> 3, k8 = lane & 7;
			const int cp = g < 2 ? g : g - 1; // column of the pass that group g sums (groups 2 and 7: none)
			const bool vlane = g != 2 && g != 7;
#pragma unroll
			for(int p0 = 0; p0 < NV; p0 += GDR_REDC) {
#pragma unroll
				for(int c = p0; c < p0 + GDR_REDC && c < NV; c++) red[(c - p0) * GDR_RED + lane] = T[c];
				wave_lds_sync();
				// (all eight reads requested before the first sum: one wait instead of one per read)
				double rv[8];
#pragma unroll
				for(int j = 0; j < 8; j++) rv[j] = red[(vlane ? cp : 0) * GDR_RED + k8 * 8 + j];
				__builtin_amdgcn_sched_barrier(0);
				double sp = ((rv[0] + rv[1]) + (rv[2] + rv[3])) + ((rv[4] + rv[5]) + (rv[6] + rv[7]));
				if(!(vlane && p0 + cp < NV)) sp = 0.0;
				sp += dpp_f64(sp, std::integral_constant<int, 0xB1>());  // quad_perm [1, 0, 3, 2]
				sp += dpp_f64(sp, std::integral_constant<int, 0x4E>());  // quad_perm [2, 3, 0, 1]
				sp += dpp_f64(sp, std::integral_constant<int, 0x141>()); // row_half_mirror
				if(vlane && k8 == 0 && p0 + cp < NV) svS[p0 + cp] = sp;
				wave_lds_sync();
			}
			if(lane >= RC_LANE0 && lane < RC_LANE0 + nR) {
				svS[GDR_VMAX + lane - RC_LANE0] = rc.val * nseg;
				vvS[lane - RC_LANE0] = rc.val;
			}
			wave_lds_sync();
			const double va = vvS[k8];
#pragma unroll
			for(int t = 0; t < 3; t++)
				if(g + 8 * t < GDR_SV) G[t] = __builtin_fma(va, svS[g + 8 * t], G[t]);
			wave_lds_sync();
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
		auto slice = [&](auto kTag, int32_t s0, uint32_t boff, bool guard) {
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
			else if(eNext >= s0 + 64) {
#pragma unroll
				for(int c = 0; c < NV; c++) T[c] += x[c];
			}
			else {
				// runs end inside the slice: rows in front of each end go to the segment it closes
				int32_t from = s0;
				while(eNext < s0 + 64) {
					const bool m = row >= from && row < eNext;
#pragma unroll
					for(int c = 0; c < NV; c++) T[c] += m ? x[c] : 0.0;
					flush(eNext);
					from = eNext;
					rc.advance(eNext, lane);
					eNext = rc.next_end();
				}
				const bool m = row >= from;
#pragma unroll
				for(int c = 0; c < NV; c++) T[c] += m ? x[c] : 0.0;
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
		for(int ch = ch0; ch < chFull; ch++) {
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
		if(chFull < ch1) { // the last, partly filled chunk of the matrix
			const uint32_t boff = (uint32_t) buf * ringBytes;
			const int32_t c0 = chFull * GDR_CH;
			gdr_dma_wait(0);
			codes(std::integral_constant<int, 0>(), boff);
			slice(std::integral_constant<int, 0>(), c0, boff, true);
			if(c0 + 64 < nRows) slice(std::integral_constant<int, 1>(), c0 + 64, boff, true);
		}
		if(HASR) flush(min(ch1 * GDR_CH, nRows));

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
				// lane (a, cs): v_a s_c summed over the segments for c = cs, cs + 8, cs + 16 (c < GDR_VMAX: varying column c)
				const int a = lane & 7, cs = lane >> 3;
#pragma unroll
				for(int tt = 0; tt < 3; tt++) {
					const int c = cs + 8 * tt;
					if(a >= nR || c >= GDR_SV) continue;
					if(c < GDR_VMAX) { if(c < NV) unsafeAtomicAdd(&gramS[c * GDR_NP + 16 + a], G[tt]); }
					else if(c - GDR_VMAX >= a && c - GDR_VMAX < nR) unsafeAtomicAdd(&gramS[(16 + a) * GDR_NP + 16 + c - GDR_VMAX], G[tt]);
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
