// Right multiply X %*% B on a compressed block (gfx950).
//
//   k_preagg          T_g = dict_g x B[cols_g, :]   (Dictionary.preaggValuesFromDense)
//   k_rmm_q1_ddc      row-parallel gather-accumulate for mat-vec, tables in LDS
//   k_rmm_rows        generic row-parallel gather for any q / DDC, RLE, uncompressed
//   k_rmm_sdc_scatter offset-list scatter for SDCZeros groups
//   k_count_nnz       non-zero count of the result
#include "../../include/cla_hip.h"
#include "cla_device.hpp"
#include <algorithm>

namespace cla {

// ---------------------------------------------------------------------------
// K1: per group dictionary x B pre-aggregation. One thread per (tuple k, output
// column c). Products and sums are rounded separately (no FMA) in column order
// h, and zero dictionary cells are skipped, as the reference does, so the
// tables are bit-identical to a scalar CPU evaluation.
// grid.y = group index; grid.y == nGroups computes constV x B.
// ---------------------------------------------------------------------------
__global__ void k_preagg(const DGroup* __restrict__ groups, int nGroups, const double* __restrict__ B, int q,
	int nCols, const double* __restrict__ constV, double* __restrict__ T, int totalVals,
	unsigned long long* __restrict__ nnz, double* __restrict__ Tpad, int squares) {
	const int g = blockIdx.y;
	const int idx = blockIdx.x * blockDim.x + threadIdx.x;
	if(g == 0 && idx == 0) *nnz = 0; // the multiply kernels behind this one on the stream count into it
	// Tpad (mat-vec on byte codes only): the same tables at a fixed stride of 256 entries, zero
	// beyond nVals, so that the gather kernel copies a slab of tables without looking up offsets
	if(Tpad != nullptr && g < nGroups && idx < 256 && idx >= groups[g].nVals) Tpad[(size_t) g * 256 + idx] = 0.0;
	if(g == nGroups) {
		if(constV == nullptr || idx >= q) return;
		double acc = 0;
		for(int c0 = 0; c0 < nCols; c0++) {
			const double a = constV[c0];
			if(squares) acc += a * a;
			else if(a != 0) acc = __dadd_rn(acc, __dmul_rn(a, B[(size_t) c0 * q + idx]));
		}
		T[(size_t) totalVals * q + idx] = acc;
		return;
	}
	const DGroup G = dgroup(groups + g);
	if(G.type == G_UNC || idx >= G.nVals * q) return;
	const int k = idx / q, c = idx - k * q;
	double acc = 0;
	for(int h = 0; h < G.nColG; h++) {
		const double v = G.dict[(size_t) k * G.nColG + h];
		if(squares) { // row sums of squares: the tuple's part beyond the constants' (q == 1)
			const double cc = constV != nullptr ? constV[G.cols[h]] : 0.0;
			acc += (v + cc) * (v + cc) - cc * cc;
		}
		else if(v != 0) acc = __dadd_rn(acc, __dmul_rn(v, B[(size_t) G.cols[h] * q + c]));
	}
	T[(size_t) (G.tblOff + k) * q + c] = acc;
	if(Tpad != nullptr) Tpad[(size_t) g * 256 + k] = acc;
}

// ---------------------------------------------------------------------------
// K2 (mat-vec): all groups DDC with the same code width CW, code streams in one
// arena with a uniform stride.
// A thread owns RPT consecutive rows and keeps their sums in registers; the
// pre-aggregated tables of a slab of groups are staged in LDS with a uniform
// stride, so code and table addresses are pure arithmetic (no per-group pointer
// loads in the hot loop). Code streams are read with 16-byte non-temporal loads,
// NB groups in flight per thread and the next batch requested before the current
// one is consumed. Groups are visited in list order, so every output cell is
// summed in the same order as the CPU algorithm.
// ---------------------------------------------------------------------------
template <int CW, int RPT, int NB>
__device__ __forceinline__ void q1_load(CodeVec<CW, RPT> (&cv)[NB], const uint8_t* myCodes, size_t arenaStride, int g,
	int gLast) {
#pragma unroll
	for(int j = 0; j < NB; j++) cv[j].load(myCodes + (size_t) min(g + j, gLast) * arenaStride);
}

// adds table[code] of NB groups; LDS slot 0 is an all-zero table that serves the
// padded batch slots beyond the slab, group gRel of the slab sits in slot gRel + 1
template <int CW, int RPT, int NB>
__device__ __forceinline__ void q1_consume(const CodeVec<CW, RPT> (&cv)[NB], const double* tbl, int tstride, int gRel,
	int nInSlab, double (&acc)[RPT]) {
#pragma unroll
	for(int j = 0; j < NB; j++) {
		const double* t = tbl + (size_t) (gRel + j < nInSlab ? gRel + j + 1 : 0) * tstride;
#pragma unroll
		for(int i = 0; i < RPT; i++) acc[i] += t[cv[j].get(i)];
	}
}

// Every slab but the last holds a multiple of 2 * Q1_NB groups (the host plans
// it so): batches of Q1_NB groups alternate between two register sets, and the
// request for the batch after next is always issued before a batch is consumed,
// also across slab boundaries. The tables of the next slab are fetched into
// registers (Q1_TPT values per thread) while the current slab is processed.
constexpr int Q1_NB = 4;
constexpr int Q1_TPT = 16;

// value f of a slab's padded table image: group f / tstride, entry f % tstride
__device__ __forceinline__ double q1_table_value(const double* __restrict__ T, const int32_t* __restrict__ tblOff,
	int4 sl, int f) {
	const int tstride = sl.z;
	if(sl.w) return T[tblOff[sl.x] + f]; // uniform nVals == tstride: the image is a plain copy
	const int g = f / tstride, i = f - g * tstride;
	const int o = tblOff[sl.x + g], n = tblOff[sl.x + g + 1] - o;
	return i < n ? T[o + i] : 0.0;
}

template <int CW, int RPT, int THREADS>
__global__ __launch_bounds__(THREADS) void k_rmm_q1_ddc(const uint8_t* __restrict__ arena, size_t arenaStride,
	int nGroups, const int4* __restrict__ slabs, int nSlabs, const int32_t* __restrict__ tblOff,
	const double* __restrict__ T, int constIdx, double* __restrict__ out, int64_t nRows,
	unsigned long long* __restrict__ nnz) {
	extern __shared__ double tbl[];
	constexpr int NB = Q1_NB;
	const int tid = threadIdx.x;
	const int64_t row0 = ((int64_t) blockIdx.x * THREADS + tid) * RPT;
	const bool full = row0 + RPT <= nRows;
	const bool any = row0 < nRows;
	const uint8_t* myCodes = arena + (size_t) row0 * CW;
	double acc[RPT];
#pragma unroll
	for(int i = 0; i < RPT; i++) acc[i] = 0.0;
	CodeVec<CW, RPT> ping[NB], pong[NB];
	if(full) q1_load<CW, RPT, NB>(ping, myCodes, arenaStride, 0, nGroups - 1);

	double stage[Q1_TPT];
	int4 sl = slabs[0];
	{
		const int total = (sl.y - sl.x) * sl.z;
#pragma unroll
		for(int k = 0; k < Q1_TPT; k++) {
			const int f = tid + k * THREADS;
			stage[k] = f < total ? q1_table_value(T, tblOff, sl, f) : 0.0;
		}
		for(int i = tid; i < sl.z; i += THREADS) tbl[i] = 0.0; // slot 0: zero table
	}

	for(int s = 0; s < nSlabs; s++) {
		const int g0 = sl.x, g1 = sl.y, tstride = sl.z;
		const int nIn = g1 - g0;
		__syncthreads(); // everyone is done with the previous slab's tables
		{
			const int total = nIn * tstride;
#pragma unroll
			for(int k = 0; k < Q1_TPT; k++) {
				const int f = tid + k * THREADS;
				if(f < total) tbl[tstride + f] = stage[k];
			}
		}
		__syncthreads();
		if(s + 1 < nSlabs) {
			sl = slabs[s + 1];
			const int total = (sl.y - sl.x) * sl.z;
#pragma unroll
			for(int k = 0; k < Q1_TPT; k++) {
				const int f = tid + k * THREADS;
				stage[k] = f < total ? q1_table_value(T, tblOff, sl, f) : 0.0;
			}
		}
		if(full) {
			for(int g = g0; g < g1; g += 2 * NB) {
				q1_load<CW, RPT, NB>(pong, myCodes, arenaStride, g + NB, nGroups - 1);
				q1_consume<CW, RPT, NB>(ping, tbl, tstride, g - g0, nIn, acc);
				q1_load<CW, RPT, NB>(ping, myCodes, arenaStride, g + 2 * NB, nGroups - 1);
				q1_consume<CW, RPT, NB>(pong, tbl, tstride, g - g0 + NB, nIn, acc);
			}
		}
		else if(any) {
			for(int g = g0; g < g1; g++) {
				const double* t = tbl + (size_t) (g - g0 + 1) * tstride;
				const uint8_t* codes = arena + (size_t) g * arenaStride;
#pragma unroll
				for(int i = 0; i < RPT; i++)
					if(row0 + i < nRows) acc[i] += t[load_code(codes, CW, row0 + i)];
			}
		}
	}

	int cnt = 0;
	if(any) {
		if(constIdx >= 0) {
			const double cadd = T[constIdx];
#pragma unroll
			for(int i = 0; i < RPT; i++) acc[i] += cadd;
		}
		if(full) {
#pragma unroll
			for(int i = 0; i < RPT; i += 2) {
				cnt += (acc[i] != 0.0) + (acc[i + 1] != 0.0);
				f64x2 v2;
				v2.x = acc[i]; v2.y = acc[i + 1];
				__builtin_nontemporal_store(v2, (f64x2*) (out + row0 + i));
			}
		}
		else {
#pragma unroll
			for(int i = 0; i < RPT; i++)
				if(row0 + i < nRows) { cnt += acc[i] != 0.0; out[row0 + i] = acc[i]; }
		}
	}
	count_add(nnz, cnt);
}

// ---------------------------------------------------------------------------
// K2 (mat-vec), byte codes: all groups DDC with uint8 codes (nVals <= 256).
// Same scheme as k_rmm_q1_ddc, specialised so that the hot loop carries no
// address arithmetic beyond code*8: every table has the fixed LDS stride of 256
// doubles, slabs hold U8_PER groups and the loop over the slab is fully unrolled,
// which turns every table base into an immediate offset of the LDS read.
// Slots of a short last slab are zero-filled (x + 0.0 leaves the sum unchanged).
// ---------------------------------------------------------------------------
constexpr int U8_RPT = 16;   // rows per thread = one 16-byte load per group

// U8_PER = groups (tables) per slab (2 KiB of LDS each), U8_NB = groups per load batch,
// Adds table[code] for NB groups x RPT rows held in registers. The NB * RPT lookups are
// issued as batches of LB LDS reads with LN batches in flight: the reads of batch b + LN - 1
// are issued before the adds of batch b, and scheduling barriers pin that order, so a wave
// keeps (LN - 1) * LB .. LN * LB reads outstanding instead of the one to three the
// scheduler chooses on its own under register pressure. Group order per row is kept
// (batches walk group-major), so the sums are bit-identical to the sequential loop.
template <int RPT, int NB, int LB, int LN>
__device__ __forceinline__ void u8_consume(const CodeVec<1, RPT> (&cv)[NB], const char* tb, double (&acc)[RPT]) {
	static_assert(RPT % LB == 0, "a batch stays inside one group");
	constexpr int NBATCH = NB * RPT / LB;
	double t[LN][LB];
	auto issue = [&](int b) {
		const int j = (b * LB) / RPT, i0 = (b * LB) % RPT;
#pragma unroll
		for(int k = 0; k < LB; k++) t[b % LN][k] = *(const double*) (tb + j * 2048 + cv[j].off8(i0 + k));
	};
#pragma unroll
	for(int b = 0; b < LN - 1 && b < NBATCH; b++) issue(b);
	__builtin_amdgcn_sched_barrier(0);
#pragma unroll
	for(int b = 0; b < NBATCH; b++) {
		if(b + LN - 1 < NBATCH) issue(b + LN - 1);
		__builtin_amdgcn_sched_barrier(0);
		const int i0 = (b * LB) % RPT;
#pragma unroll
		for(int k = 0; k < LB; k++) acc[i0 + k] += t[b % LN][k];
		__builtin_amdgcn_sched_barrier(0);
	}
}

// U8_PER is a multiple of 2 * U8_NB. The host picks the variant that pads least.
//
// FUSED (every group has one column): the tables are not read from a pre-aggregated image but made
// on the way into LDS, table_g[k] = dict_g[k] * v[col_g] (Dictionary.preaggValuesFromDense for one
// column: a zero dictionary cell stays zero whatever v holds, and 0 + d * v rounds once, so the
// entries are bit-identical to the pre-aggregation kernel's). `Tpad` is then the padded dictionary
// image (256 entries per group, zero beyond nVals), `col0` the groups' columns. Block 0 clears
// *nnzNext, the counter of the next call, so that no clearing step runs between two calls.
template <int THREADS, int U8_PER, int U8_NB, int LB, int LN, bool FUSED>
__global__ __launch_bounds__(THREADS, 4) void k_rmm_q1_u8(const uint8_t* __restrict__ arena, size_t arenaStride,
	int nGroups, const double* __restrict__ Tpad, const double* __restrict__ constTerm,
	double* __restrict__ out, int64_t nRows, unsigned long long* __restrict__ nnz,
	const int32_t* __restrict__ col0, const double* __restrict__ v, unsigned long long* __restrict__ nnzNext) {
	__shared__ double tbl[U8_PER * 256];
	__shared__ double wbufAll[(THREADS / 64) * 64 * 8]; // per-wave transpose buffers of the epilogue
	const char* tb = (const char*) tbl;
	constexpr int RPT = U8_RPT, NB = U8_NB;
	const int tid = threadIdx.x;
	const int off = tid * RPT; // first row of this thread inside a pass
	const int gLast = nGroups - 1;
	const int nPad = (nGroups + U8_PER - 1) / U8_PER * U8_PER; // groups incl. the zero-table slots of the last slab

	// The block is persistent: it owns a share of the rows and covers it in nPass passes of at most
	// THREADS * RPT rows, so all blocks finish together and the load pipeline (codes two batches
	// ahead, tables one slab ahead) keeps running from pass to pass. Shares are whole units of
	// 64 * RPT rows (the rows of one wave in one pass) and differ by at most one unit between
	// blocks: a share that ends inside a unit leaves a wave with a few live lanes that costs as
	// much as a full one (measured on 10M rows: 0.2233 ms with equal shares of 19536 rows,
	// 0.2157 ms with shares of whole units). Everything about a pass but `off` is uniform.
	constexpr int UNIT = 64 * RPT;
	const int64_t nUnits = (nRows + UNIT - 1) / UNIT;
	const int64_t unitsLo = nUnits / gridDim.x, unitsRem = nUnits % gridDim.x;
	const int64_t myUnits = unitsLo + ((int64_t) blockIdx.x < unitsRem ? 1 : 0);
	const int64_t blockBeg = ((int64_t) blockIdx.x * unitsLo + min((int64_t) blockIdx.x, unitsRem)) * UNIT;
	if(myUnits == 0 || blockBeg >= nRows) return;
	const int blockLen = (int) (min(nRows, blockBeg + myUnits * UNIT) - blockBeg);
	const int nPass = (blockLen + THREADS * RPT - 1) / (THREADS * RPT);
	// whole waves per pass (64 threads x RPT rows), so that only a block's last pass can hold a
	// partly filled wave, which has to store its rows untransposed
	const int passRows = ((blockLen + nPass - 1) / nPass + 64 * RPT - 1) / (64 * RPT) * (64 * RPT);

	int passLen = min(passRows, blockLen);
	bool full = off + RPT <= passLen;
	const uint8_t* passBase = arena + (size_t) blockBeg; // uniform; a thread's codes start at passBase + off
	uint32_t voff = full ? off : 0;

	CodeVec<1, RPT> ping[NB], pong[NB];
	if(full) u8_load<RPT, NB>(ping, passBase, voff, arenaStride, 0, gLast);

	// the tables of the next slab are fetched into registers while the current slab is processed
	constexpr int TPT = (U8_PER * 256 + THREADS - 1) / THREADS;
	double stage[TPT];
	// FUSED: a non-finite v[col] must not meet a zero dictionary cell (0 * inf); the plain product serves otherwise
	bool careful = false;
	if(FUSED) {
		static_assert(!FUSED || THREADS % 256 == 0, "a wave's table entries belong to one group");
		if(blockIdx.x == 0 && tid == 0) *nnzNext = 0;
		int bad = 0;
		for(int g = tid; g < nGroups; g += THREADS) bad |= !isfinite(v[col0[g]]);
		careful = __syncthreads_or(bad) != 0;
	}
	auto fetch = [&](int g0) { // tables g0 .. g0 + U8_PER - 1 of the padded image (zero beyond the last group)
		const int nIn = min(U8_PER, nGroups - g0) * 256;
		const double* src = Tpad + (size_t) g0 * 256;
		int tidF = tid; // laundered like tidE below: keeps the index arithmetic out of registers between uses
		asm volatile("" : "+v"(tidF));
#pragma unroll
		for(int k = 0; k < TPT; k++) {
			const int f = tidF + k * THREADS;
			if(FUSED) {
				// entry f belongs to group g0 + f / 256, the same for the whole wave: v comes through scalar loads
				const int gs = __builtin_amdgcn_readfirstlane(g0 + (tid >> 8) + k * (THREADS / 256));
				const double vv = gs < nGroups ? v[col0[gs]] : 0.0;
				const double d = f < nIn ? src[f] : 0.0;
				stage[k] = careful ? (d != 0.0 ? d * vv : 0.0) : d * vv;
			}
			else stage[k] = f < nIn ? src[f] : 0.0;
		}
	};
	fetch(0);
	const double cadd = constTerm != nullptr ? *constTerm : 0.0;
	int cnt = 0;
	for(int pass = 0; pass < nPass; pass++) {
		const int64_t passBeg = blockBeg + (int64_t) pass * passRows;
		// the first batch of the next pass is requested in the last batch slot of this pass; a
		// thread without a full next pass requests valid but unused bytes instead, so that the
		// number of loads in flight never depends on a branch
		const int nextLen = pass + 1 < nPass ? min(passRows, blockLen - (pass + 1) * passRows) : 0;
		const bool nfull = off + RPT <= nextLen;
		const uint8_t* nextBase = nextLen > 0 ? passBase + passRows : passBase; // uniform
		const uint32_t noff = nfull ? off : 0; // without a next pass: everybody re-requests the same 16 bytes
		double acc[RPT];
#pragma unroll
		for(int i = 0; i < RPT; i++) acc[i] = 0.0;
		for(int g0 = 0; g0 < nGroups; g0 += U8_PER) {
			const int nIn = min(U8_PER, nGroups - g0);
			__syncthreads();
			int tidW = tid;
			asm volatile("" : "+v"(tidW));
#pragma unroll
			for(int k = 0; k < TPT; k++) {
				const int f = tidW + k * THREADS;
				if(f < U8_PER * 256) tbl[f] = stage[k];
			}
			__syncthreads();
			fetch(g0 + U8_PER < nGroups ? g0 + U8_PER : 0);
			if(full) {
#pragma unroll
				for(int s = 0; s < U8_PER; s += 2 * NB) {
					u8_load<RPT, NB>(pong, passBase, voff, arenaStride, g0 + s + NB, gLast);
					u8_consume<RPT, NB, LB, LN>(ping, tb + s * 2048, acc);
					const int gn = g0 + s + 2 * NB;
					const bool wrap = gn >= nPad;
					u8_load<RPT, NB>(ping, wrap ? nextBase : passBase, wrap ? noff : voff, arenaStride, wrap ? 0 : gn, gLast);
					u8_consume<RPT, NB, LB, LN>(pong, tb + (s + NB) * 2048, acc);
				}
			}
			else if(off < passLen) {
				for(int g = 0; g < nIn; g++) {
					const uint8_t* codes = arena + (size_t) (g0 + g) * arenaStride + passBeg;
#pragma unroll
					for(int i = 0; i < RPT; i++)
						if(off + i < passLen) acc[i] += tbl[g * 256 + codes[off + i]];
				}
			}
		}

		// Epilogue. A thread holds 16 consecutive rows, so direct stores would touch 64
		// different lines per instruction with 16 bytes each (measured: 2.9x write
		// amplification). Waves whose 64 threads all hold full rows transpose through LDS in
		// two halves of 8 rows per thread instead, so that 8 consecutive lanes write one
		// 64-byte segment. The buffer is private to the wave and LDS executes a wave's
		// accesses in order, so no block barrier is needed.
		// (the empty asm keeps the epilogue's address arithmetic inside the pass loop: hoisted
		// out of it, it would occupy registers all through the slab loop)
		int tidE = tid;
		asm volatile("" : "+v"(tidE));
		const int wave = tidE >> 6, lane = tidE & 63;
		if((wave + 1) * 64 * RPT <= passLen) {
			double* wbuf = wbufAll + wave * (64 * 8); // 8 values per lane, XOR-swizzled against bank conflicts
			double* obase = out + passBeg + (int64_t) wave * 64 * RPT;
#pragma unroll
			for(int h = 0; h < 2; h++) {
#pragma unroll
				for(int i = 0; i < 8; i++) {
					const double v = acc[h * 8 + i] + cadd;
					cnt += v != 0.0;
					wbuf[lane * 8 + (i ^ ((lane >> 2) & 7))] = v;
				}
				__builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
				__builtin_amdgcn_wave_barrier();
				__builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
				for(int j = 0; j < 8; j++) {
					const int t = j * 64 + lane, sl = t >> 3, i = t & 7;
					__builtin_nontemporal_store(wbuf[sl * 8 + (i ^ ((sl >> 2) & 7))], obase + sl * RPT + h * 8 + i);
				}
				__builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
				__builtin_amdgcn_wave_barrier();
				__builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
			}
		}
		else if(off < passLen) {
#pragma unroll
			for(int i = 0; i < RPT; i++)
				if(off + i < passLen) {
					const double v = acc[i] + cadd;
					cnt += v != 0.0;
					out[passBeg + off + i] = v;
				}
		}
		passLen = nextLen;
		full = nfull;
		passBase = nextBase;
		voff = noff;
	}
	count_add(nnz, cnt);
}

// ---------------------------------------------------------------------------
// Generic row-parallel gather: a block owns 256 consecutive rows, a thread one row
// and a strip of output columns (blockIdx.y); groups in list order. Handles DDC,
// RLE (merged run table: one binary search per block and group, then a short
// walk) and uncompressed groups. SDCZeros groups are added afterwards.
// ---------------------------------------------------------------------------
constexpr int ROWS_QS = 8; // output columns per thread

__global__ __launch_bounds__(256) void k_rmm_rows(const DGroup* __restrict__ groups, int nGroups,
	const double* __restrict__ T, const double* __restrict__ B, int q, int constRow, double* __restrict__ out,
	int64_t nRows) {
	__shared__ int runBase;
	const int64_t r = (int64_t) blockIdx.x * 256 + threadIdx.x;
	const int c0 = blockIdx.y * ROWS_QS;
	const int nc = min(ROWS_QS, q - c0);
	const bool live = r < nRows;
	double acc[ROWS_QS];
#pragma unroll
	for(int c = 0; c < ROWS_QS; c++) acc[c] = 0.0;
	for(int g = 0; g < nGroups; g++) {
		const DGroup G = dgroup(groups + (g));
		if(G.type == G_DDC) {
			if(live) {
				const double* t = T + (size_t) (G.tblOff + load_code(G.codes, G.codeWidth, r)) * q + c0;
#pragma unroll
				for(int c = 0; c < ROWS_QS; c++)
					if(c < nc) acc[c] += t[c];
			}
		}
		else if(G.type == G_RLE) {
			__syncthreads();
			if(threadIdx.x == 0) runBase = rle_find(G.runStart, G.nRuns, (int32_t) ((int64_t) blockIdx.x * 256));
			__syncthreads();
			if(live) {
				int j = runBase;
				while(G.runStart[j + 1] <= r) j++;
				const int code = G.runCode[j];
				if(code >= 0) {
					const double* t = T + (size_t) (G.tblOff + code) * q + c0;
#pragma unroll
					for(int c = 0; c < ROWS_QS; c++)
						if(c < nc) acc[c] += t[c];
				}
			}
		}
		else if(G.type == G_UNC && live) {
#pragma unroll
			for(int c = 0; c < ROWS_QS; c++) {
				if(c >= nc) continue;
				double s = 0.0;
				for(int h = 0; h < G.nColG; h++) {
					const double a = G.dense[(size_t) r * G.nColG + h];
					if(a != 0) s = __dadd_rn(s, __dmul_rn(a, B[(size_t) G.cols[h] * q + c0 + c]));
				}
				acc[c] += s;
			}
		}
	}
	if(!live) return;
#pragma unroll
	for(int c = 0; c < ROWS_QS; c++)
		if(c < nc) out[(size_t) r * q + c0 + c] = acc[c] + (constRow >= 0 ? T[(size_t) constRow * q + c0 + c] : 0.0);
}

// One block per chunk of SDC_CK delta entries of one SDCZeros group: decode the
// rows with a wave prefix sum and add the group's table row to the output rows.
template <int W>
__global__ __launch_bounds__(256) void k_rmm_sdc_scatter(const DGroup* __restrict__ groups, int g,
	const double* __restrict__ T, int q, double* __restrict__ out) {
	const DGroup G = dgroup(groups + (g));
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

// K1 alone: T_g = dict_g x B[cols_g, :] for every group, constV x B in row totalVals.
int launch_tables(cla_block* b, const double* dB, int q) {
	const int nG = (int) b->groups.size();
	clear_stats(b);
	int rc = ensure_tables(b, (size_t) (b->totalVals + 1) * q);
	if(rc) return rc;
	const int maxWork = (b->maxVals > 1 ? b->maxVals : 1) * q;
	dim3 grid((maxWork + 255) / 256 > (q + 255) / 256 ? (maxWork + 255) / 256 : (q + 255) / 256, nG + 1);
	Prof pf(b, "k_preagg", (long) grid.x * grid.y, 256, 0, 0);
	hipLaunchKernelGGL(k_preagg, grid, dim3(256), 0, b->stream, b->dGroups, nG, dB, q, b->nCols,
		b->hasConst ? b->dConstV : nullptr, b->dTables, b->totalVals, b->dCounters, nullptr, 0);
	CLA_HIP(hipGetLastError());
	return 0;
}

// squares != 0 (q == 1, no uncompressed group): the tables hold the sum of squares of each tuple
// instead of dict x B, so that the gather yields rowSums(X^2).
// ws != nullptr: a workspace of wsDoubles doubles that the caller owns takes the place of the block's table
// buffer and nothing is allocated: kernels that need a derived format or a buffer of their own are left
// out (the tables then always come from the pre-aggregation kernel), and a block that needs them is refused.
int launch_rmm(cla_block* b, const double* dB, int q, double* dOut, unsigned long long* dNnz, int squares, double* ws,
	size_t wsDoubles) {
	const int nG = (int) b->groups.size();
	const int64_t nRows = b->nRows;
	hipStream_t st = b->stream;
	clear_stats(b);
	const bool noAlloc = ws != nullptr;
	// mat-vec on byte codes: all groups DDC in one arena, at most 256 values each
	const bool u8Path = q == 1 && nRows > 0 && b->dArena && b->arenaWidth == 1 && b->maxVals <= 256 && !(b->opt.rmmDisable & 1);
	const size_t nTbl = (size_t) (b->totalVals + 1) * q;
	const size_t nTblPad = (nTbl + 31) & ~(size_t) 31;
	const size_t need = u8Path ? nTblPad + (size_t) nG * 256 + 256 : nTbl;
	if(noAlloc) {
		if(need > wsDoubles) {
			set_error("rmm without allocation: the pre-aggregated tables need %zu bytes, the static workspace holds %zu", need * 8, wsDoubles * 8);
			return -CLA_ERR_UNSUPPORTED;
		}
	}
	else {
		const int rc = ensure_tables(b, need);
		if(rc) return rc;
	}
	double* const tables = noAlloc ? ws : b->dTables;
	double* dTpad = u8Path ? tables + nTblPad : nullptr;

	// Byte-code mat-vec with one column per group: the gather kernel makes its tables itself from the
	// padded dictionary image (built at finalize) and counts into a counter of its own that the call
	// before has cleared, so it is the only launch (K1 only runs for the constants' term, if any).
	const bool fused = u8Path && !squares && !noAlloc && b->dDictPad != nullptr && !(b->opt.rmmDisable & 2);
	const int32_t* dCol0 = fused ? (const int32_t*) (b->dDictPad + (size_t) nG * 256) : nullptr;
	if(fused) {
		b->nnzSlot = b->nnzRot;
		dNnz = b->dCounters + b->nnzSlot;
	}
	// Blocks of single-column SDCZeros lists only: the row-list kernel makes its tables from the dictionaries and
	// counts likewise into a counter that the call before has cleared: the only launch.
	if(q == 1 && !squares && !noAlloc && !u8Path && b->opt.sdcRows && nRows > 0 && dNnz == b->dCounters && rows_fusable(b)) {
		b->nnzSlot = b->nnzRot;
		const int r = launch_rmm_sdc_rows(b, -1, 0, dOut, b->dCounters + b->nnzSlot, dB, b->dCounters + (b->nnzRot % 3 + 1));
		if(r < 0) return r;
		if(r == 0) {
			b->nnzRot = b->nnzRot % 3 + 1;
			return 0;
		}
		b->nnzSlot = 0;
	}
	// K1 (also clears the non-zero counter)
	if(!fused || b->hasConst) {
		const int nK1 = fused ? 0 : nG; // fused: the constants' row only
		const int maxWork = (u8Path && !fused ? 256 : (b->maxVals > 1 ? b->maxVals : 1)) * q;
		dim3 grid(fused ? 1 : ((maxWork + 255) / 256 > (q + 255) / 256 ? (maxWork + 255) / 256 : (q + 255) / 256), nK1 + 1);
		Prof pf(b, "k_preagg", (long) grid.x * grid.y, 256, 0, 0);
		hipLaunchKernelGGL(k_preagg, grid, dim3(256), 0, st, b->dGroups, nK1, dB, q, b->nCols,
			b->hasConst ? b->dConstV : nullptr, tables, b->totalVals, dNnz, fused ? nullptr : dTpad, squares);
	}
	const int constRow = b->hasConst ? b->totalVals : -1;
	if(nRows == 0) return 0;

	if(u8Path) {
		constexpr int THREADS = 512;
		// persistent blocks: two per CU is what the register and LDS footprint allows; small
		// inputs get a block per 2048 rows
		const int perCU = 2;
		const unsigned grid = (unsigned) std::min<int64_t>((nRows + 2047) / 2048, (int64_t) g_numCU * perCU);
		const double bytes = (double) nRows * nG + (double) nRows * 8 + (double) b->totalVals * 8;
		// slab size: 16 or 20 groups, whichever leaves fewer padded table slots
		const int pad16 = (nG + 15) / 16 * 16 - nG, pad20 = (nG + 19) / 20 * 20 - nG;
		const int per = pad20 < pad16 ? 20 : 16;
		const double* constTerm = constRow >= 0 ? tables + constRow : nullptr;
		unsigned long long* nnzNext = fused ? b->dCounters + (b->nnzRot % 3 + 1) : nullptr;
		Prof pf(b, "k_rmm_q1_u8", grid, THREADS, per * 256 * 8, bytes);
#define U8_LAUNCH(PER, NBV, LB, LN, F)                                                                          \
	hipLaunchKernelGGL((k_rmm_q1_u8<THREADS, PER, NBV, LB, LN, F>), dim3(grid), dim3(THREADS), 0, st, b->dArena, \
		b->arenaStride, nG, F ? b->dDictPad : dTpad, constTerm, dOut, nRows, dNnz, dCol0, dB, nnzNext)
		if(per == 20) { if(fused) U8_LAUNCH(20, 5, 4, 2, true); else U8_LAUNCH(20, 5, 4, 2, false); }
		else { if(fused) U8_LAUNCH(16, 4, 8, 2, true); else U8_LAUNCH(16, 4, 8, 2, false); }
#undef U8_LAUNCH
		CLA_HIP(hipGetLastError());
		if(fused) b->nnzRot = b->nnzRot % 3 + 1;
		return 0;
	}
	if(q == 1 && b->dArena && b->q1LdsBytes > 0) {
		const int cw = b->arenaWidth;
		const int threads = b->q1Threads, rpt = cw == 4 ? 8 : 16;
		const int64_t rowsPerBlock = (int64_t) threads * rpt;
		const unsigned grid = (unsigned) ((nRows + rowsPerBlock - 1) / rowsPerBlock);
		const int nSlabs = (int) b->q1Slabs.size();
		const size_t lds = (size_t) b->q1LdsBytes;
		const double bytes = (double) nRows * cw * nG + (double) nRows * 8 + (double) b->totalVals * 8;
		Prof pf(b, "k_rmm_q1_ddc", grid, threads, (long) lds, bytes);
#define LAUNCH_Q1(CWV, RPTV, THR)                                                                               \
	do {                                                                                                        \
		auto kern = k_rmm_q1_ddc<CWV, RPTV, THR>;                                                               \
		CLA_HIP(allow_full_lds((const void*) kern)); \
		hipLaunchKernelGGL(kern, dim3(grid), dim3(THR), lds, st, b->dArena, b->arenaStride, nG, b->dQ1Slabs,    \
			nSlabs, b->dTblOff, tables, constRow, dOut, nRows, dNnz);                                       \
	} while(0)
#define LAUNCH_Q1_T(CWV, RPTV)                                                   \
	do {                                                                         \
		if(threads == 512) LAUNCH_Q1(CWV, RPTV, 512);                            \
		else if(threads == 1024) LAUNCH_Q1(CWV, RPTV, 1024);                     \
		else LAUNCH_Q1(CWV, RPTV, 256);                                          \
	} while(0)
		if(cw == 1) { if(rpt == 8) LAUNCH_Q1_T(1, 8); else LAUNCH_Q1_T(1, 16); }
		else if(cw == 2) { if(rpt == 8) LAUNCH_Q1_T(2, 8); else LAUNCH_Q1_T(2, 16); }
		else { if(rpt == 8) LAUNCH_Q1_T(4, 8); else LAUNCH_Q1_T(4, 16); }
#undef LAUNCH_Q1_T
#undef LAUNCH_Q1
		CLA_HIP(hipGetLastError());
		return 0;
	}

	// wide B on an all-DDC block: fused decode + fp64 MFMA (K1 above still supplies constV x B)
	if(q >= 8 && !noAlloc && !(b->opt.rmmDisable & 4)) {
		const int r = launch_rmm_mfma(b, dB, q, constRow >= 0 ? tables + (size_t) constRow * q : nullptr, dOut, dNnz);
		if(r <= 0) return r;
	}

	// narrow B on any group mix: decode rows from LDS dictionaries, B rows as scalars. A single column as well
	// where groups other than offset lists carry most of the block (the lists alone have kernels of their own
	// below): C5's X %*% v takes 1.5 ms here against 4.6 ms per row and group.
	bool vecDecode = false;
	if(q == 1) {
		int nLists = 0, nOther = 0;
		for(auto& g : b->groups) {
			if(g.d.type == G_SDCZ) nLists += g.d.nOffsets > 0;
			else nOther += g.d.type == G_UNC || g.d.nVals > 0;
		}
		vecDecode = nOther > 0 && nLists <= nOther;
	}
	// (not for the row sums of squares: the decode kernels multiply decoded values, the squares live in the tables)
	// (B wider than 16 columns: only blocks of plain streams, 16 columns of B per pass)
	if((q >= 2 || vecDecode) && !squares && !noAlloc && !(b->opt.rmmDisable & 8)) {
		const int r = launch_rmm_decode(b, dB, q, constRow >= 0 ? tables + (size_t) constRow * q : nullptr, dOut, dNnz);
		if(r <= 0) return r;
	}
	// 2 to 7 columns of B on an all-DDC block whose dictionaries the decode kernel cannot hold in LDS: the matrix-core
	// kernel on a zero-padded B (1.2 ms on C2, against 2.8 - 5 ms of the gather per row and group)
	if(q >= 2 && q < 8 && !noAlloc && !(b->opt.rmmDisable & 4)) {
		const int r = launch_rmm_mfma(b, dB, q, constRow >= 0 ? tables + (size_t) constRow * q : nullptr, dOut, dNnz);
		if(r <= 0) return r;
	}

	// wide B on a block that none of the kernels above takes: decompressed chunks of rows times B on the matrix cores
	// where that moves fewer bytes than the gather below (as a decoding kernel it multiplies every decoded value)
	if(q >= 16 && !squares && !noAlloc && !(b->opt.rmmDisable & 8)) {
		const int r = launch_rmm_decompressed(b, dB, q, dOut, dNnz);
		if(r <= 0) return r;
	}

	// generic path: row-parallel gather for DDC / RLE / uncompressed groups, then the
	// SDCZeros groups tile by tile (or per-entry scatter when their tables do not fit LDS)
	{
		const int64_t n = nRows * q;
		bool anyRowGroup = false, anySdc = false;
		for(auto& g : b->groups) {
			if(g.d.type == G_SDCZ) anySdc |= g.d.nOffsets > 0;
			else anyRowGroup = true;
		}
		if(anySdc && noAlloc) {
			set_error("rmm without allocation: SDC groups with entries need the row-tile plan, which this entry point cannot build");
			return -CLA_ERR_UNSUPPORTED;
		}
		bool needNnzPass = true;
		if(anyRowGroup || !anySdc) {
			const dim3 grid((unsigned) ((nRows + 255) / 256), (unsigned) ((q + ROWS_QS - 1) / ROWS_QS));
			Prof pf(b, "k_rmm_rows", (long) grid.x * grid.y, 256, 0, 0);
			hipLaunchKernelGGL(k_rmm_rows, grid, dim3(256), 0, st, b->dGroups, nG, tables, dB, q, constRow, dOut, nRows);
		}
		if(anySdc) {
			const int r = launch_rmm_sdc_tiles(b, q, constRow, anyRowGroup ? 1 : 0, dOut, dNnz);
			if(r < 0) return r;
			if(r == 0) needNnzPass = false;
			else {
				if(!anyRowGroup) {
					// the scatter adds on top of an initialised output
					const dim3 grid((unsigned) ((nRows + 255) / 256), (unsigned) ((q + ROWS_QS - 1) / ROWS_QS));
					Prof pf(b, "k_rmm_rows", (long) grid.x * grid.y, 256, 0, 0);
					hipLaunchKernelGGL(k_rmm_rows, grid, dim3(256), 0, st, b->dGroups, nG, tables, dB, q, constRow, dOut,
						nRows);
				}
				for(int g = 0; g < nG; g++) {
					const DGroup& G = b->groups[g].d;
					if(G.type != G_SDCZ || G.nOffsets == 0) continue;
					const unsigned sg = (unsigned) (G.nCkpt > 1 ? G.nCkpt : 1);
					Prof pf(b, "k_rmm_sdc_scatter", sg, 256, 0, 0);
					if(G.deltaWidth == 1)
						hipLaunchKernelGGL(k_rmm_sdc_scatter<1>, dim3(sg), dim3(256), 0, st, b->dGroups, g, tables, q, dOut);
					else
						hipLaunchKernelGGL(k_rmm_sdc_scatter<2>, dim3(sg), dim3(256), 0, st, b->dGroups, g, tables, q, dOut);
				}
			}
		}
		if(needNnzPass) {
			const unsigned cg = (unsigned) std::min<int64_t>((n + 256 * 8 - 1) / (256 * 8), (int64_t) g_numCU * 32);
			Prof pf(b, "k_count_nnz", cg, 256, 0, 0);
			hipLaunchKernelGGL(k_count_nnz, dim3(cg), dim3(256), 0, st, dOut, n, dNnz);
		}
	}
	CLA_HIP(hipGetLastError());
	return 0;
}

} // namespace cla
