// Left multiply pre-aggregation for blocks whose groups are all DDC with byte codes in one
// arena (the layout of the mat-vec gather): bins[g][code[g][r]] += Y[i, r].
//
// A persistent 1024-thread block owns an equal share of the rows. A thread keeps 16 values
// of Y in registers and streams the code runs of a slab of groups through a ping/pong pair
// of register batches, like k_rmm_q1_u8 does. The bins of the slab live in LDS in R copies
// (copy = lane % R, 257 doubles apart so that the copies of a bin fall into different banks):
// with skewed codes many lanes of a wave hit the same bin, and LDS serialises adds to one
// address, so R copies cut the longest chain by R. Adds return nothing, so a wave never
// waits for them. Every slab walks all rows of the block (Y is re-read per slab, it stays in
// the last-level cache) and is flushed once with global atomics.
#include "../../include/cla_hip.h"
#include "cla_device.hpp"
#include <algorithm>

namespace cla {

constexpr int LU_RPT = 16;
constexpr int LU_THREADS = 1024;
constexpr int LU_BINS = 257; // doubles per copy of a group's bins

template <int PER, int R, int NB>
__global__ __launch_bounds__(LU_THREADS) void k_lmm_u8(const DGroup* __restrict__ groups, const uint8_t* __restrict__ arena,
	size_t arenaStride, int nGroups, const double* __restrict__ Y, int64_t nRows, double* __restrict__ pre, int totalVals) {
	static_assert(PER % (2 * NB) == 0, "a slab holds whole ping/pong turns");
	extern __shared__ double bins[]; // PER * R * LU_BINS
	constexpr int RPT = LU_RPT, THREADS = LU_THREADS;
	const int tid = threadIdx.x, lane = tid & 63;
	const int off = tid * RPT;
	const int gLast = nGroups - 1;
	const int nPad = (nGroups + 2 * NB - 1) / (2 * NB) * (2 * NB);
	const double* y = Y + (size_t) blockIdx.y * nRows;
	double* dst = pre + (size_t) blockIdx.y * totalVals;

	// shares of whole units of 64 * RPT rows that differ by at most one unit between blocks (see k_rmm_q1_u8)
	constexpr int UNIT = 64 * RPT;
	const int64_t nUnits = (nRows + UNIT - 1) / UNIT;
	const int64_t unitsLo = nUnits / gridDim.x, unitsRem = nUnits % gridDim.x;
	const int64_t myUnits = unitsLo + ((int64_t) blockIdx.x < unitsRem ? 1 : 0);
	const int64_t blockBeg = ((int64_t) blockIdx.x * unitsLo + min((int64_t) blockIdx.x, unitsRem)) * UNIT;
	if(myUnits == 0 || blockBeg >= nRows) return;
	const int blockLen = (int) (min(nRows, blockBeg + myUnits * UNIT) - blockBeg);
	const int nPass = (blockLen + THREADS * RPT - 1) / (THREADS * RPT);
	const int passRows = ((blockLen + nPass - 1) / nPass + 64 * RPT - 1) / (64 * RPT) * (64 * RPT);
	auto pass_len = [&](int pass) { return pass < nPass ? min(passRows, blockLen - pass * passRows) : 0; };

	// byte offset of this lane's copy of the bins inside a group's R copies
	const int copyOff = (lane % R) * LU_BINS * 8;
	char* binBase = (char*) bins + copyOff;

	CodeVec<1, RPT> ping[NB], pong[NB];
	auto request = [&](CodeVec<1, RPT> (&cv)[NB], int pass, int g) { // codes of groups g .. g + NB - 1 for this thread's rows of `pass`
		const uint8_t* base = arena + (size_t) blockBeg + (size_t) pass * passRows;
		const uint32_t voff = off + RPT <= pass_len(pass) ? off : 0;
#pragma unroll
		for(int j = 0; j < NB; j++) cv[j].load(base + (size_t) min(g + j, gLast) * arenaStride + voff);
	};
	auto add = [&](const CodeVec<1, RPT> (&cv)[NB], int s, const double (&yv)[RPT]) { // slots s .. s + NB - 1 of the slab
#pragma unroll
		for(int j = 0; j < NB; j++) {
			char* bg = binBase + (s + j) * (R * LU_BINS * 8);
#pragma unroll
			for(int i = 0; i < RPT; i++) unsafeAtomicAdd((double*) (bg + (cv[j].get(i) << 3)), yv[i]);
		}
	};

	request(ping, 0, 0);
	for(int g0 = 0; g0 < nGroups; g0 += PER) {
		const int nIn = min(PER, nGroups - g0);
		const int gEnd = min(g0 + PER, nPad); // padded slots add into bins that are never flushed
		__syncthreads();
		for(int k = tid; k < PER * R * LU_BINS; k += THREADS) bins[k] = 0.0;
		__syncthreads();
		for(int pass = 0; pass < nPass; pass++) {
			const int passLen = pass_len(pass);
			const int64_t passBeg = blockBeg + (int64_t) pass * passRows;
			const bool full = off + RPT <= passLen;
			double yv[RPT];
			if(full) {
#pragma unroll
				for(int i = 0; i < RPT; i++) yv[i] = y[passBeg + off + i];
			}
			// what follows the last turn of this pass: the next pass of this slab, else the first pass of the next slab
			const bool lastPass = pass + 1 == nPass;
			const int nextPass = lastPass ? 0 : pass + 1;
			const int nextG = lastPass ? g0 + PER : g0;
			const bool haveNext = !lastPass || g0 + PER < nGroups;
#pragma unroll
			for(int s = 0; s < PER; s += 2 * NB) {
				if(g0 + s >= gEnd) break;
				request(pong, pass, g0 + s + NB);
				if(full) add(ping, s, yv);
				if(g0 + s + 2 * NB < gEnd) request(ping, pass, g0 + s + 2 * NB);
				else request(ping, haveNext ? nextPass : pass, haveNext ? nextG : g0);
				if(full) add(pong, s + NB, yv);
			}
			if(!full && off < passLen) { // ragged end of the matrix
				for(int g = 0; g < nIn; g++) {
					const uint8_t* codes = arena + (size_t) (g0 + g) * arenaStride + passBeg;
					for(int i = 0; off + i < passLen; i++)
						unsafeAtomicAdd((double*) (binBase + g * (R * LU_BINS * 8) + ((int) codes[off + i] << 3)), y[passBeg + off + i]);
				}
			}
		}
		__syncthreads();
		// flush: copies summed, one global add per non-zero bin
		for(int k = tid; k < nIn * 256; k += THREADS) {
			const int g = k >> 8, c = k & 255;
			const DGroup G = dgroup(groups + (g0 + g));
			if(c >= G.nVals) continue;
			double v = 0.0;
#pragma unroll
			for(int r = 0; r < R; r++) v += bins[(g * R + r) * LU_BINS + c];
			if(v != 0.0) unsafeAtomicAdd(&dst[G.tblOff + c], v);
		}
	}
}

// Returns 1 when the block is not eligible (caller uses the generic kernels), 0 when done.
int launch_lmm_u8(cla_block* b, const double* dY, int p, double* dPre) {
	const int nG = (int) b->groups.size();
	if(!(b->dArena && b->arenaWidth == 1 && b->maxVals <= 256 && nG > 0 && b->nRows > 0)) return 1;
	if(b->opt.lmmDisable & 2) return 1;
	// one persistent block per CU and row of Y; small inputs get a block per 4096 rows
	const unsigned grid = (unsigned) std::min<int64_t>((b->nRows + 4095) / 4096, std::max(1, g_numCU / std::min(p, g_numCU)));
	const double algo = (double) p * ((double) b->nRows * nG + (double) b->nRows * 8);
#define LU_LAUNCH(PER, R, NB)                                                                                   \
	do {                                                                                                        \
		const size_t lds = (size_t) PER * R * LU_BINS * 8;                                                      \
		Prof pf(b, "k_lmm_u8", (long) grid * p, LU_THREADS, (long) lds, algo);                                  \
		auto kern = k_lmm_u8<PER, R, NB>;                                                                       \
		CLA_HIP(allow_full_lds((const void*) kern)); \
		hipLaunchKernelGGL(kern, dim3(grid, p), dim3(LU_THREADS), lds, b->stream, b->dGroups, b->dArena,        \
			b->arenaStride, nG, dY, b->nRows, dPre, b->totalVals);                                              \
	} while(0)
	// 16 groups per slab with 4 copies of the bins measured best on skewed codes (0.89 ms on
	// 10M x 100; 2 copies 1.03 ms, 1 copy 1.33 ms)
	LU_LAUNCH(16, 4, 4);
#undef LU_LAUNCH
	CLA_HIP(hipGetLastError());
	return 0;
}

// ---------------------------------------------------------------------------
// The same blocks when every group has a single column: out[col_g] += sum_r Y[i, r] *
// dict_g[code_g[r]] directly, the mirror image of the mat-vec gather. Dictionaries of a slab
// of groups sit in LDS at a fixed stride, a thread keeps 16 values of Y in registers, looks
// up 16 dictionary values per group, multiplies and sums them and adds the sum into one of
// 16 LDS slots of the group; LDS reads are three to four times cheaper than the LDS adds of
// the bin kernel and there is one add per 16 rows. The reference sums Y per code first and
// multiplies once; the difference is rounding inside the 1e-12 bar.
// ---------------------------------------------------------------------------
constexpr int LD_THREADS = 512;
constexpr int LD_SLOTS = 16;

// s[j] = sum_i y[i] * table_j[code_j[i]] for NB groups; LDS reads in pinned batches of LB
// with LN batches in flight, like u8_consume of the gather kernel
template <int RPT, int NB, int LB, int LN>
__device__ __forceinline__ void u8_dot(const CodeVec<1, RPT> (&cv)[NB], const char* tb, const double (&y)[RPT], double (&s)[NB]) {
	static_assert(RPT % LB == 0, "a batch stays inside one group");
	constexpr int NBATCH = NB * RPT / LB;
	double t[LN][LB];
	auto issue = [&](int b) {
		const int j = (b * LB) / RPT, i0 = (b * LB) % RPT;
#pragma unroll
		for(int k = 0; k < LB; k++) t[b % LN][k] = *(const double*) (tb + j * 2048 + (cv[j].get(i0 + k) << 3));
	};
#pragma unroll
	for(int j = 0; j < NB; j++) s[j] = 0.0;
#pragma unroll
	for(int b = 0; b < LN - 1 && b < NBATCH; b++) issue(b);
	__builtin_amdgcn_sched_barrier(0);
#pragma unroll
	for(int b = 0; b < NBATCH; b++) {
		if(b + LN - 1 < NBATCH) issue(b + LN - 1);
		__builtin_amdgcn_sched_barrier(0);
		const int j = (b * LB) / RPT, i0 = (b * LB) % RPT;
#pragma unroll
		for(int k = 0; k < LB; k++) s[j] = __builtin_fma(y[i0 + k], t[b % LN][k], s[j]);
		__builtin_amdgcn_sched_barrier(0);
	}
}

template <int PER, int NB, int LB, int LN>
__global__ __launch_bounds__(LD_THREADS, 4) void k_lmm_u8_dot(const uint8_t* __restrict__ arena, size_t arenaStride, int nGroups,
	const double* __restrict__ dictPad, const int32_t* __restrict__ col0, const double* __restrict__ Y, int64_t nRows,
	double* __restrict__ out, int nCols, unsigned* __restrict__ done, unsigned long long* __restrict__ nnz) {
	static_assert(PER % (2 * NB) == 0, "a slab holds whole ping/pong turns");
	extern __shared__ double smem[];
	double* tbl = smem;                 // PER * 256: dictionaries of the current slab
	double* slots = smem + PER * 256;   // nGroups * LD_SLOTS partial sums, kept for the whole kernel
	const char* tb = (const char*) tbl;
	constexpr int RPT = LU_RPT, THREADS = LD_THREADS;
	const int tid = threadIdx.x;
	const int off = tid * RPT;
	const int gLast = nGroups - 1;
	const int nPad = (nGroups + PER - 1) / PER * PER;
	const double* y = Y + (size_t) blockIdx.y * nRows;

	// shares of whole units of 64 * RPT rows that differ by at most one unit between blocks (see k_rmm_q1_u8)
	constexpr int UNIT = 64 * RPT;
	const int64_t nUnits = (nRows + UNIT - 1) / UNIT;
	const int64_t unitsLo = nUnits / gridDim.x, unitsRem = nUnits % gridDim.x;
	const int64_t myUnits = unitsLo + ((int64_t) blockIdx.x < unitsRem ? 1 : 0);
	const int64_t blockBeg = ((int64_t) blockIdx.x * unitsLo + min((int64_t) blockIdx.x, unitsRem)) * UNIT;
	if(myUnits == 0 || blockBeg >= nRows) return;
	const int blockLen = (int) (min(nRows, blockBeg + myUnits * UNIT) - blockBeg);
	const int nPass = (blockLen + THREADS * RPT - 1) / (THREADS * RPT);
	const int passRows = ((blockLen + nPass - 1) / nPass + 64 * RPT - 1) / (64 * RPT) * (64 * RPT);

	for(int k = tid; k < nPad * LD_SLOTS; k += THREADS) slots[k] = 0.0;

	int passLen = min(passRows, blockLen);
	bool full = off + RPT <= passLen;
	const uint8_t* passBase = arena + (size_t) blockBeg;
	uint32_t voff = full ? off : 0;
	CodeVec<1, RPT> ping[NB], pong[NB];
	if(full) u8_load<RPT, NB>(ping, passBase, voff, arenaStride, 0, gLast);

	constexpr int TPT = (PER * 256 + THREADS - 1) / THREADS;
	double stage[TPT];
	auto fetch = [&](int g0) {
		const int nIn = min(PER, nGroups - g0) * 256;
		const double* src = dictPad + (size_t) g0 * 256;
		int tidF = tid; // laundered: keeps the index arithmetic out of registers between uses
		asm volatile("" : "+v"(tidF));
#pragma unroll
		for(int k = 0; k < TPT; k++) {
			const int f = tidF + k * THREADS;
			stage[k] = f < nIn ? src[f] : 0.0;
		}
	};
	fetch(0);
	double* mySlot = slots + (tid & (LD_SLOTS - 1));
	for(int pass = 0; pass < nPass; pass++) {
		const int64_t passBeg = blockBeg + (int64_t) pass * passRows;
		const int nextLen = pass + 1 < nPass ? min(passRows, blockLen - (pass + 1) * passRows) : 0;
		const bool nfull = off + RPT <= nextLen;
		const uint8_t* nextBase = nextLen > 0 ? passBase + passRows : passBase;
		const uint32_t noff = nfull ? off : 0;
		double yv[RPT];
#pragma unroll
		for(int i = 0; i < RPT; i++) yv[i] = full ? y[passBeg + off + i] : 0.0;
		for(int g0 = 0; g0 < nGroups; g0 += PER) {
			const int nIn = min(PER, nGroups - g0);
			__syncthreads();
			int tidW = tid;
			asm volatile("" : "+v"(tidW));
#pragma unroll
			for(int k = 0; k < TPT; k++) {
				const int f = tidW + k * THREADS;
				if(f < PER * 256) tbl[f] = stage[k];
			}
			__syncthreads();
			fetch(g0 + PER < nGroups ? g0 + PER : 0);
			if(full) {
#pragma unroll
				for(int s = 0; s < PER; s += 2 * NB) {
					double sum[NB];
					u8_load<RPT, NB>(pong, passBase, voff, arenaStride, g0 + s + NB, gLast);
					u8_dot<RPT, NB, LB, LN>(ping, tb + s * 2048, yv, sum);
#pragma unroll
					for(int j = 0; j < NB; j++) unsafeAtomicAdd(mySlot + (g0 + s + j) * LD_SLOTS, sum[j]);
					const int gn = g0 + s + 2 * NB;
					const bool wrap = gn >= nPad;
					u8_load<RPT, NB>(ping, wrap ? nextBase : passBase, wrap ? noff : voff, arenaStride, wrap ? 0 : gn, gLast);
					u8_dot<RPT, NB, LB, LN>(pong, tb + (s + NB) * 2048, yv, sum);
#pragma unroll
					for(int j = 0; j < NB; j++) unsafeAtomicAdd(mySlot + (g0 + s + NB + j) * LD_SLOTS, sum[j]);
				}
			}
			else if(off < passLen) { // ragged end of the matrix
				for(int g = 0; g < nIn; g++) {
					const uint8_t* codes = arena + (size_t) (g0 + g) * arenaStride + passBeg;
					double s = 0.0;
					for(int i = 0; off + i < passLen; i++) s += y[passBeg + off + i] * tbl[g * 256 + codes[off + i]];
					unsafeAtomicAdd(mySlot + (g0 + g) * LD_SLOTS, s);
				}
			}
		}
		passLen = nextLen;
		full = nfull;
		passBase = nextBase;
		voff = noff;
	}
	__syncthreads();
	for(int g = tid; g < nGroups; g += THREADS) {
		double v = 0.0;
#pragma unroll
		for(int k = 0; k < LD_SLOTS; k++) v += slots[g * LD_SLOTS + k];
		if(v != 0.0) unsafeAtomicAdd(&out[(size_t) blockIdx.y * nCols + col0[g]], v);
	}
	lmm_tail(done, gridDim.x * gridDim.y, out, (int) gridDim.y * nCols, nnz);
}

// All groups DDC with byte codes in one arena and one column each: the dictionaries at a fixed stride of
// 256 entries (zero beyond nVals), followed by the groups' column indexes. Built once at finalize (200 KB
// for 100 groups); the byte-code mat-vec and the dot-form left multiply read their slabs from it.
int ensure_dict_pad(cla_block* b) {
	const int nG = (int) b->groups.size();
	if(b->dDictPad != nullptr || !(b->dArena && b->arenaWidth == 1 && b->maxVals <= 256 && nG > 0 && b->nRows > 0)) return 0;
	for(int g = 0; g < nG; g++)
		if(b->groups[g].d.nColG != 1) return 0;
	std::vector<double> img((size_t) nG * 256 + (size_t) (nG + 1) / 2 + 1, 0.0);
	int32_t* cols = (int32_t*) (img.data() + (size_t) nG * 256);
	for(int g = 0; g < nG; g++) {
		const HostGroup& H = b->groups[g];
		std::copy(H.dict.begin(), H.dict.begin() + H.d.nVals, img.begin() + (size_t) g * 256);
		cols[g] = H.cols[0];
	}
	CLA_HIP(hipMalloc((void**) &b->dDictPad, img.size() * sizeof(double)));
	b->dictPadBytes = (int64_t) (img.size() * sizeof(double));
	b->derivedBytes += b->dictPadBytes;
	CLA_HIP(hipMemcpy(b->dDictPad, img.data(), img.size() * sizeof(double), hipMemcpyHostToDevice));
	return 0;
}

// Returns 1 when the block is not eligible, 0 when the groups' contributions have been added to dOut.
int launch_lmm_u8_dot(cla_block* b, const double* dY, int p, double* dOut) {
	const int nG = (int) b->groups.size();
	if(!(b->dArena && b->arenaWidth == 1 && b->maxVals <= 256 && nG > 0 && b->nRows > 0)) return 1;
	if(b->opt.lmmDisable & 1) return 1;
	// Y[row] * dict[code] summed over the rows differs from (sum of Y per code) * dict[code], the reference's order
	// (ADictionary pre-aggregation), where an infinite dictionary value meets values of Y of both signs
	if(b->dictNonFinite) return 1;
	for(int g = 0; g < nG; g++)
		if(b->groups[g].d.nColG != 1) return 1;
	constexpr int PER = 20;
	const int nPad = (nG + PER - 1) / PER * PER;
	const size_t lds = (size_t) PER * 256 * 8 + (size_t) nPad * LD_SLOTS * 8;
	if(lds > (size_t) 78 * 1024) return 1; // two blocks per CU
	if(b->dDictPad == nullptr) return 1;
	const int32_t* dCol0 = (const int32_t*) (b->dDictPad + (size_t) nG * 256);
	const int perCU = 2;
	const unsigned grid = (unsigned) std::min<int64_t>((b->nRows + 2047) / 2048, std::max(1, g_numCU * perCU / std::min(p, g_numCU * perCU)));
	const double algo = (double) p * ((double) b->nRows * nG + (double) b->nRows * 8);
	Prof pf(b, "k_lmm_u8_dot", (long) grid * p, LD_THREADS, (long) lds, algo);
	auto kern = k_lmm_u8_dot<PER, 5, 4, 2>;
	CLA_HIP(allow_full_lds((const void*) kern));
	const bool tail = b->lmmTailWanted; // (this kernel serves every group of the block)
	hipLaunchKernelGGL(kern, dim3(grid, p), dim3(LD_THREADS), lds, b->stream, b->dArena, b->arenaStride, nG, b->dDictPad, dCol0, dY,
		b->nRows, dOut, b->nCols, tail ? (unsigned*) (b->dCounters + 6) : nullptr, b->dCounters);
	b->lmmTailDone = tail;
	CLA_HIP(hipGetLastError());
	return 0;
}

} // namespace cla
