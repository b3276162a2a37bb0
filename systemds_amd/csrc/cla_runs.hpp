// Run cursors: how a wave that walks consecutive rows follows the run-length columns of a block without
// looking any row up. A run-length column (one column of a ColGroupRLE, CG/ColGroupRLE.java:104-141) is
// constant over a run, and a run is long against the 64 rows a wave handles per step, so the wave keeps per
// column the current value and the row where its run ends and only acts where a run ends inside its step.
// Lane RC_LANE0 + a of the wave is the cursor of run-length column a; a window of the next RC_WIN runs of
// every column sits in LDS and is refilled (run ends, codes, dictionary values: three dependent loads) only
// when a cursor leaves it.
#pragma once
#include "cla_device.hpp"
#include <vector>

namespace cla {

constexpr int RC_MAX = 8;     // run-length columns a wave follows
constexpr int RC_WIN = 8;     // runs per column in the wave's window (RC_MAX * RC_WIN = 64 lanes refill it)
constexpr int RC_LANE0 = 16;  // first cursor lane
constexpr int32_t RC_NEVER = 0x7fffffff;

struct RunCol {
	const int32_t* runStart;  // nRuns + 1 run starts of the merged run table (last = nRows)
	const int32_t* runCode;   // tuple per run, -1 = rows that no run covers
	const double* dict;       // nVals x nC
	double add;               // added to every value of the column (its constant where the caller wants decoded cells)
	int32_t nRuns, nC, h;     // h: the column's place in a tuple
	int32_t col;              // column of the matrix
};

// Merged run table of a block's run-length columns (k_runs.hip).
struct Mrt {
	void* base = nullptr;
	int32_t* start = nullptr;     // nSeg + 1
	int32_t* codes = nullptr;     // nSeg x nR
	int32_t* sliceRec = nullptr;  // 8 per slice: segment of the first row, run starts inside the slice, the first six of them
	double* sums = nullptr;       // nSeg x 16: workspace of the product at hand
	int nSeg = 0, nR = 0, sliceRows = 0;
	int64_t nSlices = 0, bytes = 0;
};

// Same-wave LDS traffic is ordered by the hardware; this keeps the compiler from moving accesses across.
__device__ __forceinline__ void wave_lds_sync() {
	__builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
	__builtin_amdgcn_wave_barrier();
	__builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// The cursors' state in LDS (one per wave), for kernels that are short of registers between two run ends.
struct RunPark {
	double val[RC_MAX];
	int32_t j[RC_MAX], jw[RC_MAX], end[RC_MAX];
};

struct RunCursors {
	int32_t j;     // cursor lanes: run the column is in
	int32_t jw;    // cursor lanes: run in slot 0 of the column's window
	int32_t end;   // cursor lanes: first row behind the run; RC_NEVER on all other lanes and behind the last run
	double val;    // cursor lanes: the column's value on the run
	const RunCol* cols;
	int nR;
	int32_t* winEnd;   // RC_MAX * RC_WIN, wave-private LDS
	double* winVal;

	// Window slot (a, k) = run jw_a + k of column a, loaded by lane 8 a + k.
	__device__ __forceinline__ void refill(int lane) {
		const int a = lane >> 3, k = lane & 7;
		const int jb = __shfl(j, RC_LANE0 + a, WAVE);
		int32_t e = RC_NEVER;
		double v = 0.0;
		if(a < nR) {
			const RunCol* C = as_global(cols + a);
			const int jj = jb + k;
			if(jj < C->nRuns) {
				e = as_global(C->runStart)[jj + 1];
				const int code = as_global(C->runCode)[jj];
				v = C->add + (code < 0 ? 0.0 : as_global(C->dict)[(size_t) code * C->nC + C->h]);
			}
		}
		wave_lds_sync();
		winEnd[lane] = e;
		winVal[lane] = v;
		wave_lds_sync();
		jw = j;
	}

	__device__ __forceinline__ void read_window(int lane) {
		const int a = lane - RC_LANE0;
		if(a >= 0 && a < nR) {
			end = winEnd[a * RC_WIN + (j - jw)];
			val = winVal[a * RC_WIN + (j - jw)];
		}
	}

	// Cursors at row r0 (every column's run that holds r0).
	__device__ __forceinline__ void start(const RunCol* c, int n, int32_t* we, double* wv, int32_t r0, int lane) {
		cols = c; nR = n; winEnd = we; winVal = wv;
		j = 0; jw = 0; end = RC_NEVER; val = 0.0;
		const int a = lane - RC_LANE0;
		if(a >= 0 && a < nR) {
			const RunCol* C = as_global(cols + a);
			j = rle_find(as_global(C->runStart), C->nRuns, r0);
		}
		if(nR > 0) {
			refill(lane);
			read_window(lane);
		}
	}

	__device__ __forceinline__ void park(RunPark* p, int lane) const {
		const int a = lane - RC_LANE0;
		wave_lds_sync();
		if(a >= 0 && a < RC_MAX) { p->val[a] = val; p->j[a] = j; p->jw[a] = jw; p->end[a] = end; }
		wave_lds_sync();
	}
	__device__ __forceinline__ void unpark(const RunPark* p, const RunCol* c, int n, int32_t* we, double* wv, int lane) {
		cols = c; nR = n; winEnd = we; winVal = wv;
		const int a = lane - RC_LANE0;
		j = 0; jw = 0; end = RC_NEVER; val = 0.0;
		if(a >= 0 && a < RC_MAX) { val = p->val[a]; j = p->j[a]; jw = p->jw[a]; end = p->end[a]; }
	}

	// First row at which some column's run ends (RC_NEVER: none does any more).
	__device__ __forceinline__ int32_t next_end() const {
		int32_t v = end;
		v = min(v, __builtin_amdgcn_update_dpp(v, v, 0x111, 0xf, 0xf, false)); // row_shr:1
		v = min(v, __builtin_amdgcn_update_dpp(v, v, 0x112, 0xf, 0xf, false)); // row_shr:2
		v = min(v, __builtin_amdgcn_update_dpp(v, v, 0x114, 0xf, 0xf, false)); // row_shr:4
		return __builtin_amdgcn_readlane(v, RC_LANE0 + RC_MAX - 1);
	}

	// Every column whose run ends at row e moves to its next run.
	__device__ __forceinline__ void advance(int32_t e, int lane) {
		const bool mine = end == e; // (never true outside the cursor lanes: e < RC_NEVER)
		if(mine) j++;
		if(__ballot(mine && j - jw >= RC_WIN) != 0) refill(lane);
		if(mine) read_window(lane);
	}

	// Value of column a (uniform).
	__device__ __forceinline__ double value(int a) const {
		int p[2];
		__builtin_memcpy(p, &val, 8);
		p[0] = __builtin_amdgcn_readlane(p[0], RC_LANE0 + a);
		p[1] = __builtin_amdgcn_readlane(p[1], RC_LANE0 + a);
		double r;
		__builtin_memcpy(&r, p, 8);
		return r;
	}
};

// Tail of a t(X) %*% X whose kernel is the only one of the call. The blocks have added their tiles' upper triangles
// into acc (nCols x nCols, all zero when the kernel starts); every block comes here behind its last add, and the last one
// to arrive copies acc to out, mirrored, counts out's non-zeros into *nnz and leaves acc and *done at zero for the next
// launch: what a fill of out in front of the kernel and a kernel of its own behind it would do. `lds`: 17 words of the
// block's LDS that nobody else uses any more (no static LDS here: the Gram kernels address theirs from offset zero).
__device__ __forceinline__ void gram_tail(unsigned* done, unsigned nBlocks, double* acc, double* out, int nCols, unsigned long long* nnz,
	unsigned* lds) {
	unsigned& gramTicketS = lds[0];
	int* const gramPartS = (int*) lds + 1;
	// this thread's adds have been acknowledged before the block takes its ticket (the adds, the ticket and the reads
	// below are all performed at device scope, past the caches that the chip's parts do not share)
	asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
	__syncthreads();
	if(threadIdx.x == 0) gramTicketS = atomicAdd(done, 1u);
	__syncthreads();
	if(gramTicketS != nBlocks - 1) return;
	int cnt = 0;
	for(int idx = threadIdx.x; idx < nCols * nCols; idx += blockDim.x) {
		const int i = idx / nCols, j = idx - i * nCols;
		if(j < i) continue;
		unsigned long long* cell = (unsigned long long*) acc + idx;
		const unsigned long long bits = __hip_atomic_load(cell, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
		__hip_atomic_store(cell, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
		double v;
		__builtin_memcpy(&v, &bits, 8);
		out[idx] = v;
		out[(size_t) j * nCols + i] = v;
		cnt += v != 0.0 ? (i == j ? 1 : 2) : 0;
	}
	cnt = wave_sum_i32(cnt);
	if((threadIdx.x & (WAVE - 1)) == 0) gramPartS[threadIdx.x >> 6] = cnt;
	__syncthreads();
	if(threadIdx.x == 0) {
		int s = 0;
		for(unsigned w = 0; w < (blockDim.x + WAVE - 1) / WAVE; w++) s += gramPartS[w];
		*nnz = (unsigned long long) s;
		*done = 0;
	}
}

int mrt_build(cla_block* b, const std::vector<RunCol>& runs, int sliceRows, Mrt& T);
void mrt_free(Mrt& T);
int launch_run_sums(cla_block* b, const std::vector<RunCol>& runs, const Mrt& T, const double* dB, int ld, int q, const double* dConstRow);

} // namespace cla
