// Device-side helpers shared by the kernels (gfx950, wave64).
#pragma once
#include "cla_internal.hpp"
#include <type_traits>

namespace cla {

constexpr int WAVE = 64;

// clang vector types: the non-temporal load/store builtins want these
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef double f64x2 __attribute__((ext_vector_type(2)));

// A pointer read out of a descriptor in memory is a generic pointer to the compiler, and a
// generic load also counts on the LDS counter: every wait for LDS data then waits for those
// loads too. All descriptor pointers point into device global memory; as_global says so
// (the empty asm keeps the round trip through the global address space from being folded
// away; the address-space inference then turns every access through the result into a
// global one).
template <class T>
__device__ __forceinline__ T* as_global(T* p) {
	__attribute__((address_space(1))) T* g = (__attribute__((address_space(1))) T*) p;
	asm("" : "+v"(g));
	return (T*) g;
}

// Descriptor copy whose pointers are known to be global.
__device__ __forceinline__ DGroup dgroup(const DGroup* p) {
	DGroup g = *p;
	g.codes = as_global(g.codes);
	g.dict = as_global(g.dict);
	g.cols = as_global(g.cols);
	g.deltas = as_global(g.deltas);
	g.ckpt = as_global(g.ckpt);
	g.tileIdx = as_global(g.tileIdx);
	g.runStart = as_global(g.runStart);
	g.runCode = as_global(g.runCode);
	g.dense = as_global(g.dense);
	return g;
}

// AMapToData.getIndex for the three device code widths (unsigned byte, char, int).
__device__ __forceinline__ int32_t load_code(const void* codes, int width, int64_t i) {
	if(width == 1) return ((const uint8_t*) codes)[i];
	if(width == 2) return ((const uint16_t*) codes)[i];
	return ((const int32_t*) codes)[i];
}

__device__ __forceinline__ int wave_sum_i32(int v) {
#pragma unroll
	for(int d = 32; d > 0; d >>= 1) v += __shfl_down(v, d, WAVE);
	return v;
}

__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
	for(int d = 32; d > 0; d >>= 1) v += __shfl_down(v, d, WAVE);
	return v;
}

// Adds a per-thread count into a global 64-bit counter: one atomic per wave.
__device__ __forceinline__ void count_add(unsigned long long* counter, int local) {
	const int s = wave_sum_i32(local);
	if((threadIdx.x & (WAVE - 1)) == 0 && s != 0) atomicAdd(counter, (unsigned long long) s);
}

// Tail of a left multiply whose kernel is the only one of the call: every block comes here behind its last add into
// out; the last one to arrive counts the non-zeros of out[0 .. n) into *nnz and leaves *done at zero for the next
// launch (the same is what a kernel of its own behind this one would do; done == nullptr: no tail).
__device__ __forceinline__ void lmm_tail(unsigned* done, unsigned nBlocks, const double* out, int n, unsigned long long* nnz) {
	if(done == nullptr) return;
	__shared__ unsigned ticketS;
	__shared__ int partS[16];
	// this thread's adds have been acknowledged before the block takes its ticket (the adds, the ticket and the reads
	// below are all performed at device scope, past the caches that the chip's parts do not share: no cache has to be
	// written back or invalidated, which a fence would do)
	asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
	__syncthreads();
	if(threadIdx.x == 0) ticketS = atomicAdd(done, 1u);
	__syncthreads();
	if(ticketS != nBlocks - 1) return;
	int cnt = 0;
	for(int i = threadIdx.x; i < n; i += blockDim.x) {
		// (read where the other blocks' adds were performed, not from a cache of this CU)
		const unsigned long long bits = __hip_atomic_load((const unsigned long long*) out + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
		cnt += (bits << 1) != 0ull; // != 0.0 (a NaN counts, a negative zero does not)
	}
	cnt = wave_sum_i32(cnt);
	if((threadIdx.x & (WAVE - 1)) == 0) partS[threadIdx.x >> 6] = cnt;
	__syncthreads();
	if(threadIdx.x == 0) {
		int s = 0;
		for(unsigned w = 0; w < (blockDim.x + WAVE - 1) / WAVE; w++) s += partS[w];
		*nnz = (unsigned long long) s;
		*done = 0;
	}
}

// Largest j in [0, nRuns) with runStart[j] <= row (runStart[0] == 0).
__device__ __forceinline__ int rle_find(const int32_t* __restrict__ runStart, int nRuns, int32_t row) {
	int lo = 0, hi = nRuns - 1;
	while(lo < hi) {
		const int mid = (lo + hi + 1) >> 1;
		if(runStart[mid] <= row) lo = mid; else hi = mid - 1;
	}
	return lo;
}

// Inclusive prefix sum over the 64 lanes of a wave (all lanes active) on the data-parallel
// primitives: shifts inside each row of 16 lanes, then the row totals broadcast to the rows
// behind (lane 15 of every row into rows 1 and 3, lane 31 into rows 2 and 3).
__device__ __forceinline__ int wave_scan_incl(int v) {
	v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false); // row_shr:1
	v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false); // row_shr:2
	v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false); // row_shr:4
	v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false); // row_shr:8
	v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false); // row_bcast:15
	v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false); // row_bcast:31
	return v;
}

// Sum over the 64 lanes of a wave (all lanes active), the same value in every lane: the scan
// above on the two halves of a double, total read from the last lane.
__device__ __forceinline__ double wave_sum_f64_all(double v) {
	auto dpp = [](double x, auto ctrlTag, auto rowTag) {
		constexpr int ctrl = decltype(ctrlTag)::value, rowMask = decltype(rowTag)::value;
		int p[2];
		__builtin_memcpy(p, &x, 8);
		p[0] = __builtin_amdgcn_update_dpp(0, p[0], ctrl, rowMask, 0xf, false);
		p[1] = __builtin_amdgcn_update_dpp(0, p[1], ctrl, rowMask, 0xf, false);
		double r;
		__builtin_memcpy(&r, p, 8);
		return r;
	};
	using std::integral_constant;
	v += dpp(v, integral_constant<int, 0x111>(), integral_constant<int, 0xf>());
	v += dpp(v, integral_constant<int, 0x112>(), integral_constant<int, 0xf>());
	v += dpp(v, integral_constant<int, 0x114>(), integral_constant<int, 0xf>());
	v += dpp(v, integral_constant<int, 0x118>(), integral_constant<int, 0xf>());
	v += dpp(v, integral_constant<int, 0x142>(), integral_constant<int, 0xa>());
	v += dpp(v, integral_constant<int, 0x143>(), integral_constant<int, 0xc>());
	int p[2];
	__builtin_memcpy(p, &v, 8);
	p[0] = __builtin_amdgcn_readlane(p[0], WAVE - 1);
	p[1] = __builtin_amdgcn_readlane(p[1], WAVE - 1);
	__builtin_memcpy(&v, p, 8);
	return v;
}

// One wave decodes 256 consecutive delta entries of an offset list starting at
// entry i0 from iterator state (row, emit). Lane l owns entries i0+4l .. i0+4l+3.
// A 0 entry advances the row by maxV without emitting (OffsetByte / OffsetChar
// semantics); `deltas` may be a window of the list that starts at entry winBase. On return rows[k] / didx[k] hold the absolute row and the data
// index of entry k when bit k of `mask` is set, and (row, emit) is the state
// behind the 256 entries.
template <int W>
__device__ __forceinline__ void sdc_decode256(const void* __restrict__ deltas, int64_t nDeltas, int64_t i0,
	int32_t& row, int32_t& emit, int32_t rows[4], int32_t didx[4], unsigned& mask, int64_t winBase = 0) {
	const int lane = threadIdx.x & (WAVE - 1);
	const int maxV = W == 1 ? 255 : 65535;
	const int64_t i = i0 + (int64_t) lane * 4;
	int s = 0, c = 0;
	mask = 0;
#pragma unroll
	for(int k = 0; k < 4; k++) {
		int v = -1;
		if(i + k < nDeltas) v = W == 1 ? (int) ((const uint8_t*) deltas)[i + k - winBase] : (int) ((const uint16_t*) deltas)[i + k - winBase];
		s += v < 0 ? 0 : (v == 0 ? maxV : v);
		rows[k] = s;
		didx[k] = c;
		if(v > 0) { mask |= 1u << k; c++; }
	}
	const int ps = wave_scan_incl(s), pc = wave_scan_incl(c);
	const int exs = ps - s, exc = pc - c;
#pragma unroll
	for(int k = 0; k < 4; k++) { rows[k] += row + exs; didx[k] += emit + exc; }
	row += __builtin_amdgcn_readlane(ps, WAVE - 1);
	emit += __builtin_amdgcn_readlane(pc, WAVE - 1);
}

// Walks the entries of group G with rows in [r0, r0 + tileRows) and calls f(row - r0, dataIdx)
// on the owning lane. Must be called by all 64 lanes of a wave.
template <typename F>
__device__ __forceinline__ void sdc_walk_tile(const DGroup& G, int64_t r0, int tileRows, F f) {
	// r0 and tileRows are multiples of SDC_TILE
	if(G.nOffsets <= 0) return;
	const int lane = threadIdx.x & 63;
	const int64_t rEnd = r0 + tileRows;
	if(lane == 0 && G.first >= r0 && G.first < rEnd) f((int) (G.first - r0), 0);
	const int ti = (int) (r0 / SDC_TILE);
	if(ti >= G.nTiles) return;
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
			if((mask & (1u << k)) && rows[k] < rEnd) f((int) (rows[k] - r0), didx[k]);
		i0 += 256;
	}
}

// BYTES bytes of a code stream in registers, requested as non-temporal 8/16-byte loads.
template <int BYTES>
struct RawVec;
template <>
struct RawVec<8> {
	u32x2 v;
	__device__ __forceinline__ void load(const uint8_t* p) { v = __builtin_nontemporal_load((const u32x2*) p); }
	__device__ __forceinline__ uint32_t word(int i) const { return i == 0 ? v.x : v.y; }
};
template <>
struct RawVec<16> {
	u32x4 v;
	__device__ __forceinline__ void load(const uint8_t* p) { v = __builtin_nontemporal_load((const u32x4*) p); }
	__device__ __forceinline__ uint32_t word(int i) const { return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w; }
};
template <>
struct RawVec<32> {
	u32x4 v[2];
	__device__ __forceinline__ void load(const uint8_t* p) {
		v[0] = __builtin_nontemporal_load((const u32x4*) p);
		v[1] = __builtin_nontemporal_load((const u32x4*) p + 1);
	}
	__device__ __forceinline__ uint32_t word(int i) const {
		const u32x4 q = v[i >> 2];
		const int j = i & 3;
		return j == 0 ? q.x : j == 1 ? q.y : j == 2 ? q.z : q.w;
	}
};
template <>
struct RawVec<64> {
	u32x4 v[4];
	__device__ __forceinline__ void load(const uint8_t* p) {
#pragma unroll
		for(int k = 0; k < 4; k++) v[k] = __builtin_nontemporal_load((const u32x4*) p + k);
	}
	__device__ __forceinline__ uint32_t word(int i) const {
		const u32x4 q = v[i >> 2];
		const int j = i & 3;
		return j == 0 ? q.x : j == 1 ? q.y : j == 2 ? q.z : q.w;
	}
};

// RPT codes of width CW held in registers
template <int CW, int RPT>
struct CodeVec {
	RawVec<CW * RPT> raw;
	__device__ __forceinline__ void load(const uint8_t* p) { raw.load(p); }
	__device__ __forceinline__ int get(int i) const {
		if(CW == 1) return (raw.word(i >> 2) >> (8 * (i & 3))) & 0xffu;
		if(CW == 2) return (raw.word(i >> 1) >> (16 * (i & 1))) & 0xffffu;
		return (int) raw.word(i);
	}
	// code i times 8 (the byte offset of an fp64 table entry). The compiler turns bytes 1-3 of a word into one
	// shift with a byte-select operand but byte 0 into a shift and a mask; written out, byte 0 is one
	// instruction as well, so that a table lookup costs two vector instructions (offset, add).
	__device__ __forceinline__ uint32_t off8(int i) const {
		if(CW == 1 && (i & 3) == 0) {
			uint32_t r;
			asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_0"
				: "=v"(r) : "v"(3u), "v"(raw.word(i >> 2)));
			return r;
		}
		return (uint32_t) get(i) << 3;
	}
};

// Batch request with a uniform base and a 32-bit per-thread offset: the address of every load
// is (scalar base + group * stride) + vector offset, which costs no vector arithmetic.
template <int RPT, int NB>
__device__ __forceinline__ void u8_load(CodeVec<1, RPT> (&cv)[NB], const uint8_t* base, uint32_t voff, size_t arenaStride, int g,
	int gLast) {
#pragma unroll
	for(int j = 0; j < NB; j++) cv[j].load(base + (size_t) min(g + j, gLast) * arenaStride + voff);
}

} // namespace cla
