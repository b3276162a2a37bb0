// Finalize-time and per-group helper kernels: code validation, exact integer
// counts, offset-list checkpoints and row-tile index.
#include "../../include/cla_hip.h"
#include "cla_device.hpp"
#include <algorithm>

namespace cla {

// ---------------------------------------------------------------------------
// max code of a stream (validation: every code must be < nVals)
// ---------------------------------------------------------------------------
// 16 bytes per thread and step; the elements behind the last full 16 bytes one by one
template <int W>
__global__ __launch_bounds__(256) void k_max_code(const void* __restrict__ codes, int64_t n, int* __restrict__ maxOut) {
	constexpr int PER = 16 / W;
	const int64_t nVec = n / PER;
	const u32x4* vec = (const u32x4*) codes;
	unsigned m = 0; // (a negative MapToInt entry is invalid as well: as unsigned it is a huge code)
	for(int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x; i < nVec; i += (int64_t) gridDim.x * blockDim.x) {
		const u32x4 v = __builtin_nontemporal_load(vec + i);
#pragma unroll
		for(int k = 0; k < 4; k++) {
			const unsigned x = v[k];
			if(W == 1) m = max(max(m, x & 0xffu), max(max((x >> 8) & 0xffu, (x >> 16) & 0xffu), x >> 24));
			else if(W == 2) m = max(m, max(x & 0xffffu, x >> 16));
			else m = max(m, x);
		}
	}
	if(blockIdx.x == 0 && threadIdx.x < (int) (n - nVec * PER)) {
		const int c = load_code(codes, W, nVec * PER + threadIdx.x);
		m = max(m, (unsigned) c);
	}
	m = min(m, 0x7fffffffu);
#pragma unroll
	for(int d = 32; d > 0; d >>= 1) m = max(m, (unsigned) __shfl_down((int) m, d, WAVE));
	if((threadIdx.x & 63) == 0) atomicMax(maxOut, (int) m);
}

int launch_validate_codes(cla_block* b, const void* codes, int width, int64_t n, int nVals, int* ok) {
	*ok = 1;
	if(n == 0) return 0;
	int rc = ensure_scratch(b, 64);
	if(rc) return rc;
	int* dMax = (int*) b->dScratch;
	int init = -1;
	CLA_HIP(hipMemcpyAsync(dMax, &init, sizeof(int), hipMemcpyHostToDevice, b->stream));
	if(((uintptr_t) codes & 15) != 0 || (width != 1 && width != 2 && width != 4)) {
		set_error("code stream: unaligned device buffer or width %d", width);
		return -CLA_ERR_INVALID;
	}
	const int64_t blocks = std::max<int64_t>(1, (n * width / 16 + 256 * 4 - 1) / (256 * 4));
	const unsigned grid = (unsigned) (blocks > 4096 ? 4096 : blocks);
	if(width == 1) hipLaunchKernelGGL(k_max_code<1>, dim3(grid), dim3(256), 0, b->stream, codes, n, dMax);
	else if(width == 2) hipLaunchKernelGGL(k_max_code<2>, dim3(grid), dim3(256), 0, b->stream, codes, n, dMax);
	else hipLaunchKernelGGL(k_max_code<4>, dim3(grid), dim3(256), 0, b->stream, codes, n, dMax);
	int mx = -1;
	CLA_HIP(hipMemcpyAsync(&mx, dMax, sizeof(int), hipMemcpyDeviceToHost, b->stream));
	CLA_HIP(hipStreamSynchronize(b->stream));
	*ok = mx < nVals;
	return 0;
}

// ---------------------------------------------------------------------------
// K10 counts: exact integer histogram of a code stream. Block-private bins in
// LDS (u32) when they fit, merged with integer atomics; bit-exact by
// construction. RLE groups sum their run lengths per value.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_counts_lds(const void* __restrict__ codes, int width, int64_t n, int nVals,
	int32_t* __restrict__ counts) {
	extern __shared__ unsigned int bins[];
	for(int i = threadIdx.x; i < nVals; i += blockDim.x) bins[i] = 0;
	__syncthreads();
	for(int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t) gridDim.x * blockDim.x)
		atomicAdd(&bins[load_code(codes, width, i)], 1u);
	__syncthreads();
	for(int i = threadIdx.x; i < nVals; i += blockDim.x)
		if(bins[i]) atomicAdd(&counts[i], (int) bins[i]);
}

__global__ __launch_bounds__(256) void k_counts_global(const void* __restrict__ codes, int width, int64_t n,
	int32_t* __restrict__ counts) {
	for(int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t) gridDim.x * blockDim.x)
		atomicAdd(&counts[load_code(codes, width, i)], 1);
}

// merged run table: count[code] += runStart[j+1] - runStart[j]
__global__ __launch_bounds__(256) void k_counts_rle(const int32_t* __restrict__ runStart,
	const int32_t* __restrict__ runCode, int nRuns, int32_t* __restrict__ counts) {
	const int j = blockIdx.x * blockDim.x + threadIdx.x;
	if(j >= nRuns) return;
	const int c = runCode[j];
	if(c >= 0) atomicAdd(&counts[c], runStart[j + 1] - runStart[j]);
}

int launch_counts(cla_block* b, int group, int32_t* dCounts) {
	const DGroup& G = b->groups[group].d;
	hipStream_t st = b->stream;
	CLA_HIP(hipMemsetAsync(dCounts, 0, sizeof(int32_t) * (size_t) G.nVals, st));
	if(G.type == G_RLE) {
		if(G.nRuns > 0)
			hipLaunchKernelGGL(k_counts_rle, dim3((G.nRuns + 255) / 256), dim3(256), 0, st, G.runStart, G.runCode, G.nRuns,
				dCounts);
	}
	else if(G.type == G_DDC || G.type == G_SDCZ) {
		const int64_t n = G.type == G_DDC ? b->nRows : G.nOffsets;
		if(n > 0) {
			int64_t blocks = (n + 256 * 32 - 1) / (256 * 32);
			if(blocks > g_numCU * 8) blocks = g_numCU * 8;
			const size_t lds = (size_t) G.nVals * 4;
			if(lds <= 48 * 1024)
				hipLaunchKernelGGL(k_counts_lds, dim3((unsigned) blocks), dim3(256), lds, st, G.codes, G.codeWidth, n, G.nVals,
					dCounts);
			else
				hipLaunchKernelGGL(k_counts_global, dim3((unsigned) blocks), dim3(256), 0, st, G.codes, G.codeWidth, n,
					dCounts);
		}
	}
	else {
		set_error("counts: group %d is not a dictionary-coded group", group);
		return -CLA_ERR_UNSUPPORTED;
	}
	CLA_HIP(hipGetLastError());
	return 0;
}

// ---------------------------------------------------------------------------
// Dictionary order by count. A DDC group with a dictionary beyond the first-level cache is looked up
// in global memory by the decode kernels; with skewed codes most lookups go to few tuples, and those
// share cache lines when they sit next to each other. The reference numbers tuples by first appearance
// (ColGroupFactory.java:682-703 through ACountHashMap.java:92-111), which puts frequent tuples first
// only roughly; here the block's own copy is renumbered by descending count at finalize: the codes in
// place, the dictionary rows alike. No product depends on the numbering (sums run over rows and
// columns, never over codes); the entry points that return arrays indexed by code (counts,
// co-occurrence, pre-aggregate) map their result back through HostGroup::codeOrder.
// ---------------------------------------------------------------------------
template <int W>
__global__ __launch_bounds__(256) void k_recode(void* codes, int64_t n, const uint32_t* __restrict__ lut) {
	constexpr int PER = 16 / W;
	const int64_t nVec = n / PER;
	u32x4* vec = (u32x4*) codes;
	for(int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x; i < nVec; i += (int64_t) gridDim.x * blockDim.x) {
		u32x4 v = vec[i];
#pragma unroll
		for(int k = 0; k < 4; k++) {
			if(W == 2) v[k] = lut[v[k] & 0xffffu] | (lut[v[k] >> 16] << 16);
			else v[k] = lut[v[k]];
		}
		vec[i] = v;
	}
	if(blockIdx.x == 0 && threadIdx.x < (int) (n - nVec * PER)) {
		const int64_t i = nVec * PER + threadIdx.x;
		if(W == 2) ((uint16_t*) codes)[i] = (uint16_t) lut[((const uint16_t*) codes)[i]];
		else ((uint32_t*) codes)[i] = lut[((const uint32_t*) codes)[i]];
	}
}

int reorder_ddc_by_count(cla_block* b, int group) {
	HostGroup& g = b->groups[group];
	DGroup& G = g.d;
	const int nVals = G.nVals;
	const int64_t n = b->nRows;
	// byte codes: at most 256 tuples, which the kernels hold in LDS or find in the first-level cache anyway
	if(G.type != G_DDC || (G.codeWidth != 2 && G.codeWidth != 4)) return 0;
	if((size_t) nVals * G.nColG * sizeof(double) < 16 * 1024 || n < 16 * (int64_t) nVals) return 0;
	int rc = ensure_scratch(b, sizeof(int32_t) * 2 * (size_t) nVals);
	if(rc) return rc;
	int32_t* dCounts = (int32_t*) b->dScratch;
	uint32_t* dLut = (uint32_t*) (dCounts + nVals);
	if((rc = launch_counts(b, group, dCounts))) return rc;
	std::vector<int32_t> counts(nVals);
	CLA_HIP(hipMemcpyAsync(counts.data(), dCounts, sizeof(int32_t) * (size_t) nVals, hipMemcpyDeviceToHost, b->stream));
	CLA_HIP(hipStreamSynchronize(b->stream));
	std::vector<int32_t> order(nVals); // new code -> old code
	for(int k = 0; k < nVals; k++) order[k] = k;
	std::stable_sort(order.begin(), order.end(), [&](int32_t x, int32_t y) { return counts[x] > counts[y]; });
	bool identity = true;
	for(int k = 0; k < nVals; k++) identity &= order[k] == k;
	if(identity) return 0;
	std::vector<uint32_t> lut(nVals);
	for(int k = 0; k < nVals; k++) lut[order[k]] = (uint32_t) k;
	CLA_HIP(hipMemcpyAsync(dLut, lut.data(), sizeof(uint32_t) * (size_t) nVals, hipMemcpyHostToDevice, b->stream));
	const int64_t blocks = std::max<int64_t>(1, (n * G.codeWidth / 16 + 256 * 4 - 1) / (256 * 4));
	const unsigned grid = (unsigned) std::min<int64_t>(blocks, (int64_t) g_numCU * 16);
	void* codes = const_cast<void*>(G.codes);
	Prof pf(b, "k_recode", grid, 256, 0, 2.0 * (double) n * G.codeWidth);
	if(G.codeWidth == 2) hipLaunchKernelGGL(k_recode<2>, dim3(grid), dim3(256), 0, b->stream, codes, n, dLut);
	else hipLaunchKernelGGL(k_recode<4>, dim3(grid), dim3(256), 0, b->stream, codes, n, dLut);
	CLA_HIP(hipGetLastError());
	const size_t w = (size_t) G.nColG;
	std::vector<double> nd(g.dict.size());
	for(int k = 0; k < nVals; k++) std::copy(g.dict.begin() + order[k] * w, g.dict.begin() + (order[k] + 1) * w, nd.begin() + k * w);
	g.dict.swap(nd);
	CLA_HIP(hipMemcpyAsync(const_cast<double*>(G.dict), g.dict.data(), sizeof(double) * g.dict.size(), hipMemcpyHostToDevice,
		b->stream));
	CLA_HIP(hipStreamSynchronize(b->stream));
	g.codeOrder.swap(order);
	return 0;
}

// ---------------------------------------------------------------------------
// Offset-list acceleration structures (device twin of AOffset's skip list).
// ---------------------------------------------------------------------------
// per chunk of SDC_CK entries: (sum of row increments, number of emitted rows)
template <int W>
__global__ __launch_bounds__(256) void k_sdc_chunk_sums(const void* __restrict__ deltas, int64_t nDeltas,
	int2* __restrict__ sums) {
	__shared__ int sInc[4], sNz[4];
	const int maxV = W == 1 ? 255 : 65535;
	const int64_t i0 = (int64_t) blockIdx.x * SDC_CK + threadIdx.x * 4;
	int inc = 0, nz = 0;
#pragma unroll
	for(int k = 0; k < 4; k++)
		if(i0 + k < nDeltas) {
			const int v = W == 1 ? (int) ((const uint8_t*) deltas)[i0 + k] : (int) ((const uint16_t*) deltas)[i0 + k];
			inc += v == 0 ? maxV : v;
			nz += v != 0;
		}
	inc = wave_sum_i32(inc);
	nz = wave_sum_i32(nz);
	if((threadIdx.x & 63) == 0) { sInc[threadIdx.x >> 6] = inc; sNz[threadIdx.x >> 6] = nz; }
	__syncthreads();
	if(threadIdx.x == 0) sums[blockIdx.x] = make_int2(sInc[0] + sInc[1] + sInc[2] + sInc[3], sNz[0] + sNz[1] + sNz[2] + sNz[3]);
}

// exclusive scan of the chunk sums into iterator states; entry nCkpt = final state
__global__ void k_sdc_scan(const int2* __restrict__ sums, int nCkpt, int first, OffState* __restrict__ ckpt) {
	if(threadIdx.x != 0 || blockIdx.x != 0) return;
	long long row = first;
	int emit = 1;
	for(int c = 0; c < nCkpt; c++) {
		OffState s;
		s.idx = c * SDC_CK; s.emit = emit; s.row = (int32_t) (row > 0x7fffffffLL ? 0x7fffffffLL : row); s.pad = 0;
		ckpt[c] = s;
		row += sums[c].x;
		emit += sums[c].y;
	}
	OffState s;
	s.idx = -1; s.emit = emit; s.row = (int32_t) (row > 0x7fffffffLL ? 0x7fffffffLL : row); s.pad = 0;
	ckpt[nCkpt] = s;
}

// tile t: iterator state in front of the first delta entry whose accumulated row reaches t * SDC_TILE.
// k_sdc_tile_ends writes the tiles that no entry reaches (at or in front of the first row: the initial state;
// behind the last row: the final one), k_sdc_tile_index the others: block = chunk of SDC_CK entries, a block-wide
// prefix sum gives every entry its state in front of it, and an entry writes the tiles whose first row lies
// in (row in front of it, row behind it].
__global__ __launch_bounds__(256) void k_sdc_tile_ends(const OffState* __restrict__ ckpt, int nCkpt, int64_t nDeltas, int first,
	int nTiles, OffState* __restrict__ tileIdx) {
	const int t = blockIdx.x * blockDim.x + threadIdx.x;
	if(t >= nTiles) return;
	OffState s;
	s.idx = 0; s.emit = 1; s.row = first; s.pad = 0;
	if(nCkpt > 0 && (int64_t) first < (int64_t) t * SDC_TILE) {
		s = ckpt[nCkpt];
		s.idx = (int32_t) nDeltas;
	}
	tileIdx[t] = s;
}

template <int W>
__global__ __launch_bounds__(256) void k_sdc_tile_index(const void* __restrict__ deltas, int64_t nDeltas,
	const OffState* __restrict__ ckpt, int nTiles, OffState* __restrict__ tileIdx) {
	__shared__ int sInc[4], sNz[4];
	const int maxV = W == 1 ? 255 : 65535;
	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const OffState st = ckpt[blockIdx.x];
	const int64_t i0 = (int64_t) blockIdx.x * SDC_CK + tid * 4;
	int inc[4], nz[4], incSum = 0, nzSum = 0;
#pragma unroll
	for(int k = 0; k < 4; k++) {
		inc[k] = 0; nz[k] = 0;
		if(i0 + k < nDeltas) {
			const int v = W == 1 ? (int) ((const uint8_t*) deltas)[i0 + k] : (int) ((const uint16_t*) deltas)[i0 + k];
			inc[k] = v == 0 ? maxV : v;
			nz[k] = v != 0;
		}
		incSum += inc[k]; nzSum += nz[k];
	}
	// exclusive prefix over the block: inside the wave by shuffles, across the four waves through LDS
	int incPre = incSum, nzPre = nzSum;
#pragma unroll
	for(int d = 1; d < 64; d <<= 1) {
		const int a = __shfl_up(incPre, d, 64), c = __shfl_up(nzPre, d, 64);
		if(lane >= d) { incPre += a; nzPre += c; }
	}
	if(lane == 63) { sInc[wave] = incPre; sNz[wave] = nzPre; }
	__syncthreads();
	int64_t row = (int64_t) st.row + (incPre - incSum);
	int emit = st.emit + (nzPre - nzSum);
	for(int w = 0; w < wave; w++) { row += sInc[w]; emit += sNz[w]; }
#pragma unroll
	for(int k = 0; k < 4; k++) {
		if(i0 + k >= nDeltas) break;
		const int64_t after = row + inc[k];
		for(int64_t t = row / SDC_TILE + 1; t <= after / SDC_TILE && t < nTiles; t++) {
			OffState s;
			s.idx = (int32_t) (i0 + k); s.emit = emit; s.row = (int32_t) row; s.pad = 0;
			tileIdx[t] = s;
		}
		row = after;
		emit += nz[k];
	}
}

int launch_sdc_build(cla_block* b, HostGroup& g) {
	DGroup& G = g.d;
	hipStream_t st = b->stream;
	const int nCkpt = (int) ((G.nDeltas + SDC_CK - 1) / SDC_CK);
	const int nTiles = (int) ((b->nRows + SDC_TILE - 1) / SDC_TILE);
	OffState* ckpt = nullptr;
	OffState* tiles = nullptr;
	int2* sums = nullptr;
	struct FreeSums { int2*& p; ~FreeSums() { if(p) (void) hipFree(p); } } freeSums{sums}; // on every way out
	CLA_HIP(hipMalloc((void**) &ckpt, sizeof(OffState) * (size_t) (nCkpt + 1)));
	g.owned.push_back(ckpt);
	CLA_HIP(hipMalloc((void**) &tiles, sizeof(OffState) * (size_t) (nTiles > 0 ? nTiles : 1)));
	g.owned.push_back(tiles);
	g.bytes += (int64_t) sizeof(OffState) * (nCkpt + 1 + nTiles);
	if(G.nOffsets == 0) {
		// empty list: every consumer checks nOffsets before emitting the first row
		CLA_HIP(hipMemsetAsync(ckpt, 0, sizeof(OffState) * (size_t) (nCkpt + 1), st));
		CLA_HIP(hipMemsetAsync(tiles, 0, sizeof(OffState) * (size_t) (nTiles > 0 ? nTiles : 1), st));
		CLA_HIP(hipStreamSynchronize(st));
		G.ckpt = ckpt; G.tileIdx = tiles; G.nCkpt = 0; G.nTiles = nTiles;
		return 0;
	}
	if(nCkpt > 0) {
		CLA_HIP(hipMalloc((void**) &sums, sizeof(int2) * (size_t) nCkpt));
		if(G.deltaWidth == 1)
			hipLaunchKernelGGL(k_sdc_chunk_sums<1>, dim3(nCkpt), dim3(256), 0, st, G.deltas, G.nDeltas, sums);
		else
			hipLaunchKernelGGL(k_sdc_chunk_sums<2>, dim3(nCkpt), dim3(256), 0, st, G.deltas, G.nDeltas, sums);
	}
	hipLaunchKernelGGL(k_sdc_scan, dim3(1), dim3(1), 0, st, sums, nCkpt, G.first, ckpt);
	if(nTiles > 0) {
		hipLaunchKernelGGL(k_sdc_tile_ends, dim3((nTiles + 255) / 256), dim3(256), 0, st, ckpt, nCkpt, G.nDeltas, G.first, nTiles, tiles);
		if(nCkpt > 0) {
			if(G.deltaWidth == 1)
				hipLaunchKernelGGL(k_sdc_tile_index<1>, dim3(nCkpt), dim3(256), 0, st, G.deltas, G.nDeltas, ckpt, nTiles, tiles);
			else
				hipLaunchKernelGGL(k_sdc_tile_index<2>, dim3(nCkpt), dim3(256), 0, st, G.deltas, G.nDeltas, ckpt, nTiles, tiles);
		}
	}
	OffState fin;
	CLA_HIP(hipMemcpyAsync(&fin, ckpt + nCkpt, sizeof(OffState), hipMemcpyDeviceToHost, st));
	CLA_HIP(hipStreamSynchronize(st));
	CLA_HIP(hipGetLastError());
	if(fin.row != G.last || fin.emit != G.nOffsets) {
		set_error("SDC offsets inconsistent: decoded last row %d / %d rows, declared offsetToLast %d / %lld rows",
			fin.row, fin.emit, G.last, (long long) G.nOffsets);
		return -CLA_ERR_INVALID;
	}
	if(G.last >= b->nRows) {
		set_error("SDC offsetToLast %d is outside the block (%lld rows)", G.last, (long long) b->nRows);
		return -CLA_ERR_INVALID;
	}
	G.ckpt = ckpt;
	G.tileIdx = tiles;
	G.nCkpt = nCkpt;
	G.nTiles = nTiles;
	return 0;
}

} // namespace cla
