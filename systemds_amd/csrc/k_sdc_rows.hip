// SDCZeros right multiply with one output column on row lists (gfx950).
//
//   k_rows_build      one-time transposition of the listed groups' offset and code lists into row lists
//   k_rmm_sdc_rows    out[row] = init + sum over the row's entries of T[entry]               (X %*% u)
//
// An SDCZeros group lists the rows that differ from the default; X %*% u needs, for every row, the sum of the
// table values of the groups that list it. Scattering the lists into an output tile in LDS costs one LDS add of
// a double per entry, about a cycle per lane. Here the lists are transposed once: every row gets the list of its
// entries, an entry being the 16-bit position of the (group, tuple) pair in the concatenation of the groups'
// tables. With the tables of a call in LDS a lane then owns a row: it reads its entries and sums the table
// values in a register - no atomics, no output tile, no barrier behind the table load.
//
// Layout: rows are cut into quarters of RW_Q = 256; inside a quarter the rows are sorted by their number of
// entries and dealt to the 64 lanes four at a time, long rows with short ones (the rows at places i, 127 - i,
// 128 + i and 255 - i of that order go to lane i), so that the lanes' lists are of nearly one length. A lane's list
// is its four rows' entries one after the other in groups of two (4 bytes; an odd row ends on the position of a 0.0
// behind the tables, a row without entries is one such group); bit 15 of a group marks a row's last group; the
// groups of the 64 lanes lie side by side (256 bytes, one coalesced load per wave), as many as the longest lane
// needs. perm holds, per lane, the four rows' places in the quarter. A row's entries are sorted by position, so that
// its sum does not depend on the order in which the lists were walked. A wave takes a quarter: a lane sums along its
// list, puts a sum into row order through a 2 KB buffer of the wave in LDS where a row ends, and the wave writes
// 256 consecutive rows.
#include "../../include/cla_hip.h"
#include "cla_device.hpp"
#include <algorithm>
#include <vector>

namespace cla {

constexpr int RW_WIN = SDC_TILE;   // rows per window (the conversion starts from the row-tile index)
constexpr int RW_KR = 40;          // most entries of a row (the conversion's staging area in LDS)
constexpr int RW_Q = 256;          // rows per quarter: the unit of sorting and of a wave's work
constexpr int RW_QW = RW_WIN / RW_Q; // quarters per window
constexpr int RW_F = RW_Q / 64;    // rows per lane and quarter
constexpr int RW_WAVES = 8;        // waves per block (C4: 0.110 / 0.095 / 0.086 / 0.088 / 0.097 ms with 4 / 6 / 8 / 12 / 16)
constexpr int RW_THREADS = RW_WAVES * 64;
constexpr int RW_PF = 24;          // groups of a quarter that a lane requests a quarter ahead
constexpr int RW_TBL_MAX = 16000;  // table entries of all listed groups in LDS (125 KB, next to 2 KB per wave)
constexpr uint32_t RW_LAST = 0x8000u; // a row's last group
static_assert(RW_WIN == 1024 && RW_Q == 256 && RW_F == 4 && RW_TBL_MAX < (int) RW_LAST,
	"a conversion block sorts the four quarters of a window; a row's place in its quarter is a byte; bit 15 of a position is free");

constexpr int RB_THREADS = 1024;   // threads of a conversion block (one window)

// block = window. FILL == false: the window's size in groups into winSize. FILL == true: headers, perm, data.
template <bool FILL>
__global__ __launch_bounds__(RB_THREADS) void k_rows_build(const DGroup* __restrict__ groups, const int32_t* __restrict__ list,
	const int32_t* __restrict__ gBase, int nL, int64_t nRows, uint32_t zeroIdx, uint32_t* __restrict__ winSize,
	const uint64_t* __restrict__ winOff, uint2* __restrict__ hdr, uint8_t* __restrict__ perm, uint32_t* __restrict__ data,
	int* __restrict__ overflow) {
	extern __shared__ uint32_t smemU[];
	uint32_t* cnt = smemU;                        // RW_WIN
	uint32_t* hist = cnt + RW_WIN;                // per quarter 64 (RW_KR + 1 used): rows per count, then first position per count
	uint32_t* kG = hist + 256;                     // RW_QW + 1: groups per quarter, then their prefix sums
	uint8_t* gcnt = (uint8_t*) (kG + 32);          // RW_WIN: groups of the row at (quarter, lane, turn)
	uint16_t* rowOf = (uint16_t*) (gcnt + RW_WIN); // RW_WIN: row at sorted position
	uint16_t* stage = rowOf + RW_WIN;             // RW_WIN x RW_KR
	const int tid = threadIdx.x;
	const int win = blockIdx.x;
	const int64_t r0 = (int64_t) win * RW_WIN;
	for(int k = tid; k < RW_WIN; k += RB_THREADS) cnt[k] = 0;
	if(tid < 256) hist[tid] = 0;
	if(tid < 32) kG[tid] = 0;
	__syncthreads();
	// a wave walks a group's part of the window at a time (256 offsets per step, decoded with a prefix sum over the wave)
	for(int l = tid >> 6; l < nL; l += RB_THREADS / 64) {
		const DGroup G = dgroup(groups + list[l]);
		const uint32_t gb = (uint32_t) gBase[l];
		const void* codes = G.codes;
		const int cw = G.codeWidth;
		sdc_walk_tile(G, r0, RW_WIN, [&](int rel, int di) {
			const uint32_t slot = atomicAdd(&cnt[rel], 1u);
			if(FILL && slot < (uint32_t) RW_KR) stage[rel * RW_KR + slot] = (uint16_t) (gb + (uint32_t) load_code(codes, cw, di));
		});
	}
	__syncthreads();
	// the rows of every quarter sorted by their number of entries, longest first
	bool over = false;
	for(int k = tid; k < RW_WIN; k += RB_THREADS) {
		over |= cnt[k] > (uint32_t) RW_KR;
		atomicAdd(&hist[(k / RW_Q) * 64 + min(cnt[k], (uint32_t) RW_KR)], 1u);
	}
	if(over) *overflow = 1; // a row with more entries than the staging area holds: the caller drops the row lists
	__syncthreads();
	if(tid < RW_QW) {
		uint32_t pos = tid * RW_Q;
		for(int c = RW_KR; c >= 0; c--) {
			const uint32_t n = hist[tid * 64 + c];
			hist[tid * 64 + c] = pos;
			pos += n;
		}
	}
	__syncthreads();
	for(int k = tid; k < RW_WIN; k += RB_THREADS) rowOf[atomicAdd(&hist[(k / RW_Q) * 64 + min(cnt[k], (uint32_t) RW_KR)], 1u)] = (uint16_t) k;
	__syncthreads();
	// thread = sorted position p: quarter, place s in the quarter's order -> (lane, turn)
	const int p = tid, qt = p / RW_Q, s = p % RW_Q;
	const int turn = s >> 6, lane = (turn & 1) ? 63 - (s & 63) : (s & 63);
	const int r = rowOf[p];
	const int c = (int) min(cnt[r], (uint32_t) RW_KR);
	const int gr = max(1, (c + 1) / 2);
	gcnt[(qt * 64 + lane) * RW_F + turn] = (uint8_t) gr;
	__syncthreads();
	int before = 0, all = 0;
#pragma unroll
	for(int k = 0; k < RW_F; k++) {
		const int g = gcnt[(qt * 64 + lane) * RW_F + k];
		before += k < turn ? g : 0;
		all += g;
	}
	if(turn == 0) atomicMax(&kG[qt], (uint32_t) all);
	__syncthreads();
	const uint32_t mine = kG[qt];
	uint32_t first = 0, total = 0;
#pragma unroll
	for(int k = 0; k < RW_QW; k++) {
		first += k < qt ? kG[k] : 0;
		total += kG[k];
	}
	if(!FILL) {
		if(tid == 0) winSize[win] = total;
		return;
	}
	const uint64_t base = winOff[win] + first;
	if(s == 0) hdr[(size_t) win * RW_QW + qt] = make_uint2((uint32_t) base, mine);
	perm[(((size_t) win * RW_QW + qt) * 64 + lane) * RW_F + turn] = (uint8_t) (r % RW_Q); // (position p lies in the quarter of its row)
	uint16_t* e = stage + r * RW_KR;
	for(int a = 1; a < c; a++) { // ascending positions
		const uint16_t x = e[a];
		int z = a - 1;
		for(; z >= 0 && e[z] > x; z--) e[z + 1] = e[z];
		e[z + 1] = x;
	}
	uint32_t* dst = data + (base + before) * 64 + lane;
	for(int q = 0; q < gr; q++) {
		const uint32_t lo = 2 * q < c ? e[2 * q] : zeroIdx, hi = 2 * q + 1 < c ? e[2 * q + 1] : zeroIdx;
		dst[(size_t) q * 64] = lo | hi << 16 | (q == gr - 1 ? RW_LAST : 0u);
	}
	if(turn == RW_F - 1)
		for(uint32_t q = (uint32_t) all; q < mine; q++) data[(base + q) * 64 + lane] = zeroIdx | zeroIdx << 16;
}

// block = 16 waves, all tables in LDS; a wave takes quarters in turn, a lane owns four rows of each.
// ACC == false: a row starts from constRow (or zero); ACC == true: from what other groups already wrote.
// FUSE (blocks of single-column lists only, nothing to add): the kernel makes the tables itself, T being the block's
// dictionaries and u the vector: table value = dictionary value * u[column]; block 0 clears *nnzNext, the counter of
// the next call, so that no other kernel runs in a call.
template <bool ACC, bool FUSE>
__global__ __launch_bounds__(RW_THREADS) void k_rmm_sdc_rows(const int32_t* __restrict__ tblIndex, int nTbl,
	const uint2* __restrict__ hdr, const uint32_t* __restrict__ perm, const uint32_t* __restrict__ data,
	const double* __restrict__ T, int constRow, double* __restrict__ out, int64_t nRows, int nQuarters,
	unsigned long long* __restrict__ nnz, const int32_t* __restrict__ tblCol, const double* __restrict__ u,
	unsigned long long* __restrict__ nnzNext) {
	extern __shared__ double smemD[];
	double* tbl = smemD;                 // nTbl values and a 0.0
	const int tid = threadIdx.x, lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	double* back = smemD + (nTbl + 2) / 2 * 2 + wave * RW_Q; // this wave's sums in row order
	{ // all of a thread's table values requested before the first is stored (two dependent loads each)
		constexpr int TPT = (RW_TBL_MAX + RW_THREADS - 1) / RW_THREADS;
		int32_t ti[TPT];
		double tv[TPT];
#pragma unroll
		for(int j = 0; j < TPT; j++) ti[j] = tblIndex[min(j * RW_THREADS + tid, nTbl - 1)];
#pragma unroll
		for(int j = 0; j < TPT; j++) tv[j] = T[ti[j]];
		if(FUSE) {
			double uv[TPT];
#pragma unroll
			for(int j = 0; j < TPT; j++) uv[j] = u[tblCol[min(j * RW_THREADS + tid, nTbl - 1)]];
#pragma unroll
			for(int j = 0; j < TPT; j++) tv[j] = __dmul_rn(tv[j], uv[j]);
		}
#pragma unroll
		for(int j = 0; j < TPT; j++)
			if(j * RW_THREADS + tid < nTbl) tbl[j * RW_THREADS + tid] = tv[j];
	}
	if(tid == 0) tbl[nTbl] = 0.0;
	if(FUSE && blockIdx.x == 0 && tid == 0) *nnzNext = 0;
	const double init = !ACC && constRow >= 0 ? T[constRow] : 0.0;
	__syncthreads();
	int cntNz = 0;
	// Requested a quarter ahead (two register sets take turns): the first groups of its lists, the lane's rows, the
	// start values; two quarters ahead: the quarter's header. The work on a set is straight-line code.
	struct Ahead {
		uint32_t v[RW_PF];
		uint2 h;
		uint32_t p;
		double start[RW_F];
	};
	// (a vector load although the address is uniform: a scalar load is counted with the LDS reads, whose waits would
	// then wait for it too)
	int vzero = 0;
	asm volatile("" : "+v"(vzero));
	auto header = [&](int qt) { return hdr[min(qt, nQuarters - 1) + vzero]; };
	auto request = [&](Ahead& A, int qt, const uint2 h) { // qt < nQuarters
		A.h = make_uint2((uint32_t) __builtin_amdgcn_readfirstlane((int) h.x), (uint32_t) __builtin_amdgcn_readfirstlane((int) h.y));
		const uint32_t* src = data + (size_t) A.h.x * 64 + lane;
		const int kq = (int) A.h.y; // (at least four groups: a row has one)
#pragma unroll
		for(int q = 0; q < RW_PF; q++) A.v[q] = __builtin_nontemporal_load(src + (size_t) min(q, kq - 1) * 64);
		A.p = perm[(size_t) qt * 64 + lane];
#pragma unroll
		for(int j = 0; j < RW_F; j++) {
			A.start[j] = init;
			if(ACC) A.start[j] = out[min((int64_t) qt * RW_Q + j * 64 + lane, nRows - 1)]; // (a template parameter: a load under a run-time branch is waited for at the branch's end)
		}
	};
	const int step = gridDim.x * RW_WAVES;
	auto work = [&](Ahead& A, Ahead& B, int qt, uint2& hNext) { // A holds the requests of `qt`, hNext the header of qt + step
		request(B, min(qt + step, nQuarters - 1), hNext);
		hNext = header(qt + 2 * step);
		const int kq = (int) A.h.y;
		uint32_t pw = A.p;
		double acc = 0.0;
		auto close = [&](uint32_t e) { // a group with bit 15 set ends the row at hand
			if(e & RW_LAST) {
				back[pw & 0xffu] = acc;
				acc = 0.0;
				pw >>= 8;
			}
		};
		const uint32_t none = (uint32_t) nTbl * 0x00010001u; // a group of two 0.0
		// four groups' table values requested before the first is added (a row's end is a branch: the compiler does not
		// move LDS reads across it)
#pragma unroll
		for(int q0 = 0; q0 < RW_PF; q0 += 4) {
			if(q0 < kq) {
				uint32_t e[4];
				double a[4], b2[4];
#pragma unroll
				for(int j = 0; j < 4; j++) {
					e[j] = q0 + j < kq ? A.v[q0 + j] : none;
					a[j] = tbl[e[j] & (RW_LAST - 1)];
					b2[j] = tbl[e[j] >> 16];
				}
#pragma unroll
				for(int j = 0; j < 4; j++) {
					acc = (acc + a[j]) + b2[j];
					close(e[j]);
				}
			}
		}
		const uint32_t* src = data + (size_t) A.h.x * 64 + lane;
		for(int q = RW_PF; q < kq; q++) {
			const uint32_t e = src[(size_t) q * 64];
			acc = (acc + tbl[e & (RW_LAST - 1)]) + tbl[e >> 16];
			close(e);
		}
		__builtin_amdgcn_wave_barrier(); // LDS serves a wave's accesses in order: the reads below see the sums
#pragma unroll
		for(int j = 0; j < RW_F; j++) {
			const int64_t r = (int64_t) qt * RW_Q + j * 64 + lane;
			const double res = A.start[j] + back[j * 64 + lane];
			if(r < nRows) {
				cntNz += res != 0.0;
				__builtin_nontemporal_store(res, &out[r]);
			}
		}
		__builtin_amdgcn_wave_barrier();
	};
	const int q0 = blockIdx.x * RW_WAVES + wave;
	if(q0 < nQuarters) {
		Ahead A, B;
		request(A, q0, header(q0));
		uint2 hNext = header(q0 + step);
		for(int qt = q0; qt < nQuarters; qt += 2 * step) {
			work(A, B, qt, hNext);
			if(qt + step < nQuarters) work(B, A, qt + step, hNext);
		}
	}
	count_add(nnz, cntNz);
}

// The row lists of the block's listed groups (whole-block plan), built once.
static int rows_plan(cla_block* b) {
	if(b->rowsState != 0) return 0;
	b->rowsState = -1;
	const std::vector<int32_t>& list = b->sdcList;
	const int nL = (int) list.size();
	const int nWin = (int) ((b->nRows + RW_WIN - 1) / RW_WIN);
	if(nL == 0 || nWin == 0 || b->nRows >= ((int64_t) 1 << 31) - RW_WIN) return 0;
	std::vector<int32_t> gBase(nL + 1, 0);
	double entries = 0;
	for(int l = 0; l < nL; l++) {
		const DGroup& G = b->groups[list[l]].d;
		gBase[l + 1] = gBase[l] + G.nVals;
		entries += (double) G.nOffsets;
	}
	const int nTbl = gBase[nL];
	if(nTbl > RW_TBL_MAX || nTbl >= 65535) return 0; // an entry is a 16-bit position; all tables sit in LDS
	if(entries > (double) b->nRows * (RW_KR / 2)) return 0; // dense lists: rows too long for the staging area
	if(sizeof(double) * ((size_t) nTbl + 2 + (size_t) RW_WAVES * RW_Q) > (size_t) std::min(g_ldsPerBlock, 160 * 1024)) return 0;
	std::vector<int32_t> tblIndex(nTbl), tblCol(nTbl);
	// (fusable: the listed groups are all of the block and have one column each, so that a group's dictionary sits in
	// the block's dictionary buffer where its table sits in the table buffer)
	bool fusable = (size_t) nL == b->groups.size() && !b->hasConst && b->dAllDict != nullptr;
	for(int l = 0; l < nL; l++) {
		const DGroup& G = b->groups[list[l]].d;
		fusable = fusable && G.nColG == 1 && G.dict == b->dAllDict + G.tblOff;
		for(int k = 0; k < G.nVals; k++) {
			tblIndex[gBase[l] + k] = G.tblOff + k;
			tblCol[gBase[l] + k] = b->groups[list[l]].cols[0];
		}
	}
	hipStream_t st = b->stream;
	const size_t idxBytes = 2 * ((sizeof(int32_t) * (size_t) nTbl + 15) / 16 * 16), listBytes = (sizeof(int32_t) * 2 * (size_t) nL + 15) / 16 * 16;
	const size_t sizeBytes = (sizeof(uint64_t) * (size_t) nWin + 15) / 16 * 16, hdrBytes = sizeof(uint2) * (size_t) nWin * RW_QW;
	const size_t permBytes = sizeof(uint8_t) * (size_t) nWin * RW_WIN;
	char* meta = nullptr;
	CLA_HIP(hipMalloc((void**) &meta, idxBytes + listBytes + sizeBytes + hdrBytes + permBytes + 16));
	b->dRowsMeta = meta;
	int32_t* dIdx = (int32_t*) meta;
	int32_t* dList = (int32_t*) (meta + idxBytes);
	int32_t* dBase = dList + nL;
	uint64_t* dOff = (uint64_t*) (meta + idxBytes + listBytes); // pass 1: 32-bit sizes; pass 2: 64-bit offsets
	uint2* dHdr = (uint2*) (meta + idxBytes + listBytes + sizeBytes);
	uint8_t* dPerm = (uint8_t*) (meta + idxBytes + listBytes + sizeBytes + hdrBytes);
	int* dOver = (int*) (meta + idxBytes + listBytes + sizeBytes + hdrBytes + permBytes);
	CLA_HIP(hipMemcpyAsync(dIdx, tblIndex.data(), sizeof(int32_t) * (size_t) nTbl, hipMemcpyHostToDevice, st));
	CLA_HIP(hipMemcpyAsync((char*) dIdx + idxBytes / 2, tblCol.data(), sizeof(int32_t) * (size_t) nTbl, hipMemcpyHostToDevice, st));
	CLA_HIP(hipMemcpyAsync(dList, list.data(), sizeof(int32_t) * (size_t) nL, hipMemcpyHostToDevice, st));
	CLA_HIP(hipMemcpyAsync(dBase, gBase.data(), sizeof(int32_t) * (size_t) nL, hipMemcpyHostToDevice, st));
	CLA_HIP(hipMemsetAsync(dOver, 0, sizeof(int), st));
	const size_t lds = sizeof(uint32_t) * (RW_WIN + 256 + 32) + RW_WIN + sizeof(uint16_t) * ((size_t) RW_WIN + (size_t) RW_WIN * RW_KR);
	CLA_HIP(allow_full_lds((const void*) k_rows_build<false>));
	CLA_HIP(allow_full_lds((const void*) k_rows_build<true>));
	hipLaunchKernelGGL(k_rows_build<false>, dim3(nWin), dim3(RB_THREADS), lds, st, b->dGroups, dList, dBase, nL, b->nRows, (uint32_t) nTbl,
		(uint32_t*) dOff, nullptr, nullptr, nullptr, nullptr, dOver);
	CLA_HIP(hipGetLastError());
	std::vector<uint32_t> sizes(nWin);
	int over = 0;
	CLA_HIP(hipMemcpyAsync(sizes.data(), dOff, sizeof(uint32_t) * (size_t) nWin, hipMemcpyDeviceToHost, st));
	CLA_HIP(hipMemcpyAsync(&over, dOver, sizeof(int), hipMemcpyDeviceToHost, st));
	CLA_HIP(hipStreamSynchronize(st)); // (also: the host vectors above have been read)
	if(over) return 0;
	std::vector<uint64_t> offs(nWin);
	uint64_t total = 0;
	for(int w = 0; w < nWin; w++) {
		offs[w] = total;
		total += sizes[w];
	}
	if(total > 0xfffffff0ull) return 0; // (headers hold 32-bit group offsets)
	const size_t dataBytes = (size_t) (total + 1) * 64 * sizeof(uint32_t);
	size_t freeB = 0, totalB = 0;
	CLA_HIP(hipMemGetInfo(&freeB, &totalB));
	if(dataBytes + ((size_t) 1 << 30) > freeB) return 0;
	CLA_HIP(hipMalloc((void**) &b->dRowsData, dataBytes));
	b->derivedBytes += (int64_t) (idxBytes + listBytes + sizeBytes + hdrBytes + permBytes + dataBytes);
	CLA_HIP(hipMemsetAsync((char*) b->dRowsData + dataBytes - 64 * sizeof(uint32_t), 0, 64 * sizeof(uint32_t), st));
	CLA_HIP(hipMemcpyAsync(dOff, offs.data(), sizeof(uint64_t) * (size_t) nWin, hipMemcpyHostToDevice, st));
	hipLaunchKernelGGL(k_rows_build<true>, dim3(nWin), dim3(RB_THREADS), lds, st, b->dGroups, dList, dBase, nL, b->nRows, (uint32_t) nTbl,
		nullptr, dOff, dHdr, dPerm, (uint32_t*) b->dRowsData, dOver);
	CLA_HIP(hipGetLastError());
	CLA_HIP(hipStreamSynchronize(st)); // `offs` goes out of scope
	b->rowsTbl = nTbl;
	b->rowsOff[0] = idxBytes + listBytes + sizeBytes;
	b->rowsOff[1] = idxBytes + listBytes + sizeBytes + hdrBytes;
	b->rowsColOff = idxBytes / 2;
	b->rowsFusable = fusable;
	b->rowsState = 1;
	return 0;
}

// X %*% u of all listed groups (tables in b->dTables). Returns 1 when the lists do not fit (tables beyond LDS or
// 16-bit positions, rows with too many entries), 0 when done. dU != nullptr: the kernel makes the tables itself
// (rows_fusable said it can) and clears *nnzNext.
int launch_rmm_sdc_rows(cla_block* b, int constRow, int accumulate, double* dOut, unsigned long long* dNnz, const double* dU,
	unsigned long long* nnzNext) {
	int rc = rows_plan(b);
	if(rc) return rc;
	if(b->rowsState != 1 || (dU != nullptr && !b->rowsFusable)) return 1;
	const int nQuarters = (int) ((b->nRows + RW_Q - 1) / RW_Q);
	const size_t lds = sizeof(double) * ((size_t) (b->rowsTbl + 2) / 2 * 2 + (size_t) RW_WAVES * RW_Q);
	const unsigned grid = (unsigned) std::min((nQuarters + RW_WAVES - 1) / RW_WAVES, g_numCU);
	char* meta = (char*) b->dRowsMeta;
	double algo = (double) b->nRows * 8 * (accumulate ? 2 : 1);
	for(int g : b->sdcList) algo += (double) b->groups[g].d.nDeltas * b->groups[g].d.deltaWidth + (double) b->groups[g].d.nOffsets * b->groups[g].d.codeWidth;
	Prof pf(b, "k_rmm_sdc_rows", (long) grid, RW_THREADS, (long) lds, algo);
	auto go = [&](auto kernel) {
		CLA_HIP(allow_full_lds((const void*) kernel));
		hipLaunchKernelGGL(kernel, dim3(grid), dim3(RW_THREADS), lds, b->stream, (const int32_t*) meta, b->rowsTbl,
			(const uint2*) (meta + b->rowsOff[0]), (const uint32_t*) (meta + b->rowsOff[1]), (const uint32_t*) b->dRowsData,
			dU ? (const double*) b->dAllDict : (const double*) b->dTables, constRow, dOut, b->nRows, nQuarters, dNnz,
			(const int32_t*) (meta + b->rowsColOff), dU, nnzNext);
		return 0;
	};
	if((rc = dU ? go(k_rmm_sdc_rows<false, true>) : accumulate ? go(k_rmm_sdc_rows<true, false>) : go(k_rmm_sdc_rows<false, false>))) return rc;
	CLA_HIP(hipGetLastError());
	return 0;
}

// Whether X %*% u of this block can run as the one kernel above with tables of its own (builds the row lists on
// first use).
bool rows_fusable(cla_block* b) {
	if(b->hasConst || b->hasUnc || b->hasRle || !b->hasSdc || b->nRows == 0) return false;
	for(auto& g : b->groups)
		if(g.d.type != G_SDCZ || g.d.nOffsets <= 0 || g.d.nColG != 1) return false;
	if(sdc_plan_all(b) != 0 || rows_plan(b) != 0) return false;
	return b->rowsState == 1 && b->rowsFusable;
}

} // namespace cla
