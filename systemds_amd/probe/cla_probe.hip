// Device probe: the rates and the operand layout that the kernels of this library are built on, measured
// on the device at hand with stand-alone loops. A maintainer who moves the library to another part runs it
// first; the figures quoted next to the kernels come from it.
//   1. v_mfma_f64_4x4x4_f64 operand layout (one-hot operands) against the layout k_rmm_mfma / k_tsmm_decode assume
//   2. rate of the two fp64 matrix instructions (register-only loops, 16 accumulators, 2 waves per SIMD)
//   3. streaming reads from HBM: one flat buffer, and 100 strided code streams as the byte-code mat-vec reads them
//   4. L2 -> CU: global_load_lds_dwordx4 against loads through registers, all CUs on one 256 KB region
//   5. stores of 16 bytes per lane: 1 KB contiguous per instruction, 8 rows x 128 bytes, 16 rows x 64 bytes
//   6. LDS table lookups as the mat-vec gather does them (byte -> ds_read_b64 -> add), random and conflict-free
// Usage: cla_probe            (a few seconds; every kernel is a bounded loop)
#include <hip/hip_runtime.h>
#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#define CK(x)                                                                                         \
	do {                                                                                              \
		hipError_t e_ = (x);                                                                          \
		if(e_ != hipSuccess) {                                                                        \
			printf("%s failed: %s (line %d)\n", #x, hipGetErrorString(e_), __LINE__);                 \
			exit(2);                                                                                  \
		}                                                                                             \
	} while(0)

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef double f64x4 __attribute__((ext_vector_type(4)));
#define GPTR(p) ((const __attribute__((address_space(1))) void*) (p))
#define LPTR(p) ((__attribute__((address_space(3))) void*) (p))

static int g_cus = 256;
static double g_hz = 2.4e9;
static hipEvent_t g_e0, g_e1;

template <class F>
static float time_ms(F launch, int reps) {
	launch();
	CK(hipDeviceSynchronize());
	CK(hipEventRecord(g_e0));
	for(int i = 0; i < reps; i++) launch();
	CK(hipEventRecord(g_e1));
	CK(hipEventSynchronize(g_e1));
	float ms;
	CK(hipEventElapsedTime(&ms, g_e0, g_e1));
	CK(hipGetLastError());
	return ms / reps;
}

// ---- 1. layout -------------------------------------------------------------------------------------
__global__ void k_layout(const double* A, const double* B, double* D) {
	const int l = threadIdx.x;
	D[l] = __builtin_amdgcn_mfma_f64_4x4x4f64(A[l], B[l], 0.0, 0, 0, 0);
}

// assumed: lane l, block b = (l / 4) % 4: A_b[i = l % 4][k = l / 16], B_b[k = l / 16][j = l % 4], D_b[i = l / 16][j = l % 4]
static int probe_layout() {
	double *dA, *dB, *dD;
	CK(hipMalloc(&dA, 512)); CK(hipMalloc(&dB, 512)); CK(hipMalloc(&dD, 512));
	std::vector<double> a(64), b(64), d(64);
	for(int l = 0; l < 64; l++) { a[l] = 1.0 + 0.5 * l; b[l] = 2.0 + 0.25 * ((l * 7) % 13); }
	CK(hipMemcpy(dA, a.data(), 512, hipMemcpyHostToDevice));
	CK(hipMemcpy(dB, b.data(), 512, hipMemcpyHostToDevice));
	hipLaunchKernelGGL(k_layout, dim3(1), dim3(64), 0, 0, dA, dB, dD);
	CK(hipMemcpy(d.data(), dD, 512, hipMemcpyDeviceToHost));
	int bad = 0;
	for(int l = 0; l < 64; l++) {
		const int blk = (l / 4) % 4, i = l / 16, j = l % 4;
		double s = 0;
		for(int k = 0; k < 4; k++) s += a[k * 16 + blk * 4 + i] * b[k * 16 + blk * 4 + j];
		bad += d[l] != s;
	}
	printf("layout of v_mfma_f64_4x4x4_f64: %s (%d of 64 lanes differ)\n", bad == 0 ? "as assumed" : "NOT as assumed", bad);
	CK(hipFree(dA)); CK(hipFree(dB)); CK(hipFree(dD));
	return bad;
}

// ---- 2. matrix instruction rates -------------------------------------------------------------------
template <int NACC>
__global__ __launch_bounds__(256) void k_mfma4(double* out, int iters) {
	double acc[NACC];
#pragma unroll
	for(int i = 0; i < NACC; i++) acc[i] = 0;
	const double a = out[threadIdx.x & 7], b = out[(threadIdx.x + 1) & 7];
	for(int it = 0; it < iters; it++) {
#pragma unroll
		for(int i = 0; i < NACC; i++) acc[i] = __builtin_amdgcn_mfma_f64_4x4x4f64(a, b, acc[i], 0, 0, 0);
	}
	double s = 0;
#pragma unroll
	for(int i = 0; i < NACC; i++) s += acc[i];
	out[8 + blockIdx.x * 256 + threadIdx.x] = s;
}
template <int NACC>
__global__ __launch_bounds__(256) void k_mfma16(double* out, int iters) {
	f64x4 acc[NACC];
#pragma unroll
	for(int i = 0; i < NACC; i++) acc[i] = f64x4{0, 0, 0, 0};
	const double a = out[threadIdx.x & 7], b = out[(threadIdx.x + 1) & 7];
	for(int it = 0; it < iters; it++) {
#pragma unroll
		for(int i = 0; i < NACC; i++) acc[i] = __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, acc[i], 0, 0, 0);
	}
	double s = 0;
#pragma unroll
	for(int i = 0; i < NACC; i++) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
	out[8 + blockIdx.x * 256 + threadIdx.x] = s;
}

// Two waves per SIMD (one block of 8 waves per CU): the first four waves issue matrix instructions, the last four
// vector instructions (fp64 multiply-adds or integer adds), alone and together. If the two kinds ran on units of their
// own, "together" would take as long as the longer of the two; if they share the fp64 datapath, as long as their sum.
template <int MODE_A, int MODE_B>
__global__ __launch_bounds__(512) void k_mix(double* out, int iters) {
	const int wave = threadIdx.x >> 6;
	const int mode = wave < 4 ? MODE_A : MODE_B; // 0 idle, 1 v_mfma_f64_4x4x4, 2 v_mfma_f64_16x16x4, 3 v_fma_f64, 4 v_add_u32
	const double a = out[threadIdx.x & 7], b = out[(threadIdx.x + 1) & 7];
	double s = 0;
	if(mode == 1) {
		double acc[8];
#pragma unroll
		for(int i = 0; i < 8; i++) acc[i] = 0;
		for(int it = 0; it < iters; it++)
#pragma unroll
			for(int i = 0; i < 8; i++) acc[i] = __builtin_amdgcn_mfma_f64_4x4x4f64(a, b, acc[i], 0, 0, 0);
#pragma unroll
		for(int i = 0; i < 8; i++) s += acc[i];
	}
	else if(mode == 2) {
		f64x4 acc[8];
#pragma unroll
		for(int i = 0; i < 8; i++) acc[i] = f64x4{0, 0, 0, 0};
		for(int it = 0; it < iters / 4; it++)
#pragma unroll
			for(int i = 0; i < 8; i++) acc[i] = __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, acc[i], 0, 0, 0);
#pragma unroll
		for(int i = 0; i < 8; i++) s += acc[i][0] + acc[i][3];
	}
	else if(mode == 3) {
		double acc[8];
#pragma unroll
		for(int i = 0; i < 8; i++) acc[i] = i;
		for(int it = 0; it < iters * 4; it++)
#pragma unroll
			for(int i = 0; i < 8; i++) acc[i] = __builtin_fma(acc[i], a, b);
#pragma unroll
		for(int i = 0; i < 8; i++) s += acc[i];
	}
	else if(mode == 4) {
		unsigned acc[8];
#pragma unroll
		for(int i = 0; i < 8; i++) acc[i] = threadIdx.x + i;
		const unsigned k = (unsigned) (a * 1e6);
		for(int it = 0; it < iters * 4; it++)
#pragma unroll
			for(int i = 0; i < 8; i++) acc[i] = (acc[i] + k) ^ (unsigned) it;
#pragma unroll
		for(int i = 0; i < 8; i++) s += acc[i];
	}
	out[8 + blockIdx.x * 512 + threadIdx.x] = s;
}

template <int MA, int MB>
static float mix_ms(double* out, int iters) {
	return time_ms([&] { hipLaunchKernelGGL((k_mix<MA, MB>), dim3(g_cus), dim3(512), 0, 0, out, iters); }, 2);
}

static void probe_mix() {
	double* out;
	CK(hipMalloc(&out, sizeof(double) * (8 + (size_t) g_cus * 512)));
	double h[8];
	for(int i = 0; i < 8; i++) h[i] = (double) rand() / RAND_MAX - 0.5 + 1e-7 * i;
	CK(hipMemcpy(out, h, 64, hipMemcpyHostToDevice));
	const int iters = 4000;
	const double kc = 1e-3 * g_hz / 1e3; // ms -> thousands of cycles
	const float m4 = mix_ms<1, 0>(out, iters), m16 = mix_ms<2, 0>(out, iters), f = mix_ms<0, 3>(out, iters), u = mix_ms<0, 4>(out, iters);
	printf("one wave per SIMD alone (k cycles): 4x4x4 %.0f, 16x16x4 %.0f, v_fma_f64 %.0f, integer %.0f\n", m4 * kc, m16 * kc, f * kc, u * kc);
	printf("4x4x4 with v_fma_f64 on the SIMD's other wave: %.0f (sum %.0f, longer %.0f); with integer: %.0f (sum %.0f, longer %.0f)\n",
		mix_ms<1, 3>(out, iters) * kc, (m4 + f) * kc, std::max(m4, f) * kc, mix_ms<1, 4>(out, iters) * kc, (m4 + u) * kc, std::max(m4, u) * kc);
	printf("16x16x4 with v_fma_f64 on the SIMD's other wave: %.0f (sum %.0f, longer %.0f); with integer: %.0f (sum %.0f, longer %.0f)\n",
		mix_ms<2, 3>(out, iters) * kc, (m16 + f) * kc, std::max(m16, f) * kc, mix_ms<2, 4>(out, iters) * kc, (m16 + u) * kc, std::max(m16, u) * kc);
	{
		const float both4 = mix_ms<1, 1>(out, iters), both16 = mix_ms<2, 2>(out, iters);
		// per SIMD: two waves x 8 x iters instructions of the 4 x 4 x 4 form, two waves x 8 x iters / 4 of the 16 x 16 x 4 form
		printf("sums in vector registers, two waves per SIMD: 4x4x4 %.1f TFLOP/s, %.1f cycles per instruction; 16x16x4 %.1f TFLOP/s, %.1f cycles per instruction\n",
			16.0 * iters * g_cus * 4 * 512 / both4 / 1e9, both4 * 1e-3 * g_hz / (16.0 * iters), 4.0 * iters * g_cus * 4 * 2048 / both16 / 1e9,
			both16 * 1e-3 * g_hz / (4.0 * iters));
	}
	printf("matrix instructions on both waves of a SIMD: 4x4x4 %.0f (twice alone %.0f), 16x16x4 %.0f (twice alone %.0f)\n", mix_ms<1, 1>(out, iters) * kc, 2 * m4 * kc,
		mix_ms<2, 2>(out, iters) * kc, 2 * m16 * kc);
	printf("v_fma_f64 with integer on the SIMD's other wave: %.0f (sum %.0f, longer %.0f)\n", mix_ms<3, 4>(out, iters) * kc, (f + u) * kc, std::max(f, u) * kc);
	CK(hipFree(out));
}

static void probe_mfma() {
	const int bpc = 2, blocks = g_cus * bpc; // 2 blocks of 4 waves per CU = 2 waves per SIMD
	double* out;
	CK(hipMalloc(&out, sizeof(double) * (8 + (size_t) blocks * 256)));
	double h[8];
	for(int i = 0; i < 8; i++) h[i] = (double) rand() / RAND_MAX - 0.5 + 1e-7 * i; // (all-zero operands run faster than real ones)
	CK(hipMemcpy(out, h, 64, hipMemcpyHostToDevice));
	{
		const int iters = 4000;
		const float ms = time_ms([&] { hipLaunchKernelGGL(k_mfma4<16>, dim3(blocks), dim3(256), 0, 0, out, iters); }, 2);
		const double n = 16.0 * iters * blocks * 4;
		printf("v_mfma_f64_4x4x4_f64   (512 flop):  %6.1f TFLOP/s, %5.1f cycles per instruction and SIMD\n", n * 512 / ms / 1e9,
			ms * 1e-3 * g_hz / (16.0 * iters * bpc));
	}
	{
		const int iters = 1000;
		const float ms = time_ms([&] { hipLaunchKernelGGL(k_mfma16<8>, dim3(blocks), dim3(256), 0, 0, out, iters); }, 2);
		const double n = 8.0 * iters * blocks * 4;
		printf("v_mfma_f64_16x16x4_f64 (2048 flop),  8 sums in accumulation registers (a[..] as C and D: the compiler's choice for this loop): %6.1f TFLOP/s, %5.1f cycles per instruction and SIMD\n", n * 2048 / ms / 1e9,
			ms * 1e-3 * g_hz / (8.0 * iters * bpc));
	}
	{
		const int iters = 1000;
		const float ms = time_ms([&] { hipLaunchKernelGGL(k_mfma16<16>, dim3(blocks), dim3(256), 0, 0, out, iters); }, 2);
		const double n = 16.0 * iters * blocks * 4;
		printf("v_mfma_f64_16x16x4_f64 (2048 flop), 16 sums in accumulation registers: %6.1f TFLOP/s, %5.1f cycles per instruction and SIMD\n", n * 2048 / ms / 1e9,
			ms * 1e-3 * g_hz / (16.0 * iters * bpc));
	}
	CK(hipFree(out));
}

// ---- 3. streaming reads ----------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_read_flat(const u32x4* __restrict__ p, size_t n, unsigned* sink) {
	u32x4 a = {0, 0, 0, 0};
	size_t i = (size_t) blockIdx.x * 256 + threadIdx.x;
	const size_t st = (size_t) gridDim.x * 256;
	for(; i + 3 * st < n; i += 4 * st) {
		const u32x4 x0 = __builtin_nontemporal_load(p + i), x1 = __builtin_nontemporal_load(p + i + st);
		const u32x4 x2 = __builtin_nontemporal_load(p + i + 2 * st), x3 = __builtin_nontemporal_load(p + i + 3 * st);
		a ^= x0 ^ x1 ^ x2 ^ x3;
	}
	for(; i < n; i += st) a ^= p[i];
	if((a.x ^ a.y ^ a.z ^ a.w) == 0x12345678u) sink[0] = 1;
}
// a thread reads 16 bytes at its rows from each of nG streams, NB streams in flight
template <int NB>
__global__ __launch_bounds__(512) void k_read_streams(const uint8_t* __restrict__ arena, size_t stride, int nG, int64_t nRows, unsigned* sink) {
	const int64_t row0 = ((int64_t) blockIdx.x * 512 + threadIdx.x) * 16;
	if(row0 + 16 > nRows) return;
	const uint8_t* my = arena + row0;
	u32x4 a = {0, 0, 0, 0};
	for(int g = 0; g < nG; g += NB) {
		u32x4 x[NB];
#pragma unroll
		for(int j = 0; j < NB; j++) x[j] = __builtin_nontemporal_load((const u32x4*) (my + (size_t) min(g + j, nG - 1) * stride));
#pragma unroll
		for(int j = 0; j < NB; j++) a ^= x[j];
	}
	if((a.x ^ a.y ^ a.z ^ a.w) == 0x12345678u) sink[0] = 1;
}

static void probe_stream(unsigned* sink) {
	const int64_t nRows = 10000000;
	const int nG = 100;
	const size_t stride = ((size_t) nRows + 255) & ~(size_t) 255, bytes = stride * nG;
	uint8_t* arena;
	CK(hipMalloc(&arena, bytes));
	CK(hipMemset(arena, 1, bytes));
	float best = 1e30f;
	int bestGrid = 0;
	for(int grid : {2048, 4096, 8192, 16384}) {
		const float ms = time_ms([&] { hipLaunchKernelGGL(k_read_flat, dim3(grid), dim3(256), 0, 0, (const u32x4*) arena, bytes / 16, sink); }, 5);
		if(ms < best) { best = ms; bestGrid = grid; }
	}
	printf("streaming read of 1.0 GB, one flat buffer (best of 4 grid sizes: %d blocks): %.3f ms = %.2f TB/s\n", bestGrid, best, bytes / best / 1e9);
	const unsigned grid = (unsigned) ((nRows + 512 * 16 - 1) / (512 * 16));
	const float ms = time_ms([&] { hipLaunchKernelGGL(k_read_streams<10>, dim3(grid), dim3(512), 0, 0, arena, stride, nG, nRows, sink); }, 5);
	printf("streaming read of 1.0 GB as 100 code streams, 16 bytes per lane and stream:   %.3f ms = %.2f TB/s\n", ms, bytes / ms / 1e9);
	CK(hipFree(arena));
}

// ---- 4. L2 -> CU ------------------------------------------------------------------------------------
// MODE 0: global_load_lds 16 bytes per lane; MODE 1: global_load_dwordx4 into registers
template <int MODE, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void k_l2(const unsigned char* __restrict__ src, size_t regionBytes, size_t blockStride, int rep,
	unsigned* __restrict__ sink) {
	extern __shared__ __align__(16) unsigned char lds[];
	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const unsigned char* base = src + (size_t) blockIdx.x * blockStride;
	u32x4 acc = {0, 0, 0, 0};
	for(int r = 0; r < rep; r++) {
		for(size_t off0 = (size_t) wave * 1024; off0 < regionBytes; off0 += (size_t) WAVES * 1024) {
			const size_t off = off0 + lane * 16;
			if(MODE == 0) __builtin_amdgcn_global_load_lds(GPTR(base + off), LPTR(lds + (off0 & 65535)), 16, 0, 0);
			else acc ^= __builtin_nontemporal_load((const u32x4*) (base + off));
		}
		if(MODE == 0) {
			__builtin_amdgcn_s_waitcnt(0x0f70); // vmcnt(0)
			__syncthreads();
			acc[0] ^= *(const unsigned*) (lds + tid * 4);
			__syncthreads();
		}
	}
	if(acc[0] + acc[1] + acc[2] + acc[3] == 0x12345678u) sink[0] = 1;
}

// ---- 5. stores --------------------------------------------------------------------------------------
// every block writes its own 256 KB region rep times, 16 bytes per lane, 8 KB (16 rows of 512 bytes) per wave step
template <int PATTERN>
__global__ __launch_bounds__(512) void k_store(unsigned char* __restrict__ dst, size_t regionBytes, int rep) {
	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	unsigned char* base = dst + (size_t) blockIdx.x * regionBytes;
	const u32x4 v = {(unsigned) tid, 1, 2, 3};
	for(int r = 0; r < rep; r++)
		for(size_t off0 = (size_t) wave * 8192; off0 < regionBytes; off0 += (size_t) 8 * 8192) {
#pragma unroll
			for(int p = 0; p < 8; p++) {
				size_t off;
				if(PATTERN == 0) off = off0 + p * 1024 + lane * 16;                                                             // 1 KB contiguous
				else if(PATTERN == 1) off = off0 + (size_t) ((lane >> 3) + 8 * (p & 1)) * 512 + (p >> 1) * 128 + (lane & 7) * 16; // 8 rows x 128 bytes
				else off = off0 + (size_t) (lane >> 2) * 512 + p * 64 + (lane & 3) * 16;                                        // 16 rows x 64 bytes
				__builtin_nontemporal_store(v, (u32x4*) (base + off));
			}
		}
}

static void probe_l2_and_stores(unsigned* sink) {
	const size_t region = 256 * 1024, big = (size_t) g_cus * region;
	unsigned char* d;
	CK(hipMalloc(&d, big + 4096));
	CK(hipMemset(d, 1, big + 4096));
	const int rep = 200;
	auto report = [&](const char* name, float ms, double bytesPerBlock, int blocks) {
		printf("%-58s %7.2f TB/s  %5.1f bytes per cycle and CU\n", name, bytesPerBlock * blocks / ms / 1e9, bytesPerBlock / (ms * 1e-3 * g_hz));
	};
	const size_t lds = 65536 + 1024;
	CK(hipFuncSetAttribute((const void*) k_l2<0, 8>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds));
	CK(hipFuncSetAttribute((const void*) k_l2<0, 1>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds));
	report("L2 -> LDS, global_load_lds_dwordx4, 8 waves, one region:", time_ms([&] { hipLaunchKernelGGL((k_l2<0, 8>), dim3(g_cus), dim3(512), lds, 0, d, region, (size_t) 0, rep, sink); }, 1), (double) region * rep, g_cus);
	report("L2 -> LDS, global_load_lds_dwordx4, 1 wave,  one region:", time_ms([&] { hipLaunchKernelGGL((k_l2<0, 1>), dim3(g_cus), dim3(64), lds, 0, d, region, (size_t) 0, rep, sink); }, 1), (double) region * rep, g_cus);
	report("L2 -> registers, global_load_dwordx4, 8 waves, one region:", time_ms([&] { hipLaunchKernelGGL((k_l2<1, 8>), dim3(g_cus), dim3(512), 0, 0, d, region, (size_t) 0, rep, sink); }, 1), (double) region * rep, g_cus);
	report("global_load_lds_dwordx4, 8 waves, a region per CU (64 MB):", time_ms([&] { hipLaunchKernelGGL((k_l2<0, 8>), dim3(g_cus), dim3(512), lds, 0, d, region, region, rep, sink); }, 1), (double) region * rep, g_cus);
	const int srep = 20;
	report("stores, all CUs, 1 KB contiguous per instruction:", time_ms([&] { hipLaunchKernelGGL(k_store<0>, dim3(g_cus), dim3(512), 0, 0, d, region, srep); }, 2), (double) region * srep, g_cus);
	report("stores, all CUs, 8 rows x 128 bytes per instruction:", time_ms([&] { hipLaunchKernelGGL(k_store<1>, dim3(g_cus), dim3(512), 0, 0, d, region, srep); }, 2), (double) region * srep, g_cus);
	report("stores, all CUs, 16 rows x 64 bytes per instruction:", time_ms([&] { hipLaunchKernelGGL(k_store<2>, dim3(g_cus), dim3(512), 0, 0, d, region, srep); }, 2), (double) region * srep, g_cus);
	report("stores, 8 CUs, 16 rows x 64 bytes per instruction:", time_ms([&] { hipLaunchKernelGGL(k_store<2>, dim3(8), dim3(512), 0, 0, d, region, 10 * srep); }, 2), (double) region * 10 * srep, 8);
	CK(hipFree(d));
}

// ---- 6. LDS table lookups ----------------------------------------------------------------------------
// 20 tables of 256 doubles; per table a thread looks 16 pseudo-random bytes up and adds the values to 16 sums
// (MASK = 255: any entry; MASK = 3: four entries, which cannot conflict)
template <int MASK>
__global__ __launch_bounds__(512, 4) void k_lds_lookup(double* out, int rounds) {
	__shared__ double tbl[20 * 256];
	for(int i = threadIdx.x; i < 20 * 256; i += 512) tbl[i] = 0.5 * i;
	__syncthreads();
	const char* tb = (const char*) tbl;
	unsigned x = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 12345u;
	double acc[16];
#pragma unroll
	for(int i = 0; i < 16; i++) acc[i] = 0.0;
	for(int r = 0; r < rounds; r++) {
#pragma unroll
		for(int g = 0; g < 20; g++) {
#pragma unroll
			for(int w = 0; w < 4; w++) {
				x = x * 1664525u + 1013904223u;
#pragma unroll
				for(int k = 0; k < 4; k++) acc[4 * w + k] += *(const double*) (tb + g * 2048 + (((x >> (8 * k)) & MASK) << 3));
			}
		}
	}
	double s = 0.0;
#pragma unroll
	for(int i = 0; i < 16; i++) s += acc[i];
	out[(size_t) blockIdx.x * 512 + threadIdx.x] = s;
}

static void probe_lds() {
	const int bpc = 2, blocks = g_cus * bpc, rounds = 200; // 16 waves per CU, as the mat-vec gather runs
	double* out;
	CK(hipMalloc(&out, sizeof(double) * (size_t) blocks * 512));
	const double perCU = (double) bpc * 8 * rounds * 320; // wave-level lookups per CU
	const float msAny = time_ms([&] { hipLaunchKernelGGL(k_lds_lookup<255>, dim3(blocks), dim3(512), 0, 0, out, rounds); }, 3);
	const float msFour = time_ms([&] { hipLaunchKernelGGL(k_lds_lookup<3>, dim3(blocks), dim3(512), 0, 0, out, rounds); }, 3);
	printf("LDS table lookup (byte -> ds_read_b64 -> v_add_f64), any of 256 entries: %.2f cycles per wave-level lookup and CU\n", msAny * 1e-3 * g_hz / perCU);
	printf("LDS table lookup (byte -> ds_read_b64 -> v_add_f64), one of 4 entries:   %.2f cycles per wave-level lookup and CU\n", msFour * 1e-3 * g_hz / perCU);
	CK(hipFree(out));
}

int main() {
	hipDeviceProp_t prop;
	CK(hipGetDeviceProperties(&prop, 0));
	g_cus = prop.multiProcessorCount;
	g_hz = prop.clockRate * 1e3;
	printf("%s, %d CUs, %.0f MHz\n", prop.gcnArchName, g_cus, g_hz / 1e6);
	CK(hipEventCreate(&g_e0));
	CK(hipEventCreate(&g_e1));
	unsigned* sink;
	CK(hipMalloc(&sink, 64));
	const int bad = probe_layout();
	probe_mfma();
	probe_mix();
	probe_stream(sink);
	probe_l2_and_stores(sink);
	probe_lds();
	CK(hipFree(sink));
	return bad ? 1 : 0;
}
