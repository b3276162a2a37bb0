/*
 * C test driver of libclahip.so: builds a compressed block (DDC with byte codes, DDC with char codes over
 * two columns, SDC with a default, SDCZeros, RLE, uncompressed, const) from a dense matrix it makes itself,
 * runs cla_rmm / cla_lmm / cla_tsmm / cla_mmchain / cla_decompress / cla_counts through include/cla_hip.h
 * with plain C arrays (what a JNI shim passes on) and checks every result against the same product of the
 * dense matrix accumulated in long double, within 1e-12 of sum |terms|. No Python, no C++ in between.
 *
 * Prints one line per check and "C-DRIVER OK" at the end; exit code 0 only then.
 *   cla_c_driver [nRows]
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include "cla_hip.h"

static uint64_t rng_state = 88172645463325252ull;
static uint32_t rnd(void) { /* xorshift64* */
	rng_state ^= rng_state >> 12; rng_state ^= rng_state << 25; rng_state ^= rng_state >> 27;
	return (uint32_t) ((rng_state * 2685821657736338717ull) >> 32);
}
static double rndu(void) { return (rnd() + 0.5) / 4294967296.0 * 2.0 - 1.0; }

#define CHECK(rc, what) do { if((rc) < 0) { fprintf(stderr, "%s failed: %lld (%s)\n", what, (long long) (rc), cla_last_error()); return 1; } } while(0)

enum { NCOLS = 10 };
/* columns: 0 DDC byte | 1,2 DDC char (co-coded) | 3 SDC default 1.5 | 4 SDCZeros | 5 RLE | 6,7 dense | 8 const | 9 empty */

static int fails = 0;
static void compare(const char* what, const double* got, const long double* want, const long double* scale, size_t n) {
	double worst = 0;
	for(size_t i = 0; i < n; i++) {
		const double s = (double) scale[i] > 1e-300 ? (double) scale[i] : 1e-300;
		const double e = fabs(got[i] - (double) want[i]) / s;
		if(e > worst) worst = e;
	}
	printf("%-28s worst err/scale %.3e %s\n", what, worst, worst <= 1e-12 ? "ok" : "FAIL");
	if(!(worst <= 1e-12)) fails++;
}

int main(int argc, char** argv) {
	const int64_t n = argc > 1 ? atoll(argv[1]) : 50021;
	if(cla_init(0) < 0) { fprintf(stderr, "cla_init: %s\n", cla_last_error()); return 2; }
	double* X = calloc((size_t) n * NCOLS, sizeof(double));
	cla_handle h = cla_block_create(n, NCOLS);
	if(!h || !X) { fprintf(stderr, "create: %s\n", cla_last_error()); return 2; }

	/* ---- column 0: DDC, 37 values, byte codes */
	{
		double dict[37]; uint8_t* codes = malloc((size_t) n); int32_t col = 0;
		for(int k = 0; k < 37; k++) dict[k] = rndu();
		for(int64_t r = 0; r < n; r++) { codes[r] = (uint8_t) (rnd() % 37); X[r * NCOLS + 0] = dict[codes[r]]; }
		CHECK(cla_block_add_ddc(h, &col, 1, dict, 37, codes, 1), "add_ddc u8");
		free(codes);
	}
	/* ---- columns 1,2: DDC over two columns, 700 tuples, char codes */
	{
		static double dict[700 * 2]; uint16_t* codes = malloc((size_t) n * 2); int32_t cols[2] = {1, 2};
		for(int k = 0; k < 1400; k++) dict[k] = rndu();
		for(int64_t r = 0; r < n; r++) {
			codes[r] = (uint16_t) (rnd() % 700);
			X[r * NCOLS + 1] = dict[codes[r] * 2]; X[r * NCOLS + 2] = dict[codes[r] * 2 + 1];
		}
		CHECK(cla_block_add_ddc(h, cols, 2, dict, 700, codes, 2), "add_ddc u16");
		free(codes);
	}
	/* ---- columns 3 (default 1.5) and 4 (zeros): SDC with OffsetByte lists; gaps beyond 255 use 0 entries */
	for(int which = 0; which < 2; which++) {
		const int32_t col = 3 + which;
		const double def = which == 0 ? 1.5 : 0.0;
		double dict[5];
		for(int k = 0; k < 5; k++) dict[k] = rndu();
		uint8_t* deltas = malloc((size_t) n + 16); uint8_t* codes = malloc((size_t) n + 16);
		int64_t nDeltas = 0, nOff = 0, first = -1, last = -1;
		for(int64_t r = 0; r < n; r++) {
			X[r * NCOLS + col] = def;
			/* sparse stretches (1 in 600) and dense stretches (1 in 4) */
			const int listed = ((r / 5000) % 2) ? (rnd() % 600 == 0) : (rnd() % 4 == 0);
			if(!listed) continue;
			const uint8_t code = (uint8_t) (rnd() % 5);
			X[r * NCOLS + col] = dict[code];
			if(first < 0) first = r;
			else {
				int64_t gap = r - last;
				while(gap > 255) { deltas[nDeltas++] = 0; gap -= 255; }
				deltas[nDeltas++] = (uint8_t) gap;
			}
			codes[nOff++] = code;
			last = r;
		}
		CHECK(cla_block_add_sdc(h, &col, 1, dict, 5, which == 0 ? &def : NULL, codes, 1, deltas, 1, nDeltas, (int32_t) (first < 0 ? 0 : first),
			(int32_t) last, nOff), "add_sdc");
		free(deltas); free(codes);
	}
	/* ---- column 5: RLE, 4 values, runs of 1..900 rows with uncovered rows between */
	{
		const int32_t col = 5; double dict[4];
		for(int k = 0; k < 4; k++) dict[k] = rndu();
		int32_t* rowCode = malloc(sizeof(int32_t) * (size_t) n);
		for(int64_t r = 0; r < n;) {
			const int code = (int) (rnd() % 5) - 1; /* -1: uncovered rows (zeros) */
			int64_t len = 1 + rnd() % 900;
			for(; len > 0 && r < n; len--, r++) rowCode[r] = code;
		}
		int32_t ptr[5]; uint16_t* data = malloc(sizeof(uint16_t) * 2 * (size_t) (n + 8)); int64_t nData = 0;
		for(int k = 0; k < 4; k++) {
			ptr[k] = (int32_t) nData;
			int64_t prevEnd = 0, r = 0;
			while(r < n) {
				if(rowCode[r] != k) { r++; continue; }
				int64_t s = r;
				while(r < n && rowCode[r] == k) r++;
				int64_t gap = s - prevEnd, len = r - s;
				while(gap > 65535) { data[nData++] = 65535; data[nData++] = 0; gap -= 65535; }
				data[nData++] = (uint16_t) gap; data[nData++] = (uint16_t) len; /* len <= 900 */
				prevEnd = r;
			}
		}
		ptr[4] = (int32_t) nData;
		for(int64_t r = 0; r < n; r++) X[r * NCOLS + 5] = rowCode[r] >= 0 ? dict[rowCode[r]] : 0.0;
		CHECK(cla_block_add_rle(h, &col, 1, dict, 4, ptr, data, nData), "add_rle");
		free(rowCode); free(data);
	}
	/* ---- columns 6,7: uncompressed; 8: const 2.25; 9: empty */
	{
		int32_t cols[2] = {6, 7}; double* dense = malloc(sizeof(double) * 2 * (size_t) n);
		for(int64_t r = 0; r < n; r++) for(int j = 0; j < 2; j++) X[r * NCOLS + 6 + j] = dense[r * 2 + j] = rndu();
		CHECK(cla_block_add_uncompressed(h, cols, 2, dense), "add_uncompressed");
		free(dense);
		int32_t c8 = 8, c9 = 9; double cv = 2.25;
		for(int64_t r = 0; r < n; r++) X[r * NCOLS + 8] = cv;
		CHECK(cla_block_add_const(h, &c8, 1, &cv), "add_const");
		CHECK(cla_block_add_empty(h, &c9, 1), "add_empty");
	}
	CHECK(cla_block_finalize(h), "finalize");
	printf("block: %lld x %d, %d groups, %lld bytes on the device\n", (long long) n, NCOLS, cla_block_num_groups(h), (long long) cla_block_device_bytes(h));

	/* ---- decompress: bit-exact up to the SDC default morph ((dict - default) + default) */
	{
		double* D = malloc(sizeof(double) * (size_t) n * NCOLS);
		const int64_t nnz = cla_decompress(h, D);
		CHECK(nnz, "decompress");
		double worst = 0; int64_t want = 0;
		for(size_t i = 0; i < (size_t) n * NCOLS; i++) { const double e = fabs(D[i] - X[i]); if(e > worst) worst = e; want += X[i] != 0.0; }
		printf("%-28s max abs err %.3e, nnz %lld (dense %lld) %s\n", "cla_decompress", worst, (long long) nnz, (long long) want, worst <= 4e-16 ? "ok" : "FAIL");
		if(!(worst <= 4e-16)) fails++;
		free(D);
	}
	/* ---- X %*% B, q = 1 and q = 6 */
	for(int q = 1; q <= 6; q += 5) {
		double* B = malloc(sizeof(double) * NCOLS * q); double* out = malloc(sizeof(double) * (size_t) n * q);
		long double* want = malloc(sizeof(long double) * (size_t) n * q); long double* sc = malloc(sizeof(long double) * (size_t) n * q);
		for(int i = 0; i < NCOLS * q; i++) B[i] = rndu();
		CHECK(cla_rmm(h, B, q, out), "rmm");
		for(int64_t r = 0; r < n; r++) for(int j = 0; j < q; j++) {
			long double s = 0, a = 0;
			for(int c = 0; c < NCOLS; c++) { const long double t = (long double) X[r * NCOLS + c] * B[c * q + j]; s += t; a += fabsl(t); }
			want[r * q + j] = s; sc[r * q + j] = a;
		}
		compare(q == 1 ? "cla_rmm X %*% v" : "cla_rmm X %*% B (10x6)", out, want, sc, (size_t) n * q);
		free(B); free(out); free(want); free(sc);
	}
	/* ---- Y %*% X, 3 rows */
	{
		const int p = 3;
		double* Y = malloc(sizeof(double) * (size_t) n * p); double out[3 * NCOLS]; long double want[3 * NCOLS], sc[3 * NCOLS];
		for(size_t i = 0; i < (size_t) n * p; i++) Y[i] = rndu();
		CHECK(cla_lmm(h, Y, p, out), "lmm");
		for(int i = 0; i < p; i++) for(int c = 0; c < NCOLS; c++) {
			long double s = 0, a = 0;
			for(int64_t r = 0; r < n; r++) { const long double t = (long double) Y[(size_t) i * n + r] * X[r * NCOLS + c]; s += t; a += fabsl(t); }
			want[i * NCOLS + c] = s; sc[i * NCOLS + c] = a;
		}
		compare("cla_lmm Y %*% X (3 rows)", out, want, sc, 3 * NCOLS);
		free(Y);
	}
	/* ---- t(X) %*% X and the chain t(X) %*% (w * (X %*% v)) */
	{
		double out[NCOLS * NCOLS]; long double want[NCOLS * NCOLS], sc[NCOLS * NCOLS];
		CHECK(cla_tsmm(h, out), "tsmm");
		for(int a = 0; a < NCOLS; a++) for(int b = 0; b < NCOLS; b++) {
			long double s = 0, m = 0;
			for(int64_t r = 0; r < n; r++) { const long double t = (long double) X[r * NCOLS + a] * X[r * NCOLS + b]; s += t; m += fabsl(t); }
			want[a * NCOLS + b] = s; sc[a * NCOLS + b] = m;
		}
		compare("cla_tsmm t(X) %*% X", out, want, sc, NCOLS * NCOLS);
		double v[NCOLS], chain[NCOLS]; double* w = malloc(sizeof(double) * (size_t) n);
		for(int c = 0; c < NCOLS; c++) v[c] = rndu();
		for(int64_t r = 0; r < n; r++) w[r] = rndu();
		CHECK(cla_mmchain(h, v, w, 1, chain), "mmchain");
		long double cw[NCOLS] = {0}, cs[NCOLS] = {0};
		for(int64_t r = 0; r < n; r++) {
			long double s = 0, m = 0;
			for(int c = 0; c < NCOLS; c++) { const long double t = (long double) X[r * NCOLS + c] * v[c]; s += t; m += fabsl(t); }
			for(int c = 0; c < NCOLS; c++) { cw[c] += X[r * NCOLS + c] * (w[r] * s); cs[c] += fabsl(X[r * NCOLS + c]) * fabsl(w[r]) * m; }
		}
		compare("cla_mmchain XtwXv", chain, cw, cs, NCOLS);
		free(w);
	}
	/* ---- counts of group 0 (exact integers) */
	{
		int32_t counts[37]; int64_t total = 0;
		CHECK(cla_counts(h, 0, counts), "counts");
		for(int k = 0; k < 37; k++) total += counts[k];
		printf("%-28s sum %lld %s\n", "cla_counts group 0", (long long) total, total == n ? "ok" : "FAIL");
		if(total != n) fails++;
	}
	/* ---- error behaviour: a negative code and a message, the process lives on */
	{
		double dummy[4] = {0};
		const int64_t rc = cla_rmm(h, dummy, 0, dummy);
		printf("%-28s %lld \"%s\" %s\n", "cla_rmm with nColB = 0", (long long) rc, cla_last_error(), rc == -CLA_ERR_INVALID ? "ok" : "FAIL");
		if(rc != -CLA_ERR_INVALID) fails++;
	}
	cla_block_free(h);
	free(X);
	if(fails) { printf("C-DRIVER FAILED (%d checks)\n", fails); return 1; }
	printf("C-DRIVER OK\n");
	return 0;
}
