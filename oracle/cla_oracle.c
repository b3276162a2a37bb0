/*
 * TEST INFRASTRUCTURE ONLY — see cla_oracle.h. CPU restatement of the
 * SystemDS compressed multiply path. Not linked into the product.
 *
 * Reference path shorthands: C/ = src/main/java/org/apache/sysds/runtime/compress/,
 * CG/ = C/colgroup/.
 */
#define _GNU_SOURCE
#include "cla_oracle.h"
#include <math.h>
#include <pthread.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static __thread char g_err[512];
const char* ora_last_error(void) { return g_err; }
#define FAIL(code, ...) do { snprintf(g_err, sizeof(g_err), __VA_ARGS__); return (code); } while(0)

static inline int imax(int a, int b) { return a > b ? a : b; }
static inline int64_t lmin(int64_t a, int64_t b) { return a < b ? a : b; }
static inline int64_t lmax(int64_t a, int64_t b) { return a > b ? a : b; }

/* AMapToData.getIndex: MapToByte `_data[n] & 0xFF` (CG/mapping/MapToByte.java:67-69),
 * MapToChar `_data[n]` (unsigned 16 bit), MapToInt `_data[n]`. */
static inline int32_t code_at(const void* codes, int w, int64_t i) {
	if(w == 1) return ((const uint8_t*) codes)[i];
	if(w == 2) return ((const uint16_t*) codes)[i];
	return ((const int32_t*) codes)[i];
}

/* ------------------------------------------------------------------------- */
/* Map width: CG/mapping/MapToFactory.java:102-117                            */
/* ------------------------------------------------------------------------- */
int ora_map_width(int64_t nUnique) {
	if(nUnique <= 1) return 0;          /* MapToZero */
	if(nUnique <= 256) return 1;        /* (Bit), UByte <=128, Byte <=256 */
	if(nUnique <= 65536) return 2;      /* MapToChar */
	if(nUnique <= 8388607) return 3;    /* MapToCharPByte */
	return 4;                           /* MapToInt */
}

/* ------------------------------------------------------------------------- */
/* AOffset codec: CG/offset/OffsetFactory.java:238-340 (encode),              */
/* OffsetByte.java:200-212 / OffsetChar.java:172-183 (decode).                */
/* ------------------------------------------------------------------------- */
/* calcSize, OffsetFactory.java:283-293 */
int64_t ora_offset_encoded_size(const int32_t* rows, int64_t n, int width) {
	const int maxV = width == 1 ? 255 : 65535;
	int64_t sz = 0;
	for(int64_t i = 1; i < n; i++) {
		if(rows[i] <= rows[i - 1]) FAIL(-1, "offset rows must be strictly increasing at %lld", (long long) i);
		sz += 1 + (rows[i] - rows[i - 1] - 1) / maxV;
	}
	return sz;
}

/* createByte / createChar, OffsetFactory.java:246-335. The first row is kept
 * outside the delta array (offsetToFirst). A delta that is an exact multiple
 * of maxV is written as (div-1) zero entries followed by maxV; otherwise div
 * zero entries followed by the remainder. */
int64_t ora_offset_encode(const int32_t* rows, int64_t n, int width, void* deltas, int64_t cap) {
	const int maxV = width == 1 ? 255 : 65535;
	if(n > 0 && rows[0] < 0) FAIL(-1, "Invalid negative offset");
	int64_t p = 0;
	for(int64_t i = 1; i < n; i++) {
		const int gap = rows[i] - rows[i - 1];
		if(gap <= 0) FAIL(-1, "invalid offset construction with negative sequences");
		const int div = gap / maxV, mod = gap % maxV;
		const int nz = mod == 0 ? div - 1 : div;
		const int v = mod == 0 ? maxV : mod;
		if(p + nz + 1 > cap) FAIL(-1, "offset encode: capacity exceeded");
		for(int z = 0; z < nz; z++, p++) {
			if(width == 1) ((uint8_t*) deltas)[p] = 0; else ((uint16_t*) deltas)[p] = 0;
		}
		if(width == 1) ((uint8_t*) deltas)[p++] = (uint8_t) v; else ((uint16_t*) deltas)[p++] = (uint16_t) v;
	}
	return p;
}

/* Iterator: OffsetByte.java:200-212. */
typedef struct {
	const void* d; int w; int64_t idx, nDeltas; int32_t row; int64_t dataIdx;
} off_it;
static inline void off_init(off_it* it, const ora_group* g) {
	it->d = g->deltas; it->w = g->deltaWidth; it->idx = 0; it->nDeltas = g->nDeltas; it->row = g->first; it->dataIdx = 0;
}
static inline int off_has_next(const off_it* it) { return it->idx < it->nDeltas; }
static inline int32_t off_next(off_it* it) {
	const int maxV = it->w == 1 ? 255 : 65535;
	int v = it->w == 1 ? ((const uint8_t*) it->d)[it->idx] : ((const uint16_t*) it->d)[it->idx];
	while(v == 0) {
		it->row += maxV;
		it->idx++;
		v = it->w == 1 ? ((const uint8_t*) it->d)[it->idx] : ((const uint16_t*) it->d)[it->idx];
	}
	it->row += v;
	it->idx++;
	it->dataIdx++;
	return it->row;
}

int64_t ora_offset_decode(const void* deltas, int width, int64_t nDeltas, int32_t first, int32_t* rows, int64_t cap) {
	ora_group g; memset(&g, 0, sizeof(g));
	g.deltas = deltas; g.deltaWidth = width; g.nDeltas = nDeltas; g.first = first;
	off_it it; off_init(&it, &g);
	int64_t n = 0;
	if(cap < 1) FAIL(-1, "offset decode: capacity");
	rows[n++] = it.row;
	while(off_has_next(&it)) {
		if(n >= cap) FAIL(-1, "offset decode: capacity");
		rows[n++] = off_next(&it);
	}
	return n;
}

/* Java object-size estimates that drive byte-vs-char selection:
 * utils/MemoryEstimates.java:68-106, OffsetByte.java estimateInMemorySize,
 * OffsetChar.java:88-92, OffsetFactory.java:105-140, :238-244. */
static double byte_array_cost(int64_t len) {
	double size = 28;
	if(len <= 4) size += 4;
	else { size += len; int64_t diff = (len - 4) % 8; if(diff > 0) size += 8 - diff; }
	return size;
}
static double char_array_cost(int64_t len) {
	double size = 28;
	if(len <= 2) size += 4;
	else { size += len * 2; int64_t diff = (len * 2 - 4) % 8; if(diff > 0) size += 8 - diff; }
	return size;
}
int ora_offset_choose_width(const int32_t* rows, int64_t n) {
	if(n < 3) return 0; /* OffsetEmpty / OffsetSingle / OffsetTwo */
	const int64_t endLength = n - 1;
	const int64_t range = (int64_t) rows[n - 1] - rows[0];
	const int64_t corrB = lmax(range - endLength * 256, 0) / 256;
	const int64_t corrC = lmax(range - endLength * 65535, 0) / 65535;
	const long byteSize = (long) (16 + 4 + 4 + 4 + 8 + byte_array_cost(endLength + corrB));
	const long charSize = (long) (16 + 4 + 4 + 8 + char_array_cost(endLength + corrC));
	return byteSize < charSize ? 1 : 2;
}

/* ------------------------------------------------------------------------- */
/* RLE codec: CG/ColGroupRLE.java:1073-1157 (genRLEBitmap), decode            */
/* :114-117 (rs = re + data[p]; re = rs + data[p+1]).                         */
/* ------------------------------------------------------------------------- */
int64_t ora_rle_encode(const int32_t* offsets, int64_t len, uint16_t* out, int64_t cap) {
	const int CM = 65535;
	int64_t p = 0;
#define PUT(a, b) do { if(p + 2 > cap) FAIL(-1, "rle encode: capacity"); out[p++] = (uint16_t) (a); out[p++] = (uint16_t) (b); } while(0)
	if(len <= 0) return 0;
	int64_t lastRunEnd = 0;
	int64_t firstOff = offsets[0];
	while(firstOff > CM) { PUT(CM, 0); firstOff -= CM; lastRunEnd += CM; }
	int64_t curRunOff = firstOff, curRunLen = 1;
	for(int64_t i = 1; i < len; i++) {
		const int64_t absOffset = offsets[i];
		const int64_t curRunEnd = lastRunEnd + curRunOff + curRunLen;
		if(absOffset > curRunEnd || curRunLen >= CM) {
			PUT(curRunOff, curRunLen);
			lastRunEnd = curRunEnd;
			curRunOff = absOffset - lastRunEnd;
			while(curRunOff > CM) { PUT(CM, 0); lastRunEnd += CM; curRunOff -= CM; }
			curRunLen = 1;
		}
		else
			curRunLen++;
	}
	PUT(curRunOff, curRunLen);
#undef PUT
	return p;
}

int64_t ora_rle_decode(const uint16_t* data, int64_t nData, int32_t* rows, int64_t cap) {
	int64_t n = 0;
	int64_t rs = 0, re = 0;
	for(int64_t p = 0; p + 1 < nData; p += 2) {
		rs = re + data[p];
		re = rs + data[p + 1];
		for(int64_t r = rs; r < re; r++) {
			if(n >= cap) FAIL(-1, "rle decode: capacity");
			rows[n++] = (int32_t) r;
		}
	}
	return n;
}

/* ------------------------------------------------------------------------- */
/* Dictionary.preaggValuesFromDense: CG/dictionary/Dictionary.java:893-908    */
/* ret[k,i] += v * b[cols[h]*cut + i] for v = dict[k,h] != 0 (no FMA).        */
/* ------------------------------------------------------------------------- */
void ora_preagg_values_from_dense(const double* dict, int nVals, const int32_t* cols, int nColG, const double* B,
	int q, double* out) {
	memset(out, 0, sizeof(double) * (size_t) nVals * q);
	for(int k = 0; k < nVals; k++) {
		double* o = out + (size_t) k * q;
		for(int h = 0; h < nColG; h++) {
			const double v = dict[(size_t) k * nColG + h];
			const double* b = B + (size_t) cols[h] * q;
			if(v != 0)
				for(int i = 0; i < q; i++) {
					const double prod = v * b[i];
					o[i] += prod;
				}
		}
	}
}

/* ------------------------------------------------------------------------- */
/* Counts: MapTo*.getCounts (CG/mapping/MapToByte.java:168-187,               */
/* AMapToData.java:408-419); RLE sums run lengths (CG/ColGroupRLE.java:259-265)*/
/* ------------------------------------------------------------------------- */
int ora_counts(const ora_group* g, int64_t nRows, int32_t* counts) {
	memset(counts, 0, sizeof(int32_t) * (size_t) g->nVals);
	if(g->type == ORA_DDC) {
		for(int64_t r = 0; r < nRows; r++) counts[code_at(g->codes, g->codeWidth, r)]++;
	}
	else if(g->type == ORA_SDC) {
		for(int64_t j = 0; j < g->nOffsets; j++) counts[code_at(g->codes, g->codeWidth, j)]++;
	}
	else if(g->type == ORA_RLE) {
		for(int k = 0; k < g->nVals; k++)
			for(int p = g->ptr[k]; p < g->ptr[k + 1]; p += 2) counts[k] += g->rle[p + 1];
	}
	else
		FAIL(-1, "counts: unsupported group type %d", g->type);
	return 0;
}

/* ------------------------------------------------------------------------- */
/* Per-row code materialisation used by the brute-force helpers below.        */
/* code -1 = row not covered (zero tuple for SDCZeros / RLE gaps).            */
/* ------------------------------------------------------------------------- */
static int32_t* row_codes(const ora_group* g, int64_t nRows) {
	int32_t* rc = (int32_t*) malloc(sizeof(int32_t) * (size_t) lmax(nRows, 1));
	if(!rc) return NULL;
	if(g->type == ORA_DDC) {
		for(int64_t r = 0; r < nRows; r++) rc[r] = code_at(g->codes, g->codeWidth, r);
	}
	else if(g->type == ORA_SDC) {
		for(int64_t r = 0; r < nRows; r++) rc[r] = -1;
		if(g->nOffsets > 0) {
			off_it it; off_init(&it, g);
			rc[it.row] = code_at(g->codes, g->codeWidth, 0);
			while(off_has_next(&it)) { int32_t row = off_next(&it); rc[row] = code_at(g->codes, g->codeWidth, it.dataIdx); }
		}
	}
	else if(g->type == ORA_RLE) {
		for(int64_t r = 0; r < nRows; r++) rc[r] = -1;
		for(int k = 0; k < g->nVals; k++) {
			int64_t rs = 0, re = 0;
			for(int p = g->ptr[k]; p < g->ptr[k + 1]; p += 2) {
				rs = re + g->rle[p]; re = rs + g->rle[p + 1];
				for(int64_t r = rs; r < re && r < nRows; r++) rc[r] = k;
			}
		}
	}
	else { free(rc); return NULL; }
	return rc;
}

/* Integer co-occurrence N[a,b] = #{r : code_a(r)=a and code_b(r)=b}: the
 * integer form of APreAgg.preAggregateThatIndexStructure (CG/APreAgg.java:87-110,
 * CG/mapping/AMapToData.java:429-493). Brute force, exact. */
int ora_cooc(const ora_group* a, const ora_group* b, int64_t nRows, int64_t* out) {
	int32_t* ca = row_codes(a, nRows);
	int32_t* cb = row_codes(b, nRows);
	if(!ca || !cb) { free(ca); free(cb); FAIL(-1, "cooc: unsupported group type"); }
	memset(out, 0, sizeof(int64_t) * (size_t) a->nVals * b->nVals);
	for(int64_t r = 0; r < nRows; r++)
		if(ca[r] >= 0 && cb[r] >= 0) out[(size_t) ca[r] * b->nVals + cb[r]]++;
	free(ca); free(cb);
	return 0;
}

/* ------------------------------------------------------------------------- */
/* Additive decompression of one group into rows [rl,ru) of a dense block of  */
/* nColOut columns. `values` is the (possibly pre-aggregated) dictionary and  */
/* `colIdx` the output columns (nC of them).                                   */
/*  DDC : CG/ColGroupDDC.java:137-225 (+ AMapToData.decompressToRange :947-976)*/
/*  SDCZ: CG/ColGroupSDCZeros.java:122-315                                     */
/*  RLE : CG/ColGroupRLE.java:104-141                                          */
/* ------------------------------------------------------------------------- */
typedef struct {
	const ora_group* g;
	const double* values; /* nVals x nC */
	const int32_t* colIdx;
	int nC;
	const double* dense;  /* UNC result block (nRows x nC) */
	off_it cursor;        /* SDC: cached iterator (AOffset.cacheIterator, CG/offset/AOffset.java:212-227) */
	int64_t lastRu;       /* SDC: upper row of the previous call served by `cursor` */
} dec_group;

static void dec_ddc(const dec_group* d, double* out, int nColOut, int64_t rl, int64_t ru) {
	const ora_group* g = d->g;
	const int nC = d->nC;
	if(nC == 1 && nColOut == 1) {
		for(int64_t r = rl; r < ru; r++) out[r] += d->values[code_at(g->codes, g->codeWidth, r)];
	}
	else {
		for(int64_t r = rl; r < ru; r++) {
			const double* v = d->values + (size_t) code_at(g->codes, g->codeWidth, r) * nC;
			double* c = out + (size_t) r * nColOut;
			for(int j = 0; j < nC; j++) c[d->colIdx[j]] += v[j];
		}
	}
}

static void dec_sdcz(dec_group* d, double* out, int nColOut, int64_t rl, int64_t ru) {
	const ora_group* g = d->g;
	if(g->nOffsets <= 0) return;
	/* AOffset.getIterator(rl) (CG/offset/AOffset.java:177-230): continue from the
	 * cached position when the caller moves forward, restart otherwise. */
	if(rl < d->lastRu) off_init(&d->cursor, g);
	d->lastRu = ru;
	off_it it = d->cursor;
	while(it.row < rl && off_has_next(&it)) off_next(&it);
	const int nC = d->nC;
	while(it.row < ru) {
		if(it.row >= rl) {
			const double* v = d->values + (size_t) code_at(g->codes, g->codeWidth, it.dataIdx) * nC;
			double* c = out + (size_t) it.row * nColOut;
			for(int j = 0; j < nC; j++) c[d->colIdx[j]] += v[j];
		}
		if(!off_has_next(&it)) { it.row = INT32_MAX; break; }
		off_next(&it);
	}
	d->cursor = it;
}

static void dec_rle(const dec_group* d, double* out, int nColOut, int64_t rl, int64_t ru) {
	const ora_group* g = d->g;
	const int nC = d->nC;
	for(int k = 0; k < g->nVals; k++) {
		const double* v = d->values + (size_t) k * nC;
		int64_t rs = 0, re = 0;
		for(int p = g->ptr[k]; p < g->ptr[k + 1]; p += 2) {
			rs = re + g->rle[p];
			re = rs + g->rle[p + 1];
			if(re <= rl) continue;
			if(rs >= ru) break;
			const int64_t a = lmax(rs, rl), b = lmin(re, ru);
			for(int64_t r = a; r < b; r++) {
				double* c = out + (size_t) r * nColOut;
				for(int j = 0; j < nC; j++) c[d->colIdx[j]] += v[j];
			}
		}
	}
}

static void dec_unc(const dec_group* d, double* out, int nColOut, int64_t rl, int64_t ru) {
	const int nC = d->nC;
	for(int64_t r = rl; r < ru; r++) {
		const double* v = d->dense + (size_t) r * nC;
		double* c = out + (size_t) r * nColOut;
		for(int j = 0; j < nC; j++) c[d->colIdx[j]] += v[j];
	}
}

static void dec_any(dec_group* d, double* out, int nColOut, int64_t rl, int64_t ru) {
	switch(d->g->type) {
		case ORA_DDC: dec_ddc(d, out, nColOut, rl, ru); break;
		case ORA_SDC: dec_sdcz(d, out, nColOut, rl, ru); break;
		case ORA_RLE: dec_rle(d, out, nColOut, rl, ru); break;
		case ORA_UNC: dec_unc(d, out, nColOut, rl, ru); break;
		default: break;
	}
}

/* ------------------------------------------------------------------------- */
/* Pre-filter: CLALibUtils.filterGroups (C/lib/CLALibUtils.java:188-206),     */
/* SDC.extractCommon (CG/ColGroupSDC.java:483-489; dict - default tuple,       */
/* Dictionary.java:838-846), ColGroupConst.addToCommon                         */
/* (CG/ColGroupConst.java:330-362).                                            */
/* Returns per-group dictionaries to use (malloc'd where morphed).             */
/* ------------------------------------------------------------------------- */
typedef struct {
	int n;                 /* number of filtered (kept) groups */
	const ora_group** g;   /* kept groups in list order */
	double** dictOwned;    /* NULL or owned morphed dictionary */
	const double** dict;   /* dictionary to use for kept group i */
	double* constV;        /* nCols, or NULL when nothing was filtered */
} filtered;

static int should_prefilter(const ora_group* groups, int nG) {
	/* CLALibUtils.shouldPreFilter (C/lib/CLALibUtils.java:90-98): morphing (SDC
	 * with default), const or empty groups. */
	for(int i = 0; i < nG; i++) {
		const ora_group* g = &groups[i];
		if((g->type == ORA_SDC && g->def) || g->type == ORA_CONST || g->type == ORA_EMPTY) return 1;
	}
	return 0;
}

static void filtered_free(filtered* f) {
	if(!f) return;
	if(f->dictOwned) for(int i = 0; i < f->n; i++) free(f->dictOwned[i]);
	free(f->dictOwned); free(f->dict); free(f->g); free(f->constV);
	memset(f, 0, sizeof(*f));
}

static int filter_groups(const ora_group* groups, int nG, int nCols, filtered* f) {
	memset(f, 0, sizeof(*f));
	f->g = (const ora_group**) calloc((size_t) imax(nG, 1), sizeof(void*));
	f->dictOwned = (double**) calloc((size_t) imax(nG, 1), sizeof(void*));
	f->dict = (const double**) calloc((size_t) imax(nG, 1), sizeof(void*));
	const int filt = should_prefilter(groups, nG);
	if(filt) f->constV = (double*) calloc((size_t) imax(nCols, 1), sizeof(double));
	for(int i = 0; i < nG; i++) {
		const ora_group* g = &groups[i];
		if(g->type == ORA_EMPTY) continue;
		if(g->type == ORA_CONST) {
			for(int j = 0; j < g->nColG; j++) f->constV[g->cols[j]] += g->dict[j];
			continue;
		}
		const int id = f->n++;
		f->g[id] = g;
		f->dict[id] = g->dict;
		if(g->type == ORA_SDC && g->def) {
			double* dz = (double*) malloc(sizeof(double) * (size_t) g->nVals * g->nColG);
			for(int k = 0; k < g->nVals; k++)
				for(int j = 0; j < g->nColG; j++)
					dz[(size_t) k * g->nColG + j] = g->dict[(size_t) k * g->nColG + j] - g->def[j];
			for(int j = 0; j < g->nColG; j++) f->constV[g->cols[j]] += g->def[j];
			f->dictOwned[id] = dz;
			f->dict[id] = dz;
		}
	}
	return 0;
}

/* ------------------------------------------------------------------------- */
/* Tiny thread pool: run nTasks tasks on k threads (the reference creates a    */
/* pool per call, R/util/CommonThreadPool.java:65-145).                        */
/* ------------------------------------------------------------------------- */
typedef void (*task_fn)(void* ctx, int task);
typedef struct { task_fn fn; void* ctx; int nTasks; int next; pthread_mutex_t mu; } pool_t;
static void* pool_worker(void* a) {
	pool_t* p = (pool_t*) a;
	for(;;) {
		pthread_mutex_lock(&p->mu);
		const int t = p->next < p->nTasks ? p->next++ : -1;
		pthread_mutex_unlock(&p->mu);
		if(t < 0) break;
		p->fn(p->ctx, t);
	}
	return NULL;
}
static void run_tasks(task_fn fn, void* ctx, int nTasks, int k) {
	if(k <= 1 || nTasks <= 1) { for(int t = 0; t < nTasks; t++) fn(ctx, t); return; }
	pool_t p; p.fn = fn; p.ctx = ctx; p.nTasks = nTasks; p.next = 0; pthread_mutex_init(&p.mu, NULL);
	const int nt = k < nTasks ? k : nTasks;
	pthread_t* th = (pthread_t*) malloc(sizeof(pthread_t) * (size_t) nt);
	for(int i = 0; i < nt; i++) pthread_create(&th[i], NULL, pool_worker, &p);
	for(int i = 0; i < nt; i++) pthread_join(th[i], NULL);
	free(th); pthread_mutex_destroy(&p.mu);
}

/* ------------------------------------------------------------------------- */
/* Right multiply: CLALibRightMultBy.RMM (C/lib/CLALibRightMultBy.java:208-258)*/
/*  per group ADictBasedColGroup.rightMultByMatrix (CG/ADictBasedColGroup.java */
/*  :246-275) -> preaggValuesFromDense; ColGroupUncompressed.rightMultByMatrix */
/*  (CG/ColGroupUncompressed.java:888-927); constV %*% B (:247-252);           */
/*  CLALibDecompress.decompressDense (C/lib/CLALibDecompress.java:310-357,     */
/*  DecompressDenseTask :401-444, addVector :531-618).                         */
/* ------------------------------------------------------------------------- */
typedef struct {
	dec_group* dg; int nDG; const double* constB; double* out; int q; int64_t nRows; int64_t blklen;
	int64_t* nnzPerTask;
} rmm_ctx;

static void rmm_task(void* vctx, int t) {
	rmm_ctx* c = (rmm_ctx*) vctx;
	const int64_t rl = (int64_t) t * c->blklen, ru = lmin(rl + c->blklen, c->nRows);
	const int64_t sub = imax(32768 / c->q, 128); /* DecompressDenseTask._blklen :417 */
	/* each task owns private SDC cursors (thread-local iterator cache in the reference) */
	dec_group* dg = (dec_group*) malloc(sizeof(dec_group) * (size_t) imax(c->nDG, 1));
	memcpy(dg, c->dg, sizeof(dec_group) * (size_t) c->nDG);
	for(int i = 0; i < c->nDG; i++) if(dg[i].g->type == ORA_SDC) { off_init(&dg[i].cursor, dg[i].g); dg[i].lastRu = 0; }
	int64_t nnz = 0;
	for(int64_t b = rl; b < ru; b += sub) {
		const int64_t e = lmin(b + sub, ru);
		for(int i = 0; i < c->nDG; i++) dec_any(&dg[i], c->out, c->q, b, e);
		if(c->constB)
			for(int64_t r = b; r < e; r++) for(int j = 0; j < c->q; j++) c->out[(size_t) r * c->q + j] += c->constB[j];
		for(int64_t r = b; r < e; r++) for(int j = 0; j < c->q; j++) nnz += c->out[(size_t) r * c->q + j] != 0;
	}
	free(dg);
	c->nnzPerTask[t] = nnz;
}

int64_t ora_rmm(const ora_group* groups, int nG, int64_t nRows, int nCols, const double* B, int q, double* out, int k) {
	if(nRows < 0 || nCols <= 0 || q <= 0) FAIL(-1, "rmm: bad dims");
	memset(out, 0, sizeof(double) * (size_t) nRows * q);
	filtered f;
	filter_groups(groups, nG, nCols, &f);
	int32_t* allCols = (int32_t*) malloc(sizeof(int32_t) * (size_t) q);
	for(int j = 0; j < q; j++) allCols[j] = j;
	dec_group* dg = (dec_group*) calloc((size_t) imax(f.n, 1), sizeof(dec_group));
	double** owned = (double**) calloc((size_t) imax(f.n, 1), sizeof(double*));
	int nDG = 0;
	for(int i = 0; i < f.n; i++) {
		const ora_group* g = f.g[i];
		dec_group d; memset(&d, 0, sizeof(d));
		d.g = g; d.colIdx = allCols; d.nC = q;
		if(g->type == ORA_UNC) {
			/* dense group x B[cols,:] (LibMatrixMult.matrixMult), kept as an
			 * uncompressed overlapping group */
			double* u = (double*) calloc((size_t) lmax(nRows, 1) * q, sizeof(double));
			for(int64_t r = 0; r < nRows; r++)
				for(int h = 0; h < g->nColG; h++) {
					const double a = g->dense[(size_t) r * g->nColG + h];
					if(a != 0) for(int j = 0; j < q; j++) u[(size_t) r * q + j] += a * B[(size_t) g->cols[h] * q + j];
				}
			d.dense = u; owned[nDG] = u;
		}
		else {
			double* T = (double*) malloc(sizeof(double) * (size_t) g->nVals * q);
			ora_preagg_values_from_dense(f.dict[i], g->nVals, g->cols, g->nColG, B, q, T);
			/* Dictionary.create returns null for an all-zero array
			 * (CG/dictionary/Dictionary.java:65-78) -> group dropped */
			int allZero = 1;
			for(size_t z = 0; z < (size_t) g->nVals * q; z++) if(T[z] != 0) { allZero = 0; break; }
			if(allZero) { free(T); continue; }
			d.values = T; owned[nDG] = T;
		}
		dg[nDG++] = d;
	}
	double* constB = NULL;
	if(f.constV) {
		constB = (double*) calloc((size_t) q, sizeof(double));
		int any = 0;
		for(int c0 = 0; c0 < nCols; c0++) {
			const double a = f.constV[c0];
			if(a != 0) for(int j = 0; j < q; j++) constB[j] += a * B[(size_t) c0 * q + j];
		}
		for(int j = 0; j < q; j++) any |= constB[j] != 0;
		if(!any) { free(constB); constB = NULL; } /* mmTemp.isEmpty() -> null, :251 */
	}
	const int kk = imax(k, 1);
	rmm_ctx c;
	c.dg = dg; c.nDG = nDG; c.constB = constB; c.out = out; c.q = q; c.nRows = nRows;
	c.blklen = lmax(nRows / kk, 512); /* CLALibDecompress.java:315 */
	const int nTasks = (int) ((nRows + c.blklen - 1) / c.blklen);
	c.nnzPerTask = (int64_t*) calloc((size_t) imax(nTasks, 1), sizeof(int64_t));
	run_tasks(rmm_task, &c, nTasks, kk);
	int64_t nnz = 0;
	for(int t = 0; t < nTasks; t++) nnz += c.nnzPerTask[t];
	free(c.nnzPerTask);
	for(int i = 0; i < nDG; i++) free(owned[i]);
	free(owned); free(dg); free(constB); free(allCols);
	filtered_free(&f);
	return nnz;
}

/* CLALibDecompress.decompressDense of the block itself (C/lib/CLALibDecompress.java:310-357):
 * every group adds dict[code] into its own columns, SDC defaults and const rows
 * included. Single threaded. */
int ora_decompress(const ora_group* groups, int nG, int64_t nRows, int nCols, double* out) {
	memset(out, 0, sizeof(double) * (size_t) nRows * nCols);
	filtered f;
	filter_groups(groups, nG, nCols, &f);
	for(int i = 0; i < f.n; i++) {
		dec_group d; memset(&d, 0, sizeof(d));
		d.g = f.g[i]; d.values = f.dict[i]; d.colIdx = f.g[i]->cols; d.nC = f.g[i]->nColG; d.dense = f.g[i]->dense;
		if(d.g->type == ORA_SDC) off_init(&d.cursor, d.g);
		dec_any(&d, out, nCols, 0, nRows);
	}
	if(f.constV)
		for(int64_t r = 0; r < nRows; r++) for(int j = 0; j < nCols; j++) out[(size_t) r * nCols + j] += f.constV[j];
	filtered_free(&f);
	return 0;
}

/* ------------------------------------------------------------------------- */
/* Left multiply pre-aggregation (first step of LMM).                          */
/*  DDC : AMapToData.preAggregateDense (CG/mapping/AMapToData.java:214-330)    */
/*  SDCZ: AOffset.preAggregateDenseMap (CG/offset/AOffset.java:288-430)        */
/*  RLE : ColGroupRLE.preAggregateDense (CG/ColGroupRLE.java:759-796)          */
/* pre[i, code(r)] += Y[i, r], rows of X visited in ascending order, columns   */
/* [cl,cu) of Y only.                                                          */
/* ------------------------------------------------------------------------- */
static void preagg_range(const ora_group* g, const double* Y, int64_t nRows, int rl, int ru, int64_t cl, int64_t cu,
	double* pre, off_it* cursor) {
	const int nv = g->nVals;
	if(g->type == ORA_DDC) {
		for(int i = rl; i < ru; i++) {
			const double* y = Y + (size_t) i * nRows;
			double* p = pre + (size_t) (i - rl) * nv;
			for(int64_t r = cl; r < cu; r++) p[code_at(g->codes, g->codeWidth, r)] += y[r];
		}
	}
	else if(g->type == ORA_SDC) {
		if(g->nOffsets <= 0) return;
		off_it it = *cursor;
		while(it.row < cl && off_has_next(&it)) off_next(&it);
		while(it.row < cu) {
			if(it.row >= cl) {
				const int c = code_at(g->codes, g->codeWidth, it.dataIdx);
				for(int i = rl; i < ru; i++) pre[(size_t) (i - rl) * nv + c] += Y[(size_t) i * nRows + it.row];
			}
			if(!off_has_next(&it)) { it.row = INT32_MAX; break; }
			off_next(&it);
		}
		*cursor = it;
	}
	else if(g->type == ORA_RLE) {
		for(int k = 0; k < nv; k++) {
			int64_t rs = 0, re = 0;
			for(int p = g->ptr[k]; p < g->ptr[k + 1]; p += 2) {
				rs = re + g->rle[p];
				re = rs + g->rle[p + 1];
				if(re <= cl) continue;
				if(rs >= cu) break;
				const int64_t a = lmax(rs, cl), b = lmin(re, cu);
				for(int i = rl; i < ru; i++) {
					const double* y = Y + (size_t) i * nRows;
					double* o = pre + (size_t) (i - rl) * nv + k;
					for(int64_t r = a; r < b; r++) *o += y[r];
				}
			}
		}
	}
}

int ora_preaggregate_dense(const ora_group* g, int64_t nRows, const double* Y, int p, double* preAgg) {
	if(g->type != ORA_DDC && g->type != ORA_SDC && g->type != ORA_RLE) FAIL(-1, "preaggregate: not an APreAgg group");
	memset(preAgg, 0, sizeof(double) * (size_t) p * g->nVals);
	off_it cur; memset(&cur, 0, sizeof(cur));
	if(g->type == ORA_SDC) off_init(&cur, g);
	preagg_range(g, Y, nRows, 0, p, 0, nRows, preAgg, &cur);
	return 0;
}

/* ------------------------------------------------------------------------- */
/* Left multiply: CLALibLeftMultBy.LMM (C/lib/CLALibLeftMultBy.java:286-346),  */
/* LMMWithPreAggDense (:731-790; 4 rows x 4 groups x 2048 columns blocking),   */
/* APreAgg.mmWithDictionary (CG/APreAgg.java:312-322) + addMatrixToResult      */
/* (CG/ColGroupUtils.java:283-311), rowSum (:827-885), outerProduct (:530-599),*/
/* LMMParallelNoTempOut task split (:367-405),                                 */
/* ColGroupUncompressed.leftMultByMatrixNoPreAgg (CG/ColGroupUncompressed.java */
/* :428-539).                                                                  */
/* ------------------------------------------------------------------------- */
typedef struct {
	const filtered* f; const double* Y; int p; int64_t nRows; int nCols; double* out;
	int rowBlock; int s; int nPa; const int* paIdx; int nNpa; const int* npaIdx; double* rowSums;
	int nRowBlocks;
} lmm_ctx;

static void lmm_preagg_task(const lmm_ctx* c, int rl, int ru, int off, int skip) {
	const int colBZ = 2048, rowBlockSize = 4, colGroupBlocking = 4;
	double* preAgg[4] = {0, 0, 0, 0};
	size_t preCap[4] = {0, 0, 0, 0};
	off_it cur[4];
	for(int rlt = rl; rlt < ru; rlt += rowBlockSize) {
		const int rut = rlt + rowBlockSize < ru ? rlt + rowBlockSize : ru;
		for(int gl = off; gl < c->nPa; gl += colGroupBlocking * skip) {
			const int gu = gl + colGroupBlocking * skip < c->nPa ? gl + colGroupBlocking * skip : c->nPa;
			for(int j = gl, p = 0; j < gu; j += skip, p++) {
				const ora_group* g = c->f->g[c->paIdx[j]];
				const size_t len = (size_t) (rut - rlt) * g->nVals;
				if(preCap[p] < len) { free(preAgg[p]); preAgg[p] = (double*) malloc(sizeof(double) * len); preCap[p] = len; }
				memset(preAgg[p], 0, sizeof(double) * len);
				if(g->type == ORA_SDC) off_init(&cur[p], g);
			}
			for(int64_t clt = 0; clt < c->nRows; clt += colBZ) {
				const int64_t cut = lmin(clt + colBZ, c->nRows);
				for(int j = gl, p = 0; j < gu; j += skip, p++)
					preagg_range(c->f->g[c->paIdx[j]], c->Y, c->nRows, rlt, rut, clt, cut, preAgg[p], &cur[p]);
			}
			for(int j = gl, p = 0; j < gu; j += skip, p++) {
				const int gi = c->paIdx[j];
				const ora_group* g = c->f->g[gi];
				const double* dict = c->f->dict[gi];
				/* tmp = preAgg %*% dict ; out[i, cols] += tmp */
				for(int i = rlt; i < rut; i++) {
					const double* pa = preAgg[p] + (size_t) (i - rlt) * g->nVals;
					for(int jj = 0; jj < g->nColG; jj++) {
						double s = 0;
						for(int kk = 0; kk < g->nVals; kk++) s += pa[kk] * dict[(size_t) kk * g->nColG + jj];
						c->out[(size_t) i * c->nCols + g->cols[jj]] += s;
					}
				}
			}
		}
	}
	for(int p = 0; p < 4; p++) free(preAgg[p]);
}

static void lmm_unc(const lmm_ctx* c, const ora_group* g, int rl, int ru) {
	for(int i = rl; i < ru; i++) {
		const double* y = c->Y + (size_t) i * c->nRows;
		for(int j = 0; j < g->nColG; j++) {
			double s = 0;
			for(int64_t r = 0; r < c->nRows; r++) s += y[r] * g->dense[(size_t) r * g->nColG + j];
			c->out[(size_t) i * c->nCols + g->cols[j]] += s;
		}
	}
}

static void lmm_rowsum(const lmm_ctx* c, int rl, int ru) {
	/* rowSum is accumulated per 2048-column block (:766-767, :876-884) */
	for(int i = rl; i < ru; i++) {
		const double* y = c->Y + (size_t) i * c->nRows;
		for(int64_t clt = 0; clt < c->nRows; clt += 2048) {
			const int64_t cut = lmin(clt + 2048, c->nRows);
			double tmp = 0;
			for(int64_t r = clt; r < cut; r++) tmp += y[r];
			c->rowSums[i] += tmp;
		}
	}
}

static void lmm_task(void* vctx, int t) {
	const lmm_ctx* c = (const lmm_ctx*) vctx;
	const int perBlock = c->nNpa + c->s + (c->rowSums ? 1 : 0);
	const int blk = t / perBlock, sub = t % perBlock;
	const int rl = blk * c->rowBlock, ru = rl + c->rowBlock < c->p ? rl + c->rowBlock : c->p;
	if(sub < c->nNpa) lmm_unc(c, c->f->g[c->npaIdx[sub]], rl, ru);
	else if(sub < c->nNpa + c->s) lmm_preagg_task(c, rl, ru, sub - c->nNpa, c->s);
	else lmm_rowsum(c, rl, ru);
}

int64_t ora_lmm(const ora_group* groups, int nG, int64_t nRows, int nCols, const double* Y, int p, double* out, int k) {
	if(nRows < 0 || nCols <= 0 || p <= 0) FAIL(-1, "lmm: bad dims");
	memset(out, 0, sizeof(double) * (size_t) p * nCols);
	filtered f;
	filter_groups(groups, nG, nCols, &f);
	int* paIdx = (int*) malloc(sizeof(int) * (size_t) imax(f.n, 1));
	int* npaIdx = (int*) malloc(sizeof(int) * (size_t) imax(f.n, 1));
	int nPa = 0, nNpa = 0;
	for(int i = 0; i < f.n; i++) {
		if(f.g[i]->type == ORA_UNC) npaIdx[nNpa++] = i; else paIdx[nPa++] = i;
	}
	const int kk = imax(k, 1);
	lmm_ctx c;
	c.f = &f; c.Y = Y; c.p = p; c.nRows = nRows; c.nCols = nCols; c.out = out;
	c.nPa = nPa; c.paIdx = paIdx; c.nNpa = nNpa; c.npaIdx = npaIdx;
	c.rowSums = f.constV ? (double*) calloc((size_t) p, sizeof(double)) : NULL;
	if(kk == 1 || nPa + nNpa <= 1) {
		/* LMMTaskExec (:512-528) */
		c.rowBlock = p; c.s = nPa > 0 ? 1 : 0; c.nRowBlocks = 1;
		for(int i = 0; i < nNpa; i++) lmm_unc(&c, f.g[npaIdx[i]], 0, p);
		if(nPa > 0) lmm_preagg_task(&c, 0, p, 0, 1);
		if(c.rowSums) lmm_rowsum(&c, 0, p);
	}
	else {
		c.s = nPa < kk ? nPa : kk;
		c.rowBlock = imax(p / kk, 1);
		c.nRowBlocks = (p + c.rowBlock - 1) / c.rowBlock;
		const int perBlock = nNpa + c.s + (c.rowSums ? 1 : 0);
		run_tasks(lmm_task, &c, c.nRowBlocks * perBlock, kk);
	}
	if(c.rowSums) {
		/* outerProductRangeContiguous (:563-575) */
		for(int i = 0; i < p; i++) {
			const double vl = c.rowSums[i];
			if(vl != 0) for(int j = 0; j < nCols; j++) out[(size_t) i * nCols + j] += vl * f.constV[j];
		}
	}
	int64_t nnz = 0;
	for(size_t z = 0; z < (size_t) p * nCols; z++) nnz += out[z] != 0;
	free(c.rowSums); free(paIdx); free(npaIdx);
	filtered_free(&f);
	return nnz;
}

/* ------------------------------------------------------------------------- */
/* TSMM: CLALibTSMM.leftMultByTransposeSelf (C/lib/CLALibTSMM.java:59-94)      */
/* ------------------------------------------------------------------------- */
/* DictLibMatrixMult.addToUpperTriangle (CG/dictionary/DictLibMatrixMult.java:47-54) */
static inline void add_upper(int nCols, int row, int col, double* res, double val) {
	if(row == col) res[(size_t) row * nCols + col] += val + val;
	else if(row > col) res[(size_t) col * nCols + row] += val;
	else res[(size_t) row * nCols + col] += val;
}

/* AColGroupCompressed.tsmmDense (CG/AColGroupCompressed.java:226-241) */
static void tsmm_self(const ora_group* g, const double* dict, const int32_t* counts, double* res, int nCols) {
	const int nC = g->nColG;
	for(int k = 0; k < g->nVals; k++) {
		const int scale = counts[k];
		for(int i = 0; i < nC; i++) {
			const double v = dict[(size_t) k * nC + i] * scale;
			if(v != 0)
				for(int j = i; j < nC; j++)
					res[(size_t) g->cols[i] * nCols + g->cols[j]] += v * dict[(size_t) k * nC + j];
		}
	}
}

/* APreAgg.preAggregateThatIndexStructure (CG/APreAgg.java:87-110): `self` is the
 * target index structure, `that` supplies codes + dictionary.
 *   P[code_self(r), :] += dict_that[code_that(r), :]  for rows covered by both.
 * DDC_DDC AMapToData.java:429-493, DDC_SDCZ :504-567, SDCZ_DDC :578-634,
 * SDCZ_SDCZ :636-747, RLE_DDC :749-780, DDC_RLE :782-794,
 * ColGroupRLE.preAggregateThat* (CG/ColGroupRLE.java:835-955),
 * ColGroupSDCZeros.preAggregateThat* (CG/ColGroupSDCZeros.java:682-753).
 * All variants visit matching rows in ascending row order; restated here on
 * materialised per-row codes (row order preserved, so the fp64 sums agree). */
static double* preagg_that(const ora_group* self, const ora_group* that, const double* dictThat, int64_t nRows) {
	const int nC = that->nColG;
	double* P = (double*) calloc((size_t) self->nVals * nC, sizeof(double));
	int32_t* cs = row_codes(self, nRows);
	int32_t* ct = row_codes(that, nRows);
	for(int64_t r = 0; r < nRows; r++)
		if(cs[r] >= 0 && ct[r] >= 0) {
			const double* v = dictThat + (size_t) ct[r] * nC;
			double* o = P + (size_t) cs[r] * nC;
			for(int j = 0; j < nC; j++) o[j] += v[j];
		}
	free(cs); free(ct);
	return P;
}

/* DictLibMatrixMult.MMToUpperTriangleDenseDense (DictLibMatrixMult.java:527-601):
 * adds t(left) %*% right at (rowsLeft x colsRight), folded into the upper
 * triangle. */
static void mm_to_upper(const double* left, int lSize, const int32_t* rowsLeft, const double* right, int rSize,
	const int32_t* colsRight, int commonDim, double* res, int nCols) {
	for(int k = 0; k < commonDim; k++)
		for(int i = 0; i < lSize; i++) {
			const double vl = left[(size_t) k * lSize + i];
			if(vl != 0)
				for(int j = 0; j < rSize; j++)
					add_upper(nCols, rowsLeft[i], colsRight[j], res, vl * right[(size_t) k * rSize + j]);
		}
}

/* APreAgg.tsmmAPreAgg (CG/APreAgg.java:153-179) for g.tsmmAColGroup(h): this=g, lg=h. */
static void tsmm_pair(const ora_group* g, const double* dg, const ora_group* h, const double* dh, int64_t nRows,
	double* res, int nCols) {
	const int left = (double) g->nVals * g->nColG < (double) h->nVals * h->nColG; /* shouldPreAggregateLeft :302-310 */
	if(left) {
		double* lpa = preagg_that(g, h, dh, nRows); /* nVals_g x nCol_h */
		mm_to_upper(lpa, h->nColG, h->cols, dg, g->nColG, g->cols, g->nVals, res, nCols);
		free(lpa);
	}
	else {
		double* rpa = preagg_that(h, g, dg, nRows); /* nVals_h x nCol_g */
		mm_to_upper(dh, h->nColG, h->cols, rpa, g->nColG, g->cols, h->nVals, res, nCols);
		free(rpa);
	}
}

typedef struct {
	const filtered* f; int64_t nRows; int nCols; double* res; int nTasks; int* ti; int* tj; double** priv;
} tsmm_ctx;

static void tsmm_task(void* vctx, int t) {
	tsmm_ctx* c = (tsmm_ctx*) vctx;
	const int i = c->ti[t], j = c->tj[t];
	const ora_group* g = c->f->g[i];
	if(i == j) {
		int32_t* counts = (int32_t*) malloc(sizeof(int32_t) * (size_t) imax(g->nVals, 1));
		ora_counts(g, c->nRows, counts);
		tsmm_self(g, c->f->dict[i], counts, c->res, c->nCols);
		free(counts);
	}
	else
		tsmm_pair(g, c->f->dict[i], c->f->g[j], c->f->dict[j], c->nRows, c->res, c->nCols);
}

int64_t ora_tsmm(const ora_group* groups, int nG, int64_t nRows, int nCols, double* out, int k) {
	memset(out, 0, sizeof(double) * (size_t) nCols * nCols);
	int hasUnc = 0;
	for(int i = 0; i < nG; i++) hasUnc |= groups[i].type == ORA_UNC;
	if(nG >= nCols || hasUnc) {
		/* :73-77 decompress + LibMatrixMult.matrixMultTransposeSelf (upper triangle, then mirrored) */
		double* D = (double*) malloc(sizeof(double) * (size_t) lmax(nRows, 1) * nCols);
		ora_decompress(groups, nG, nRows, nCols, D);
		for(int64_t r = 0; r < nRows; r++) {
			const double* d = D + (size_t) r * nCols;
			for(int i = 0; i < nCols; i++) {
				const double a = d[i];
				if(a != 0) for(int j = i; j < nCols; j++) out[(size_t) i * nCols + j] += a * d[j];
			}
		}
		free(D);
	}
	else {
		filtered f;
		filter_groups(groups, nG, nCols, &f);
		tsmm_ctx c;
		c.f = &f; c.nRows = nRows; c.nCols = nCols; c.res = out;
		c.nTasks = f.n * (f.n + 1) / 2;
		c.ti = (int*) malloc(sizeof(int) * (size_t) imax(c.nTasks, 1));
		c.tj = (int*) malloc(sizeof(int) * (size_t) imax(c.nTasks, 1));
		int t = 0;
		for(int i = 0; i < f.n; i++) for(int j = i; j < f.n; j++) { c.ti[t] = i; c.tj[t] = j; t++; }
		/* tasks write disjoint rectangles of the upper triangle for non-overlapping groups (:135-154) */
		run_tasks(tsmm_task, &c, c.nTasks, imax(k, 1));
		free(c.ti); free(c.tj);
		if(f.constV) {
			/* addCorrectionLayer (:103-108, :156-166) with colSum of the filtered groups */
			double* cs = (double*) calloc((size_t) nCols, sizeof(double));
			for(int i = 0; i < f.n; i++) {
				const ora_group* g = f.g[i];
				int32_t* counts = (int32_t*) malloc(sizeof(int32_t) * (size_t) imax(g->nVals, 1));
				ora_counts(g, nRows, counts);
				for(int kk = 0; kk < g->nVals; kk++)
					for(int j = 0; j < g->nColG; j++) cs[g->cols[j]] += f.dict[i][(size_t) kk * g->nColG + j] * counts[kk];
				free(counts);
			}
			for(int row = 0; row < nCols; row++) {
				const double v1l = f.constV[row];
				const double v2l = cs[row] + f.constV[row] * (double) nRows;
				for(int col = row; col < nCols; col++)
					out[(size_t) row * nCols + col] += v1l * cs[col] + v2l * f.constV[col];
			}
			free(cs);
		}
		filtered_free(&f);
	}
	/* LibMatrixMult.copyUpperToLowerTriangle + nnz (R/matrix/data/LibMatrixMult.java:4769) */
	int64_t nnz = 0;
	for(int i = 0; i < nCols; i++)
		for(int j = i; j < nCols; j++) {
			const double v = out[(size_t) i * nCols + j];
			out[(size_t) j * nCols + i] = v;
			if(v != 0) nnz += (i == j) ? 1 : 2;
		}
	return nnz;
}

/* ------------------------------------------------------------------------- */
/* Compressed x compressed: CLALibLeftMultBy.leftMultByMatrixTransposed for    */
/* two compressed blocks, single-threaded form                                 */
/* (C/lib/CLALibLeftMultBy.java:100-112, 249-284): out = t(left) %*% right.    */
/* ------------------------------------------------------------------------- */
/* DictLibMatrixMult.MMDictsDenseDense (CG/dictionary/DictLibMatrixMult.java:195-215);
 * scale != NULL: MMDictsScalingDenseDense (:217-237) */
static void mm_dicts(const double* left, int lSize, const int32_t* rowsLeft, const double* right, int rSize,
	const int32_t* colsRight, int commonDim, const int32_t* scale, double* res, int resCols) {
	for(int k = 0; k < commonDim; k++)
		for(int i = 0; i < lSize; i++) {
			const double vl = scale ? left[(size_t) k * lSize + i] * scale[k] : left[(size_t) k * lSize + i];
			if(vl != 0)
				for(int j = 0; j < rSize; j++)
					res[(size_t) rowsLeft[i] * resCols + colsRight[j]] += vl * right[(size_t) k * rSize + j];
		}
}

/* pre-aggregate of a dense column block over a group's index structure, rows in ascending order:
 * P[code(r), i] += D[r, i]  (APreAgg.preAggregate on the transposed uncompressed data,
 * CG/APreAgg.java:234-249, CG/ColGroupUncompressed.java:741-783) */
static double* preagg_dense_cols(const ora_group* g, const double* D, int nC, int64_t nRows) {
	double* P = (double*) calloc((size_t) imax(g->nVals, 1) * nC, sizeof(double));
	int32_t* c = row_codes(g, nRows);
	for(int64_t r = 0; r < nRows; r++)
		if(c[r] >= 0)
			for(int i = 0; i < nC; i++) P[(size_t) c[r] * nC + i] += D[(size_t) r * nC + i];
	free(c);
	return P;
}

/* rhs.leftMultByAColGroup(lhs, ret, nRows): APreAgg.java:70-79, 211-249; ColGroupUncompressed.java:732-825 */
static void left_mult_by_group(const ora_group* rhs, const double* dr, const ora_group* lhs, const double* dl,
	int64_t nRows, double* res, int resCols) {
	const int lc = lhs->nColG, rc = rhs->nColG;
	if(lhs->type == ORA_UNC && rhs->type == ORA_UNC) {
		/* t(lhs data) %*% rhs data, rows in ascending order */
		for(int64_t r = 0; r < nRows; r++)
			for(int i = 0; i < lc; i++) {
				const double a = lhs->dense[(size_t) r * lc + i];
				if(a != 0)
					for(int j = 0; j < rc; j++)
						res[(size_t) lhs->cols[i] * resCols + rhs->cols[j]] += a * rhs->dense[(size_t) r * rc + j];
			}
	}
	else if(lhs->type == ORA_UNC) {
		/* rhs pre-aggregates the transposed left data, then times its dictionary (APreAgg.java:234-249) */
		double* P = preagg_dense_cols(rhs, lhs->dense, lc, nRows); /* nVals_r x lc */
		mm_dicts(P, lc, lhs->cols, dr, rc, rhs->cols, rhs->nVals, NULL, res, resCols);
		free(P);
	}
	else if(rhs->type == ORA_UNC) {
		/* lhs pre-aggregates the transposed right data one column at a time (ColGroupUncompressed.java:741-783) */
		double* P = preagg_dense_cols(lhs, rhs->dense, rc, nRows); /* nVals_l x rc */
		mm_dicts(dl, lc, lhs->cols, P, rc, rhs->cols, lhs->nVals, NULL, res, resCols);
		free(P);
	}
	else if(lhs->codes == rhs->codes && lhs->type == rhs->type && lhs->deltas == rhs->deltas && lhs->rle == rhs->rle) {
		/* same index structure: the dictionaries meet directly, scaled by the counts (:216-220) */
		int32_t* counts = (int32_t*) malloc(sizeof(int32_t) * (size_t) imax(rhs->nVals, 1));
		ora_counts(rhs, nRows, counts);
		mm_dicts(dl, lc, lhs->cols, dr, rc, rhs->cols, rhs->nVals, counts, res, resCols);
		free(counts);
	}
	else if((double) rhs->nVals * rc < (double) lhs->nVals * lc) { /* shouldPreAggregateLeft (:302-310) */
		double* lpa = preagg_that(lhs, rhs, dr, nRows); /* nVals_l x rc */
		mm_dicts(dl, lc, lhs->cols, lpa, rc, rhs->cols, lhs->nVals, NULL, res, resCols);
		free(lpa);
	}
	else {
		double* rpa = preagg_that(rhs, lhs, dl, nRows); /* nVals_r x lc */
		mm_dicts(rpa, lc, lhs->cols, dr, rc, rhs->cols, rhs->nVals, NULL, res, resCols);
		free(rpa);
	}
}

/* AColGroup.colSum of the filtered groups (CLALibUtils.getColSum, C/lib/CLALibUtils.java:267-269) */
static double* filtered_col_sum(const filtered* f, int nCols, int64_t nRows) {
	double* cs = (double*) calloc((size_t) imax(nCols, 1), sizeof(double));
	for(int i = 0; i < f->n; i++) {
		const ora_group* g = f->g[i];
		if(g->type == ORA_UNC) {
			for(int64_t r = 0; r < nRows; r++)
				for(int j = 0; j < g->nColG; j++) cs[g->cols[j]] += g->dense[(size_t) r * g->nColG + j];
			continue;
		}
		int32_t* counts = (int32_t*) malloc(sizeof(int32_t) * (size_t) imax(g->nVals, 1));
		ora_counts(g, nRows, counts);
		for(int kk = 0; kk < g->nVals; kk++)
			for(int j = 0; j < g->nColG; j++) cs[g->cols[j]] += f->dict[i][(size_t) kk * g->nColG + j] * counts[kk];
		free(counts);
	}
	return cs;
}

int64_t ora_lmm_compressed(const ora_group* right, int nGR, int nColsR, const ora_group* left, int nGL, int nColsL,
	int64_t nRows, double* out) {
	if(nRows < 0 || nColsR <= 0 || nColsL <= 0) FAIL(-1, "lmm_compressed: bad dims");
	memset(out, 0, sizeof(double) * (size_t) nColsL * nColsR);
	filtered fR, fL;
	filter_groups(right, nGR, nColsR, &fR);
	filter_groups(left, nGL, nColsL, &fL);
	for(int j = 0; j < fL.n; j++)
		for(int i = 0; i < fR.n; i++)
			left_mult_by_group(fR.g[i], fR.dict[i], fL.g[j], fL.dict[j], nRows, out, nColsR);
	const double* cL = fL.constV;
	const double* cR = fR.constV;
	if(cL && cR) /* outerProductWithScaling (:639-648) */
		for(int row = 0; row < nColsL; row++) {
			const double v = cL[row] * (double) (int) nRows;
			for(int col = 0; col < nColsR; col++) out[(size_t) row * nColsR + col] += v * cR[col];
		}
	if(cL) { /* left constants x column sums of the right groups (:558-569) */
		double* cs = filtered_col_sum(&fR, nColsR, nRows);
		for(int row = 0; row < nColsL; row++)
			if(cL[row] != 0)
				for(int col = 0; col < nColsR; col++) out[(size_t) row * nColsR + col] += cL[row] * cs[col];
		free(cs);
	}
	if(cR) { /* column sums of the left groups x right constants */
		double* cs = filtered_col_sum(&fL, nColsL, nRows);
		for(int row = 0; row < nColsL; row++)
			if(cs[row] != 0)
				for(int col = 0; col < nColsR; col++) out[(size_t) row * nColsR + col] += cs[row] * cR[col];
		free(cs);
	}
	filtered_free(&fR); filtered_free(&fL);
	int64_t nnz = 0;
	for(size_t z = 0; z < (size_t) nColsL * nColsR; z++) nnz += out[z] != 0;
	return nnz;
}

/* ------------------------------------------------------------------------- */
/* MMChain: CLALibMMChain.mmChain (C/lib/CLALibMMChain.java:92-148):           */
/* t(X) %*% (w * (X %*% v)) ; ctype 0 = XtXv, 1 = XtwXv.                       */
/* ------------------------------------------------------------------------- */
int64_t ora_mmchain(const ora_group* groups, int nG, int64_t nRows, int nCols, const double* v, const double* w,
	int ctype, double* out, int k) {
	double* tmp = (double*) malloc(sizeof(double) * (size_t) lmax(nRows, 1));
	if(ora_rmm(groups, nG, nRows, nCols, v, 1, tmp, k) < 0) { free(tmp); return -1; }
	if(ctype == 1) {
		if(!w) { free(tmp); FAIL(-1, "mmchain: XtwXv needs w"); }
		for(int64_t r = 0; r < nRows; r++) tmp[r] *= w[r];
	}
	const int64_t nnz = ora_lmm(groups, nG, nRows, nCols, tmp, 1, out, k);
	free(tmp);
	return nnz;
}
