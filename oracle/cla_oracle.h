/*
 * TEST INFRASTRUCTURE ONLY — CPU restatement ("oracle") of the compressed
 * linear algebra multiply path of Apache SystemDS.
 *
 * Nothing in the product (systemds_amd/, include/) links, imports or calls this.
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg use it,
 * and only as the checker / the timed CPU baseline.
 *
 * Every function cites the reference file:line it follows. Paths are relative
 * to src/main/java/org/apache/sysds/runtime/compress/ of the reference tree
 * (C/ below), colgroup/ is CG/.
 *
 * How each function is pinned (see tests/test_oracle_*.py):
 *   offset codec      : reference-held known-answer row lists
 *                       (src/test/.../compress/offset/OffsetTests.java:78-140),
 *                       exact pre-aggregate sums (OffsetPreAggTests.java:50-350)
 *   rle codec         : encode/decode round trip + structural rules of
 *                       genRLEBitmap (CG/ColGroupRLE.java:1073-1157)
 *   decompress        : closed form dict[code[r]] (brute force in numpy)
 *   rmm / lmm / tsmm  : equal D@B, Y@D, D.T@D of the brute-force decompressed D,
 *                       checked against math.fsum truth; the reference's own
 *                       tests are differential in exactly this way
 *                       (CompressedTestBase.java:609-626, 666-685, 865-884)
 *   lmm_compressed    : equal t(D_left) @ D_right of the two brute-force decompressed
 *                       blocks, checked against math.fsum truth (the reference's test is
 *                       differential the same way, CompressedTestBase.java:726-760)
 *   counts / cooc     : numpy.bincount / np.add.at brute force (exact integers)
 */
#ifndef CLA_ORACLE_H
#define CLA_ORACLE_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { ORA_DDC = 0, ORA_SDC = 1, ORA_RLE = 2, ORA_UNC = 3, ORA_CONST = 4, ORA_EMPTY = 5 };

/* One column group, all arrays borrowed. Mirrors the fields of
 * ColGroupDDC (CG/ColGroupDDC.java:79-113), ColGroupSDC/SDCZeros
 * (CG/ColGroupSDC.java:68-117, CG/ColGroupSDCZeros.java:76-104),
 * ColGroupRLE (CG/ColGroupRLE.java:53-91, CG/AColGroupOffset.java:36-55),
 * ColGroupUncompressed, ColGroupConst, ColGroupEmpty. */
typedef struct ora_group {
	int32_t type;
	int32_t nColG;
	int32_t nVals;
	int32_t codeWidth;   /* bytes per code: 1 (MapToByte/UByte), 2 (MapToChar), 4 (MapToInt) */
	const int32_t* cols; /* nColG global column ids */
	const double* dict;  /* nVals x nColG row-major; CONST: 1 x nColG */
	const void* codes;   /* DDC: nRows codes; SDC: nOffsets codes */
	const double* def;   /* SDC default tuple (nColG) or NULL for SDCZeros */
	const void* deltas;  /* SDC: AOffset delta entries (uint8 or uint16) */
	int32_t deltaWidth;  /* 1 = OffsetByte, 2 = OffsetChar */
	int32_t first;       /* offsetToFirst */
	int32_t last;        /* offsetToLast */
	int32_t pad0;
	int64_t nDeltas;
	int64_t nOffsets;    /* number of rows in the offset list (0 => empty list) */
	const int32_t* ptr;  /* RLE: nVals+1 positions into rle[] */
	const uint16_t* rle; /* RLE: (gap, runLength) pairs */
	int64_t nData;       /* RLE: length of rle[] */
	const double* dense; /* UNC: nRows x nColG row-major */
} ora_group;

/* ---- codecs ---- */
int64_t ora_offset_encoded_size(const int32_t* rows, int64_t n, int width);
int64_t ora_offset_encode(const int32_t* rows, int64_t n, int width, void* deltas, int64_t cap);
int64_t ora_offset_decode(const void* deltas, int width, int64_t nDeltas, int32_t first, int32_t* rows, int64_t cap);
int ora_offset_choose_width(const int32_t* rows, int64_t n);
int64_t ora_rle_encode(const int32_t* rows, int64_t n, uint16_t* out, int64_t cap);
int64_t ora_rle_decode(const uint16_t* data, int64_t nData, int32_t* rows, int64_t cap);
int ora_map_width(int64_t nUnique);

/* ---- group-level pieces ---- */
void ora_preagg_values_from_dense(const double* dict, int nVals, const int32_t* cols, int nColG, const double* B,
	int q, double* out);
int ora_counts(const ora_group* g, int64_t nRows, int32_t* counts);
int ora_cooc(const ora_group* a, const ora_group* b, int64_t nRows, int64_t* out);
int ora_decompress(const ora_group* groups, int nG, int64_t nRows, int nCols, double* out);
int ora_preaggregate_dense(const ora_group* g, int64_t nRows, const double* Y, int p, double* preAgg);

/* ---- drivers (k = thread count as the reference's int k) ---- */
int64_t ora_rmm(const ora_group* groups, int nG, int64_t nRows, int nCols, const double* B, int q, double* out, int k);
int64_t ora_lmm(const ora_group* groups, int nG, int64_t nRows, int nCols, const double* Y, int p, double* out, int k);
int64_t ora_tsmm(const ora_group* groups, int nG, int64_t nRows, int nCols, double* out, int k);
/* t(left) %*% right for two compressed blocks of nRows rows each; out is nColsL x nColsR row-major */
int64_t ora_lmm_compressed(const ora_group* right, int nGR, int nColsR, const ora_group* left, int nGL, int nColsL,
	int64_t nRows, double* out);
int64_t ora_mmchain(const ora_group* groups, int nG, int64_t nRows, int nCols, const double* v, const double* w,
	int ctype, double* out, int k);

const char* ora_last_error(void);

#ifdef __cplusplus
}
#endif
#endif
