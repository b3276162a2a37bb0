/*
 * cla_hip.h — C ABI of libclahip.so: the compressed linear algebra (CLA)
 * multiply path of Apache SystemDS on one AMD MI355X (gfx950), hand-written HIP.
 *
 * This is the boundary a SystemDS maintainer binds with JNI or Panama FFM from
 * org.apache.sysds.runtime.compress. It follows the conventions of the
 * reference's existing native bridge (utils/NativeHelper.java:361-418,
 * src/main/cpp/systemds.cpp:64-84): primitive arrays in, the number of
 * non-zeros (a long) out, a negative value on failure so that the caller falls
 * back to its Java kernel (R/matrix/data/LibMatrixNative.java:123-135).
 *
 * Granularity: one call per CLALib* driver on a whole CompressedMatrixBlock,
 * so code streams, offset lists, run lists and dictionaries stay resident in
 * HBM between calls. The per-group virtual methods of AColGroup
 * (CG/AColGroup.java:353-462) are served by cla_counts / cla_cooc /
 * cla_preagg / cla_decompress.
 *
 * Reference paths: C/ = src/main/java/org/apache/sysds/runtime/compress/,
 * CG/ = C/colgroup/.
 *
 * Conventions
 *  - All matrices are dense row-major fp64 (Java DenseBlockFP64).
 *  - Host pointers are borrowed only for the duration of the call.
 *  - `_dev` variants take device pointers (HBM) and run asynchronously on the
 *    block's stream up to the final non-zero count read-back; `_dev_async`
 *    variants leave that count in a device counter (cla_block_nnz reads it on
 *    request) and return without waiting for the stream.
 *  - No exceptions cross the boundary (every entry point catches what the host
 *    code below it may throw, std::bad_alloc included); errors are negative
 *    return codes and cla_last_error() (thread local) explains them.
 *  - Calls on different blocks are thread safe; calls on one block are
 *    serialised internally (one HIP stream per block).
 */
#ifndef CLA_HIP_H
#define CLA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct cla_block* cla_handle;

/* error codes (returned negated) */
enum {
	CLA_OK = 0,
	CLA_ERR_INVALID = 1,     /* bad argument / shape (Java: DMLCompressionException) */
	CLA_ERR_UNSUPPORTED = 2, /* encoding or combination not handled (Java: NotImplementedException) */
	CLA_ERR_DEVICE = 3,      /* HIP runtime error, no device, out of memory */
	CLA_ERR_STATE = 4        /* block not finalized / already finalized */
};

/* Library bring-up: replaces NativeHelper's load/initialise step
 * (utils/NativeHelper.java:109-360). Selects the HIP device; fails (negative)
 * when no gfx950 device is visible — the product never computes on the CPU. */
int cla_init(int device);
/* Human readable reason of the last failure on this thread. */
const char* cla_last_error(void);
/* Device/library facts as a JSON object (name, CUs, LDS bytes, HBM bytes). */
int cla_device_info(char* json, size_t cap);

/* ---- CompressedMatrixBlock construction (C/CompressedMatrixBlock.java:119-132) ---- */
cla_handle cla_block_create(int64_t nRows, int32_t nCols);
void cla_block_free(cla_handle h);

/* ColGroupDDC (CG/ColGroupDDC.java:79-113): X[r, cols] = dict[codes[r]].
 * codeWidth 1 = MapToByte/MapToUByte (unsigned, `& 0xFF`), 2 = MapToChar,
 * 4 = MapToInt (CG/mapping/MapToFactory.java:102-117). codes has nRows entries. */
int cla_block_add_ddc(cla_handle h, const int32_t* cols, int32_t nColG, const double* dict, int32_t nVals,
	const void* codes, int32_t codeWidth);

/* ColGroupSDC / ColGroupSDCZeros (CG/ColGroupSDC.java:68-117,
 * CG/ColGroupSDCZeros.java:76-104) with the raw AOffset arrays
 * (CG/offset/OffsetByte.java, OffsetChar.java): `deltas` holds nDeltas entries
 * of deltaWidth bytes (1 or 2), a 0 entry means "+255 (or +65535) and no row".
 * The list has nOffsets rows from offsetToFirst to offsetToLast; codes has
 * nOffsets entries. defaultTuple NULL => SDCZeros. nOffsets may be 1 or 2 with
 * nDeltas 0 / 1 (OffsetSingle / OffsetTwo). */
int cla_block_add_sdc(cla_handle h, const int32_t* cols, int32_t nColG, const double* dict, int32_t nVals,
	const double* defaultTuple, const void* codes, int32_t codeWidth, const void* deltas, int32_t deltaWidth,
	int64_t nDeltas, int32_t offsetToFirst, int32_t offsetToLast, int64_t nOffsets);

/* ColGroupRLE (CG/ColGroupRLE.java:53-91, CG/AColGroupOffset.java:36-55):
 * ptr[nVals+1] positions into data[]; data = (gap, runLength) char pairs. */
int cla_block_add_rle(cla_handle h, const int32_t* cols, int32_t nColG, const double* dict, int32_t nVals,
	const int32_t* ptr, const uint16_t* data, int64_t nData);

/* ColGroupUncompressed (dense MatrixBlock nRows x nColG, row-major). */
int cla_block_add_uncompressed(cla_handle h, const int32_t* cols, int32_t nColG, const double* values);
/* ColGroupConst (CG/ColGroupConst.java): every row equals `row`. */
int cla_block_add_const(cla_handle h, const int32_t* cols, int32_t nColG, const double* row);
/* ColGroupEmpty. */
int cla_block_add_empty(cla_handle h, const int32_t* cols, int32_t nColG);

/* Ends construction: validates codes < nVals, builds the device-side
 * acceleration structures (offset checkpoints and row-tile index — the
 * device twin of AOffset's skip list, CG/offset/AOffset.java:177-199 — and the
 * merged run table for RLE) and the pre-filter of CLALibUtils.filterGroups
 * (C/lib/CLALibUtils.java:188-206: SDC default -> constV, dict - default). */
int cla_block_finalize(cla_handle h);

/* Use an existing HIP stream (hipStream_t) for all work of this block. */
int cla_block_set_stream(cla_handle h, void* hipStream);
/* Per-block switch between the alternative kernels of a driver (each a complete implementation of the
 * same product: the reference likewise holds several variants per product, e.g. the pre-aggregating and
 * the decompressing right multiply, CG/ColGroupDDC.java:647-692). The defaults are the tuned dispatch.
 *   tsmm_route      0 cost model, 1 one pass per pair of groups, 2 decoded Gram matrix
 *   tsmm_chunks     1 / 0: more than 64 columns as pairs of column chunks
 *   tsmm_wide_dense 0 / 1, tsmm_mfma 1 / 0, tsmm_pair_dot 1 / 0
 *   tsmm_narrow     1 / 0: decoded Gram matrix with a last column block of at most 4 columns on the 4x4x4 matrix instruction
 *   expand_streams  1 / 0: one code per row for small RLE / SDCZeros groups (set before the first multiply)
 *   rmm_disable     bit 0 byte-code mat-vec kernel, 1 its fused tables, 2 matrix-core kernel, 3 decode kernels (tile, stream and
 *                   the decompressed rows times a wide B)
 *   rmm_direct      1 / 0: X %*% B on blocks of plain streams with codes read straight from global memory, 16 columns of B per pass
 *                   (0: at most 16 columns of B on the tile kernel on the matrix cores, wider B per row and group)
 *   lmm_disable     bit 0 dot form on byte codes, bit 1 byte-code bin kernel
 *   sdc_packed      1 / 0: packed SDCZeros lists for the mat-vecs
 *   sdc_lanes       1 / 0: SDCZeros mat-vecs on lane-major copies of the lists, one lane per group
 *   sdc_rows        1 / 0: SDCZeros X %*% v on row lists (the lists transposed), one lane per row
 *   lmm_joint       1 / 0: Y %*% X (16 rows of Y per pass) on a block that is not mostly offset lists in passes over the decoded
 *                   rows on the matrix cores; blocks of more than 64 columns, or whose code tiles exceed LDS together, go chunk of
 *                   columns by chunk (sub-blocks kept with the block); single-column byte-code blocks only from 13 rows of Y
 *                   on (the kernel reports non-finite values of Y and the host looks, i.e. waits for the stream once per call;
 *                   such a Y takes the bin kernels)
 *   tsmm_one_kernel 1 / 0: t(X) %*% X of a whole block of at most 64 columns on the decoded Gram kernels as the call's only
 *                   kernel (its blocks add into an accumulator kept with the block, nCols x nCols doubles; the last block
 *                   to finish writes the output, mirrored, and the count of its non-zeros and clears the accumulator)
 *                   instead of a fill of the output in front of the kernel and a mirror-and-count kernel behind it
 *   ddc_reorder     1 / 0 (read by cla_block_finalize): the block's copy of a DDC group with two- or four-byte codes and a
 *                   dictionary of 16 KiB or more is renumbered by descending count of the tuples (codes in place, dictionary
 *                   rows alike), so that the tuples most rows refer to share cache lines. The reference numbers tuples by
 *                   first appearance (CG/ColGroupFactory.java:682-703); no product depends on the numbering, and cla_counts,
 *                   cla_cooc and cla_preagg answer in the caller's numbering either way
 * Blocks derived from this one (overlapping results, joint blocks) inherit the values at the time of the call
 * that uses them. Returns 0, or -CLA_ERR_INVALID for an unknown key or value. */
int cla_block_set_option(cla_handle h, const char* key, int32_t value);
int32_t cla_block_num_groups(cla_handle h);
/* Dimensions of the block (CompressedMatrixBlock.getNumRows / getNumColumns) and the number of tuples of a group's
 * dictionary (AColGroupValue.getNumValues; 0 for groups without one): what a binding needs to check the lengths
 * of the arrays a caller hands it. Negative: -CLA_ERR_INVALID. */
int64_t cla_block_num_rows(cla_handle h);
int32_t cla_block_num_cols(cla_handle h);
int32_t cla_block_group_num_values(cla_handle h, int32_t group);
/* Bytes of HBM held by the block's compressed representation. */
int64_t cla_block_device_bytes(cla_handle h);
/* Bytes of HBM held by the formats the library has derived from that representation so far (padded
 * dictionary image at finalize; packed SDCZeros lists, one-code-per-row streams and cached counts on the
 * first call of the driver that uses them). */
int64_t cla_block_derived_bytes(cla_handle h);

/* Frees every format the library derived from the block since finalize (and the blocks it made from it for its own
 * use); the next call that wants one builds it again. Waits for the block's stream. It has no counterpart in the reference,
 * whose derived state (cached counts, pre-aggregates) is soft-referenced and goes under memory pressure
 * (CG/AColGroupValue.java getCounts); here the caller decides. Returns 0 or a negative error. */
int cla_block_drop_derived(cla_handle h);
/* Builds now what the first call of the named products would build (so that a caller can pay for it at upload
 * instead of inside the first multiply): each product runs once on operands of zeros in temporary device
 * buffers (for CLA_PRODUCT_RMM an output of nRows x nColB doubles) that are freed before the call returns.
 * nColB: columns of B of the right multiplies to come (which forms a right multiply uses depends on it; 1 for
 * X %*% v), nRowY: rows of Y of the left multiplies; either is ignored when its product is not named. Waits for
 * the stream. It has no counterpart in the reference. Returns 0 or a negative error. */
#define CLA_PRODUCT_RMM 1u
#define CLA_PRODUCT_LMM 2u
#define CLA_PRODUCT_TSMM 4u
int cla_block_prepare(cla_handle h, uint32_t products, int32_t nColB, int32_t nRowY);

/* ---- multiply drivers ---- */

/* CLALibRightMultBy.rightMultByMatrix with allowOverlap=false (RMM,
 * C/lib/CLALibRightMultBy.java:51-102, 208-258): out[nRows x nColB] = X %*% B,
 * B is nCols x nColB. Returns nnz(out) or a negative error. */
int64_t cla_rmm(cla_handle h, const double* B, int32_t nColB, double* out);
int64_t cla_rmm_dev(cla_handle h, const double* dB, int32_t nColB, double* dOut);
/* The same without the wait: returns 0 once the kernels are queued on the block's stream (or a negative
 * error); the non-zero count stays in a device counter until cla_block_nnz asks for it. */
int cla_rmm_dev_async(cla_handle h, const double* dB, int32_t nColB, double* dOut);
/* cla_rmm_dev for callers that cannot allocate device memory (tight serving loops, harnesses that forbid
 * hipMalloc). It has no counterpart in the reference. The pre-aggregated tables dict_g x B and the non-zero
 * counter live in a static device array of 4 MiB that the library holds per GPU until the process ends; the
 * call makes no hipMalloc / hipFree and builds no derived format, so it always takes the table-reading kernels
 * (never the matrix-core or decode kernels). -CLA_ERR_UNSUPPORTED when the tables ((sum of dictionary sizes
 * + 1) x nColB doubles, plus 256 per group for byte-code mat-vecs) exceed the array, or when the block holds
 * SDC groups with entries (their row-tile plan is an allocation). All calls on one GPU share the array: the
 * library serialises them (a lock per GPU, held until the call's kernels have finished), so calls on different
 * blocks from different threads are safe and run one after the other. The call waits for the block's stream
 * before it returns (it cannot run under stream capture). The count returned by cla_block_nnz is not updated
 * by this entry point. */
int64_t cla_rmm_dev_noalloc(cla_handle h, const double* dB, int32_t nColB, double* dOut);
/* nnz of the result of the last driver call on this block (MatrixBlock.recomputeNonZeros of the reference
 * drivers, C/lib/CLALibRightMultBy.java:98); waits for the block's stream. */
int64_t cla_block_nnz(cla_handle h);

/* CLALibLeftMultBy.leftMultByMatrix (C/lib/CLALibLeftMultBy.java:126-145,
 * 286-346): out[nRowY x nCols] = Y %*% X, Y is nRowY x nRows.
 * The _dev_async form returns without waiting except where the block takes the one-pass kernel on the decoded rows
 * (option lmm_joint, blocks that are neither byte-code DDC nor mostly offset lists): that kernel reports a value
 * of Y that is not finite, the host reads the flag (one wait for the block's stream per call) and such a Y takes
 * the bin kernels. The same holds for cla_mmchain_dev_async, whose second half is this product. */
int64_t cla_lmm(cla_handle h, const double* Y, int32_t nRowY, double* out);
int64_t cla_lmm_dev(cla_handle h, const double* dY, int32_t nRowY, double* dOut);
int cla_lmm_dev_async(cla_handle h, const double* dY, int32_t nRowY, double* dOut);

/* CLALibTSMM.leftMultByTransposeSelf (C/lib/CLALibTSMM.java:59-94):
 * out[nCols x nCols] = t(X) %*% X, full symmetric. Blocks no compressed form takes (overlapping
 * groups, an uncompressed group of more than 32 columns among more than 64, a pair of groups whose
 * pre-aggregate exceeds LDS, code tiles, list windows or dictionaries that exceed LDS in the decode
 * kernel) are decompressed in chunks of rows (at most 512 MiB of scratch kept with the block) and
 * multiplied on the matrix cores, as the reference's own fallback does (:73-77). */
int64_t cla_tsmm(cla_handle h, double* out);
int64_t cla_tsmm_dev(cla_handle h, double* dOut);
int cla_tsmm_dev_async(cla_handle h, double* dOut);

/* CLALibLeftMultBy.leftMultByMatrixTransposed for two compressed blocks
 * (C/lib/CLALibLeftMultBy.java:100-112, 170-284): out[nColsLeft x nColsRight] = t(left) %*% right,
 * both blocks with the same number of rows. Every group of `left` meets every group of `right`
 * once (AColGroup.leftMultByAColGroup), the filtered constants of both sides enter through the
 * outer products with the column sums. Returns nnz(out) or a negative error. Shapes no compressed
 * form takes (overlapping groups; beyond 64 columns of both blocks together an uncompressed group
 * of more than 32 columns) go through the decompressed joint rows, as the reference's decompressing
 * fallback does. The first call on a pair of handles builds a
 * small joint descriptor (and, on more than 64 joint columns, descriptors of column chunks). */
int64_t cla_lmm_compressed(cla_handle right, cla_handle left, double* out);
int64_t cla_lmm_compressed_dev(cla_handle right, cla_handle left, double* dOut);

/* CLALibRightMultBy.rightMultByMatrix with allowOverlap (RMMOverlapping,
 * C/lib/CLALibRightMultBy.java:157-201): X %*% B kept compressed. Every group with row data
 * returns a group over all nColB output columns that shares its index structure (codes,
 * offsets, runs) with the source group and holds the dictionary dict_g x B[cols_g, :]
 * (ADictBasedColGroup.rightMultByMatrix, CG/ADictBasedColGroup.java:246-275); constants go
 * through B into the new block's constants. Only the small dictionary products are computed;
 * the returned block (nRows x nColB, overlapping groups) takes every entry point that is
 * linear in the groups (cla_rmm, cla_lmm, cla_mmchain, cla_decompress, sums) and borrows the
 * device copies of the source block, which stays alive until both handles are freed. An
 * uncompressed group returns an uncompressed group over all output columns that holds its rows times
 * B[cols_g, :] (CG/ColGroupUncompressed.java:888-927), owned by the new block.
 * NULL on failure (cla_last_error). */
cla_handle cla_rmm_overlapping(cla_handle h, const double* B, int32_t nColB);

/* CLALibMMChain.mmChain (C/lib/CLALibMMChain.java:92-148):
 * out[nCols] = t(X) %*% (w * (X %*% v)); ctype 0 = XtXv (w ignored), 1 = XtwXv,
 * 2 = XtXvy: t(X) %*% ((X %*% v) - w) (C/lib/CLALibMMChain.java:52). */
int64_t cla_mmchain(cla_handle h, const double* v, const double* w, int32_t ctype, double* out);
int64_t cla_mmchain_dev(cla_handle h, const double* dV, const double* dW, int32_t ctype, double* dOut);
int cla_mmchain_dev_async(cla_handle h, const double* dV, const double* dW, int32_t ctype, double* dOut);

/* CLALibDecompress.decompressDense (C/lib/CLALibDecompress.java:310-357):
 * out[nRows x nCols] = X. */
int64_t cla_decompress(cla_handle h, double* out);
int64_t cla_decompress_dev(cla_handle h, double* dOut);

/* CLALibCompAgg.aggregateUnary (C/lib/CLALibCompAgg.java:78-127) for the operators whose
 * per-group form is counts x dictionary (AColGroupCompressed.unaryAggregateOperations,
 * CG/AColGroupCompressed.java:137-205): op = sum, sum of squares, min, max; dir = all cells
 * (out[1]), per row (out[nRows]), per column (out[nCols]). Returns the number of non-zero
 * cells of the result. What has no such form is aggregated over decompressed chunks of rows (at most
 * 256 MiB of scratch), as CLALibCompAgg.decompressingAggregate does (C/lib/CLALibCompAgg.java:220-232,
 * 419-452, 605-720): everything but plain sums on overlapping groups, row minima / maxima, row sums of
 * squares next to an uncompressed group or over an SDC group with a non-zero default (its tuples are held
 * relative to the default, so their squares would come from a cancelling difference). */
enum cla_agg_op { CLA_AGG_SUM = 0, CLA_AGG_SUMSQ = 1, CLA_AGG_MIN = 2, CLA_AGG_MAX = 3 };
enum cla_agg_dir { CLA_AGG_ALL = 0, CLA_AGG_ROW = 1, CLA_AGG_COL = 2 };
int64_t cla_aggregate(cla_handle h, int32_t op, int32_t dir, double* out);
int64_t cla_aggregate_dev(cla_handle h, int32_t op, int32_t dir, double* dOut);

/* ---- per-group pieces (AColGroup surface) ---- */

/* AMapToData.getCounts / ColGroupRLE.getCounts (CG/mapping/AMapToData.java:408-419,
 * CG/mapping/MapToByte.java:168-187, CG/ColGroupRLE.java:259-265): exact integer
 * histogram of group `group`'s code stream, nVals entries. */
int cla_counts(cla_handle h, int32_t group, int32_t* counts);

/* Integer co-occurrence between two groups of the block:
 * out[a * nVals_B + b] = #{rows r : code_A(r) = a and code_B(r) = b}, rows not
 * covered by an SDCZeros/RLE group are skipped. This is the exact-integer form
 * of APreAgg.preAggregateThatIndexStructure (CG/APreAgg.java:87-110,
 * CG/mapping/AMapToData.java:429-794). */
int cla_cooc(cla_handle h, int32_t groupA, int32_t groupB, int64_t* out);

/* APreAgg.preAggregateDense (CG/APreAgg.java:137-151; DDC
 * CG/mapping/AMapToData.java:214-330, SDCZ CG/offset/AOffset.java:288-430, RLE
 * CG/ColGroupRLE.java:759-796): preAgg[nRowY x nVals] with
 * preAgg[i, code(r)] += Y[i, r]. */
int cla_preagg(cla_handle h, int32_t group, const double* Y, int32_t nRowY, double* preAgg);

/* ---- introspection (the twin of the reference's -stats timers,
 * utils/DMLCompressionStatistics.java:44-125) ---- */
/* enable != 0: bracket every kernel of this block with HIP events on its stream. */
int cla_block_profile(cla_handle h, int enable);
/* JSON with the kernels launched by the last driver call on this block: launch
 * geometry, algorithmic bytes and (when profiling) milliseconds. */
int cla_stats(cla_handle h, char* json, size_t cap);

/* Diagnostic: throws inside the library (kind 0 std::bad_alloc, 1 std::length_error, 2 a non-standard
 * exception, 3 an over-long std::vector reservation) and returns what an entry point returns for it:
 * -CLA_ERR_DEVICE for a failed allocation, -CLA_ERR_INVALID otherwise, 0 for an unknown kind. Needs no
 * device. It is how a binding checks that nothing unwinds into the JVM (JNI code must not let C++
 * exceptions escape, src/main/cpp/systemds.cpp has none to begin with). */
int cla_selftest_exception(int kind);

#ifdef __cplusplus
}
#endif
#endif
