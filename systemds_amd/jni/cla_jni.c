/*
 * JNI shim between org.apache.sysds.utils.ClaHipNative (ClaHipNative.java in this directory) and
 * libclahip.so (include/cla_hip.h). Same pattern as the reference's own bridge
 * (src/main/cpp/systemds.cpp:38-84): arrays are pinned with GetPrimitiveArrayCritical, inputs are
 * released with JNI_ABORT (no copy back), outputs with 0 (copy back when the VM handed out a copy).
 * No JNI call is made while an array is pinned; the library throws no C++ exception across its
 * boundary, so nothing can unwind through these frames. Array references are checked for NULL and for the
 * length the library will read or write before anything is pinned.
 * This file has not been compiled or run where it was written (no JDK there): it is the binding as a
 * maintainer would add it, checked by reading only.
 *
 * Build (needs a JDK; systemds_amd/build.py compiles it when $JAVA_HOME/include/jni.h exists):
 *   cc -O2 -fPIC -shared -I$JAVA_HOME/include -I$JAVA_HOME/include/linux -Iinclude \
 *      systemds_amd/jni/cla_jni.c -o libclahip_jni.so -Lsystemds_amd -lclahip
 */
#include <jni.h>
#include <stddef.h>
#include "cla_hip.h"

#define FN(name) Java_org_apache_sysds_utils_ClaHipNative_##name
#define H(h) ((cla_handle) (intptr_t) (h))

/* Length of a Java array, -1 for a NULL reference (GetArrayLength on NULL crashes the VM). */
static jlong len(JNIEnv* env, jarray a) { return a ? (jlong) (*env)->GetArrayLength(env, a) : -1; }
/* An array the library reads or writes `need` elements of: not NULL and long enough. Checked before anything is
 * pinned: a short array would otherwise be a heap overwrite inside a critical region. */
static int holds(JNIEnv* env, jarray a, jlong need) { return need >= 0 && len(env, a) >= need; }

/* pin / unpin; a NULL Java array pins to NULL */
static void* pin(JNIEnv* env, jarray a) { return a ? (*env)->GetPrimitiveArrayCritical(env, a, NULL) : NULL; }
static void unpin_in(JNIEnv* env, jarray a, void* p) { if(a && p) (*env)->ReleasePrimitiveArrayCritical(env, a, p, JNI_ABORT); }
static void unpin_out(JNIEnv* env, jarray a, void* p) { if(a && p) (*env)->ReleasePrimitiveArrayCritical(env, a, p, 0); }

JNIEXPORT jint JNICALL FN(init)(JNIEnv* env, jclass c, jint device) { (void) env; (void) c; return cla_init(device); }

JNIEXPORT jstring JNICALL FN(lastError)(JNIEnv* env, jclass c) { (void) c; return (*env)->NewStringUTF(env, cla_last_error()); }

JNIEXPORT jlong JNICALL FN(blockCreate)(JNIEnv* env, jclass c, jlong nRows, jint nCols) {
	(void) env; (void) c;
	return (jlong) (intptr_t) cla_block_create(nRows, nCols);
}

JNIEXPORT void JNICALL FN(blockFree)(JNIEnv* env, jclass c, jlong h) { (void) env; (void) c; cla_block_free(H(h)); }

JNIEXPORT jint JNICALL FN(addDDC)(JNIEnv* env, jclass c, jlong h, jintArray cols, jdoubleArray dict, jint nVals,
	jobject codes, jint codeWidth) {
	(void) c;
	if(!cols || !holds(env, dict, (jlong) nVals * len(env, cols)) || !holds(env, (jarray) codes, cla_block_num_rows(H(h)))) return -CLA_ERR_INVALID;
	const jint nColG = (*env)->GetArrayLength(env, cols);
	jint* pc = pin(env, cols);
	double* pd = pin(env, dict);
	void* pk = pin(env, (jarray) codes);
	const jint rc = (pc && pd) ? cla_block_add_ddc(H(h), (const int32_t*) pc, nColG, pd, nVals, pk, codeWidth) : -CLA_ERR_INVALID;
	unpin_in(env, (jarray) codes, pk);
	unpin_in(env, dict, pd);
	unpin_in(env, cols, pc);
	return rc;
}

JNIEXPORT jint JNICALL FN(addSDC)(JNIEnv* env, jclass c, jlong h, jintArray cols, jdoubleArray dict, jint nVals,
	jdoubleArray defaultTuple, jobject codes, jint codeWidth, jobject deltas, jint deltaWidth, jlong nDeltas, jint offsetToFirst,
	jint offsetToLast, jlong nOffsets) {
	(void) c;
	if(!cols || !holds(env, dict, (jlong) nVals * len(env, cols)) || (defaultTuple && !holds(env, defaultTuple, len(env, cols))) ||
		(nOffsets > 0 && (!holds(env, (jarray) codes, nOffsets) || !holds(env, (jarray) deltas, nDeltas)))) return -CLA_ERR_INVALID;
	const jint nColG = (*env)->GetArrayLength(env, cols);
	jint* pc = pin(env, cols);
	double* pd = pin(env, dict);
	double* pt = pin(env, defaultTuple);
	void* pk = pin(env, (jarray) codes);
	void* po = pin(env, (jarray) deltas);
	const jint rc = (pc && pd) ? cla_block_add_sdc(H(h), (const int32_t*) pc, nColG, pd, nVals, pt, pk, codeWidth, po, deltaWidth,
		nDeltas, offsetToFirst, offsetToLast, nOffsets) : -CLA_ERR_INVALID;
	unpin_in(env, (jarray) deltas, po);
	unpin_in(env, (jarray) codes, pk);
	unpin_in(env, defaultTuple, pt);
	unpin_in(env, dict, pd);
	unpin_in(env, cols, pc);
	return rc;
}

JNIEXPORT jint JNICALL FN(addRLE)(JNIEnv* env, jclass c, jlong h, jintArray cols, jdoubleArray dict, jint nVals, jintArray ptr,
	jcharArray data) {
	(void) c;
	if(!cols || !data || !holds(env, dict, (jlong) nVals * len(env, cols)) || !holds(env, ptr, (jlong) nVals + 1)) return -CLA_ERR_INVALID;
	const jint nColG = (*env)->GetArrayLength(env, cols);
	const jlong nData = (*env)->GetArrayLength(env, data);
	jint* pc = pin(env, cols);
	double* pd = pin(env, dict);
	jint* pp = pin(env, ptr);
	jchar* pr = pin(env, data);
	const jint rc = (pc && pd && pp) ? cla_block_add_rle(H(h), (const int32_t*) pc, nColG, pd, nVals, (const int32_t*) pp,
		(const uint16_t*) pr, nData) : -CLA_ERR_INVALID;
	unpin_in(env, data, pr);
	unpin_in(env, ptr, pp);
	unpin_in(env, dict, pd);
	unpin_in(env, cols, pc);
	return rc;
}

/* cols + one double array */
#define ADD_COLS_VALUES(name, call)                                                                         \
	JNIEXPORT jint JNICALL FN(name)(JNIEnv* env, jclass c, jlong h, jintArray cols, jdoubleArray values) { \
		(void) c;                                                                                           \
		if(!cols || !values) return -CLA_ERR_INVALID;                                                       \
		const jint nColG = (*env)->GetArrayLength(env, cols);                                               \
		jint* pc = pin(env, cols);                                                                          \
		double* pv = pin(env, values);                                                                      \
		const jint rc = pc ? call(H(h), (const int32_t*) pc, nColG, pv) : -CLA_ERR_INVALID;                 \
		unpin_in(env, values, pv);                                                                          \
		unpin_in(env, cols, pc);                                                                            \
		return rc;                                                                                          \
	}
ADD_COLS_VALUES(addUncompressed, cla_block_add_uncompressed)
ADD_COLS_VALUES(addConst, cla_block_add_const)

JNIEXPORT jint JNICALL FN(addEmpty)(JNIEnv* env, jclass c, jlong h, jintArray cols) {
	(void) c;
	if(!cols) return -CLA_ERR_INVALID;
	const jint nColG = (*env)->GetArrayLength(env, cols);
	jint* pc = pin(env, cols);
	const jint rc = pc ? cla_block_add_empty(H(h), (const int32_t*) pc, nColG) : -CLA_ERR_INVALID;
	unpin_in(env, cols, pc);
	return rc;
}

JNIEXPORT jint JNICALL FN(finalizeBlock)(JNIEnv* env, jclass c, jlong h) { (void) env; (void) c; return cla_block_finalize(H(h)); }

JNIEXPORT jint JNICALL FN(setOption)(JNIEnv* env, jclass c, jlong h, jstring key, jint value) {
	(void) c;
	const char* k = (*env)->GetStringUTFChars(env, key, NULL);
	if(!k) return -CLA_ERR_INVALID;
	const jint rc = cla_block_set_option(H(h), k, value);
	(*env)->ReleaseStringUTFChars(env, key, k);
	return rc;
}

JNIEXPORT jint JNICALL FN(dropDerived)(JNIEnv* env, jclass c, jlong h) { (void) env; (void) c; return cla_block_drop_derived(H(h)); }

JNIEXPORT jint JNICALL FN(prepare)(JNIEnv* env, jclass c, jlong h, jint products, jint nColB, jint nRowY) {
	(void) env; (void) c;
	return cla_block_prepare(H(h), (uint32_t) products, nColB, nRowY);
}

JNIEXPORT jlong JNICALL FN(derivedBytes)(JNIEnv* env, jclass c, jlong h) { (void) env; (void) c; return cla_block_derived_bytes(H(h)); }

/* one input array, one output array */
JNIEXPORT jlong JNICALL FN(rmm)(JNIEnv* env, jclass c, jlong h, jdoubleArray B, jint nColB, jdoubleArray out) {
	(void) c;
	const jlong nR = cla_block_num_rows(H(h)), nC = cla_block_num_cols(H(h));
	if(nColB <= 0 || !holds(env, B, nC * nColB) || !holds(env, out, nR * nColB)) return -CLA_ERR_INVALID;
	double* b = pin(env, B);
	double* o = pin(env, out);
	const jlong nnz = (b && o) ? cla_rmm(H(h), b, nColB, o) : -CLA_ERR_INVALID;
	unpin_out(env, out, o);
	unpin_in(env, B, b);
	return nnz;
}

JNIEXPORT jlong JNICALL FN(lmm)(JNIEnv* env, jclass c, jlong h, jdoubleArray Y, jint nRowY, jdoubleArray out) {
	(void) c;
	const jlong nR = cla_block_num_rows(H(h)), nC = cla_block_num_cols(H(h));
	if(nRowY <= 0 || !holds(env, Y, nR * nRowY) || !holds(env, out, nC * nRowY)) return -CLA_ERR_INVALID;
	double* y = pin(env, Y);
	double* o = pin(env, out);
	const jlong nnz = (y && o) ? cla_lmm(H(h), y, nRowY, o) : -CLA_ERR_INVALID;
	unpin_out(env, out, o);
	unpin_in(env, Y, y);
	return nnz;
}

JNIEXPORT jlong JNICALL FN(tsmm)(JNIEnv* env, jclass c, jlong h, jdoubleArray out) {
	(void) c;
	const jlong nC = cla_block_num_cols(H(h));
	if(!holds(env, out, nC * nC)) return -CLA_ERR_INVALID;
	double* o = pin(env, out);
	const jlong nnz = o ? cla_tsmm(H(h), o) : -CLA_ERR_INVALID;
	unpin_out(env, out, o);
	return nnz;
}

JNIEXPORT jlong JNICALL FN(mmchain)(JNIEnv* env, jclass c, jlong h, jdoubleArray v, jdoubleArray w, jint ctype, jdoubleArray out) {
	(void) c;
	const jlong nR = cla_block_num_rows(H(h)), nC = cla_block_num_cols(H(h));
	if(!holds(env, v, nC) || (w && !holds(env, w, nR)) || !holds(env, out, nC)) return -CLA_ERR_INVALID;
	double* pv = pin(env, v);
	double* pw = pin(env, w);
	double* o = pin(env, out);
	const jlong nnz = (pv && o) ? cla_mmchain(H(h), pv, pw, ctype, o) : -CLA_ERR_INVALID;
	unpin_out(env, out, o);
	unpin_in(env, w, pw);
	unpin_in(env, v, pv);
	return nnz;
}

JNIEXPORT jlong JNICALL FN(rmmOverlapping)(JNIEnv* env, jclass c, jlong h, jdoubleArray B, jint nColB) {
	(void) c;
	if(nColB <= 0 || !holds(env, B, (jlong) cla_block_num_cols(H(h)) * nColB)) return 0;
	double* b = pin(env, B);
	const jlong r = b ? (jlong) (intptr_t) cla_rmm_overlapping(H(h), b, nColB) : 0;
	unpin_in(env, B, b);
	return r;
}

JNIEXPORT jlong JNICALL FN(lmmCompressed)(JNIEnv* env, jclass c, jlong hRight, jlong hLeft, jdoubleArray out) {
	(void) c;
	if(!holds(env, out, (jlong) cla_block_num_cols(H(hLeft)) * cla_block_num_cols(H(hRight)))) return -CLA_ERR_INVALID;
	double* o = pin(env, out);
	const jlong nnz = o ? cla_lmm_compressed(H(hRight), H(hLeft), o) : -CLA_ERR_INVALID;
	unpin_out(env, out, o);
	return nnz;
}

JNIEXPORT jlong JNICALL FN(decompress)(JNIEnv* env, jclass c, jlong h, jdoubleArray out) {
	(void) c;
	if(!holds(env, out, cla_block_num_rows(H(h)) * cla_block_num_cols(H(h)))) return -CLA_ERR_INVALID;
	double* o = pin(env, out);
	const jlong nnz = o ? cla_decompress(H(h), o) : -CLA_ERR_INVALID;
	unpin_out(env, out, o);
	return nnz;
}

JNIEXPORT jlong JNICALL FN(aggregate)(JNIEnv* env, jclass c, jlong h, jint op, jint dir, jdoubleArray out) {
	(void) c;
	/* (CLA_AGG_ALL one value, CLA_AGG_ROW one per row, CLA_AGG_COL one per column) */
	if(!holds(env, out, dir == CLA_AGG_ALL ? 1 : dir == CLA_AGG_ROW ? cla_block_num_rows(H(h)) : cla_block_num_cols(H(h)))) return -CLA_ERR_INVALID;
	double* o = pin(env, out);
	const jlong nnz = o ? cla_aggregate(H(h), op, dir, o) : -CLA_ERR_INVALID;
	unpin_out(env, out, o);
	return nnz;
}

JNIEXPORT jint JNICALL FN(counts)(JNIEnv* env, jclass c, jlong h, jint group, jintArray counts) {
	(void) c;
	if(!holds(env, counts, cla_block_group_num_values(H(h), group))) return -CLA_ERR_INVALID;
	jint* p = pin(env, counts);
	const jint rc = p ? cla_counts(H(h), group, (int32_t*) p) : -CLA_ERR_INVALID;
	unpin_out(env, counts, p);
	return rc;
}

JNIEXPORT jint JNICALL FN(cooc)(JNIEnv* env, jclass c, jlong h, jint groupA, jint groupB, jlongArray out) {
	(void) c;
	if(!holds(env, out, (jlong) cla_block_group_num_values(H(h), groupA) * cla_block_group_num_values(H(h), groupB))) return -CLA_ERR_INVALID;
	jlong* p = pin(env, out);
	const jint rc = p ? cla_cooc(H(h), groupA, groupB, (int64_t*) p) : -CLA_ERR_INVALID;
	unpin_out(env, out, p);
	return rc;
}

JNIEXPORT jint JNICALL FN(preagg)(JNIEnv* env, jclass c, jlong h, jint group, jdoubleArray Y, jint nRowY, jdoubleArray preAgg) {
	(void) c;
	if(nRowY <= 0 || !holds(env, Y, cla_block_num_rows(H(h)) * nRowY) ||
		!holds(env, preAgg, (jlong) nRowY * cla_block_group_num_values(H(h), group))) return -CLA_ERR_INVALID;
	double* y = pin(env, Y);
	double* p = pin(env, preAgg);
	const jint rc = (y && p) ? cla_preagg(H(h), group, y, nRowY, p) : -CLA_ERR_INVALID;
	unpin_out(env, preAgg, p);
	unpin_in(env, Y, y);
	return rc;
}
