/*
 * Native declarations of libclahip.so for SystemDS (package org.apache.sysds.utils, next to
 * NativeHelper: src/main/java/org/apache/sysds/utils/NativeHelper.java:361-418). One static
 * native per entry point of include/cla_hip.h that the compressed multiply drivers call; the JNI
 * side is cla_jni.c in this directory.
 *
 * Conventions, as in NativeHelper and LibMatrixNative (runtime/matrix/data/LibMatrixNative.java:
 * 123-135): primitive arrays in, the number of non-zeros (a long) out, a negative value means
 * "not done on the device" and the caller keeps its Java path; lastError() explains it.
 *
 * This file needs a JDK to compile; the build image of this repository has none, so it is kept
 * as source for the maintainer who adds the binding.
 */
package org.apache.sysds.utils;

public final class ClaHipNative {
	private static boolean loaded = false;

	private ClaHipNative() {
	}

	/** Loads the JNI shim (which links libclahip.so) and selects the device; false = keep the Java path. */
	public static synchronized boolean load(int device) {
		if(loaded)
			return true;
		try {
			System.loadLibrary("clahip_jni");
			loaded = init(device) == 0;
		}
		catch(UnsatisfiedLinkError e) {
			loaded = false;
		}
		return loaded;
	}

	// ---- library
	public static native int init(int device);

	public static native String lastError();

	// ---- CompressedMatrixBlock construction (compress/CompressedMatrixBlock.java:119-132)
	public static native long blockCreate(long nRows, int nCols);

	public static native void blockFree(long h);

	/** codes: byte[] (MapToByte / MapToUByte), char[] (MapToChar) or int[] (MapToInt); codeWidth 1 / 2 / 4. */
	public static native int addDDC(long h, int[] cols, double[] dict, int nVals, Object codes, int codeWidth);

	/** deltas: byte[] (OffsetByte.offsets) or char[] (OffsetChar.offsets); defaultTuple null = SDCZeros. */
	public static native int addSDC(long h, int[] cols, double[] dict, int nVals, double[] defaultTuple, Object codes,
		int codeWidth, Object deltas, int deltaWidth, long nDeltas, int offsetToFirst, int offsetToLast, long nOffsets);

	public static native int addRLE(long h, int[] cols, double[] dict, int nVals, int[] ptr, char[] data);

	public static native int addUncompressed(long h, int[] cols, double[] values);

	public static native int addConst(long h, int[] cols, double[] row);

	public static native int addEmpty(long h, int[] cols);

	public static native int finalizeBlock(long h);

	public static native int setOption(long h, String key, int value);

	/** Frees every format the library derived from the block since finalizeBlock; the next call that wants one builds it again. */
	public static native int dropDerived(long h);

	/** Product bits of prepare. */
	public static final int PRODUCT_RMM = 1, PRODUCT_LMM = 2, PRODUCT_TSMM = 4;

	/** Builds now what the first call of the named products would build (nColB / nRowY: the widths of the operands to come). */
	public static native int prepare(long h, int products, int nColB, int nRowY);

	/** Bytes of device memory held by the derived formats. */
	public static native long derivedBytes(long h);

	// ---- drivers (compress/lib/CLALibRightMultBy, CLALibLeftMultBy, CLALibTSMM, CLALibMMChain, ...)
	public static native long rmm(long h, double[] B, int nColB, double[] out);

	public static native long lmm(long h, double[] Y, int nRowY, double[] out);

	public static native long tsmm(long h, double[] out);

	/** ctype 0 XtXv, 1 XtwXv, 2 XtXvy (MapMultChain.ChainType). */
	public static native long mmchain(long h, double[] v, double[] w, int ctype, double[] out);

	/** cla_rmm_overlapping: handle of the overlapping result block, 0 = not supported. */
	public static native long rmmOverlapping(long h, double[] B, int nColB);

	/** cla_lmm_compressed: out = t(left) %*% right. */
	public static native long lmmCompressed(long hRight, long hLeft, double[] out);

	public static native long decompress(long h, double[] out);

	/** op 0 sum, 1 sumSq, 2 min, 3 max; dir 0 all cells, 1 per row, 2 per column. */
	public static native long aggregate(long h, int op, int dir, double[] out);

	// ---- per-group pieces (AColGroup surface)
	public static native int counts(long h, int group, int[] counts);

	public static native int cooc(long h, int groupA, int groupB, long[] out);

	public static native int preagg(long h, int group, double[] Y, int nRowY, double[] preAgg);
}
