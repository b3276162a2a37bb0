"""The C-ABI library loads and exports every symbol include/cla_hip.h declares."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    src = open(os.path.join(ROOT, "include", "cla_hip.h")).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(cla_[a-z_0-9]+)\s*\(", src)))


def test_header_declares_the_expected_surface():
    syms = declared_symbols()
    for s in ("cla_init", "cla_block_create", "cla_block_add_ddc", "cla_block_add_sdc", "cla_block_add_rle",
              "cla_block_finalize", "cla_rmm", "cla_lmm", "cla_tsmm", "cla_counts", "cla_cooc"):
        assert s in syms


def test_library_exports_every_declared_symbol():
    from systemds_amd import capi
    assert os.path.exists(capi.LIB_PATH), "libclahip.so not built: run __graft_entry__.build()"
    lib = ctypes.CDLL(capi.LIB_PATH)
    missing = [s for s in declared_symbols() if not hasattr(lib, s)]
    assert not missing, missing
    # the ctypes table binds exactly the declared surface
    assert sorted(capi.SIGNATURES) == declared_symbols()


def test_product_fails_loudly_without_gpu_or_init():
    """No CPU fallback: without a device every entry point reports an error."""
    import torch
    from systemds_amd import capi
    lib = capi.load_library()
    if torch.cuda.is_available():
        return
    assert lib.cla_init(0) < 0
    assert b"GPU only" in lib.cla_last_error()
    assert not lib.cla_block_create(10, 2)


def test_no_exception_crosses_the_boundary():
    """Host code below the entry points may throw (std::bad_alloc from a vector, std::length_error from an
    absurd size): every entry point turns that into a negative code and a message. Needs no device."""
    from systemds_amd import capi
    lib = capi.load_library()
    assert lib.cla_selftest_exception(0) == capi.ERR_DEVICE
    assert b"allocation" in lib.cla_last_error()
    assert lib.cla_selftest_exception(1) == capi.ERR_INVALID
    assert b"selftest" in lib.cla_last_error()
    assert lib.cla_selftest_exception(2) == capi.ERR_INVALID
    assert lib.cla_selftest_exception(3) == capi.ERR_INVALID
    assert lib.cla_selftest_exception(99) == 0


def test_jni_shim_covers_the_java_natives():
    """systemds_amd/jni: every `static native` of ClaHipNative.java has a shim function in cla_jni.c, and the
    shim only calls symbols that include/cla_hip.h declares (neither file can be compiled without a JDK)."""
    jni = os.path.join(ROOT, "systemds_amd", "jni")
    java = open(os.path.join(jni, "ClaHipNative.java")).read()
    shim = open(os.path.join(jni, "cla_jni.c")).read()
    natives = re.findall(r"public static native \S+\s+(\w+)\(", java)
    assert len(natives) >= 20
    shims = set(re.findall(r"FN\((\w+)\)\(", shim)) | set(re.findall(r"ADD_COLS_VALUES\((\w+),", shim))
    shims -= {"name"}  # the macro's own parameter
    assert sorted(natives) == sorted(shims)
    called = set(re.findall(r"\b(cla_[a-z_0-9]+)\s*\(", re.sub(r"/\*.*?\*/", "", shim, flags=re.S)))
    called |= set(re.findall(r"ADD_COLS_VALUES\(\w+, (cla_\w+)\)", shim))
    assert called and called <= set(declared_symbols()), called - set(declared_symbols())
