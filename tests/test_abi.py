"""The C-ABI library loads and exports exactly what include/dsx.h and include/dsx_testing.h (the tests' switches) declare (no
GPU, no compute calls)."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "dsx.h")).read() + open(os.path.join(ROOT, "include", "dsx_testing.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dsx_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = declared_functions()
    for must in ["dsx_init", "dsx_sparse_z", "dsx_sparse_layer_forward", "dsx_fc_forward", "dsx_topk", "dsx_topk_filtered",
                 "dsx_knn_search", "dsx_knn_topk", "dsx_malloc", "dsx_memcpy_h2d"]:
        assert must in names


def test_library_exports_every_declared_symbol(pkg):
    lib = pkg.load_library()
    for name in declared_functions():
        assert hasattr(lib, name), "libdsx_hip.so does not export %s" % name


def test_python_signatures_cover_the_header(pkg):
    bound = set(pkg.SIGNATURES) | set(pkg.SPECIAL_RESTYPES)
    assert bound == set(declared_functions())


def test_header_compiles_as_c():
    import subprocess
    import tempfile
    with tempfile.TemporaryDirectory() as d:
        src = os.path.join(d, "t.c")
        open(src, "w").write('#include "dsx.h"\n#include "dsx_testing.h"\nint main(void) { return DSX_OK; }\n')
        subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), "-c", src, "-o",
                               os.path.join(d, "t.o")])


def test_calls_before_init_fail_loudly(pkg):
    lib = pkg.load_library()
    if lib.dsx_is_initialized():
        pytest.skip("library already initialised in this process")
    p = C.c_void_p()
    rc = lib.dsx_malloc(C.byref(p), 16)
    assert rc == -3 and b"dsx_init" in lib.dsx_last_error()
    assert lib.dsx_topk(None, None, None, 1, 1, 1) == -3
    assert lib.dsx_sync() == -3


def test_missing_library_raises(pkg, monkeypatch):
    monkeypatch.setattr(pkg, "_lib", None)
    monkeypatch.setattr(pkg, "LIB_PATH", "/nonexistent/libdsx_hip.so")
    with pytest.raises(pkg.DsxError):
        pkg.load_library()
