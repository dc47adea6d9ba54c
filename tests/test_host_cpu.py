"""Host-side C++ layer without a GPU: the C++ unit-test program, the network-file reader against an independent writer
(scipy's NetCDF module), this build's writer against scipy's reader, and the exported C ABI of libdsstne_amd.so."""
import os
import re
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CPP = os.path.join(ROOT, "tests", "cpp")
EXE = os.path.join(CPP, "test_host_cpu")


def need_exe():
    if not os.path.exists(EXE):
        pytest.fail("%s is missing: run __graft_entry__.build()" % EXE)


def test_cpp_host_unit_tests(tmp_path):
    need_exe()
    r = subprocess.run([EXE, str(tmp_path), os.path.join(ROOT, "tests", "golden", "ldl")], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert r.returncode == 0, r.stdout[-3000:]
    assert "0 failed" in r.stdout


def test_cpp_host_unit_tests_under_the_sanitizers(tmp_path):
    """The same program with the whole host layer compiled with -fsanitize=address,undefined (tests/cpp: make asan)."""
    exe = EXE + "_asan"
    if not os.path.exists(exe):
        pytest.fail("%s is missing: run __graft_entry__.build()" % exe)
    env = dict(os.environ, ASAN_OPTIONS="verify_asan_link_order=0:detect_leaks=0", UBSAN_OPTIONS="halt_on_error=1")
    r = subprocess.run([exe, str(tmp_path), os.path.join(ROOT, "tests", "golden", "ldl")], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                       timeout=600, env=env)
    assert r.returncode == 0, r.stdout[-4000:]
    assert "0 failed" in r.stdout and "runtime error" not in r.stdout and "AddressSanitizer" not in r.stdout


def test_network_reader_against_scipy_writer(tmp_path):
    """A network file written by an independent NetCDF implementation (classic CDF-2, signed attribute types) with the
    reference's attribute and variable names (engine/NNNetwork.cpp:1933-1971, NNLayer.cpp:3447-3500, NNWeight.cpp:853-900)."""
    need_exe()
    from scipy.io import netcdf_file
    rng = np.random.default_rng(3)
    W = rng.standard_normal(5 * 3).astype(np.float32)
    b = rng.standard_normal(3).astype(np.float32)
    path = str(tmp_path / "scipy_net.nc")
    f = netcdf_file(path, "w", version=2)
    f.version = np.float32(0.9)
    f.name = "from-scipy"
    f.kind = np.int32(1)
    f.errorFunction = np.int32(3)
    f.layers = np.int32(2)
    f.weights = np.int32(1)
    for i, (name, kind, nx, act, attr, ds) in enumerate([("Input", 0, 5, 0, 1, "in"), ("Output", 2, 3, 2, 0, "out")]):
        p = "layer%d_" % i
        setattr(f, p + "name", name)
        setattr(f, p + "kind", np.int32(kind))
        setattr(f, p + "type", np.int32(0))
        setattr(f, p + "dataSet", ds)
        for d, v in (("Nx", nx), ("Ny", 1), ("Nz", 1), ("Nw", 1), ("dimensions", 1)):
            setattr(f, p + d, np.int32(v))
        setattr(f, p + "activation", np.int32(act))
        setattr(f, p + "attributes", np.int32(attr))
        setattr(f, p + "sources", np.int32(1 if i else 0))
        if i:
            setattr(f, p + "source0", "Input")
        setattr(f, p + "skips", np.int32(0))
    f.weight0_inputLayer = "Input"
    f.weight0_outputLayer = "Output"
    f.weight0_width = np.int32(3)
    f.weight0_height = np.int32(5)
    f.weight0_length = np.int32(1)
    f.weight0_bShared = np.int32(0)
    f.createDimension("weight0_biasDim", 3)
    f.createDimension("weight0_weightDim", 15)
    f.createVariable("weight0_bias", "f4", ("weight0_biasDim",))[:] = b
    f.createVariable("weight0_weights", "f4", ("weight0_weightDim",))[:] = W
    f.close()
    r = subprocess.run([EXE, "--dump-network", path], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=60)
    assert r.returncode == 0, r.stdout
    out = r.stdout
    assert "name=from-scipy kind=1 errorFunction=3 layers=2 weights=1" in out
    assert "layer Input kind=0 Nx=5 activation=0 attributes=1 dataSet=in sources=0" in out
    assert "layer Output kind=2 Nx=3 activation=2 attributes=0 dataSet=out sources=1" in out
    m = re.search(r"weight Input->Output width=3 height=5 shared=0 nweights=15 wsum=(\S+) bsum=(\S+)", out)
    assert m, out
    assert abs(float(m.group(1)) - float((W.astype(np.float64) * np.arange(1, 16)).sum())) < 1e-5
    assert abs(float(m.group(2)) - float((b.astype(np.float64) * np.arange(1, 4)).sum())) < 1e-5


def test_writer_against_scipy_reader(tmp_path):
    need_exe()
    from scipy.io import netcdf_file
    path = str(tmp_path / "ours.nc")
    r = subprocess.run([EXE, "--write-cdf2", path], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=60)
    assert r.returncode == 0, r.stdout
    f = netcdf_file(path, "r", mmap=False)
    assert f.title == b"written by NcClassic" and int(f.answer) == 42 and float(f.ratio) == 0.375
    assert np.array_equal(f.variables["fv"][:], np.array([1.5, -2.25, 3.0, 1e-3, 7.0], dtype=np.float32))
    assert np.array_equal(f.variables["iv"][:], np.array([-7, 0, 123456789], dtype=np.int32))
    assert np.array_equal(f.variables["dv"][:], np.array([3.141592653589793, -1e100]))
    f.close()


def test_host_library_exports_its_header(pkg):
    import ctypes as C
    text = open(os.path.join(ROOT, "include", "dsstne_capi.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    declared = sorted(set(re.findall(r"\b(dsstne_[a-z0-9_]+)\s*\(", text)))
    assert "dsstne_predict" in declared and "dsstne_knn_search" in declared
    from amazon_dsstne_amd import host_api
    lib = host_api.load_host_library()
    for name in declared:
        assert hasattr(lib, name), "libdsstne_amd.so does not export %s" % name
    assert set(host_api.SIGNATURES) == set(declared)
