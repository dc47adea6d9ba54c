"""The product's NetCDF-4 (HDF5) reader against fixtures written by the HDF5 library itself (tests/golden/nc4, made by
tests/golden/nc4/make_fixtures.py): every fixture must give exactly what its classic original gives, whatever the HDF5
file-format generation (old-style groups and headers, HDF5 1.8's dense storage, the newest superblock) and whatever the storage
layout (contiguous, chunked).  CPU only.

What this pins: the container.  What it cannot pin: a file written by DSSTNE itself (none exists, and neither netCDF-C nor
netcdf-cxx4 is installed); the fixtures follow netCDF-C's published description of how it lays a NetCDF-4 file out."""
import glob
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
NC4 = os.path.join(ROOT, "tests", "golden", "nc4")
DUMP = os.path.join(ROOT, "tests", "cpp", "nc_dump")
HOST = os.path.join(ROOT, "tests", "cpp", "test_host_cpu")
FIXTURES = sorted(f for f in glob.glob(os.path.join(NC4, "*.nc")) if not f.endswith(".classic.nc"))


def dump(path, expect=0):
    r = subprocess.run([DUMP, path], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=60)
    assert r.returncode == expect, (path, r.returncode, r.stdout[-500:], r.stderr[-500:])
    return r.stdout, r.stderr


def test_fixtures_are_there():
    assert os.path.exists(DUMP) and os.path.exists(HOST), "tests/cpp programs are missing: run __graft_entry__.build()"
    assert len(FIXTURES) >= 14
    gens = {os.path.basename(f).split(".")[1] for f in FIXTURES}
    assert gens == {"earliest", "v18", "latest", "plain"}


@pytest.mark.parametrize("fixture", FIXTURES, ids=[os.path.basename(f) for f in FIXTURES])
def test_netcdf4_fixture_reads_like_its_classic_original(fixture):
    original = os.path.join(NC4, os.path.basename(fixture).split(".")[0] + ".classic.nc")
    got, err = dump(fixture)
    want, err0 = dump(original)
    assert "container 4" in err and "container 5" in err0
    assert got == want
    assert got.count("\n") > 5


def test_fixture_generations_differ_on_disk():
    """The three generations really are different containers: superblock versions 0, 2 and 3."""
    def superblock(path):
        with open(path, "rb") as f:
            head = f.read(9)
        assert head[:8] == b"\x89HDF\r\n\x1a\n"
        return head[8]
    assert superblock(os.path.join(NC4, "net.earliest.nc")) == 0
    assert superblock(os.path.join(NC4, "net.v18.nc")) == 2
    assert superblock(os.path.join(NC4, "net.latest.nc")) == 3
    # dense storage is in play: fractal heaps and version 2 B-trees in the 1.8-style file, symbol-table nodes in the old-style one
    new = open(os.path.join(NC4, "tied.v18.nc"), "rb").read()
    old = open(os.path.join(NC4, "tied.plain.nc"), "rb").read()
    assert b"FRHP" in new and b"BTHD" in new and b"BTIN" in new and b"OHDR" in new and b"OCHK" in new
    assert b"SNOD" in old and b"HEAP" in old and b"FRHP" not in old and b"OHDR" not in old
    # the oldest superblock with the new headers and dense storage that tracking creation order brings: what netCDF-C writes since it
    # lowered the format bound
    mid = open(os.path.join(NC4, "tied.earliest.nc"), "rb").read()
    assert b"OHDR" in mid and b"FRHP" in mid and b"SNOD" not in mid
    chunked = open(os.path.join(NC4, "big.earliest.c7.nc"), "rb").read()
    assert chunked.count(b"TREE") > 3      # chunk indexes of 143 chunks: more than one B-tree node per variable


@pytest.mark.parametrize("name", ["net.earliest.nc", "net.v18.nc", "net.latest.nc", "net.earliest.c7.nc", "net.v18.c7.nc", "tied.v18.nc",
                                  "tied.earliest.nc", "tied.plain.nc", "net.plain.c5.nc"])
def test_network_descriptor_from_netcdf4(name):
    """LoadNNNetworkDescriptorNetCDF (the first half of LoadNeuralNetworkNetCDF, engine/NNNetwork.cpp:3761-4057) on a NetCDF-4 file."""
    def descriptor(path):
        r = subprocess.run([HOST, "--dump-network", path], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=60)
        assert r.returncode == 0, r.stdout[-1000:]
        return [l for l in r.stdout.splitlines() if l.startswith(("name=", "layer ", "weight "))]
    got = descriptor(os.path.join(NC4, name))
    want = descriptor(os.path.join(NC4, name.split(".")[0] + ".classic.nc"))
    assert got == want and len(got) >= 3


def test_big_fixture_values():
    """The values themselves, against what make_fixtures.py wrote (same generator, same seed)."""
    rng = np.random.default_rng(2016)
    values = rng.standard_normal(1000).astype(np.float32)
    index = rng.integers(0, 1 << 32, 1000, dtype=np.uint64).astype(np.uint32)
    offsets = np.cumsum(rng.integers(0, 1 << 40, 1000, dtype=np.uint64), dtype=np.uint64)
    out, _ = dump(os.path.join(NC4, "big.v18.c7.nc"))
    lines = {l.split(" ", 2)[1]: l for l in out.splitlines()}
    assert lines["offsets"].split(":")[1].split() == [str(int(v)) for v in offsets]
    assert lines["index"].split(":")[1].split() == [str(int(v)) for v in index]
    assert lines["values"].split(":")[1].split() == ["f%08x" % v for v in values.view(np.uint32)]
    assert lines["aUInt64"].endswith(": %d" % (1 << 63)) and lines["anInt64"].endswith(": %d" % -(1 << 40))
    assert lines["name"] == 'att name text "three long variables"' and lines["empty"] == 'att empty text ""'
    assert lines["emptyDim"] == "dim emptyDim 0" and lines["nothing"].startswith("var nothing type 5 count 0:")


def test_damaged_files_are_refused_not_crashed_on(tmp_path):
    """Truncations and random byte damage: the reader either still reads the file or reports an error; it never crashes, hangs
    or allocates without bound."""
    rng = np.random.default_rng(7)
    for name in ("net.earliest.nc", "tied.v18.nc", "tied.plain.nc", "big.earliest.c7.nc", "big.latest.nc"):
        data = open(os.path.join(NC4, name), "rb").read()
        cases = []
        for cut in (9, 40, 96, 200, 1000, len(data) // 2, len(data) - 1):
            cases.append(data[:cut])
        for _ in range(40):
            b = bytearray(data)
            for _ in range(int(rng.integers(1, 8))):
                at = int(rng.integers(8, min(len(b), 6000)))      # headers, heaps and indexes sit at the front
                b[at] = int(rng.integers(0, 256))
            cases.append(bytes(b))
        for i, blob in enumerate(cases):
            p = tmp_path / ("damaged_%d.nc" % i)
            p.write_bytes(blob)
            r = subprocess.run([DUMP, str(p)], stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=60)
            assert r.returncode in (0, 1), "%s case %d: exit %d %s" % (name, i, r.returncode, r.stderr[-300:])
