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
DUMP_ASAN = os.path.join(ROOT, "tests", "cpp", "nc_dump_asan")   # the readers built with -fsanitize=address,undefined (make asan)
ASAN_ENV = dict(os.environ, ASAN_OPTIONS="verify_asan_link_order=0:detect_leaks=0:abort_on_error=0", UBSAN_OPTIONS="halt_on_error=1")
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


def run_asan(args, timeout=300):
    assert os.path.exists(DUMP_ASAN), "tests/cpp/nc_dump_asan is missing: run __graft_entry__.build()"
    return subprocess.run([DUMP_ASAN] + args, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=timeout, env=ASAN_ENV)


@pytest.mark.parametrize("fixture", FIXTURES, ids=[os.path.basename(f) for f in FIXTURES])
def test_fixtures_read_cleanly_under_the_sanitizers(fixture):
    r = run_asan([fixture])
    assert r.returncode == 0, r.stderr[-2000:]
    assert "runtime error" not in r.stderr and "AddressSanitizer" not in r.stderr
    assert r.stdout == dump(fixture)[0]


def test_single_byte_damage_under_the_sanitizers(tmp_path):
    """Every byte of the first 1,500 of four fixtures (superblock, root header, the first heaps and indexes) set to four other
    values, one at a time, read by the sanitizer build in one process per fixture: a read or write outside a buffer, a signed
    overflow or a misaligned access ends that process with a report; damage that is merely wrong data or a refused file does not."""
    procs = []
    for name in ("net.earliest.nc", "tied.v18.nc", "tied.plain.nc", "big.earliest.c7.nc"):
        assert os.path.exists(DUMP_ASAN), "tests/cpp/nc_dump_asan is missing: run __graft_entry__.build()"
        procs.append((name, subprocess.Popen([DUMP_ASAN, "--sweep", os.path.join(NC4, name), "0", "1500", str(tmp_path / (name + ".tmp"))],
                                             stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, env=ASAN_ENV)))
    for name, p in procs:
        out, err = p.communicate(timeout=600)
        assert p.returncode == 0, "%s: exit %d\n%s" % (name, p.returncode, err[-3000:])
        assert "copies still read" in out and "runtime error" not in err


def patched(data, at, value_le16):
    b = bytearray(data)
    b[at:at + 2] = int(value_le16).to_bytes(2, "little")
    return bytes(b)


def test_attribute_sizes_beyond_the_message_are_refused(tmp_path):
    """An attribute message whose datatype or dataspace size field points past the end of the message (the cursor used to be
    moved there unchecked and the value copied from outside the block).  Version 1 messages (old-style file): version, reserved,
    name size, datatype size, dataspace size (2 bytes each), name; version 3 (new-style): ... one byte of character set, name."""
    cases = []
    old = open(os.path.join(NC4, "tied.plain.nc"), "rb").read()
    name = b"version\x00"
    pos = old.index(name)
    assert old[pos - 8] == 1 and int.from_bytes(old[pos - 6:pos - 4], "little") == len(name)      # a version 1 attribute message
    for field in (pos - 4, pos - 2):
        for value in (0xFFF8, 0x7FF0, 0x0400):
            cases.append(patched(old, field, value))
    new = open(os.path.join(NC4, "net.v18.nc"), "rb").read()
    pos = new.index(name)
    assert new[pos - 9] == 3 and int.from_bytes(new[pos - 7:pos - 5], "little") == len(name)       # a version 3 attribute message
    for field in (pos - 5, pos - 3):
        for value in (0xFFFF, 0x7FF0, 0x0400):
            cases.append(patched(new, field, value))
    for i, blob in enumerate(cases):
        p = tmp_path / ("attr_%d.nc" % i)
        p.write_bytes(blob)
        r = run_asan([str(p)])
        assert r.returncode == 1 and r.stdout.startswith("error:"), (i, r.returncode, r.stdout[:300], r.stderr[-1500:])
