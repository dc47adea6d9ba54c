#!/usr/bin/env python3
"""Regenerates the NetCDF-4 fixtures of this directory (TEST INFRASTRUCTURE, run by `make fixtures`).

1. The classic originals: the network and dataset files that the C++ unit-test program tests/cpp/test_host_cpu writes with this
   build's own classic writer (net: a 3-layer network with weights; tied: a network from a JSON definition with 272 attributes;
   analog / boolean: sparse dataset files), plus `small`: a 256 -> 32 -> 256 network file written here with the reference's names
   (the GPU tests predict with it), and `big`: three 1,000-element variables (float, uint32, uint64) and attributes of
   every numeric type, written here as a CDF-5 file straight from the classic format's definition.
2. Each original converted by ./classic_to_nc4, i.e. written by the HDF5 library itself in the layout of the netCDF-C library, in
   several HDF5 file-format generations and storage layouts.

The tests (tests/test_netcdf4.py) read every fixture with the product's own parser and compare with the classic original."""
import os
import shutil
import struct
import subprocess
import sys
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(os.path.dirname(HERE)))

NC_TYPES = {np.dtype(np.int8): 1, np.dtype(np.int16): 3, np.dtype(np.int32): 4, np.dtype(np.float32): 5, np.dtype(np.float64): 6,
            np.dtype(np.uint8): 7, np.dtype(np.uint16): 8, np.dtype(np.uint32): 9, np.dtype(np.int64): 10, np.dtype(np.uint64): 11}


def write_cdf5(path, dims, atts, variables):
    """dims: [(name, length)], atts: [(name, str or numpy array)], variables: [(name, dim index, numpy array)]."""
    def name(s):
        b = s.encode()
        return struct.pack(">Q", len(b)) + b + b"\0" * ((4 - len(b) % 4) % 4)

    def values(a):
        b = a.astype(a.dtype.newbyteorder(">")).tobytes()
        return b + b"\0" * ((4 - len(b) % 4) % 4)

    def header(begins):
        h = b"CDF\x05" + struct.pack(">Q", 0)
        h += struct.pack(">IQ", 0x0A, len(dims)) + b"".join(name(n) + struct.pack(">Q", l) for n, l in dims)
        h += struct.pack(">IQ", 0x0C, len(atts))
        for n, v in atts:
            if isinstance(v, str):
                b = v.encode()
                h += name(n) + struct.pack(">IQ", 2, len(b)) + b + b"\0" * ((4 - len(b) % 4) % 4)
            else:
                v = np.atleast_1d(v)
                h += name(n) + struct.pack(">IQ", NC_TYPES[v.dtype], v.size) + values(v)
        h += struct.pack(">IQ", 0x0B, len(variables))
        for (n, d, a), begin in zip(variables, begins):
            vsize = (a.nbytes + 3) // 4 * 4
            h += name(n) + struct.pack(">QQ", 1, d) + struct.pack(">IQ", 0, 0) + struct.pack(">IQQ", NC_TYPES[a.dtype], vsize, begin)
        return h
    begins = [0] * len(variables)
    pos = len(header(begins))
    for i, (_, _, a) in enumerate(variables):
        begins[i] = pos
        pos += (a.nbytes + 3) // 4 * 4
    with open(path, "wb") as f:
        f.write(header(begins))
        for _, _, a in variables:
            f.write(values(a))


def small_network():
    """The network of the `small` fixtures: 256 sparse inputs -> 32 ReLU -> 256 sigmoid, weights from tests/dsx_support/synth.py
    (seed 4242), so that a test can rebuild the same problem and ask the oracle what the network must predict."""
    sys.path.insert(0, ROOT)
    import __graft_entry__ as entry
    entry.load_package()
    from dsx_support import synth
    return synth.autoencoder("small-nc4", 4242, 256, [32], 16, 5, 1, 1.0, 12, 0.5, (1, 40), bias_std=0.3)


def write_small_network(path):
    """A network file with the reference's attribute and variable names (engine/NNNetwork.cpp:1933-1971, engine/NNLayer.cpp:3447-3500,
    engine/NNWeight.cpp:853-900), CDF-5 container."""
    p = small_network()
    u = np.uint32
    atts = [("version", np.float32(0.9)), ("name", p.name), ("kind", u(1)), ("errorFunction", u(3)), ("layers", u(3)), ("weights", u(2))]
    layers = [("Input", 0, 256, 3, 1, "input", []), ("Hidden", 1, 32, 2, 0, "", ["Input"]), ("Output", 2, 256, 0, 0, "output", ["Hidden"])]
    for i, (name, kind, nx, act, attr, ds, sources) in enumerate(layers):
        q = "layer%d_" % i
        atts += [(q + "name", name), (q + "kind", u(kind)), (q + "type", u(0)), (q + "dataSet", ds), (q + "Nx", u(nx)), (q + "Ny", u(1)),
                 (q + "Nz", u(1)), (q + "Nw", u(1)), (q + "dimensions", u(1)), (q + "activation", u(act)), (q + "attributes", u(attr)),
                 (q + "sources", u(len(sources)))]
        atts += [(q + "source%d" % j, s) for j, s in enumerate(sources)]
        atts += [(q + "skips", u(0))]
    dims, variables = [], []
    for i, (a, b) in enumerate([("Input", "Hidden"), ("Hidden", "Output")]):
        q = "weight%d_" % i
        W, bias = p.weights[i], p.biases[i]
        atts += [(q + "inputLayer", a), (q + "outputLayer", b), (q + "width", np.uint64(W.shape[1])), (q + "height", np.uint64(W.shape[0])),
                 (q + "length", np.uint64(1)), (q + "bShared", u(0))]
        dims += [(q + "biasDim", bias.size), (q + "weightDim", W.size)]
        variables += [(q + "bias", 2 * i, bias), (q + "weights", 2 * i + 1, W.reshape(-1))]
    write_cdf5(path, dims, atts, variables)


def main():
    tool = os.path.join(HERE, "classic_to_nc4")
    exe = os.path.join(ROOT, "tests", "cpp", "test_host_cpu")
    if not os.path.exists(tool) or not os.path.exists(exe):
        sys.exit("build ./classic_to_nc4 (make) and tests/cpp/test_host_cpu first")
    for old in os.listdir(HERE):
        if old.endswith(".nc"):
            os.remove(os.path.join(HERE, old))
    with tempfile.TemporaryDirectory() as tmp:
        subprocess.run([exe, tmp, os.path.join(ROOT, "tests", "golden", "ldl")], check=True, stdout=subprocess.DEVNULL)
        for n in ("net", "tied", "analog", "boolean"):
            shutil.copy(os.path.join(tmp, n + ".nc"), os.path.join(HERE, n + ".classic.nc"))
    write_small_network(os.path.join(HERE, "small.classic.nc"))
    rng = np.random.default_rng(2016)
    write_cdf5(os.path.join(HERE, "big.classic.nc"),
               [("floatDim", 1000), ("indexDim", 1000), ("offsetDim", 1000), ("emptyDim", 0)],
               [("name", "three long variables"), ("empty", ""), ("aByte", np.int8(-7)), ("aShort", np.int16(-12345)), ("anInt", np.int32(-7 << 20)),
                ("aFloat", np.float32(0.1)), ("aDouble", np.float64(1.0) / 3), ("aUByte", np.uint8(250)), ("aUShort", np.uint16(65000)),
                ("aUInt", np.uint32(4000000000)), ("anInt64", np.int64(-1) << 40), ("aUInt64", np.uint64(1) << np.uint64(63)),
                ("several", np.arange(5, dtype=np.float32) * np.float32(1.5)), ("pair", np.array([1, 1 << 40], dtype=np.uint64))],
               [("values", 0, rng.standard_normal(1000).astype(np.float32)),
                ("index", 1, rng.integers(0, 1 << 32, 1000, dtype=np.uint64).astype(np.uint32)),
                ("offsets", 2, np.cumsum(rng.integers(0, 1 << 40, 1000, dtype=np.uint64), dtype=np.uint64)),
                ("nothing", 3, np.zeros(0, dtype=np.float32))])
    # (original, HDF5 generation, chunk elements or 0 for contiguous storage)
    plan = [("net", "earliest", 0), ("net", "v18", 0), ("net", "latest", 0), ("net", "earliest", 7), ("net", "v18", 7),
            ("tied", "v18", 0), ("tied", "earliest", 0), ("tied", "plain", 0), ("net", "plain", 5),
            ("analog", "earliest", 0), ("analog", "v18", 0), ("boolean", "v18", 2),
            ("small", "earliest", 0), ("small", "v18", 1000),
            ("big", "earliest", 7), ("big", "v18", 7), ("big", "latest", 0), ("big", "earliest", 0)]
    for name, gen, chunk in plan:
        out = os.path.join(HERE, "%s.%s%s.nc" % (name, gen, (".c%d" % chunk) if chunk else ""))
        cmd = [tool, os.path.join(HERE, name + ".classic.nc"), out, gen] + ([str(chunk)] if chunk else [])
        subprocess.run(cmd, check=True)
        print("%-28s %7d bytes" % (os.path.basename(out), os.path.getsize(out)))


if __name__ == "__main__":
    main()
