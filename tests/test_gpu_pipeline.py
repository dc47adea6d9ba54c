"""End-to-end parity on the GPU: sparse input -> FC stack -> filtered top-K through the C ABI vs the CPU oracle."""
import os

import numpy as np
import pytest

from parity import assert_close, assert_topk_parity, assert_units_close

pytestmark = pytest.mark.gpu


def say(msg):
    print("[case] " + msg, flush=True)


def run_and_compare(pkg, dsx, orc, p, position=0, batch=None, filtered=True, guided=False, fallback_rows=0):
    from dsx_support.pipeline import DevicePipeline
    pipe = DevicePipeline(p, dsx, guided=guided)
    pipe.step(position, batch, filtered=filtered)
    keys, idx = pipe.results(batch)
    unit = pipe.output_unit(batch)
    _, ref_unit, _, _ = orc.forward(p, position, batch, filtered=False, want_unit=True, want_topk=False)
    _, _, ref_keys, ref_idx = orc.forward(p, position, batch, filtered=filtered)
    assert_units_close(unit, ref_unit, p, position, "%s output activations" % p.name, max_fallback_rows=fallback_rows)
    ref_scores = ref_unit.copy()
    if filtered:
        b = p.batch if batch is None else batch
        orc.lib().orc_apply_filter(ref_scores.ctypes.data, b, ref_scores.shape[1], 0, position,
                                   p.index.ctypes.data if p.index is not None else None, p.start.ctypes.data, p.end.ctypes.data,
                                   p.sparse_index.ctypes.data, None)
    n = assert_topk_parity(keys, idx, ref_keys, ref_idx, ref_scores, p.name)
    say("%s: top-%d parity ok (%d tie-equivalent index differences)" % (p.name, p.k, n))
    return pipe, keys, idx, unit


def test_cfg1_tiny_vs_oracle_and_golden(pkg, dsx, orc, synth):
    p = synth.config(1)
    _, keys, idx, unit = run_and_compare(pkg, dsx, orc, p)
    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "cfg1_golden.npz"))
    assert_close(unit, g["unit"], "cfg1 output vs fp64 golden", rel=1e-4, abs_floor=1e-3)
    assert np.array_equal(idx, g["idx"])          # the fixture's smallest score gap is 3.8e-5: no near-ties
    assert_close(keys, g["keys"], "cfg1 scores vs golden")


def test_cfg1_unfiltered_and_partial_batch(pkg, dsx, orc, synth):
    p = synth.config(1, batches=3)
    run_and_compare(pkg, dsx, orc, p, position=32, filtered=False)
    run_and_compare(pkg, dsx, orc, p, position=70, batch=26, filtered=True)   # last, short batch (engine/NNNetwork.cpp:1415-1417)


def test_cfg2_catalogue_full_size(pkg, dsx, orc, synth):
    p = synth.config(2)
    say("cfg2 batch nnz = %d" % p.batch_nnz())
    pipe, keys, idx, unit = run_and_compare(pkg, dsx, orc, p)
    # size-independent properties: own inputs never recommended, scores descending, score == activation at the index
    rows = np.arange(p.batch)[:, None]
    assert np.array_equal(unit[rows, idx], keys)
    assert np.all(np.diff(keys, axis=1) <= 0)
    for b in range(p.batch):
        assert not set(idx[b].tolist()) & set(p.sparse_index[int(p.start[b]):int(p.end[b])].tolist())
    # idempotence: a second pass gives bit-identical results
    pipe.step()
    k2, i2 = pipe.results()
    assert np.array_equal(k2.view(np.uint32), keys.view(np.uint32)) and np.array_equal(i2, idx)


def test_cfg3_analog_indexed_reduced_batch(pkg, dsx, orc, synth):
    # configuration 3 at full layer widths (27278 -> 1024 -> 1024 -> 27278, analog values, indexed rows), 512 of the 4096 rows
    p = synth.autoencoder("cfg3-analog-indexed-b512", 1003, 27278, [1024, 1024], 512, 10, 1, 1.0, 144, 1.0, (5, 2000), analog=True,
                          indexed=True)
    # 8 of the 512 rows hold an output that differs from the fp32 oracle's by more than 1e-4 (worst 1.5e-4: small sigmoids behind
    # sums over 1,024 ReLU units, where two fp32 summation orders part); those rows are judged against float64
    run_and_compare(pkg, dsx, orc, p, fallback_rows=8)


def test_cfg4_large_catalogue_reduced(pkg, dsx, orc, synth):
    # configuration 4's shape class (hidden 512, top-100, Zipf 1.1, 1..1000 non-zeros) at 200,000 items and 256 rows
    p = synth.autoencoder("cfg4-large-200k-b256", 1004, 200000, [512], 256, 100, 1, 1.1, 50, 1.0, (1, 1000))
    run_and_compare(pkg, dsx, orc, p)


def test_nonzero_bias_and_odd_widths(pkg, dsx, orc, synth):
    p = synth.autoencoder("odd-widths", 77, 3001, [70, 33], 45, 17, 2, 1.0, 30, 0.8, (0, 200), bias_std=0.5)
    run_and_compare(pkg, dsx, orc, p, position=45)


def test_cfg2_guided_topk_matches_scan_and_oracle(pkg, dsx, orc, synth):
    # the output layer leaves segment maxima and the top-K reads only the segments that can hold a result: same answers
    p = synth.config(2)
    for filtered in (True, False):
        _, k_scan, i_scan, _ = run_and_compare(pkg, dsx, orc, p, filtered=filtered)
        pipe, k_gd, i_gd, unit = run_and_compare(pkg, dsx, orc, p, filtered=filtered, guided=True)
        assert pipe.seg_width.value == 64
        assert np.array_equal(i_gd, i_scan) and np.array_equal(k_gd.view(np.uint32), k_scan.view(np.uint32))
        # the maxima themselves: exact maxima of the stored activations
        sm = pipe.seg_max.numpy()
        N = unit.shape[1]
        pad = np.full((unit.shape[0], sm.shape[1] * 64), -np.inf, dtype=np.float32)
        pad[:, :N] = unit
        assert np.array_equal(sm, pad.reshape(unit.shape[0], -1, 64).max(axis=2))


def test_cfg3_guided_with_saturated_scores(pkg, dsx, orc, synth):
    # 1024-wide hidden layers saturate many sigmoids at 1.0f: whole segments tie at the bound and the guided kernel has to read
    # most of the row; indexed, analog filter rows
    p = synth.autoencoder("cfg3-analog-indexed-b512", 1003, 27278, [1024, 1024], 512, 10, 1, 1.0, 144, 1.0, (5, 2000), analog=True,
                          indexed=True)
    _, k_scan, i_scan, _ = run_and_compare(pkg, dsx, orc, p, fallback_rows=8)     # (the same 8 rows as in the test above)
    _, k_gd, i_gd, _ = run_and_compare(pkg, dsx, orc, p, guided=True, fallback_rows=8)
    assert np.array_equal(i_gd, i_scan) and np.array_equal(k_gd.view(np.uint32), k_scan.view(np.uint32))


def test_every_launch_waited_for_when_dsx_sync_is_set():
    """DSX_SYNC=1 (the reference's SYNCHRONOUS build, engine/GpuTypes.h:147-176): every kernel is waited for right after its
    launch.  A fresh process, because the switch is read by dsx_init; the tiny configuration through every kernel of the path."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = ("import __graft_entry__ as e; e.smoke(); pkg = e.load_package(); "
            "import ctypes as C; lib = pkg.load_library(); print('sync', C.c_int.in_dll(lib, 'dsx_debug_sync_launches').value)")
    r = subprocess.run([sys.executable, "-c", code], cwd=root, env=dict(os.environ, DSX_SYNC="1"), stdout=subprocess.PIPE,
                       stderr=subprocess.STDOUT, text=True, timeout=300)
    assert r.returncode == 0, r.stdout[-3000:]
    assert "smoke ok" in r.stdout
    launches = int(r.stdout.split("sync")[-1].split()[0])
    assert launches >= 3, "DSX_SYNC=1 waited for %d launches" % launches   # sparse layer, output layer, top-K
