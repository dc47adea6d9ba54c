"""The C++ inference classes (NNNetwork, NNDataSet<T>, DsstneContext, KnnExactGpu) on the GPU, driven through their
C ABI and through C++ programs that mirror the reference's own tests and its native embedding example."""
import os
import subprocess

import numpy as np
import pytest

from parity import assert_close, assert_topk_parity, assert_units_close

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CPP = os.path.join(ROOT, "tests", "cpp")


def say(msg):
    print("[case] " + msg, flush=True)


def run_exe(name, *args, timeout=300):
    exe = os.path.join(CPP, name)
    if not os.path.exists(exe):
        pytest.fail("%s is missing: run __graft_entry__.build()" % exe)
    r = subprocess.run([exe] + [str(a) for a in args], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=timeout)
    return r.returncode, r.stdout


def test_reference_dataset_and_buffer_unit_tests():
    """tst/amazon/dsstne/engine/TestNNDataSet.cpp and TestGpuBuffer.cpp, re-typed against this build's headers."""
    rc, out = run_exe("test_dataset_gpu")
    assert rc == 0 and "0 failed" in out, out[-3000:]


def host_forward(pkg, dsx, orc, p, filtered=True, boolean=None, position=0):
    from amazon_dsstne_amd import host_api
    net = host_api.Network(p, max_k=p.k)
    try:
        net.bind_input(boolean=boolean)
        net.predict_batch(position)
        rows = min(p.batch, p.examples - position)
        net.topk(p.k, filter_dataset="input" if filtered else None)
        keys, idx = net.get_topk(rows)
        unit = net.units(rows=p.batch)[:rows]
    finally:
        net.close()
    _, ref_unit, _, _ = orc.forward(p, position, rows, filtered=False, want_unit=True, want_topk=False)
    _, _, ref_keys, ref_idx = orc.forward(p, position, rows, filtered=filtered)
    assert_units_close(unit, ref_unit, p, position, p.name + " units via NNNetwork")
    ref_scores = ref_unit.copy()
    if filtered:
        orc.lib().orc_apply_filter(ref_scores.ctypes.data, rows, ref_scores.shape[1], 0, position,
                                   p.index.ctypes.data if p.index is not None else None, p.start.ctypes.data, p.end.ctypes.data,
                                   p.sparse_index.ctypes.data, None)
    n = assert_topk_parity(keys, idx, ref_keys, ref_idx, ref_scores, p.name + " via NNNetwork")
    say("%s through NNNetwork::PredictBatch: parity ok (%d tie-equivalent)" % (p.name, n))


def test_network_api_cfg1(pkg, dsx, orc, synth):
    host_forward(pkg, dsx, orc, synth.config(1), filtered=True)
    host_forward(pkg, dsx, orc, synth.config(1), filtered=False)


def test_network_api_public_constructor_data_runs_analog_kernel(pkg, dsx, orc, synth):
    # 0/1 data fed through the public API is Sparse but not Boolean and runs the analog kernel with values 1
    # (engine/NNTypes.cpp:501-524, dispatch engine/NNTypes.h:527-545); the result must equal the Boolean path's.
    host_forward(pkg, dsx, orc, synth.config(1), filtered=True, boolean=False)


def test_network_api_cfg2_full(pkg, dsx, orc, synth):
    # output layer of 27,278 units: the forward pass leaves segment maxima and both top-K calls are the guided ones
    host_forward(pkg, dsx, orc, synth.config(2), filtered=True)
    host_forward(pkg, dsx, orc, synth.config(2), filtered=False)


def test_topk_after_units_were_overwritten(pkg, dsx, orc, synth):
    # the segment maxima of the forward pass must not outlive the units they describe
    from amazon_dsstne_amd import host_api
    p = synth.config(2)
    rng = np.random.default_rng(3)
    fresh = rng.random((p.batch, p.widths[-1]), dtype=np.float32)
    net = host_api.Network(p, max_k=p.k)
    try:
        net.bind_input()
        net.predict_batch(0)
        net.set_units(fresh)
        net.topk(p.k, filter_dataset=None)
        keys, idx = net.get_topk(p.batch)
        net.topk(p.k, filter_dataset="input")
        fkeys, fidx = net.get_topk(p.batch)
    finally:
        net.close()
    rk, ri = orc.topk(fresh, p.k)
    assert np.array_equal(idx, ri) and np.array_equal(keys.view(np.uint32), rk.view(np.uint32))
    rk, ri = orc.topk_filtered(fresh, p.k, 0, None, p.start, p.end, p.sparse_index, None)
    assert np.array_equal(fidx, ri) and np.array_equal(fkeys.view(np.uint32), rk.view(np.uint32))


def test_network_api_positions_and_short_last_batch(pkg, dsx, orc, synth):
    p = synth.autoencoder("three-batches", 21, 2000, [96], 64, 12, batches=3, zipf_s=1.0, nnz_mean=25, nnz_sigma=0.8, nnz_clip=(0, 300),
                          bias_std=0.2)
    p.examples -= 20            # 172 rows: the last batch is short (engine/NNNetwork.cpp:1415-1417)
    p.unique_examples -= 20
    p.start, p.end = p.start[:172], p.end[:172]
    host_forward(pkg, dsx, orc, p, position=64)
    host_forward(pkg, dsx, orc, p, position=128)


def test_network_api_analog_indexed(pkg, dsx, orc, synth):
    p = synth.autoencoder("analog-indexed-small", 1003, 27278, [256, 256], 128, 10, 1, 1.0, 144, 1.0, (5, 2000), analog=True, indexed=True)
    host_forward(pkg, dsx, orc, p)


def test_native_embedding_example(pkg, dsx, orc, synth, tmp_path):
    """java/src/test/native/main.cpp flow in C++: network file -> DsstneContext -> descriptors -> LoadSparseData ->
    PredictBatch -> kCalculateTopK; compared with the oracle's unfiltered top-K."""
    from amazon_dsstne_amd import host_api
    p = synth.config(1)
    net = host_api.Network(p)
    netfile = str(tmp_path / "cfg1.nc")
    net.save(netfile)
    net.close()
    inputs = tmp_path / "inputs.txt"
    with open(inputs, "w") as f:
        for r in range(p.batch):
            f.write(" ".join(str(int(i)) for i in p.sparse_index[int(p.start[r]):int(p.end[r])]) + "\n")
    rc, out = run_exe("predict_main", netfile, inputs, p.batch, p.k)
    assert rc == 0, out[-3000:]
    rows = [l for l in out.splitlines() if l and l[0].isdigit() and "\t" in l]
    assert len(rows) == p.batch, out[-2000:]
    idx = np.zeros((p.batch, p.k), dtype=np.uint32)
    keys = np.zeros((p.batch, p.k), dtype=np.float32)
    for r, line in enumerate(rows):
        cells = [c for c in line.split("\t")[1].split(",") if c]
        for j, c in enumerate(cells):
            i, s = c.split(":")
            idx[r, j], keys[r, j] = int(i), float(s)
    _, ref_unit, ref_keys, ref_idx = orc.forward(p, filtered=False, want_unit=True)
    assert_topk_parity(keys, idx, ref_keys, ref_idx, ref_unit, "native embedding example")


def test_predict_tool_end_to_end(pkg, dsx, orc, synth, tmp_path):
    """utils/Predict.cpp's flow with the reference's flags: index files + samples text -> dataset file -> network file ->
    batches of PredictBatch + NNRecsGenerator::generateRecs (top-5K on the device with the samples filter, K written)."""
    from amazon_dsstne_amd import host_api
    exe = os.path.join(ROOT, "amazon-dsstne_amd", "predict")
    if not os.path.exists(exe):
        pytest.fail("%s is missing: run __graft_entry__.build()" % exe)
    p = synth.config(1, batches=3)          # 96 samples, batch 32, 1024 items, top-10
    p.examples -= 7                          # 89 samples: the last batch is short
    p.unique_examples -= 7
    p.start, p.end = p.start[:89], p.end[:89]
    net = host_api.Network(p, dataset="gl_input")
    netfile = str(tmp_path / "net.nc")
    net.save(netfile)
    net.close()
    N = p.widths[0]
    with open(tmp_path / "in.idx", "w") as f:
        for i in range(N):
            f.write("item%d\t%d\n" % (i, i))
    with open(tmp_path / "out.idx", "w") as f:
        for i in reversed(range(N)):       # order of the lines does not matter
            f.write("item%d\t%d\n" % (i, i))
    rows = []
    for r in range(p.examples):
        cols = p.sparse_index[int(p.start[r]):int(p.end[r])]
        rows.append("user%d\t" % r + ":".join("item%d,1" % c for c in cols))
    (tmp_path / "samples.txt").write_text("\n".join(rows) + "\n")
    # the filter file lists every sample's own items with multiplier 0 (no value given)
    with open(tmp_path / "filter.txt", "w") as f:
        for r in range(p.examples):
            cols = p.sparse_index[int(p.start[r]):int(p.end[r])]
            f.write("user%d\t" % r + ":".join("item%d" % c for c in cols) + "\n")
    recs = tmp_path / "recs.txt"
    r = subprocess.run([exe, "-d", "gl", "-n", netfile, "-r", str(tmp_path / "samples.txt"), "-i", str(tmp_path / "in.idx"), "-o",
                        str(tmp_path / "out.idx"), "-f", str(tmp_path / "filter.txt"), "-s", str(recs), "-k", str(p.k), "-b", str(p.batch),
                        "-p", "8.6f"], cwd=str(tmp_path), stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    assert r.returncode == 0, r.stdout[-3000:]
    lines = recs.read_text().splitlines()
    assert len(lines) == p.examples, r.stdout[-2000:]
    idx = np.zeros((p.examples, p.k), dtype=np.uint32)
    keys = np.zeros((p.examples, p.k), dtype=np.float32)
    for n, line in enumerate(lines):
        who, cells = line.split("\t")
        assert who == "user%d" % n
        cells = [c for c in cells.split(":") if c]
        assert len(cells) == p.k
        for j, c in enumerate(cells):
            name, score = c.split(",")
            idx[n, j], keys[n, j] = int(name[4:]), float(score)
    ref_keys = np.zeros_like(keys)
    ref_idx = np.zeros_like(idx)
    ref_scores = np.zeros((p.examples, N), dtype=np.float32)
    for pos in range(0, p.examples, p.batch):
        rows_here = min(p.batch, p.examples - pos)
        _, u, _, _ = orc.forward(p, pos, rows_here, filtered=False, want_unit=True, want_topk=False)
        _, _, k_, i_ = orc.forward(p, pos, rows_here, filtered=True)
        orc.lib().orc_apply_filter(u.ctypes.data, rows_here, N, 0, pos, None, p.start.ctypes.data, p.end.ctypes.data,
                                   p.sparse_index.ctypes.data, None)
        ref_keys[pos:pos + rows_here], ref_idx[pos:pos + rows_here], ref_scores[pos:pos + rows_here] = k_, i_, u
    mism = idx != ref_idx
    if mism.any():
        rws, cls = np.nonzero(mism)
        gap = np.abs(ref_scores[rws, idx[rws, cls]].astype(np.float64) - ref_keys[rws, cls].astype(np.float64))
        assert gap.max() < 1e-5
    assert np.allclose(keys, ref_keys, rtol=1e-4, atol=2e-6)        # printed with six decimals


def test_soft_errors_do_not_abort(pkg, dsx, synth, capfd):
    from amazon_dsstne_amd import host_api
    p = synth.config(1)
    net = host_api.Network(p, max_k=20)
    try:
        net.bind_input()
        lib = net.lib
        # SetPosition out of range: message, position unchanged (engine/NNNetwork.cpp:732-745); prediction still works
        assert lib.dsstne_predict_batch(net.ctx, 10_000) == 0
        # k above the context's maxK is refused
        assert lib.dsstne_topk(net.ctx, b"Output", 21, None) != 0
        assert b"maxK" in lib.dsstne_last_error()
        assert lib.dsstne_topk(net.ctx, b"NoSuchLayer", 5, None) != 0
        assert lib.dsstne_get_units(net.ctx, b"Input", None, 1) != 0      # a fast-sparse input layer has no unit buffer
        assert lib.dsstne_load_sparse_data(net.ctx, b"nope", None, None, None, None) != 0
        # loader exceptions surface as error codes: start[0] != 0, and more non-zeros than the dataset can hold
        s = np.ones(p.examples, dtype=np.uint64)
        e = np.full(p.examples, 2, dtype=np.uint64)
        i = np.zeros(4, dtype=np.uint32)
        assert lib.dsstne_load_sparse_data(net.ctx, b"input", s.ctypes.data, e.ctypes.data, None, i.ctypes.data) != 0
        assert b"zero indexed" in lib.dsstne_last_error()
        s[:] = 0
        e[:] = 10_000_000
        assert lib.dsstne_load_sparse_data(net.ctx, b"input", s.ctypes.data, e.ctypes.data, None, i.ctypes.data) != 0
        assert b"Not enough space" in lib.dsstne_last_error()
    finally:
        net.close()
    assert "Invalid position setting" in capfd.readouterr().out


def test_knn_api(pkg, dsx, orc, synth, tmp_path):
    import ctypes as C
    from amazon_dsstne_amd import host_api
    lib = host_api.load_host_library()
    p = synth.knn_config(seed=5, items=20011, queries=37, dim=48, k=20)
    knn = lib.dsstne_knn_create(64, 32)
    assert knn
    try:
        items = np.ascontiguousarray(p.items)
        assert lib.dsstne_knn_load(knn, items.ctypes.data, items.shape[0], items.shape[1], None) == 0, lib.dsstne_last_error()
        scores = np.empty((37, 20), dtype=np.float32)
        idx = np.empty((37, 20), dtype=np.uint32)
        q = np.ascontiguousarray(p.queries)
        assert lib.dsstne_knn_search(knn, 20, q.ctypes.data, 37, scores.ctypes.data, idx.ctypes.data) == 0, lib.dsstne_last_error()
        full = p.queries.astype(np.float64) @ p.items.astype(np.float64).T
        order = np.argsort(-full, axis=1, kind="stable")[:, :20]
        mism = idx != order
        if mism.any():
            r, c = np.nonzero(mism)
            assert np.abs(full[r, idx[r, c]] - full[r, order[r, c]]).max() < 1e-5
        assert_close(scores, np.take_along_axis(full, idx.astype(np.int64), axis=1), "knn scores", rel=1e-4, abs_floor=0.05)
        g, t = C.c_float(), C.c_float()
        lib.dsstne_knn_elapsed(knn, C.byref(g), C.byref(t))
        assert g.value > 0 and t.value > 0
        # k > maxK -> std::invalid_argument (knn/KnnExactGpu.cu:49-54); size > batch likewise
        assert lib.dsstne_knn_search(knn, 33, q.ctypes.data, 37, scores.ctypes.data, idx.ctypes.data) != 0
        assert b"maxK" in lib.dsstne_last_error()
        assert lib.dsstne_knn_search(knn, 20, q.ctypes.data, 65, scores.ctypes.data, idx.ctypes.data) != 0
        # text-file loading: keys are labels, results come back in load order
        path = tmp_path / "items.txt"
        with open(path, "w") as f:
            for i in range(50):
                f.write("item%d\t%s\n" % (i, " ".join("%.8g" % v for v in p.items[i])))
        assert lib.dsstne_knn_load_file(knn, str(path).encode(), b"\t", b" ") == 0, lib.dsstne_last_error()
        s2 = np.empty((5, 3), dtype=np.float32)
        i2 = np.empty((5, 3), dtype=np.uint32)
        q2 = np.ascontiguousarray(p.items[:5])
        assert lib.dsstne_knn_search(knn, 3, q2.ctypes.data, 5, s2.ctypes.data, i2.ctypes.data) == 0, lib.dsstne_last_error()
        assert i2[:, 0].tolist() == [0, 1, 2, 3, 4] and np.allclose(s2[:, 0], 1.0, atol=1e-5)
    finally:
        lib.dsstne_knn_destroy(knn)


def test_knn_api_split_products(pkg, dsx, orc, synth):
    """KnnData(…, DataType::FP32Split): the fp32 table as bf16 planes, scores as exact as fp32 storage gives them."""
    from amazon_dsstne_amd import host_api
    lib = host_api.load_host_library()
    p = synth.knn_config(seed=7, items=23456, queries=50, dim=72, k=24)
    knn = lib.dsstne_knn_create_typed(64, 32, b"fp32-split")
    assert knn, lib.dsstne_last_error()
    try:
        items = np.ascontiguousarray(p.items)
        assert lib.dsstne_knn_load(knn, items.ctypes.data, items.shape[0], items.shape[1], None) == 0, lib.dsstne_last_error()
        scores = np.empty((50, 24), dtype=np.float32)
        idx = np.empty((50, 24), dtype=np.uint32)
        q = np.ascontiguousarray(p.queries)
        assert lib.dsstne_knn_search(knn, 24, q.ctypes.data, 50, scores.ctypes.data, idx.ctypes.data) == 0, lib.dsstne_last_error()
        full = p.queries.astype(np.float64) @ p.items.astype(np.float64).T
        order = np.argsort(-full, axis=1, kind="stable")[:, :24]
        mism = idx != order
        if mism.any():
            r, c = np.nonzero(mism)
            assert np.abs(full[r, idx[r, c]] - full[r, order[r, c]]).max() < 1e-5
        # fp32 accuracy: unit vectors, so the scores are within a few fp32 roundings of the exact ones
        assert np.abs(scores - np.take_along_axis(full, idx.astype(np.int64), axis=1)).max() < 2e-6
    finally:
        lib.dsstne_knn_destroy(knn)


def test_knn_api_fp16_storage(pkg, dsx, orc, synth):
    """KnnData(…, DataType::FP16) + KnnExactGpu::search: table and queries rounded to fp16, fp32 scores (knn/KnnData.cpp:209-216,
    knn/KnnExactGpu.cu:108-116); a partial batch (size < batchSize) as the JNI passes it."""
    from amazon_dsstne_amd import host_api
    lib = host_api.load_host_library()
    p = synth.knn_config(seed=6, items=12345, queries=21, dim=40, k=16)
    assert not lib.dsstne_knn_create_typed(64, 32, b"fp8")
    assert b"Unknown DataType" in lib.dsstne_last_error()
    knn = lib.dsstne_knn_create_typed(64, 32, b"fp16")
    assert knn, lib.dsstne_last_error()
    try:
        items = np.ascontiguousarray(p.items)
        assert lib.dsstne_knn_load(knn, items.ctypes.data, items.shape[0], items.shape[1], None) == 0, lib.dsstne_last_error()
        scores = np.empty((21, 16), dtype=np.float32)
        idx = np.empty((21, 16), dtype=np.uint32)
        q = np.ascontiguousarray(p.queries)
        assert lib.dsstne_knn_search(knn, 16, q.ctypes.data, 21, scores.ctypes.data, idx.ctypes.data) == 0, lib.dsstne_last_error()
        it16 = p.items.astype(np.float16).astype(np.float64)
        q16 = p.queries.astype(np.float16).astype(np.float64)
        full = q16 @ it16.T
        order = np.argsort(-full, axis=1, kind="stable")[:, :16]
        mism = idx != order
        if mism.any():
            r, c = np.nonzero(mism)
            assert np.abs(full[r, idx[r, c]] - full[r, order[r, c]]).max() < 1e-5
        assert_close(scores, np.take_along_axis(full, idx.astype(np.int64), axis=1), "knn fp16 scores", rel=1e-4, abs_floor=0.05)
        # the rounding is visible: against the unrounded operands the scores are off by more than fp32 summation explains
        exact = p.queries.astype(np.float64) @ p.items.astype(np.float64).T
        assert np.abs(scores - np.take_along_axis(exact, idx.astype(np.int64), axis=1)).max() > 1e-5
    finally:
        lib.dsstne_knn_destroy(knn)


def reference_batches(orc, p, positions):
    out = []
    for pos in positions:
        rows = min(p.batch, p.examples - pos)
        _, unit, _, _ = orc.forward(p, pos, rows, filtered=False, want_unit=True, want_topk=False)
        _, _, keys, idx = orc.forward(p, pos, rows, filtered=True)
        scores = unit.copy()
        orc.lib().orc_apply_filter(scores.ctypes.data, rows, scores.shape[1], 0, pos, None, p.start.ctypes.data, p.end.ctypes.data,
                                   p.sparse_index.ctypes.data, None)
        out.append((rows, keys, idx, scores))
    return out


@pytest.mark.parametrize("config,batches,lanes", [(1, 9, 2), (2, 4, 2), (1, 5, 1), (1, 40, 2), (1, 11, 3), (2, 6, 4), (1, 40, 4)])
def test_streamed_batches_on_two_lanes(pkg, dsx, orc, synth, config, batches, lanes):
    """Batches handed over as host arrays one after the other (NNDataSet::LoadSparseData, as the reference's JNI predict feeds
    it): the dataset holds one batch, every load replaces it, and the results of batch i are collected while batch i + 1 is
    already queued.  The loads go to the set of device arrays of the lane the batch will run on, lane after lane in turn; every
    batch must still see its own data, as input and as filter."""
    import copy
    from amazon_dsstne_amd import host_api
    big = synth.config(config, batches=batches)
    positions = list(range(0, big.examples, big.batch))
    want = reference_batches(orc, big, positions)

    def batch_arrays(pos):
        s, e = big.start[pos:pos + big.batch], big.end[pos:pos + big.batch]
        lo, hi = int(s[0]), int(e[-1])
        data = None if big.sparse_data is None else np.ascontiguousarray(big.sparse_data[lo:hi])
        return (np.ascontiguousarray(s - lo), np.ascontiguousarray(e - lo), data, np.ascontiguousarray(big.sparse_index[lo:hi]))

    one = copy.copy(big)                      # a dataset of one batch with room for the largest of them
    one.examples = one.unique_examples = big.batch
    room = max(int(big.end[pos + big.batch - 1] - big.start[pos]) for pos in positions)
    one.start, one.end = np.zeros(big.batch, np.uint64), np.zeros(big.batch, np.uint64)
    one.sparse_index = np.zeros(room, np.uint32)
    one.sparse_data = None if big.sparse_data is None else np.zeros(room, big.sparse_data.dtype)
    net = host_api.Network(one, max_k=big.k)
    try:
        net.bind_input()
        if lanes != 2:
            net.set_lanes(lanes)
        got = []
        for n, pos in enumerate(positions):
            net.load_sparse(*batch_arrays(pos))
            net.predict_batch(0)
            net.topk(big.k, filter_dataset="input")
            if lanes >= 2 and n > 0:
                got.append(net.get_topk_previous(big.batch))            # the batch before, while this one runs
            elif lanes == 1:
                got.append(net.get_topk(big.batch))
        if lanes >= 2:
            got.append(net.get_topk(big.batch))
        for n, ((rows, keys, idx, scores), (gk, gi)) in enumerate(zip(want, got)):
            assert_topk_parity(gk, gi, keys, idx, scores, "%s streamed batch %d on %d lane(s)" % (big.name, n, lanes))
        # the same data predicted twice after one load (the second batch runs on the lane that did not take the upload),
        # and two loads in a row (the second finds the lane guess of the first unused)
        net.load_sparse(*batch_arrays(positions[1]))
        for rep in range(2):
            net.predict_batch(0)
            net.topk(big.k, filter_dataset="input")
        gk, gi = net.get_topk(big.batch)
        assert_topk_parity(gk, gi, want[1][1], want[1][2], want[1][3], big.name + " second predict after one load")
        net.load_sparse(*batch_arrays(positions[2]))
        net.load_sparse(*batch_arrays(positions[0]))
        net.predict_batch(0)
        net.topk(big.k, filter_dataset="input")
        gk, gi = net.get_topk(big.batch)
        assert_topk_parity(gk, gi, want[0][1], want[0][2], want[0][3], big.name + " after two loads in a row")
    finally:
        net.close()


@pytest.mark.parametrize("config,batches,lanes", [(1, 7, 2), (2, 3, 2), (1, 9, 3), (2, 5, 4), (1, 7, 4)])
def test_two_lanes_keep_batches_apart(pkg, dsx, orc, synth, config, batches, lanes):
    """Consecutive PredictBatch calls take turns on the sets of buffers and streams of two to four lanes (NNNetwork::SetLanes).
    A loop that issues batch i+1 before it collects batch i must get every batch's own results; the last batch is short."""
    from amazon_dsstne_amd import host_api
    p = synth.config(config, batches=batches)
    short = p.batch // 3
    p.examples -= short
    p.unique_examples -= short
    p.start, p.end = p.start[:p.examples], p.end[:p.examples]
    positions = list(range(0, p.examples, p.batch))
    want = reference_batches(orc, p, positions)
    net = host_api.Network(p, max_k=p.k)
    try:
        net.bind_input()
        if lanes != 2:
            net.set_lanes(lanes)
        got = []
        for n, pos in enumerate(positions):
            net.predict_batch(pos)
            net.topk(p.k, filter_dataset="input")
            if n > 0:
                got.append(net.get_topk_previous(want[n - 1][0]))       # the batch before, while this one runs
        got.append(net.get_topk(want[-1][0]))
        for n, ((rows, keys, idx, scores), (gk, gi)) in enumerate(zip(want, got)):
            assert_topk_parity(gk, gi, keys, idx, scores, "%s batch %d on two lanes" % (p.name, n))
        # many batches in flight without reading anything back, then the last two
        for rep in range(3):
            for pos in positions:
                net.predict_batch(pos)
                net.topk(p.k, filter_dataset="input")
        gk, gi = net.get_topk(want[-1][0])
        assert_topk_parity(gk, gi, want[-1][1], want[-1][2], want[-1][3], p.name + " last batch after a run")
        gk, gi = net.get_topk_previous(want[-2][0])
        assert_topk_parity(gk, gi, want[-2][1], want[-2][2], want[-2][3], p.name + " batch before the last after a run")
        # units of the current batch, and a new input upload between batches (orders both lanes)
        net.predict_batch(positions[1])
        unit = net.units(rows=p.batch)
        _, ref_unit, _, _ = orc.forward(p, positions[1], p.batch, filtered=False, want_unit=True, want_topk=False)
        assert_units_close(unit, ref_unit, p, positions[1], p.name + " units on several lanes")
        net.load_sparse(p.start, p.end, p.sparse_data, p.sparse_index)
        net.predict_batch(positions[0])
        net.topk(p.k, filter_dataset="input")
        gk, gi = net.get_topk(want[0][0])
        assert_topk_parity(gk, gi, want[0][1], want[0][2], want[0][3], p.name + " after a reload")
        # one lane: the reference's single set of buffers
        net.set_lanes(1)
        with pytest.raises(host_api.DsxError):
            net.get_topk_previous(1)
        for n, pos in enumerate(positions[:2]):
            net.predict_batch(pos)
            net.topk(p.k, filter_dataset="input")
            gk, gi = net.get_topk(want[n][0])
            assert_topk_parity(gk, gi, want[n][1], want[n][2], want[n][3], "%s batch %d on one lane" % (p.name, n))
        net.set_lanes(lanes)
        for n, pos in enumerate(positions[:3]):
            net.predict_batch(pos)
            net.topk(p.k, filter_dataset="input")
        gk, gi = net.get_topk(want[2][0])
        assert_topk_parity(gk, gi, want[2][1], want[2][2], want[2][3], p.name + " back on %d lanes" % lanes)
        gk, gi = net.get_topk_previous(want[1][0])
        assert_topk_parity(gk, gi, want[1][1], want[1][2], want[1][3], p.name + " back on %d lanes, batch before" % lanes)
    finally:
        net.close()


def test_unit_buffer_read_with_a_bare_hipmemcpy(pkg, dsx, orc, synth):
    """The reference's callers follow PredictBatch with GetUnitBuffer and a plain cudaMemcpy on the default stream
    (utils/NNRecsGenerator.cpp:83, java/src/main/native/com_amazon_dsstne_Dsstne.cpp:366).  The same pattern with hipMemcpy from the
    HIP runtime itself, not through this library: every batch read this way must be that batch's finished activations, on several
    lanes (the pointer goes round as many buffers) and on one."""
    import ctypes as C
    from amazon_dsstne_amd import host_api
    hip = C.CDLL("libamdhip64.so")
    hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
    hip.hipMemcpy.restype = C.c_int
    p = synth.config(2, batches=3)
    N = p.widths[-1]
    refs = [orc.forward(p, pos, p.batch, filtered=False, want_unit=True, want_topk=False)[1] for pos in (0, p.batch, 2 * p.batch)]
    net = host_api.Network(p, max_k=p.k)
    try:
        net.bind_input()
        for lanes in (2, 1, 4, 3):
            net.set_lanes(lanes)
            seen = set()
            for rep in range(2):
                for n, pos in enumerate((0, p.batch, 2 * p.batch)):
                    net.predict_batch(pos)
                    ptr = net.unit_buffer("Output")
                    seen.add(ptr)
                    got = np.empty((p.batch, N), dtype=np.float32)
                    assert hip.hipMemcpy(got.ctypes.data, ptr, got.nbytes, 2) == 0     # hipMemcpyDeviceToHost, null stream
                    assert_close(got, refs[n], "units of batch %d read with hipMemcpy (%d lanes)" % (n, lanes), rel=1e-4, abs_floor=1e-3)
            assert len(seen) == lanes
    finally:
        net.close()


def test_network_file_in_netcdf4_container_predicts(pkg, dsx, orc, synth, tmp_path):
    """LoadNeuralNetworkNetCDF on NetCDF-4 (HDF5) network files, the container the reference writes: the fixtures of
    tests/golden/nc4 (written by the HDF5 library, old and new file-format generations, contiguous and chunked) through the
    native embedding example (DsstneContext -> PredictBatch -> kCalculateTopK) must print what the classic file prints, and
    that must be what the oracle predicts for the same weights."""
    nc4 = os.path.join(ROOT, "tests", "golden", "nc4")
    p = synth.autoencoder("small-nc4", 4242, 256, [32], 16, 5, 1, 1.0, 12, 0.5, (1, 40), bias_std=0.3)   # as make_fixtures.py builds it
    inputs = tmp_path / "inputs.txt"
    with open(inputs, "w") as f:
        for r in range(p.batch):
            f.write(" ".join(str(int(i)) for i in p.sparse_index[int(p.start[r]):int(p.end[r])]) + "\n")
    outs = {}
    for name in ("small.classic.nc", "small.earliest.nc", "small.v18.c1000.nc"):
        rc, out = run_exe("predict_main", os.path.join(nc4, name), inputs, p.batch, p.k)
        assert rc == 0, out[-3000:]
        outs[name] = [l for l in out.splitlines() if l and l[0].isdigit() and "\t" in l]
        assert len(outs[name]) == p.batch, out[-2000:]
    assert outs["small.earliest.nc"] == outs["small.classic.nc"] and outs["small.v18.c1000.nc"] == outs["small.classic.nc"]
    idx = np.zeros((p.batch, p.k), dtype=np.uint32)
    keys = np.zeros((p.batch, p.k), dtype=np.float32)
    for r, line in enumerate(outs["small.v18.c1000.nc"]):
        for j, c in enumerate(c for c in line.split("\t")[1].split(",") if c):
            i, s = c.split(":")
            idx[r, j], keys[r, j] = int(i), float(s)
    _, ref_unit, ref_keys, ref_idx = orc.forward(p, filtered=False, want_unit=True)
    assert_topk_parity(keys, idx, ref_keys, ref_idx, ref_unit, "network from a NetCDF-4 file")


def test_wide_output_layer_is_deferred_and_materialised_on_demand(pkg, dsx, orc, synth):
    """An output layer of 131,072 units or more is not stored by PredictBatch: CalculateFilteredTopK / CalculateTopK run it
    together with the top-K (dsx_fc_topk), GetUnits computes it when asked, and SetDeferredOutput(false) stores it as the
    reference does.  All three must agree with the oracle, batch after batch on two lanes (the deferred state travels with the
    lane's buffers), the last batch being short."""
    from amazon_dsstne_amd import host_api
    p = synth.autoencoder("wide-140k", 31, 140000, [64], 48, 20, batches=3, zipf_s=1.1, nnz_mean=30, nnz_sigma=0.8, nnz_clip=(1, 400))
    short = 11
    p.examples -= short
    p.unique_examples -= short
    p.start, p.end = p.start[:p.examples], p.end[:p.examples]
    positions = list(range(0, p.examples, p.batch))
    want = reference_batches(orc, p, positions)
    dsx.dsx_fc_topk_flagged(1)
    net = host_api.Network(p, max_k=p.k)
    try:
        net.bind_input()
        for deferred in (True, False):
            net.set_deferred_output(deferred)
            got = []
            for n, pos in enumerate(positions):
                net.predict_batch(pos)
                net.topk(p.k, filter_dataset="input")
                if n > 0:
                    got.append(net.get_topk_previous(want[n - 1][0]))
            got.append(net.get_topk(want[-1][0]))
            for n, ((rows, keys, idx, scores), (gk, gi)) in enumerate(zip(want, got)):
                assert_topk_parity(gk, gi, keys, idx, scores, "%s batch %d, deferred=%s" % (p.name, n, deferred))
        # unfiltered top-K of a deferred layer, then its units on demand, then the top-K again from the stored units
        net.set_deferred_output(True)
        net.predict_batch(positions[1])
        net.topk(p.k, filter_dataset=None)
        k1, i1 = net.get_topk(p.batch)
        _, ref_unit, ref_keys, ref_idx = orc.forward(p, positions[1], p.batch, filtered=False, want_unit=True)
        assert_topk_parity(k1, i1, ref_keys, ref_idx, ref_unit, "deferred, unfiltered")
        unit = net.units(rows=p.batch)
        assert_units_close(unit, ref_unit, p, positions[1], "units of a deferred layer, computed on demand")
        net.topk(p.k, filter_dataset=None)
        k2, i2 = net.get_topk(p.batch)
        assert_topk_parity(k2, i2, ref_keys, ref_idx, ref_unit, "after the units were asked for")
        rows = np.arange(p.batch)[:, None]
        assert np.array_equal(unit[rows, i2], k2)          # now the scores are the stored units, bit for bit
        assert dsx.dsx_fc_topk_flagged(0) == 0
    finally:
        net.close()
