"""Pins the CPU oracle against independent evidence (no GPU needed).

Each oracle function is checked against something that is NOT a re-typing of its own formula: the reference's own
topKsort compiled from utils/Utils.cpp (oracle/_ref), numpy float64 linear algebra and sorting, torch-CPU as a second
implementation of the forward pass, brute force on tiny inputs, and special cases with closed-form answers, chosen so
that a dropped term, a wrong index or a transposed operand fails at least one of them.
"""
import numpy as np
import pytest

from parity import assert_close, check_topk_invariants

A_SPARSE, A_BOOLEAN, A_INDEXED, A_WEIGHTED = 1, 2, 64, 128
T_UINT, T_INT, T_LLINT, T_ULLINT, T_FLOAT, T_DOUBLE, _, _, T_UCHAR, T_CHAR = range(10)


def np_topk(scores, k):
    """Independent top-K: full lexicographic sort on (-score, index)."""
    batch, width = scores.shape
    keys = np.full((batch, k), -np.float32(999999999999999.0), dtype=np.float32)
    idx = np.zeros((batch, k), dtype=np.uint32)
    for b in range(batch):
        order = np.lexsort((np.arange(width), -scores[b].astype(np.float64)))[:k]
        keys[b, :len(order)] = scores[b, order]
        idx[b, :len(order)] = order
    return keys, idx


def random_csr(rng, rows, width, max_nnz, allow_empty=True, empty_rows=()):
    counts = rng.integers(0 if allow_empty else 1, max_nnz + 1, size=rows)
    for r in empty_rows:
        counts[r] = 0
    start = np.zeros(rows, dtype=np.uint64)
    end = np.zeros(rows, dtype=np.uint64)
    cols = []
    pos = 0
    for r in range(rows):
        c = rng.choice(width, size=int(counts[r]), replace=False).astype(np.uint32)
        cols.append(c)
        start[r] = pos
        pos += len(c)
        end[r] = pos
    idx = np.concatenate(cols).astype(np.uint32) if pos else np.zeros(0, dtype=np.uint32)
    return start, end, idx


def dense_from_csr(start, end, idx, vals, rows, width):
    X = np.zeros((rows, width), dtype=np.float64)
    for r in range(rows):
        for t in range(int(start[r]), int(end[r])):
            X[r, idx[t]] += 1.0 if vals is None else float(vals[t])
    return X


# ---------------------------------------------------------------------------------------------------------------- top-K

# (batch, k, features) of tst/gputests/TestSort.cpp:208-211; the row pitch there is the feature count rounded up to 128
# with zero padding, and the padded pitch is what the kernel is given as its width.
TESTSORT_SHAPES = [(128, 128, 1024), (128, 128, 100000), (128, 64, 1024), (128, 32, 64), (128, 1, 64)]


@pytest.mark.parametrize("batch,k,nfeat", TESTSORT_SHAPES)
def test_topk_matches_reference_topksort(orc, rng, batch, k, nfeat):
    if orc.ref_lib() is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    if nfeat > 10000:
        batch = 16
    stride = (nfeat + 127) // 128 * 128
    scores = np.zeros((batch, stride), dtype=np.float32)
    scores[:, :nfeat] = rng.random((batch, nfeat), dtype=np.float32)
    keys, idx = orc.topk(scores, k)
    for b in range(batch):
        rk, rv = orc.ref_topksort(scores[b, :nfeat], k)   # TestSort.cpp:96 sorts the first nFeatures entries on the CPU
        # the reference leaves the order of equal keys open: keys must agree exactly, indices wherever keys are unique
        assert np.array_equal(keys[b], rk)
        uniq = np.concatenate(([True], rk[1:] != rk[:-1])) & np.concatenate((rk[:-1] != rk[1:], [True]))
        assert np.array_equal(idx[b][uniq], rv[uniq])
        assert np.array_equal(scores[b, idx[b]], keys[b])


@pytest.mark.parametrize("batch,width,k", [(7, 33, 5), (3, 64, 64), (4, 1000, 256), (2, 5, 8), (1, 1, 1), (5, 300, 100)])
def test_topk_bruteforce_and_ties(orc, rng, batch, width, k):
    scores = rng.integers(0, 8, size=(batch, width)).astype(np.float32) / 4 - 1   # many exact ties, both signs, zeros
    keys, idx = orc.topk(scores, k)
    rk, ri = np_topk(scores, k)
    assert np.array_equal(keys, rk)
    assert np.array_equal(idx, ri)
    check_topk_invariants(scores, keys, idx, k)
    if k > width:   # engine/kernels.cu:3221-3224 sentinel
        assert np.all(keys[:, width:] == -np.float32(999999999999999.0)) and np.all(idx[:, width:] == 0)


def test_topk_negative_zero_ties_with_positive_zero(orc):
    scores = np.array([[-0.0, 0.0, -1.0, 0.0]], dtype=np.float32)
    keys, idx = orc.topk(scores, 3)
    assert idx.tolist() == [[0, 1, 3]]


def test_knn_topk_ignores_padding(orc, rng):
    scores = rng.random((6, 40), dtype=np.float32)
    scores[:, 37:] = 100.0   # garbage in the pad columns must never surface (knn/topk.cu:37)
    keys, idx = orc.topk(scores, 5, width=37)
    rk, ri = np_topk(scores[:, :37], 5)
    assert np.array_equal(keys, rk) and np.array_equal(idx, ri)


def test_topk_kv(orc, rng):
    keys_in = rng.random((5, 200), dtype=np.float32)
    vals_f = rng.random((5, 200), dtype=np.float32)
    vals_u = rng.integers(0, 1 << 31, size=(5, 200)).astype(np.uint32)
    rk, ri = np_topk(keys_in, 17)
    k1, v1 = orc.topk_kv(keys_in, vals_f, 17)
    k2, v2 = orc.topk_kv(keys_in, vals_u, 17)
    rows = np.arange(5)[:, None]
    assert np.array_equal(k1, rk) and np.array_equal(v1, vals_f[rows, ri])
    assert np.array_equal(k2, rk) and np.array_equal(v2, vals_u[rows, ri])
    if orc.ref_lib() is not None:   # topKsort<float, float> with explicit payloads (utils/Utils.cpp:207-250)
        import ctypes
        R = orc.ref_lib()
        tk = np.empty(17, dtype=np.float32)
        tv = np.empty(17, dtype=np.float32)
        row_k, row_v = keys_in[0].copy(), vals_f[0].copy()
        R.ref_topksort_f32_f32(row_k.ctypes.data, row_v.ctypes.data, 200, tk.ctypes.data, tv.ctypes.data, 17)
        assert np.array_equal(tk, k1[0]) and np.array_equal(tv, v1[0])


# ------------------------------------------------------------------------------------------------------------- sparse Z

def test_sparse_z_boolean_equals_dense_product(orc, rng):
    rows, width, stride = 40, 300, 37
    start, end, idx = random_csr(rng, rows, width, 60, empty_rows=(3, 17))
    W = rng.standard_normal((width, stride)).astype(np.float32)
    bias = rng.standard_normal(stride).astype(np.float32)
    unit0 = np.tile(bias, (rows, 1))
    got = orc.sparse_z(A_SPARSE | A_BOOLEAN, T_FLOAT, 0, rows, stride, W, None, start, end, idx, None, None, unit0, 1.0)
    X = dense_from_csr(start, end, idx, None, rows, width)
    ref = X @ W.astype(np.float64) + bias
    assert_close(got, ref, "sparse Z vs dense fp64", rel=2e-5, abs_floor=1.0)
    empty = np.nonzero(start == end)[0]
    assert len(empty) > 0
    assert np.array_equal(got[empty], unit0[empty])   # empty row: untouched (bias only)


def test_sparse_z_special_cases(orc):
    W = np.arange(12, dtype=np.float32).reshape(4, 3) + 0.5
    start = np.array([0, 1, 1, 3], dtype=np.uint64)
    end = np.array([1, 1, 3, 5], dtype=np.uint64)
    idx = np.array([2, 1, 1, 0, 3], dtype=np.uint32)   # row0: {2}; row1: empty; row2: {1,1} duplicate; row3: {0,3}
    unit0 = np.full((4, 3), 10.0, dtype=np.float32)
    got = orc.sparse_z(A_SPARSE | A_BOOLEAN, T_FLOAT, 0, 4, 3, W, None, start, end, idx, None, None, unit0, 1.0)
    assert np.array_equal(got[0], 10 + W[2])            # single non-zero: bias + W[idx] exactly
    assert np.array_equal(got[1], unit0[1])             # empty
    assert np.array_equal(got[2], 10 + 2 * W[1])        # duplicates add twice
    assert np.array_equal(got[3], 10 + W[0] + W[3])
    # beta = 0 discards the previous contents, beta = 2 scales them; empty rows stay untouched either way
    g0 = orc.sparse_z(A_SPARSE | A_BOOLEAN, T_FLOAT, 0, 4, 3, W, None, start, end, idx, None, None, unit0, 0.0)
    g2 = orc.sparse_z(A_SPARSE | A_BOOLEAN, T_FLOAT, 0, 4, 3, W, None, start, end, idx, None, None, unit0, 2.0)
    assert np.array_equal(g0[0], W[2]) and np.array_equal(g2[0], 20 + W[2])
    assert np.array_equal(g0[1], unit0[1]) and np.array_equal(g2[1], unit0[1])


def test_sparse_z_position_index_weight(orc, rng):
    rows, width, stride, batch = 50, 120, 16, 8
    start, end, idx = random_csr(rng, rows, width, 20, allow_empty=False)
    W = rng.standard_normal((width, stride)).astype(np.float32)
    dw = rng.random(rows, dtype=np.float32) + 0.5
    perm = rng.permutation(rows).astype(np.uint32)
    zero = np.zeros((batch, stride), dtype=np.float32)
    X = dense_from_csr(start, end, idx, None, rows, width)
    full = X @ W.astype(np.float64)
    # position offsets the row window
    got = orc.sparse_z(A_SPARSE | A_BOOLEAN, T_FLOAT, 11, batch, stride, W, None, start, end, idx, None, None, zero, 0.0)
    assert_close(got, full[11:19], "position", rel=2e-5, abs_floor=1.0)
    # indexed: batch row b is stored row index[position + b] (engine/kernels.cu:750)
    got = orc.sparse_z(A_SPARSE | A_BOOLEAN | A_INDEXED, T_FLOAT, 5, batch, stride, W, perm, start, end, idx, None, None, zero, 0.0)
    assert_close(got, full[perm[5:13]], "indexed", rel=2e-5, abs_floor=1.0)
    # weighted: the whole row is scaled by its data weight, looked up at the resolved row
    got = orc.sparse_z(A_SPARSE | A_BOOLEAN | A_INDEXED | A_WEIGHTED, T_FLOAT, 5, batch, stride, W, perm, start, end, idx, dw, None, zero, 0.0)
    assert_close(got, full[perm[5:13]] * dw[perm[5:13]][:, None], "weighted", rel=2e-5, abs_floor=1.0)
    # the Indexed / Weighted arrays are ignored unless the attribute bit is set (engine/NNTypes.h:527-545)
    got = orc.sparse_z(A_SPARSE | A_BOOLEAN, T_FLOAT, 5, batch, stride, W, perm, start, end, idx, dw, None, zero, 0.0)
    assert_close(got, full[5:13], "attribute gating", rel=2e-5, abs_floor=1.0)


@pytest.mark.parametrize("dtype,tag,scale", [(np.float32, T_FLOAT, 1.0), (np.float64, T_DOUBLE, 1.0), (np.int32, T_INT, 1.0),
                                             (np.uint32, T_UINT, 1.0), (np.int64, T_LLINT, 1.0), (np.uint64, T_ULLINT, 1.0),
                                             (np.uint8, T_UCHAR, 1 / 256), (np.int8, T_CHAR, 1 / 256)])
def test_sparse_z_analog_types(orc, rng, dtype, tag, scale):
    rows, width, stride = 12, 90, 9
    start, end, idx = random_csr(rng, rows, width, 25)
    if np.issubdtype(dtype, np.floating):
        vals = (rng.integers(1, 11, size=len(idx)) * 0.5).astype(dtype)
    elif dtype == np.int8:
        vals = rng.integers(-100, 100, size=len(idx)).astype(dtype)
    else:
        vals = rng.integers(0, 200, size=len(idx)).astype(dtype)
    W = rng.standard_normal((width, stride)).astype(np.float32)
    zero = np.zeros((rows, stride), dtype=np.float32)
    got = orc.sparse_z(A_SPARSE, tag, 0, rows, stride, W, None, start, end, idx, None, vals, zero, 0.0)
    X = dense_from_csr(start, end, idx, vals.astype(np.float64) * scale, rows, width)   # engine/kernels.cu:923,998: bytes / 256
    assert_close(got, X @ W.astype(np.float64), "analog %s" % dtype.__name__, rel=5e-5, abs_floor=1.0)


def test_sparse_z_integer_weight_truncation(orc):
    # generic analog kernel keeps w * value in a T (engine/kernels.cu:828,848): with T = int the product is truncated
    W = np.ones((1, 1), dtype=np.float32)
    start, end = np.array([0], dtype=np.uint64), np.array([1], dtype=np.uint64)
    idx = np.zeros(1, dtype=np.uint32)
    vals = np.array([3], dtype=np.int32)
    dw = np.array([0.5], dtype=np.float32)
    got = orc.sparse_z(A_SPARSE | A_WEIGHTED, T_INT, 0, 1, 1, W, None, start, end, idx, dw, vals, np.zeros((1, 1), np.float32), 0.0)
    assert got[0, 0] == 1.0   # int(0.5 * 3) = 1, not 1.5


# -------------------------------------------------------------------------------------------------- loaders, bias, GEMM

def test_clear_unit(orc, rng):
    b = [rng.standard_normal(7).astype(np.float32) for _ in range(4)]
    for n in range(5):
        got = orc.clear_unit(b[:n], 7, 3)
        ref = np.zeros(7, dtype=np.float32)
        for i in range(n):
            ref = ref + b[i] if i else b[0].copy()
        assert np.array_equal(got, np.tile(ref, (3, 1)))


def test_load_sparse_input_unit(orc, rng):
    rows, width = 9, 50
    start, end, idx = random_csr(rng, rows, width, 12)
    vals = rng.integers(1, 200, size=len(idx)).astype(np.uint8)
    dw = rng.random(rows, dtype=np.float32) + 1
    got = orc.load_sparse_input_unit(A_SPARSE | A_BOOLEAN | A_WEIGHTED, T_FLOAT, 2, 5, width, None, start, end, idx, dw, None)
    X = dense_from_csr(start, end, idx, None, rows, width)
    assert np.array_equal(got, (X[2:7] * dw[2:7, None]).astype(np.float32))
    # analog loader has no 8-bit rescaling (engine/kernels.cu:215-234)
    got = orc.load_sparse_input_unit(A_SPARSE, T_UCHAR, 0, rows, width, None, start, end, idx, None, vals)
    assert np.array_equal(got, dense_from_csr(start, end, idx, vals, rows, width).astype(np.float32))


def test_load_input_unit(orc, rng):
    data = rng.integers(0, 255, size=(6, 10)).astype(np.uint8)
    got = orc.load_input_unit(T_UCHAR, 1, 4, 10, None, data)
    assert np.array_equal(got, (data[1:5].astype(np.float32) * np.float32(1 / 256) - np.float32(0.5)))   # engine/kernels.cu:463
    datac = rng.integers(-128, 127, size=(6, 10)).astype(np.int8)
    got = orc.load_input_unit(T_CHAR, 0, 6, 10, None, datac)
    assert np.array_equal(got, datac.astype(np.float32) * np.float32(1 / 128))                          # engine/kernels.cu:476
    dataf = rng.standard_normal((6, 10)).astype(np.float32)
    perm = rng.permutation(6).astype(np.uint32)
    got = orc.load_input_unit(T_FLOAT, 2, 3, 10, perm, dataf)
    assert np.array_equal(got, dataf[perm[2:5]])


@pytest.mark.parametrize("transposed", [False, True])
def test_sgemm_vs_fp64(orc, rng, transposed):
    B, k, n = 13, 70, 29
    X = rng.standard_normal((B, k)).astype(np.float32)
    W = rng.standard_normal((k, n)).astype(np.float32)
    Z0 = rng.standard_normal((B, n)).astype(np.float32)
    got = orc.sgemm_acc(X, W.T.copy() if transposed else W, Z0, transposed)
    assert_close(got, Z0 + X.astype(np.float64) @ W.astype(np.float64), "sgemm", rel=2e-5, abs_floor=1.0)


def test_activations_closed_form(orc):
    x = np.linspace(-12, 12, 481).astype(np.float32)
    x64 = x.astype(np.float64)
    cases = {
        0: 1 / (1 + np.exp(-x64)),
        1: np.tanh(x64),
        2: np.maximum(0, x64),
        3: x64,
        11: np.maximum(x64, 0.2 * x64),
        10: np.where(x64 > 0, x64, 1.5 * (np.exp(x64) - 1)),
        12: np.where(x64 > 0, 1.05 * x64, 1.05 * 1.5 * (np.exp(x64) - 1)),
        4: x64, 5: x64, 6: x64, 8: x64, 9: x64,   # kinds CalculateActivation has no case for (engine/NNLayer.cpp:1646-1683)
    }
    for act, ref in cases.items():
        got = orc.activation(x, act, slope=0.2, alpha=1.5, lam=1.05)
        assert_close(got, ref, "activation %d" % act, rel=1e-6, abs_floor=1e-6)


def test_softmax(orc, rng):
    z = (rng.standard_normal((4, 50)) * 5).astype(np.float32)
    got = orc.softmax(z)
    e = np.exp(z.astype(np.float64) - z.max(axis=1, keepdims=True))
    assert_close(got, e / e.sum(axis=1, keepdims=True), "softmax", rel=1e-5, abs_floor=1e-9)


# ---------------------------------------------------------------------------------------------------------------- filter

def test_filter_definition(orc, rng):
    batch, width = 6, 40
    scores = rng.random((batch, width), dtype=np.float32) + 0.1
    start, end, idx = random_csr(rng, batch, width + 10, 8)      # some indexes fall outside [0, width): ignored
    mul = rng.random(len(idx), dtype=np.float32) * 2
    expect = scores.copy()
    for b in range(batch):
        for t in range(int(start[b]), int(end[b])):
            if idx[t] < width:
                expect[b, idx[t]] = mul[t] * expect[b, idx[t]]   # utils/Filters.cpp:62
    k1, i1 = orc.topk_filtered(scores, 7, 0, None, start, end, idx, mul)
    rk, ri = np_topk(expect, 7)
    assert np.array_equal(k1, rk) and np.array_equal(i1, ri)
    # default multiplier 0 (utils/Filters.cpp:108-121): filtered items never surface while enough others remain
    k0, i0 = orc.topk_filtered(scores, 7, 0, None, start, end, idx, None)
    for b in range(batch):
        assert not set(i0[b].tolist()) & set(idx[int(start[b]):int(end[b])].tolist())
    # ... and surface with score +0.0, lowest index first, once everything else is used up
    small = np.array([[0.5, 0.25, 0.75, 0.9]], dtype=np.float32)
    s1, e1 = np.array([0], dtype=np.uint64), np.array([3], dtype=np.uint64)
    kk, ii = orc.topk_filtered(small, 4, 0, None, s1, e1, np.array([3, 0, 3], dtype=np.uint32), None)
    assert ii.tolist() == [[2, 1, 0, 3]] and kk.tolist() == [[0.75, 0.25, 0.0, 0.0]]


# ------------------------------------------------------------------------------------------------------------------- KNN

def test_knn_vs_numpy(orc, synth):
    p = synth.knn_config(seed=7, items=1003, queries=9, dim=24, k=10)
    cm, rows, pad = p.column_major_padded()
    cm[:, rows - pad:] = 99.0   # the reference leaves the pad rows uninitialised (knn/KnnData.cpp:336-340)
    scores, idx = orc.knn_search(cm, rows, pad, 24, p.queries, 10)
    full = p.queries.astype(np.float64) @ p.items.astype(np.float64).T
    rk, ri = np_topk(full.astype(np.float32), 10)
    assert np.array_equal(idx, ri)
    assert_close(scores, np.take_along_axis(full, ri.astype(np.int64), axis=1), "knn scores", rel=1e-5, abs_floor=1.0)
    # an item queried with itself comes back first with score 1
    s2, i2 = orc.knn_search(cm, rows, pad, 24, p.items[:5], 3)
    assert i2[:, 0].tolist() == [0, 1, 2, 3, 4] and np.allclose(s2[:, 0], 1.0, atol=1e-6)


def test_merge_knn(orc):
    import ctypes as C
    s0 = np.array([[0.9, 0.5, 0.1]], dtype=np.float32)
    s1 = np.array([[0.9, 0.7, 0.2]], dtype=np.float32)
    i0 = np.array([[10, 11, 12]], dtype=np.uint32)
    i1 = np.array([[20, 21, 22]], dtype=np.uint32)
    sc = (C.c_void_p * 2)(s0.ctypes.data, s1.ctypes.data)
    ix = (C.c_void_p * 2)(i0.ctypes.data, i1.ctypes.data)
    out_s = np.empty((1, 3), dtype=np.float32)
    out_i = np.empty((1, 3), dtype=np.uint32)
    out_d = np.empty((1, 3), dtype=np.uint32)
    orc.lib().orc_merge_knn(3, 1, 3, 2, sc, ix, out_s.ctypes.data, out_i.ctypes.data, out_d.ctypes.data)
    # strict '<' (knn/KnnExactGpu.cu:183): on the 0.9 tie the lower device wins
    assert out_s.tolist() == [[np.float32(0.9), np.float32(0.9), np.float32(0.7)]]
    assert out_i.tolist() == [[10, 20, 21]] and out_d.tolist() == [[0, 1, 1]]


# ------------------------------------------------------------------------------------------------------------ end to end

def test_forward_vs_torch_cpu(orc, synth):
    torch = pytest.importorskip("torch")
    p = synth.autoencoder("t", 5, 300, [48, 32], 20, 6, zipf_s=1.0, nnz_mean=12, nnz_sigma=0.7, nnz_clip=(0, 40), bias_std=0.3)
    _, unit, _, _ = orc.forward(p, filtered=False, want_unit=True, want_topk=False)
    X = torch.zeros(p.batch, p.widths[0], dtype=torch.float64)
    for r in range(p.batch):
        X[r, torch.from_numpy(p.sparse_index[int(p.start[r]):int(p.end[r])].astype(np.int64))] = 1
    h = X
    for l, (W, b) in enumerate(zip(p.weights, p.biases)):
        h = h @ torch.from_numpy(W).double() + torch.from_numpy(b).double()
        h = torch.relu(h) if p.acts[l] == 2 else torch.sigmoid(h)
    assert_close(unit, h.numpy(), "forward vs torch fp64", rel=2e-5, abs_floor=1e-4)
    _, _, keys, idx = orc.forward(p, filtered=True)
    masked = unit.copy()
    for r in range(p.batch):
        masked[r, p.sparse_index[int(p.start[r]):int(p.end[r])]] *= 0
    rk, ri = np_topk(masked, p.k)
    assert np.array_equal(idx, ri) and np.array_equal(keys, rk)


def test_cfg1_golden(orc, synth):
    """Expected top-10 of the tiny configuration computed by tests/golden/make_cfg1_golden.py with numpy float64 only."""
    import os
    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "cfg1_golden.npz"))
    p = synth.config(1)
    assert int(p.sparse_index.astype(np.uint64).sum()) == int(g["input_checksum"])   # same synthetic bytes as when recorded
    _, unit, _, _ = orc.forward(p, filtered=False, want_unit=True, want_topk=False)
    _, _, keys, idx = orc.forward(p, filtered=True)
    assert_close(unit, g["unit"], "cfg1 output vs fp64 golden", rel=2e-5, abs_floor=1e-4)
    assert np.array_equal(idx, g["idx"])
    assert_close(keys, g["keys"], "cfg1 top-10 scores", rel=2e-5)
