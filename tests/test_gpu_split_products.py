"""The dense layer with fp32 products formed from bf16 matrix instructions (dsx_fc_split / dsx_fc_forward_split) against the
CPU oracle, against fp64, and against the fp32 kernel it stands in for (needs an MI355X).

Tolerance: 1e-4 relative to the scale of the sums, as for dsx_fc_forward; on top of that the mode has to be as close to the
fp64 product as the fp32 kernel is (it claims fp32 accuracy, not only the tolerance)."""
import ctypes as C

import numpy as np
import pytest

from parity import assert_close, assert_topk_parity, assert_units_close

pytestmark = pytest.mark.gpu


def say(msg):
    print("[case] " + msg, flush=True)


def dev(pkg, a):
    return None if a is None else pkg.DeviceArray.from_numpy(a)


def planes_of(pkg, dsx, d, ld, k_major, rows, k):
    planes = pkg.DeviceArray((dsx.dsx_fc_split_bytes(rows, k) // 4,), np.uint32)
    pkg.check(dsx.dsx_fc_split(d.ptr, ld, k_major, rows, k, planes.ptr))
    return planes


def bf16_planes_to_float(words, rows, k):
    """Undo the layout of dsx_fc_split on the host: returns the three planes as float64 arrays [rows][k]."""
    rp, kb = (rows + 255) // 256 * 256, (k + 15) // 16 * 2
    halves = words.view(np.uint16).reshape(3, kb, rp, 8)
    f = (halves.astype(np.uint32) << 16).view(np.float32).astype(np.float64)      # [p][kb][r][8]
    f = f.transpose(0, 2, 1, 3).reshape(3, rp, kb * 8)
    return f, rp, kb * 8


@pytest.mark.parametrize("rows,k,k_major", [(5, 3, 0), (130, 17, 0), (257, 40, 1), (128, 16, 1), (1, 129, 1)])
def test_split_planes_sum_back_to_the_input(pkg, dsx, rng, rows, k, k_major):
    """hi + mid + lo is the fp32 input exactly (three times eight significant bits), the padding is zero, and each plane is what
    rounding to nearest-even leaves of the one before (so that |mid| <= ulp_bf16(hi) / 2 and so on)."""
    say("split planes rows=%d k=%d k_major=%d" % (rows, k, k_major))
    x = (rng.standard_normal((rows, k)) * np.exp(4 * rng.standard_normal((rows, k)))).astype(np.float32)
    x[0, 0] = 0.0
    x[rows - 1, k - 1] = np.float32(1.0) + np.float32(2.0 ** -23)      # needs all three planes
    ld = (rows if k_major else k) + 3
    src = np.zeros((k, ld) if k_major else (rows, ld), dtype=np.float32)
    if k_major:
        src[:, :rows] = x.T
    else:
        src[:, :k] = x
    d = dev(pkg, src)
    planes = planes_of(pkg, dsx, d, ld, k_major, rows, k)
    f, rp, kp = bf16_planes_to_float(planes.numpy(), rows, k)
    total = f[0] + f[1] + f[2]
    assert np.array_equal(total[:rows, :k], x.astype(np.float64))
    assert not total[rows:].any() and not total[:, k:].any()
    hi = f[0][:rows, :k]
    nz = hi != 0
    assert np.all(np.abs(f[1][:rows, :k][nz]) <= np.abs(hi[nz]) * 2.0 ** -8)
    assert np.all(np.abs(f[2][:rows, :k][nz]) <= np.abs(hi[nz]) * 2.0 ** -16)


def test_split_planes_special_values(pkg, dsx):
    x = np.array([[np.inf, -np.inf, np.nan, 3.3e38, -3.4e38, 1e-40, -0.0, 65504.0]], dtype=np.float32)
    d = dev(pkg, x)
    planes = planes_of(pkg, dsx, d, 8, 0, 1, 8)
    f, _, _ = bf16_planes_to_float(planes.numpy(), 1, 8)
    total = (f[0] + f[1] + f[2])[0, :8]
    assert total[0] == np.inf and total[1] == -np.inf and np.isnan(total[2])
    assert np.isfinite(total[3]) and abs(total[3] / 3.3e38 - 1) < 2.0 ** -7          # kept to bf16 precision, not turned into inf
    assert np.isfinite(total[4]) and abs(total[4] / -3.4e38 - 1) < 2.0 ** -7
    assert total[7] == 65504.0 and total[6] == 0.0
    assert abs(total[5] - 1e-40) <= 2.0 ** -134                                         # subnormal: to half a bf16 subnormal step


SHAPES = [(300, 100, 1000), (130, 17, 257), (1, 128, 129), (257, 130, 128), (64, 512, 3000), (1024, 128, 5000), (1, 1, 1), (257, 1, 5),
          (40, 4100, 300), (513, 33, 1)]


@pytest.fixture(params=[128, 256])
def tile_rows(request, pkg, dsx):
    """Both tile heights of the kernel on every shape (by itself it takes 256 rows only for long sums over many tiles)."""
    pkg.check(dsx.dsx_testing_set_split_tile_rows(request.param))
    yield request.param
    pkg.check(dsx.dsx_testing_set_split_tile_rows(0))


def test_fc_split_tile_rows_argument(pkg, dsx):
    assert dsx.dsx_testing_set_split_tile_rows(64) != 0
    pkg.check(dsx.dsx_testing_set_split_tile_rows(0))


@pytest.mark.parametrize("B,k,n", SHAPES)
def test_fc_split_vs_oracle_fp64_and_fp32_kernel(pkg, dsx, orc, rng, tile_rows, B, k, n):
    say("fc_forward_split B=%d k=%d n=%d, tiles of %d rows" % (B, k, n, tile_rows))
    X = (rng.standard_normal((B, k)) * np.exp(rng.standard_normal((B, k)))).astype(np.float32)
    W = (rng.standard_normal((k, n)) * 0.1).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    dX, dW, db = dev(pkg, X), dev(pkg, W), dev(pkg, bias)
    xp = planes_of(pkg, dsx, dX, k, 0, B, k)
    wp = planes_of(pkg, dsx, dW, n, 1, n, k)
    Z = pkg.DeviceArray.from_numpy(np.full((B, n + 3), 55.0, dtype=np.float32))
    pkg.check(dsx.dsx_fc_forward_split(xp.ptr, wp.ptr, db.ptr, Z.ptr, n + 3, B, k, n, 0, 3, None, None, None))
    got = Z.numpy()
    assert np.all(got[:, n:] == 55.0)                                   # nothing written past n
    got = got[:, :n]
    ref = orc.sgemm_acc(X, W, orc.clear_unit([bias], n, B))
    scale = np.abs(X).astype(np.float64) @ np.abs(W).astype(np.float64) + np.abs(bias)   # what the rounding errors scale with
    assert_close(got, ref, "split fc vs oracle", rel=1e-4, abs_floor=max(0.1 * float(scale.max()), 1e-2))
    exact = X.astype(np.float64) @ W.astype(np.float64) + bias
    Zf = pkg.DeviceArray.from_numpy(np.zeros((B, n), dtype=np.float32))
    pkg.check(dsx.dsx_fc_forward(dX.ptr, k, dW.ptr, 0, db.ptr, Zf.ptr, n, B, k, n, 0, 3, None))
    err_split = float((np.abs(got - exact) / scale).max())
    err_f32 = float((np.abs(Zf.numpy() - exact) / scale).max())
    say("  max error / sum |x||w|: split %.3e, fp32 kernel %.3e" % (err_split, err_f32))
    assert err_split <= 2.0 * err_f32 + 2.0 ** -23                      # as close to fp64 as fp32 multiplication is (a missing 2^-16 term: 1e-5)
    assert err_split < 2e-6


def test_fc_split_infinite_operand_gives_nan_only_where_it_takes_part(pkg, dsx, rng):
    """The stated limit of the mode: an Inf operand sits in the first plane with zeros behind it, so the six-term sum holds
    Inf x 0 (or +Inf and -Inf from planes of opposite sign) and the sums it takes part in come out NaN or +/-Inf, where the fp32
    kernel gives +/-Inf.  Every other sum is unaffected."""
    B, k, n = 130, 48, 200
    X = rng.standard_normal((B, k)).astype(np.float32)
    W = rng.standard_normal((k, n)).astype(np.float32)
    X[7, 5] = np.inf
    W[9, 33] = -np.inf
    dX, dW = dev(pkg, X), dev(pkg, W)
    xp = planes_of(pkg, dsx, dX, k, 0, B, k)
    wp = planes_of(pkg, dsx, dW, n, 1, n, k)
    Z = pkg.DeviceArray((B, n), np.float32)
    pkg.check(dsx.dsx_fc_forward_split(xp.ptr, wp.ptr, None, Z.ptr, n, B, k, n, 0, 3, None, None, None))
    Zf = pkg.DeviceArray((B, n), np.float32)
    pkg.check(dsx.dsx_fc_forward(dX.ptr, k, dW.ptr, 0, None, Zf.ptr, n, B, k, n, 0, 3, None))
    got, plain = Z.numpy(), Zf.numpy()
    touched = np.zeros((B, n), dtype=bool)
    touched[7, :] = True
    touched[:, 33] = True
    assert np.all(~np.isfinite(got[touched])) and np.all(~np.isfinite(plain[touched]))
    assert np.isnan(got[touched]).any()                                  # Inf x 0, or Inf - Inf between the planes' terms
    assert np.isinf(plain[7, 0]) and np.isinf(plain[0, 33])              # the fp32 kernel keeps the infinity
    clean = ~touched
    assert np.all(np.isfinite(got[clean]))
    assert_close(got[clean], plain[clean], "sums without a non-finite operand", rel=1e-4, abs_floor=1.0)


@pytest.mark.parametrize("act", [0, 1, 2, 10, 11, 12])
@pytest.mark.parametrize("accumulate", [0, 1])
def test_fc_split_epilogue(pkg, dsx, orc, rng, tile_rows, act, accumulate):
    B, k, n = 70, 48, 150
    X = rng.standard_normal((B, k)).astype(np.float32)
    W = (rng.standard_normal((k, n)) * 0.3).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    Z0 = rng.standard_normal((B, n)).astype(np.float32)
    params = pkg.ActParams(0.2, 1.5, 1.05)
    dX, dW, db = dev(pkg, X), dev(pkg, W), dev(pkg, bias)
    xp = planes_of(pkg, dsx, dX, k, 0, B, k)
    wp = planes_of(pkg, dsx, dW, n, 1, n, k)
    Z = pkg.DeviceArray.from_numpy(Z0)
    pkg.check(dsx.dsx_fc_forward_split(xp.ptr, wp.ptr, db.ptr, Z.ptr, n, B, k, n, accumulate, act, C.byref(params), None, None))
    pre = orc.clear_unit([bias], n, B) + (Z0 if accumulate else 0)
    ref = orc.activation(orc.sgemm_acc(X, W, pre), act, 0.2, 1.5, 1.05)
    # (sums of 48 products of size 0.3 that cancel to almost nothing carry the rounding of their terms: 1e-4 of a tenth of a typical sum)
    assert_close(Z.numpy(), ref, "split fc epilogue", rel=1e-4, abs_floor=0.1)


def test_fc_split_transposed_weights_and_pitched_input(pkg, dsx, orc, rng):
    B, k, n = 90, 70, 130
    X = rng.standard_normal((B, k + 6)).astype(np.float32)       # row pitch larger than k
    Wt = (rng.standard_normal((n, k)) * 0.2).astype(np.float32)  # [n][k]: shared transposed weight (engine/NNLayer.cpp:1065-1072)
    dX, dW = dev(pkg, X), dev(pkg, Wt)
    xp = planes_of(pkg, dsx, dX, k + 6, 0, B, k)
    wp = planes_of(pkg, dsx, dW, k, 0, n, k)                      # a column of W is a row of the stored matrix
    Z = pkg.DeviceArray.from_numpy(np.zeros((B, n), dtype=np.float32))
    pkg.check(dsx.dsx_fc_forward_split(xp.ptr, wp.ptr, None, Z.ptr, n, B, k, n, 0, 3, None, None, None))
    ref = orc.sgemm_acc(np.ascontiguousarray(X[:, :k]), Wt, np.zeros((B, n), dtype=np.float32), transposed=True)
    assert_close(Z.numpy(), ref, "split fc, transposed weights", rel=1e-4, abs_floor=0.5)


def test_fc_split_segment_maxima_and_arguments(pkg, dsx, rng, tile_rows):
    B, k, n = 300, 64, 1000
    X = rng.standard_normal((B, k)).astype(np.float32)
    W = (rng.standard_normal((k, n)) * 0.2).astype(np.float32)
    dX, dW = dev(pkg, X), dev(pkg, W)
    xp = planes_of(pkg, dsx, dX, k, 0, B, k)
    wp = planes_of(pkg, dsx, dW, n, 1, n, k)
    Z = pkg.DeviceArray((B, n), np.float32)
    nseg = (n + 63) // 64
    sm = pkg.DeviceArray((B, nseg), np.float32)
    sw = C.c_uint32(7)
    pkg.check(dsx.dsx_fc_forward_split(xp.ptr, wp.ptr, None, Z.ptr, n, B, k, n, 0, 0, None, sm.ptr, C.byref(sw)))
    assert sw.value == 64
    unit = Z.numpy()
    pad = np.full((B, nseg * 64), -np.inf, dtype=np.float32)
    pad[:, :n] = unit
    assert np.array_equal(sm.numpy(), pad.reshape(B, nseg, 64).max(axis=2))
    # argument errors are reported, not run
    assert dsx.dsx_fc_forward_split(None, wp.ptr, None, Z.ptr, n, B, k, n, 0, 0, None, None, None) != 0
    assert dsx.dsx_fc_forward_split(xp.ptr, wp.ptr, None, Z.ptr, n - 1, B, k, n, 0, 0, None, None, None) != 0
    assert dsx.dsx_fc_forward_split(xp.ptr, wp.ptr, None, Z.ptr, n, B, k, n, 0, 7, None, None, None) != 0      # softmax is a row operation
    assert dsx.dsx_fc_forward_split(xp.ptr, wp.ptr, None, Z.ptr, n, B, k, n, 0, 0, None, sm.ptr, None) != 0
    assert dsx.dsx_fc_split(dX.ptr, k - 1, 0, B, k, xp.ptr) != 0
    assert dsx.dsx_fc_forward_split(xp.ptr, wp.ptr, None, Z.ptr, n, 0, k, n, 0, 0, None, None, None) == 0       # empty batch: nothing to do


def test_cfg2_with_split_products_matches_the_oracle(pkg, dsx, orc, synth):
    """Config 2 end to end with the output layer in this mode, scanning and guided top-K: activations within 1e-4 of the oracle's,
    indexes the oracle's except where its scores are closer than 1e-5."""
    from dsx_support.pipeline import DevicePipeline
    p = synth.config(2)
    _, ref_unit, _, _ = orc.forward(p, 0, None, filtered=False, want_unit=True, want_topk=False)
    _, _, ref_keys, ref_idx = orc.forward(p, 0, None, filtered=True)
    ref_scores = ref_unit.copy()
    orc.lib().orc_apply_filter(ref_scores.ctypes.data, p.batch, ref_scores.shape[1], 0, 0, None, p.start.ctypes.data, p.end.ctypes.data,
                               p.sparse_index.ctypes.data, None)
    for guided in (False, True):
        pipe = DevicePipeline(p, dsx, guided=guided, split=True)
        pipe.step()
        keys, idx = pipe.results()
        unit = pipe.output_unit()
        assert_units_close(unit, ref_unit, p, 0, "cfg2 output activations (split products)")
        nd = assert_topk_parity(keys, idx, ref_keys, ref_idx, ref_scores, "cfg2 split products guided=%s" % guided)
        say("cfg2 split products, guided=%s: parity ok (%d tie-equivalent index differences)" % (guided, nd))
        rows = np.arange(p.batch)[:, None]
        assert np.array_equal(unit[rows, idx], keys)


def host_forward_split(orc, p, lanes=2, batches=(0,)):
    """PredictBatch + filtered top-K through the class API with NNNetwork::SetSplitProducts(true), compared with the oracle."""
    from amazon_dsstne_amd import host_api
    net = host_api.Network(p, max_k=p.k)
    try:
        net.set_lanes(lanes)
        net.set_split_products(True)
        net.bind_input()
        for position in batches:
            rows = min(p.batch, p.examples - position)
            net.predict_batch(position)
            net.topk(p.k, filter_dataset="input")
            keys, idx = net.get_topk(rows)
            unit = net.units(rows=p.batch)[:rows]
            _, ref_unit, _, _ = orc.forward(p, position, rows, filtered=False, want_unit=True, want_topk=False)
            _, _, ref_keys, ref_idx = orc.forward(p, position, rows, filtered=True)
            assert_units_close(unit, ref_unit, p, position, p.name + " units, split products")
            ref_scores = ref_unit.copy()
            orc.lib().orc_apply_filter(ref_scores.ctypes.data, rows, ref_scores.shape[1], 0, position,
                                       p.index.ctypes.data if p.index is not None else None, p.start.ctypes.data, p.end.ctypes.data,
                                       p.sparse_index.ctypes.data, None)
            nd = assert_topk_parity(keys, idx, ref_keys, ref_idx, ref_scores, p.name + " split products")
            say("%s at %d, %d lanes, split products through NNNetwork: parity ok (%d tie-equivalent)" % (p.name, position, lanes, nd))
        return net
    except Exception:
        net.close()
        raise


def test_network_api_split_products_cfg2(pkg, dsx, orc, synth):
    p = synth.config(2, batches=3)
    for lanes in (1, 2):
        host_forward_split(orc, p, lanes=lanes, batches=(0, 1024, 2048)).close()


def test_network_api_split_products_hidden_layer_and_new_weights(pkg, dsx, orc, synth):
    """A network whose hidden layers are wide enough for the mode too (4096 rows x 2048 units: 512 tiles of 128 x 128), and weights replaced
    after the planes were built: the next batch must be computed from the new weights."""
    p = synth.autoencoder("split-wide-hidden", 31, 5000, [256, 2048], 4096, 10, 1, 1.0, 40, 0.8, (1, 300), bias_std=0.1)
    net = host_forward_split(orc, p)
    try:
        rng = np.random.default_rng(5)
        p.weights[1] = (rng.standard_normal(p.weights[1].shape) * 0.02).astype(np.float32)
        p.weights[2] = (rng.standard_normal(p.weights[2].shape) * 0.02).astype(np.float32)
        net.set_weights("Hidden1", "Hidden2", weights=p.weights[1])
        net.set_weights("Hidden2", "Output", weights=p.weights[2])
        net.predict_batch(0)
        unit = net.units(rows=p.batch)
        _, ref_unit, _, _ = orc.forward(p, 0, p.batch, filtered=False, want_unit=True, want_topk=False)
        assert_units_close(unit, ref_unit, p, 0, "units after SetWeights, split products")
        # and back: the fp32 kernels give the same within the tolerance
        net.set_split_products(False)
        net.predict_batch(0)
        plain = net.units(rows=p.batch)
        assert_units_close(plain, ref_unit, p, 0, "units with the mode switched off again")
        assert not np.array_equal(plain, unit)          # (the two modes round differently: the first pass did take the other kernel)
    finally:
        net.close()


def test_network_api_split_products_deferred_wide_output(pkg, dsx, orc, synth):
    """An output layer wide enough to be computed together with its top-K (131,072 units or more): with split products that call is
    dsx_fc_topk_split; the units asked for afterwards come from the storing kernel of the same mode."""
    p = synth.autoencoder("split-wide-output", 1004, 140000, [512], 256, 100, 1, 1.1, 50, 1.0, (1, 1000))
    host_forward_split(orc, p).close()


# ---------------------------------------------------------------------------------------------------------------- exact KNN

def knn_split_search(pkg, dsx, cm, rows, pad, dim, queries_m, k):
    dI, dQ = dev(pkg, cm), dev(pkg, queries_m)
    planes = planes_of(pkg, dsx, dI, rows, 1, rows, dim)            # the column-major table: vector r is column r
    nq = queries_m.shape[0]
    scores = pkg.DeviceArray((nq, k), np.float32)
    idx = pkg.DeviceArray((nq, k), np.uint32)
    el = (C.c_float * 2)()
    pkg.check(dsx.dsx_knn_search_split(planes.ptr, rows, pad, dim, dQ.ptr, nq, k, scores.ptr, idx.ptr, None, 0, el))
    return scores.numpy(), idx.numpy(), el


@pytest.mark.parametrize("items,queries,dim,k,blocks", [(1003, 9, 24, 10, 0), (50000, 64, 256, 100, 0), (30011, 70, 64, 100, 1024),
                                                         (9000, 130, 256, 10, 1024), (26000, 33, 36, 200, 1024), (100, 3, 8, 100, 0),
                                                         (5000, 1, 4, 256, 1024)])
def test_knn_search_split(pkg, dsx, orc, synth, items, queries, dim, k, blocks):
    """dsx_knn_search_split against the oracle, through the scanned first block alone and (blocks = 1,024: a first block of 1,024
    items) through the candidate ranges."""
    say("knn split products items=%d queries=%d dim=%d k=%d first block %d" % (items, queries, dim, k, blocks))
    p = synth.knn_config(seed=11, items=items, queries=queries, dim=dim, k=k)
    cm, rows, pad = p.column_major_padded()
    cm[:, rows - pad:] = 50.0     # pad rows must never be returned (knn/KnnData.cpp:336-340 leaves them uninitialised)
    dsx.dsx_testing_set_knn_block_columns(blocks)
    try:
        got_s, got_i, el = knn_split_search(pkg, dsx, cm, rows, pad, dim, p.queries, k)
        path = dsx.dsx_knn_last_search_path()
    finally:
        dsx.dsx_testing_set_knn_block_columns(0)
    assert path == (1 if blocks else 0), path          # DSX_KNN_PATH_CANDIDATES where there are ranges after the first block
    ref_s, ref_i = orc.knn_search(cm, rows, pad, dim, p.queries, k)
    full = p.queries.astype(np.float64) @ p.items.astype(np.float64).T
    assert got_i.max() < items
    mism = got_i != ref_i
    if mism.any():   # different rounding may swap neighbours whose scores differ by less than 1e-5
        r, c = np.nonzero(mism)
        assert np.abs(full[r, got_i[r, c]] - full[r, ref_i[r, c]]).max() < 1e-5
    assert_close(got_s, np.take_along_axis(full, got_i.astype(np.int64), axis=1), "knn scores, split products", rel=1e-4, abs_floor=0.05)
    assert np.all(np.diff(got_s, axis=1) <= 0)
    assert el[0] > 0 and el[1] > 0


@pytest.mark.parametrize("B,k,n,act", [(1024, 128, 128, 2), (200, 256, 96, 0), (33, 128, 50, 3), (700, 512, 300, 2)])
def test_fc_forward_planes_matches_forward_then_split(pkg, dsx, rng, B, k, n, act):
    """dsx_fc_forward_planes = dsx_fc_forward + dsx_fc_split of its result, bit for bit (result and planes; the small-layer kernel
    writes the planes itself, other shapes run the splitter behind the layer), also over stale contents of the planes buffer."""
    say("fc_forward_planes B=%d k=%d n=%d act=%d" % (B, k, n, act))
    X = rng.standard_normal((B, k)).astype(np.float32)
    W = (rng.standard_normal((k, n)) * 0.2).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    dX, dW, db = dev(pkg, X), dev(pkg, W), dev(pkg, bias)
    words = dsx.dsx_fc_split_bytes(B, n) // 4
    Z1 = pkg.DeviceArray((B, n), np.float32)
    P1 = pkg.DeviceArray.from_numpy(np.zeros(words, dtype=np.uint32))
    pkg.check(dsx.dsx_fc_forward(dX.ptr, k, dW.ptr, 0, db.ptr, Z1.ptr, n, B, k, n, 0, act, None))
    pkg.check(dsx.dsx_fc_split(Z1.ptr, n, 0, B, n, P1.ptr))
    Z2 = pkg.DeviceArray((B, n), np.float32)
    P2 = pkg.DeviceArray.from_numpy(np.zeros(words, dtype=np.uint32))
    pkg.check(dsx.dsx_fc_forward_planes(dX.ptr, k, dW.ptr, 0, db.ptr, Z2.ptr, n, B, k, n, act, None, P2.ptr))
    assert np.array_equal(Z1.numpy().view(np.uint32), Z2.numpy().view(np.uint32))
    f1, rp, kp = bf16_planes_to_float(P1.numpy(), B, n)
    f2, _, _ = bf16_planes_to_float(P2.numpy(), B, n)
    assert np.array_equal(f1[:, :B, :], f2[:, :B, :])                       # every valid row, k padding included
    assert not f2[:, B:, :].any()                                           # rows beyond the batch stay as they were (zero)
