"""dsx_fc_topk (output layer + filtered top-K without storing the layer's result) against the two-call path
(dsx_fc_forward, then dsx_topk_filtered over the stored result) and the CPU oracle, through the C ABI.  Needs an MI355X."""
import ctypes as C

import numpy as np
import pytest

from parity import assert_close, assert_topk_parity
from test_oracle import random_csr

pytestmark = pytest.mark.gpu

ACT_SIGMOID, ACT_TANH, ACT_RELU, ACT_LINEAR, ACT_LRELU, ACT_ELU = 0, 1, 2, 3, 11, 10


def say(msg):
    print("[case] " + msg, flush=True)


def dev(pkg, a):
    return None if a is None else pkg.DeviceArray.from_numpy(a)


MODE = {"split": False}


@pytest.fixture(params=["fp32", "split"])
def knobs(request, dsx):
    """Every test runs twice: dsx_fc_topk, and dsx_fc_topk_split (the same call with the products formed from bf16 matrix
    instructions; the two-call path it is compared with stays the fp32 one)."""
    MODE["split"] = request.param == "split"
    dsx.dsx_fc_topk_flagged(1)
    yield dsx
    MODE["split"] = False
    dsx.dsx_testing_set_fc_topk_first_columns(0)
    dsx.dsx_testing_set_fc_topk_candidate_capacity(0)
    dsx.dsx_fc_topk_flagged(1)


def run_both(pkg, dsx, orc, X, W, bias, act, k, position=0, index=None, start=None, end=None, fidx=None, what=""):
    """Runs dsx_fc_topk and the two-call path; checks the fused result against the stored scores under the parity rules and
    against the oracle's filtered top-k of the oracle's own scores.  Returns (keys, idx, stored unit, two-call keys, two-call idx)."""
    batch, kdim = X.shape
    n = W.shape[1]
    dX, dW, db = dev(pkg, X), dev(pkg, W), dev(pkg, bias)
    di, ds, de, dx = (dev(pkg, a) for a in (index, start, end, fidx))
    params = pkg.ActParams(0.01, 1.0, 1.0)
    keys = pkg.DeviceArray.from_numpy(np.full((batch, k), 7.0, dtype=np.float32))
    vals = pkg.DeviceArray.from_numpy(np.full((batch, k), 7, dtype=np.uint32))
    if MODE["split"]:
        xp = pkg.DeviceArray((dsx.dsx_fc_split_bytes(batch, kdim) // 4,), np.uint32)
        wp = pkg.DeviceArray((dsx.dsx_fc_split_bytes(n, kdim) // 4,), np.uint32)
        pkg.check(dsx.dsx_fc_split(dX.ptr, kdim, 0, batch, kdim, xp.ptr))
        pkg.check(dsx.dsx_fc_split(dW.ptr, n, 1, n, kdim, wp.ptr))
        pkg.check(dsx.dsx_fc_topk_split(dX.ptr, kdim, dW.ptr, xp.ptr, wp.ptr, pkg.ptr(db), batch, kdim, n, act, C.byref(params), k, keys.ptr,
                                        vals.ptr, position, pkg.ptr(di), pkg.ptr(ds), pkg.ptr(de), pkg.ptr(dx)))
    else:
        pkg.check(dsx.dsx_fc_topk(dX.ptr, kdim, dW.ptr, pkg.ptr(db), batch, kdim, n, act, C.byref(params), k, keys.ptr, vals.ptr, position,
                                  pkg.ptr(di), pkg.ptr(ds), pkg.ptr(de), pkg.ptr(dx)))
    Z = pkg.DeviceArray((batch, n), np.float32)
    pkg.check(dsx.dsx_fc_forward(dX.ptr, kdim, dW.ptr, 0, pkg.ptr(db), Z.ptr, n, batch, kdim, n, 0, act, C.byref(params)))
    k2 = pkg.DeviceArray((batch, k), np.float32)
    v2 = pkg.DeviceArray((batch, k), np.uint32)
    if fidx is None:
        pkg.check(dsx.dsx_topk(Z.ptr, k2.ptr, v2.ptr, batch, n, k))
    else:
        pkg.check(dsx.dsx_topk_filtered(Z.ptr, k2.ptr, v2.ptr, batch, n, k, position, pkg.ptr(di), ds.ptr, de.ptr, dx.ptr, None))
    gk, gi, unit, tk, ti = keys.numpy(), vals.numpy(), Z.numpy(), k2.numpy(), v2.numpy()
    scores = unit.copy()
    if fidx is not None:
        orc.lib().orc_apply_filter(scores.ctypes.data, batch, n, 0, position, index.ctypes.data if index is not None else None,
                                   start.ctypes.data, end.ctypes.data, fidx.ctypes.data, None)
    m = min(k, n)
    assert_topk_parity(gk[:, :m], gi[:, :m], tk[:, :m], ti[:, :m], scores, what + " fused vs two calls")
    assert np.all(np.diff(gk.astype(np.float64), axis=1) <= 0)
    return gk, gi, unit, tk, ti


def layer(rng, batch, kdim, n, scale=0.3):
    X = rng.standard_normal((batch, kdim), dtype=np.float32)
    W = (rng.standard_normal((kdim, n), dtype=np.float32) * np.float32(scale)).astype(np.float32)
    bias = (rng.standard_normal(n, dtype=np.float32) * np.float32(0.2)).astype(np.float32)
    return X, W, bias


@pytest.mark.parametrize("n", [27278, 27279, 27280])      # rows of W aligned to 8, 4 and 16 bytes: three load widths
def test_fc_topk_catalogue_shape(pkg, dsx, orc, rng, knobs, n):
    batch, kdim, k = 300, 128, 10
    say("fc_topk n=%d" % n)
    X, W, bias = layer(rng, batch, kdim, n)
    start, end, fidx = random_csr(rng, batch, n, 400, empty_rows=(2,))
    gk, gi, unit, _, _ = run_both(pkg, dsx, orc, X, W, bias, ACT_SIGMOID, k, 0, None, start, end, fidx, "n=%d" % n)
    for b in range(batch):
        assert not set(gi[b].tolist()) & set(fidx[int(start[b]):int(end[b])].tolist())
    assert dsx.dsx_fc_topk_flagged(0) == 0
    # against the oracle's own forward arithmetic
    ref = orc.activation(orc.sgemm_acc(X, W, np.tile(bias, (batch, 1))), ACT_SIGMOID)
    assert_close(unit, ref, "stored layer", rel=1e-4, abs_floor=1e-3)
    rk, ri = orc.topk_filtered(ref, k, 0, None, start, end, fidx, None)
    scores = ref.copy()
    orc.lib().orc_apply_filter(scores.ctypes.data, batch, n, 0, 0, None, start.ctypes.data, end.ctypes.data, fidx.ctypes.data, None)
    assert_topk_parity(gk, gi, rk, ri, scores, "fused vs oracle")


@pytest.mark.parametrize("act", [ACT_SIGMOID, ACT_TANH, ACT_RELU, ACT_LINEAR, ACT_LRELU])
@pytest.mark.parametrize("k", [1, 33, 100, 256])
def test_fc_topk_ranges_activations_and_k(pkg, dsx, orc, rng, knobs, act, k):
    # a first block of 256 columns, so that 6,001 columns run several candidate ranges
    dsx.dsx_testing_set_fc_topk_first_columns(256)
    batch, kdim, n = 150, 64, 6001
    say("fc_topk act=%d k=%d" % (act, k))
    X, W, bias = layer(rng, batch, kdim, n)
    rows = 400
    start, end, fidx = random_csr(rng, rows, n + 30, 200)        # some indexes beyond the width: ignored
    index = rng.permutation(rows).astype(np.uint32)
    run_both(pkg, dsx, orc, X, W, bias, act, k, 17, index, start, end, fidx, "act=%d k=%d" % (act, k))
    run_both(pkg, dsx, orc, X, W, bias, act, k, what="unfiltered act=%d k=%d" % (act, k))


def test_fc_topk_unsupported_shapes_say_so(pkg, dsx, rng):
    X, W, bias = layer(rng, 8, 64, 500)
    dX, dW = dev(pkg, X), dev(pkg, W)
    keys = pkg.DeviceArray((8, 4), np.float32)
    vals = pkg.DeviceArray((8, 4), np.uint32)
    assert dsx.dsx_fc_topk(dX.ptr, 64, dW.ptr, None, 8, 64, 500, ACT_ELU, None, 4, keys.ptr, vals.ptr, 0, None, None, None, None) == -5
    assert dsx.dsx_fc_topk(dX.ptr + 4, 64, dW.ptr, None, 7, 60, 500, ACT_SIGMOID, None, 4, keys.ptr, vals.ptr, 0, None, None, None, None) == -5
    assert dsx.dsx_fc_topk(dX.ptr, 64, dW.ptr, None, 8, 64, 500, ACT_SIGMOID, None, 0, keys.ptr, vals.ptr, 0, None, None, None, None) == -1
    assert dsx.dsx_fc_topk_supported(64, dX.ptr, ACT_SIGMOID, None, None) == 1
    assert dsx.dsx_fc_topk_supported(64, dX.ptr, ACT_SIGMOID, None, dW.ptr) == 0     # filters with multipliers need the stored scores


def test_fc_topk_small_layers_and_short_rows(pkg, dsx, orc, rng, knobs):
    # narrower than the first block: the whole layer goes through the scratch matrix; k above the width leaves sentinels
    for batch, kdim, n, k in [(40, 64, 700, 20), (3, 16, 9, 12), (130, 128, 3000, 5)]:
        X, W, bias = layer(rng, batch, kdim, n)
        start, end, fidx = random_csr(rng, batch, n, min(n - 1, 50))
        gk, gi, _, tk, ti = run_both(pkg, dsx, orc, X, W, bias, ACT_SIGMOID, k, 0, None, start, end, fidx, "n=%d" % n)
        if not MODE["split"]:      # the same kernel, the same scan: bit for bit (split products round differently: parity rules, above)
            assert np.array_equal(gi, ti) and np.array_equal(gk.view(np.uint32), tk.view(np.uint32))


def test_fc_topk_ties_and_full_lists_are_recomputed_exactly(pkg, dsx, orc, rng, knobs):
    """Scores tied in their thousands: integer operands give exactly representable sums whatever the order, a ReLU turns half of
    them into the same 0, and a saturated sigmoid into the same 1.  Lists fill up, the rows are recomputed on the device, and
    the result must be the two-call path's bit for bit (score descending, then the lower column)."""
    dsx.dsx_testing_set_fc_topk_first_columns(256)
    dsx.dsx_testing_set_fc_topk_candidate_capacity(512)          # a third of row 5's columns tie at the top: more than a list holds
    batch, kdim, n, k = 70, 32, 9000, 50
    X = rng.integers(-2, 3, size=(batch, kdim)).astype(np.float32)
    W = rng.integers(-2, 3, size=(kdim, n)).astype(np.float32)
    bias = rng.integers(-1, 2, size=n).astype(np.float32)
    X[5] = 0.0                                           # every score of this row is act(bias): three distinct values
    start, end, fidx = random_csr(rng, batch, n, 300)
    for act in (ACT_RELU, ACT_LINEAR):
        dsx.dsx_fc_topk_flagged(1)
        gk, gi, _, tk, ti = run_both(pkg, dsx, orc, X, W, bias, act, k, 0, None, start, end, fidx, "ties act=%d" % act)
        assert np.array_equal(gi, ti) and np.array_equal(gk.view(np.uint32), tk.view(np.uint32))
    assert dsx.dsx_fc_topk_flagged(1) == 1               # row 5 at least filled its list
    # saturated sigmoids: 1.0f in every column, more than even a full-size list holds
    dsx.dsx_testing_set_fc_topk_candidate_capacity(0)
    Xs = np.abs(X) + 1.0
    Ws = np.abs(W) * 3.0 + 1.0
    gk, gi, _, tk, ti = run_both(pkg, dsx, orc, Xs.astype(np.float32), Ws.astype(np.float32), bias, ACT_SIGMOID, k, 0, None, start, end, fidx,
                                 "saturated")
    assert np.array_equal(gi, ti) and np.all(gk == 1.0)
    assert dsx.dsx_fc_topk_flagged(1) == 1


@pytest.mark.parametrize("act", [ACT_RELU, ACT_LINEAR, ACT_TANH, ACT_LRELU])
def test_fc_topk_listed_columns_score_zero_not_nothing(pkg, dsx, orc, rng, knobs, act):
    """utils/Filters.cpp:62 multiplies a listed column's score by 0 and kCalculateTopK then sees that zero: in a row with fewer
    than k scores above 0 the listed columns come back, lower column first.  Most scores here are negative (or a ReLU's 0), every
    row has listed columns on both sides of the first block, and the fused call must give the two-call path's result bit for bit."""
    dsx.dsx_testing_set_fc_topk_first_columns(256)
    batch, kdim, n, k = 48, 32, 5000, 40
    X = rng.integers(1, 3, size=(batch, kdim)).astype(np.float32)
    W = -rng.integers(0, 3, size=(kdim, n)).astype(np.float32)           # exact sums whatever the order
    bias = np.zeros(n, dtype=np.float32)
    W[:, rng.choice(n, 12, replace=False)] *= -1.0                        # a dozen columns score above 0: fewer than k
    start, end, fidx = random_csr(rng, batch, n, 120, empty_rows=(3,))
    say("fc_topk listed zeros act=%d" % act)
    dsx.dsx_fc_topk_flagged(1)
    gk, gi, unit, tk, ti = run_both(pkg, dsx, orc, X, W, bias, act, k, 0, None, start, end, fidx, "listed zeros act=%d" % act)
    assert np.array_equal(gi, ti) and np.array_equal(gk.view(np.uint32), tk.view(np.uint32))
    listed_back = sum(len(set(gi[b].tolist()) & set(fidx[int(start[b]):int(end[b])].tolist())) for b in range(batch))
    assert listed_back > 0, "the case does not reach a listed column"
    rk, ri = orc.topk_filtered(unit, k, 0, None, start, end, fidx, None)
    assert np.array_equal(gi, ri) and np.array_equal(gk, rk)              # (-0.0 == 0.0: the oracle keeps the product's sign)


def test_fc_topk_tiny_lists_overflow_on_ordinary_data(pkg, dsx, orc, rng, knobs):
    # 64 words per row and range: ordinary rows overflow, most rows are recomputed; results still under the parity rules
    dsx.dsx_testing_set_fc_topk_first_columns(128)
    dsx.dsx_testing_set_fc_topk_candidate_capacity(64)
    batch, kdim, n, k = 90, 128, 8000, 30
    X, W, bias = layer(rng, batch, kdim, n)
    start, end, fidx = random_csr(rng, batch, n, 500)
    run_both(pkg, dsx, orc, X, W, bias, ACT_SIGMOID, k, 0, None, start, end, fidx, "tiny lists")
    assert dsx.dsx_fc_topk_flagged(1) == 1
