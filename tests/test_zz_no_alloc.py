"""dsx_topk_filtered_static (the entry point that allocates nothing: partial lists in a fixed device array) against
dsx_topk_filtered / dsx_topk, bit for bit, through the C ABI.  Two calls in a row, the second with a smaller input, so that
whatever the first call left in the shared scratch is still there when the second one runs.  Needs an MI355X."""
import numpy as np
import pytest

from parity import assert_topk_exact, check_topk_invariants
from test_oracle import random_csr

pytestmark = pytest.mark.gpu


def say(msg):
    print("[case] " + msg, flush=True)


def dev(pkg, a):
    return None if a is None else pkg.DeviceArray.from_numpy(a)


def both_calls(pkg, dsx, scores, k, start, end, fidx, fmul):
    """Returns (static keys, static idx, reference keys, reference idx): the reference is dsx_topk_filtered, or dsx_topk when
    there is no filter."""
    batch, width = scores.shape
    d, ds, de, dx, dm = (dev(pkg, x) for x in (scores, start, end, fidx, fmul))
    out = []
    for static in (True, False):
        keys = pkg.DeviceArray.from_numpy(np.full((batch, k), 123.0, dtype=np.float32))
        vals = pkg.DeviceArray.from_numpy(np.full((batch, k), 77, dtype=np.uint32))
        if static:
            pkg.check(dsx.dsx_topk_filtered_static(d.ptr, keys.ptr, vals.ptr, batch, width, k, 0, None, pkg.ptr(ds), pkg.ptr(de),
                                                   pkg.ptr(dx), pkg.ptr(dm)))
        elif fidx is None:
            pkg.check(dsx.dsx_topk(d.ptr, keys.ptr, vals.ptr, batch, width, k))
        else:
            pkg.check(dsx.dsx_topk_filtered(d.ptr, keys.ptr, vals.ptr, batch, width, k, 0, None, ds.ptr, de.ptr, dx.ptr, pkg.ptr(dm)))
        out += [keys.numpy(), vals.numpy()]
    return out


def test_static_scratch_two_calls_second_smaller(pkg, dsx, orc, rng):
    # (batch, width, k, longest filter row): the first case splits every row over many segments (6 rows on 256 CUs) and, being wider
    # than 262,080 columns with a filter, over at least three because of the bitmap; the second is smaller in every dimension and
    # still split; the third has one segment per row and touches no scratch
    for batch, width, k, maxnnz in [(6, 600000, 100, 1000), (4, 70000, 10, 300), (2048, 3000, 16, 50)]:
        say("static filtered batch=%d width=%d k=%d" % (batch, width, k))
        scores = rng.random((batch, width), dtype=np.float32)
        start, end, fidx = random_csr(rng, batch, width, maxnnz, empty_rows=(1,))
        fmul = (rng.random(len(fidx), dtype=np.float32) * 3).astype(np.float32)
        sk, si, rk, ri = both_calls(pkg, dsx, scores, k, start, end, fidx, fmul)
        assert_topk_exact(sk, si, rk, ri, "static vs dsx_topk_filtered")
        ok, oi = orc.topk_filtered(scores, k, 0, None, start, end, fidx, fmul)
        assert_topk_exact(sk, si, ok, oi, "static vs oracle")


def test_static_scratch_unfiltered_then_smaller(pkg, dsx, orc, rng):
    # 300 rows: 4 workgroups per row (300 * 4 * 256 = 307,200 words of lists); then a smaller call whose lists overlay the first call's
    for batch, width, k in [(300, 40000, 256), (5, 90000, 7), (1500, 3000, 256)]:
        say("static unfiltered batch=%d width=%d k=%d" % (batch, width, k))
        scores = rng.standard_normal((batch, width), dtype=np.float32)
        scores[0, ::2] = scores[0, 1]          # ties across segments: order by column
        sk, si, rk, ri = both_calls(pkg, dsx, scores, k, None, None, None, None)
        assert_topk_exact(sk, si, rk, ri, "static vs dsx_topk")
        check_topk_invariants(scores, sk, si, k)


def test_static_scratch_rejects_what_cannot_fit(pkg, dsx, rng):
    # filtered, 600,000 columns: the bitmap needs 3 segments per row; 4,000 rows x 3 x 256 words > 2^21 -> clear error, nothing launched
    batch, width, k = 4000, 600000, 256
    scores = pkg.DeviceArray((16, 16), np.float32)     # never read: the call must fail before any launch
    keys = pkg.DeviceArray((16, 16), np.float32)
    vals = pkg.DeviceArray((16, 16), np.uint32)
    start = pkg.DeviceArray((batch,), np.uint64)
    rc = dsx.dsx_topk_filtered_static(scores.ptr, keys.ptr, vals.ptr, batch, width, k, 0, None, start.ptr, start.ptr, start.ptr, None)
    assert rc == -1
    assert b"fixed scratch" in dsx.dsx_last_error()
    pkg.check(dsx.dsx_sync())
