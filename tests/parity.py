"""Comparison rules of the parity tests.

Integer / index work on identical inputs: bit exact.  Floating point: scores within 1e-4 relative of the oracle, top-K
indices identical except where the oracle's own scores of the two candidates differ by less than 1e-5 (ties are broken by
the lower index on both sides, so exact ties agree as well).
"""
import numpy as np

REL_TOL = 1e-4
TIE_GAP = 1e-5


def assert_close(got, ref, what="values", rel=REL_TOL, abs_floor=1e-6):
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    err = np.abs(got - ref) / np.maximum(np.abs(ref), abs_floor)
    worst = float(err.max()) if err.size else 0.0
    assert worst <= rel, "%s: max relative error %.3g > %.1g at %s (got %r, ref %r)" % (
        what, worst, rel, np.unravel_index(int(err.argmax()), err.shape), got.flat[int(err.argmax())], ref.flat[int(err.argmax())])
    return worst


def assert_topk_exact(keys, idx, ref_keys, ref_idx, what="top-K"):
    assert np.array_equal(idx, ref_idx), "%s: indices differ in %d slots" % (what, int((idx != ref_idx).sum()))
    assert np.array_equal(keys.view(np.uint32), ref_keys.view(np.uint32)), "%s: keys differ bitwise" % what


def assert_topk_parity(keys, idx, ref_keys, ref_idx, ref_scores, what="top-K"):
    """ref_scores: the oracle's score matrix (after filtering) that ref_keys/ref_idx were selected from."""
    assert keys.shape == ref_keys.shape and idx.shape == ref_idx.shape
    mism = idx != ref_idx
    if mism.any():
        rows, cols = np.nonzero(mism)
        gap = np.abs(ref_scores[rows, idx[rows, cols]].astype(np.float64) - ref_keys[rows, cols].astype(np.float64))
        assert gap.max() < TIE_GAP, "%s: %d index mismatches outside near-ties, worst oracle score gap %.3g" % (
            what, int((gap >= TIE_GAP).sum()), float(gap.max()))
    assert_close(keys, ref_keys, what + " scores")
    return int(mism.sum())


def check_topk_invariants(scores, keys, idx, k, width=None):
    """Size-independent properties of a correct top-K: sorted, consistent, and nothing outside beats the k-th."""
    batch = scores.shape[0]
    width = scores.shape[1] if width is None else width
    m = min(k, width)
    assert np.all(idx[:, :m] < width)
    rows = np.arange(batch)[:, None]
    assert np.array_equal(scores[rows, idx[:, :m]] + np.float32(0), keys[:, :m]), "reported key is not the score at the reported index"
    d = np.diff(keys[:, :m].astype(np.float64), axis=1)
    assert np.all(d <= 0), "keys are not descending"
    same = d == 0
    if same.any():
        assert np.all(np.diff(idx[:, :m].astype(np.int64), axis=1)[same] > 0), "equal keys are not in ascending index order"
    for b in range(batch):
        assert len(set(idx[b, :m].tolist())) == m, "duplicate index in row %d" % b
    if m < width:
        masked = scores[:, :width].copy()
        masked[rows, idx[:, :m]] = -np.inf
        assert np.all(masked.max(axis=1) <= keys[:, m - 1]), "an unselected score beats the k-th key"
