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


def forward_f64(p, rows):
    """The chain network of a synth.Problem in float64 for the given batch positions (numpy only): the ground truth that both
    the fp32 oracle and the GPU approximate."""
    sig = lambda z: 1.0 / (1.0 + np.exp(-z))
    acts = {0: sig, 1: np.tanh, 2: lambda z: np.maximum(z, 0.0), 3: lambda z: z}
    out = []
    for b in rows:
        r = int(p.index[b]) if p.index is not None else int(b)
        s, e = int(p.start[r]), int(p.end[r])
        cols = p.sparse_index[s:e]
        vals = np.ones(e - s) if p.sparse_data is None else p.sparse_data[s:e].astype(np.float64)
        h = p.biases[0].astype(np.float64) + vals @ p.weights[0][cols].astype(np.float64)
        h = acts[p.acts[0]](h)
        for l in range(1, len(p.weights)):
            h = acts[p.acts[l]](p.biases[l].astype(np.float64) + h @ p.weights[l].astype(np.float64))
        out.append(h)
    return np.asarray(out)


FALLBACK_LOG = []  # one (what, rows compared, rows judged against float64, worst relative error vs the oracle) per call


def assert_units_close(got, ref, p, position=0, what="activations", rel=REL_TOL, abs_floor=1e-3, positions=None, max_fallback_rows=0):
    """Layer outputs against the fp32 oracle: every row within `rel` of it (relative to max(|ref|, abs_floor)).

    `max_fallback_rows` (0 unless the caller states a ceiling) is how many rows may miss that and be judged against the float64
    ground truth instead: where deep sums cancel, two fp32 summation orders part by more than `rel`, and such a row passes if
    its largest deviation from the truth is at most twice the oracle's own, plus one part in 10^6 of the row's largest value.
    Every call prints one `[parity]` line with the number of rows that took this second rule and the worst error against the
    oracle, and appends the same to FALLBACK_LOG.  Row i of got / ref is batch position `position + i`, or positions[i]."""
    got64, ref64 = np.asarray(got, dtype=np.float64), np.asarray(ref, dtype=np.float64)
    err = np.abs(got64 - ref64) / np.maximum(np.abs(ref64), abs_floor)
    worst = float(err.max()) if err.size else 0.0
    bad_rows = np.nonzero((err > rel).any(axis=1))[0]
    FALLBACK_LOG.append((what, int(got64.shape[0]), int(bad_rows.size), worst))
    print("[parity] %s: %d rows, %d beyond %.0e of the oracle (ceiling %d), worst relative error %.3g" % (
        what, got64.shape[0], bad_rows.size, rel, max_fallback_rows, worst), flush=True)
    if bad_rows.size == 0:
        return worst
    assert bad_rows.size <= max_fallback_rows, "%s: %d rows differ from the oracle by more than %.0e (ceiling %d), worst %.3g" % (
        what, bad_rows.size, rel, max_fallback_rows, worst)
    truth = forward_f64(p, (position + bad_rows) if positions is None else np.asarray(positions)[bad_rows])
    e_got = np.abs(got64[bad_rows] - truth)
    e_ref = np.abs(ref64[bad_rows] - truth)
    # rounding errors fall on different elements in the two computations: compare their levels row by row
    level_got, level_ref = e_got.max(axis=1), e_ref.max(axis=1)
    worse = level_got > 2.0 * level_ref + 1e-6 * np.abs(truth).max(axis=1) + 1e-9
    print("[parity] %s: the %d rows against float64: largest deviation %.3g, the oracle's %.3g" % (
        what, bad_rows.size, float(level_got.max()), float(level_ref.max())), flush=True)
    assert not worse.any(), "%s: %d rows are further from the float64 result than the fp32 oracle is (worst %.3g vs oracle %.3g)" % (
        what, int(worse.sum()), float(level_got.max()), float(level_ref.max()))
    return worst
