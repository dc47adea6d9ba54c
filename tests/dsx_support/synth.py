"""Seeded synthetic workloads of the inference path: the five benchmark configurations and smaller relatives for tests.

Everything is generated with numpy's PCG64 from an explicit seed, so the CPU container and the GPU box produce the same
bytes.  Weights are always *given* to the network (never randomised on the device): the reference initialises weights
with cuRAND streams that cannot be reproduced, so parity is defined on supplied weights.

Weights are N(0, 0.01) read as variance 0.01 (standard deviation 0.1): with a smaller spread every sigmoid output of the
deep configurations collapses to 0.5 +- 1e-5 and the top-K comparison would only see ties.
"""
import os
from concurrent.futures import ThreadPoolExecutor

import numpy as np

from amazon_dsstne_amd import (ACT_RELU, ACT_SIGMOID, ATTR_BOOLEAN, ATTR_INDEXED, ATTR_SPARSE, T_FLOAT)

WEIGHT_STD = 0.1


class Problem:
    """One synthetic workload: a chain network plus a sparse input dataset."""

    def __init__(self):
        self.name = ""
        self.batch = 0
        self.widths = []          # [input width, layer 1 width, ..., output width]
        self.acts = []            # activation ordinal per layer
        self.weights = []         # W[l]: [widths[l]][widths[l+1]] fp32 row-major
        self.biases = []          # b[l]: [widths[l+1]] fp32
        self.k = 10
        self.attributes = ATTR_SPARSE | ATTR_BOOLEAN
        self.data_type = T_FLOAT
        self.examples = 0         # rows addressable through position (+ index)
        self.unique_examples = 0  # rows stored
        self.start = None         # uint64 [unique_examples]
        self.end = None           # uint64 [unique_examples]
        self.sparse_index = None  # uint32 [nnz]
        self.sparse_data = None   # values (None for Boolean data)
        self.index = None         # uint32 [examples] (Indexed datasets)
        self.data_weight = None
        self.law = {}             # how the workload was drawn (for reports): weight spread, index law, non-zeros per row

    @property
    def nnz(self):
        return int(self.sparse_index.shape[0])

    def batch_nnz(self, position=0, batch=None):
        batch = self.batch if batch is None else batch
        rows = np.arange(position, position + batch)
        if self.index is not None:
            rows = self.index[rows]
        return int((self.end[rows] - self.start[rows]).sum())


BIG = 1 << 26        # arrays of this many elements or more are drawn chunk by chunk on several threads
CHUNK = 1 << 24


def _threads():
    return min(16, os.cpu_count() or 4)


def normal_f32(rng, shape, scale=1.0):
    """N(0, scale^2) fp32 array.  Small arrays come straight from `rng`; big ones (config 4's matrices, the KNN table) are drawn
    in chunks of 2^24 values, each from its own PCG64 stream seeded from `rng`, on several threads: the same bytes for the same
    seed whatever the number of threads."""
    n = int(np.prod(shape, dtype=np.int64))
    if n < BIG:
        a = rng.standard_normal(shape, dtype=np.float32)
        if scale != 1.0:
            a *= np.float32(scale)
        return a
    flat = np.empty(n, dtype=np.float32)
    seeds = rng.integers(0, 1 << 62, size=(n + CHUNK - 1) // CHUNK)

    def fill(i):
        out = flat[i * CHUNK:(i + 1) * CHUNK]
        np.random.default_rng(int(seeds[i])).standard_normal(out=out, dtype=np.float32)
        if scale != 1.0:
            out *= np.float32(scale)
    with ThreadPoolExecutor(_threads()) as ex:
        list(ex.map(fill, range(len(seeds))))
    return flat.reshape(shape)


def make_weights(rng, widths, bias_std=0.0):
    ws, bs = [], []
    for i in range(len(widths) - 1):
        ws.append(normal_f32(rng, (widths[i], widths[i + 1]), WEIGHT_STD))
        if bias_std > 0:
            bs.append(rng.standard_normal(widths[i + 1], dtype=np.float32) * np.float32(bias_std))
        else:
            bs.append(np.zeros(widths[i + 1], dtype=np.float32))
    return ws, bs


def lognormal_counts(rng, rows, mean, sigma, lo, hi):
    """Non-zeros per row: lognormal with the given arithmetic mean, clipped to [lo, hi]."""
    mu = np.log(mean) - 0.5 * sigma * sigma
    c = np.rint(rng.lognormal(mu, sigma, rows)).astype(np.int64)
    return np.clip(c, lo, hi)


def zipf_rows(rng, n_items, s, counts):
    """CSR rows whose columns follow Zipf(s) over a random permutation of the items, distinct and ascending per row."""
    perm = rng.permutation(n_items).astype(np.uint32)
    p = 1.0 / np.power(np.arange(1, n_items + 1, dtype=np.float64), s)
    cdf = np.cumsum(p)
    cdf /= cdf[-1]
    rows = len(counts)
    start = np.zeros(rows, dtype=np.uint64)
    end = np.zeros(rows, dtype=np.uint64)
    chunks = []
    pos = 0
    for r in range(rows):
        c = int(min(counts[r], n_items))
        got = np.empty(0, dtype=np.int64)
        while got.shape[0] < c:
            draw = np.searchsorted(cdf, rng.random(2 * c + 16), side="left")
            draw = np.minimum(draw, n_items - 1)
            merged = np.concatenate([got, draw])
            _, first = np.unique(merged, return_index=True)
            got = merged[np.sort(first)]
        cols = np.sort(perm[got[:c]])
        chunks.append(cols)
        start[r] = pos
        pos += c
        end[r] = pos
    idx = np.concatenate(chunks).astype(np.uint32) if chunks else np.zeros(0, dtype=np.uint32)
    return start, end, idx


def uniform_rows(rng, n_items, counts):
    rows = len(counts)
    start = np.zeros(rows, dtype=np.uint64)
    end = np.zeros(rows, dtype=np.uint64)
    chunks = []
    pos = 0
    for r in range(rows):
        c = int(counts[r])
        cols = np.sort(rng.choice(n_items, size=c, replace=False)).astype(np.uint32)
        chunks.append(cols)
        start[r] = pos
        pos += c
        end[r] = pos
    idx = np.concatenate(chunks).astype(np.uint32) if chunks else np.zeros(0, dtype=np.uint32)
    return start, end, idx


def autoencoder(name, seed, n_items, hidden, batch, k, batches=1, zipf_s=None, nnz_mean=16, nnz_sigma=0.0, nnz_clip=(1, 1 << 30),
                analog=False, indexed=False, bias_std=0.0):
    """Sparse-input autoencoder: n_items -> hidden... (ReLU) -> n_items (sigmoid), top-k over the output."""
    rng = np.random.default_rng(seed)
    p = Problem()
    p.name = name
    p.batch = batch
    p.k = k
    p.widths = [n_items] + list(hidden) + [n_items]
    p.acts = [ACT_RELU] * len(hidden) + [ACT_SIGMOID]
    p.weights, p.biases = make_weights(rng, p.widths, bias_std)
    rows = batch * batches
    if nnz_sigma > 0:
        counts = lognormal_counts(rng, rows, nnz_mean, nnz_sigma, nnz_clip[0], nnz_clip[1])
    else:
        counts = np.full(rows, nnz_mean, dtype=np.int64)
    if zipf_s is None:
        p.start, p.end, p.sparse_index = uniform_rows(rng, n_items, counts)
    else:
        p.start, p.end, p.sparse_index = zipf_rows(rng, n_items, zipf_s, counts)
    p.unique_examples = rows
    p.examples = rows
    p.attributes = ATTR_SPARSE
    if analog:
        # rating-like values 0.5, 1.0, ..., 5.0
        p.sparse_data = (rng.integers(1, 11, size=p.sparse_index.shape[0]).astype(np.float32) * np.float32(0.5))
        p.data_type = T_FLOAT
    else:
        p.attributes |= ATTR_BOOLEAN
    if indexed:
        p.attributes |= ATTR_INDEXED
        p.index = rng.permutation(rows).astype(np.uint32)
    p.law = {"seed": seed, "weight_std": WEIGHT_STD, "bias_std": bias_std,
             "index_law": ("uniform without replacement" if zipf_s is None else "Zipf(s=%g) over a random permutation of the items, without replacement within a row" % zipf_s),
             "nnz_per_row": ("%d" % nnz_mean if nnz_sigma <= 0 else "lognormal(mean %g, sigma %g) clipped to [%d, %d]" % (nnz_mean, nnz_sigma, nnz_clip[0], nnz_clip[1])),
             "values": ("0.5 .. 5.0 in steps of 0.5, uniform" if analog else "1 (Boolean)"), "indexed_rows": bool(indexed)}
    return p


def config(n, seed=None, batches=1):
    """The five configurations of the benchmark definition (1-based)."""
    if n == 1:
        return autoencoder("cfg1-tiny", 1001 if seed is None else seed, 1024, [64], 32, 10, batches, None, 16)
    if n == 2:
        return autoencoder("cfg2-catalogue-27278", 1002 if seed is None else seed, 27278, [128, 128, 128], 1024, 10, batches, 1.0, 144,
                           1.0, (5, 2000))
    if n == 3:
        return autoencoder("cfg3-analog-indexed-27278", 1003 if seed is None else seed, 27278, [1024, 1024], 4096, 10, batches, 1.0, 144,
                           1.0, (5, 2000), analog=True, indexed=True)
    if n == 4:
        return autoencoder("cfg4-large-1M", 1004 if seed is None else seed, 1000000, [512], 4096, 100, batches, 1.1, 50, 1.0, (1, 1000))
    raise ValueError("config %r: 1..4 are networks; use knn_config() for 5" % (n,))


class KnnProblem:
    def __init__(self):
        self.name = ""
        self.items = None      # [M][D] fp32 row-major, rows L2-normalised
        self.queries = None    # [Q][D]
        self.k = 100

    def column_major_padded(self, pad_to=8):
        """Item table as KnnData::load builds it (knn/KnnData.cpp:186-207): rows padded to a multiple of 8, column-major."""
        m, d = self.items.shape
        rows = (m + pad_to - 1) // pad_to * pad_to
        t = np.empty((d, rows), dtype=np.float32)
        t[:, m:] = 0
        step = 1 << 16

        def block(r0):
            t[:, r0:min(r0 + step, m)] = self.items[r0:r0 + step].T
        with ThreadPoolExecutor(_threads()) as ex:
            list(ex.map(block, range(0, m, step)))
        return t, rows, rows - m


def knn_config(seed=1005, items=2000000, queries=4096, dim=256, k=100):
    rng = np.random.default_rng(seed)
    p = KnnProblem()
    p.name = "cfg5-knn-%dx%d" % (items, dim)
    p.k = k
    it = normal_f32(rng, (items, dim))
    step = 1 << 16

    def normalise(r0):
        blk = it[r0:r0 + step]
        blk /= np.linalg.norm(blk, axis=1, keepdims=True)
    with ThreadPoolExecutor(_threads()) as ex:
        list(ex.map(normalise, range(0, items, step)))
    q = rng.standard_normal((queries, dim), dtype=np.float32)
    q /= np.linalg.norm(q, axis=1, keepdims=True)
    p.items, p.queries = it, q
    return p
