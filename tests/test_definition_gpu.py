"""Networks built from JSON definition files (LoadNeuralNetworkJSON, engine/NNNetwork.cpp:2792-3760) on the GPU: layers sized
from data sets, weight initialisation schemes (engine/NNWeight.cpp:500-561), and the forward pass of a definition with several
sources, a skip connection and tied (shared, transposed) weights (engine/NNLayer.cpp:994-1168) against fp64 numpy."""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LDL = os.path.join(ROOT, "tests", "golden", "ldl")

ATTR_SPARSE, ATTR_BOOLEAN = 1, 2
T_UINT, T_FLOAT = 0, 4


def write_dataset_file(path, datasets):
    """datasets: list of (name, width, start, end, index, values or None) written with the attribute and variable names the
    reference's dataset files carry (engine/NNTypes.cpp:1081-1358), through scipy's independent NetCDF writer."""
    from scipy.io import netcdf_file
    f = netcdf_file(path, "w", version=2)
    f.datasets = np.int32(len(datasets))
    for n, (name, width, start, end, index, values) in enumerate(datasets):
        s = str(n)
        setattr(f, "name" + s, name)
        setattr(f, "attributes" + s, np.int32(ATTR_SPARSE | (ATTR_BOOLEAN if values is None else 0)))
        setattr(f, "kind" + s, np.int32(0))
        setattr(f, "dataType" + s, np.int32(T_UINT if values is None else T_FLOAT))
        setattr(f, "dimensions" + s, np.int32(1))
        setattr(f, "width" + s, np.int32(width))
        f.createDimension("examplesDim" + s, len(start))
        f.createDimension("sparseDataDim" + s, len(index))
        for var, arr in (("sparseStart", start), ("sparseEnd", end)):
            v = f.createVariable(var + s, "i", ("examplesDim" + s,))
            v[:] = np.asarray(arr, dtype=np.int32)
        v = f.createVariable("sparseIndex" + s, "i", ("sparseDataDim" + s,))
        v[:] = np.asarray(index, dtype=np.int32)
        if values is not None:
            v = f.createVariable("sparseData" + s, "f", ("sparseDataDim" + s,))
            v[:] = np.asarray(values, dtype=np.float32)
    f.close()


def random_rows(rng, rows, width, lo, hi):
    start, end, index = [], [], []
    for _ in range(rows):
        n = int(rng.integers(lo, hi + 1))
        cols = np.sort(rng.choice(width, size=n, replace=False))
        start.append(len(index))
        index.extend(int(c) for c in cols)
        end.append(len(index))
    return np.array(start, np.uint64), np.array(end, np.uint64), np.array(index, np.uint32)


def dense(rows, width, start, end, index, values=None):
    X = np.zeros((rows, width), dtype=np.float64)
    for r in range(rows):
        for j in range(int(start[r]), int(end[r])):
            X[r, index[j]] += 1.0 if values is None else float(values[j])
    return X


def sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


def test_movielens_definition_sizes_layers_and_initialises_weights(pkg, dsx, orc, synth, tmp_path):
    """The reference's MovieLens sample definition: input and output are "auto", so both take the data sets' width; hidden
    and output weights start from the default scheme (Xavier: uniform, |w| <= sqrt(6 / (n_in + n_out)) / 2, biases 0);
    the seed fixes the values.  Prediction then agrees with the CPU restatement fed the same weights."""
    from amazon_dsstne_amd import host_api
    p = synth.config(1, batches=2)                   # 64 rows over 1024 items, 16 per row, batch 32
    N = p.widths[0]
    path = str(tmp_path / "gl.nc")
    write_dataset_file(path, [("gl_input", N, p.start, p.end, p.sparse_index, None), ("gl_output", N, p.start, p.end, p.sparse_index, None)])
    definition = os.path.join(LDL, "movielens_config.json")
    net = host_api.DefinedNetwork(definition, path, p.batch, p.k, seed=7)
    W1, b1 = net.get_weights("Input", "Hidden", N, 128)
    W2, b2 = net.get_weights("Hidden", "Output", 128, N)
    bound = 0.5 * np.sqrt(6.0 / (N + 128))
    for W in (W1, W2):
        assert np.abs(W).max() <= bound * (1 + 1e-6)
        assert np.abs(W).max() > 0.98 * bound                   # the range is used
        assert abs(W.mean()) < 0.02 * bound
        assert abs(W.std() - bound / np.sqrt(3.0)) < 0.02 * bound   # a uniform law, not a normal one
    assert not np.array_equal(W1.ravel()[:4096], W2.ravel()[:4096])
    assert (b1 == 0).all() and (b2 == 0).all()

    # same weights into the CPU restatement: Input -> Hidden (sigmoid) -> Output (sigmoid), top-10 with the input filter
    p.widths = [N, 128, N]
    p.acts = [0, 0]
    p.weights, p.biases = [W1, W2], [b1, b2]
    for pos in (0, 32):
        net.predict_batch(pos)
        got = net.units("Output", rows=p.batch, width=N)
        _, want, _, _ = orc.forward(p, pos, p.batch, filtered=False, want_unit=True, want_topk=False)
        _, _, keys, idx = orc.forward(p, pos, p.batch, filtered=True)
        assert np.allclose(got, want, rtol=1e-4, atol=1e-6)
        net.topk(p.k, filter_dataset="gl_input")
        gk, gi = net.get_topk(p.batch)
        mism = gi != idx
        if mism.any():
            r, c = np.nonzero(mism)
            assert np.abs(want[r, gi[r, c]].astype(np.float64) - keys[r, c]).max() < 1e-5
            for row in range(p.batch):                               # and a swapped-in item is never one of the row's own
                own = p.sparse_index[int(p.start[pos + row]):int(p.end[pos + row])]
                assert not np.isin(gi[row], own).any()
        assert np.allclose(gk, keys, rtol=1e-4, atol=1e-7)
    net.close()

    # the seed decides the starting weights
    again = host_api.DefinedNetwork(definition, path, p.batch, p.k, seed=7)
    W1b, _ = again.get_weights("Input", "Hidden", N, 128)
    again.close()
    other = host_api.DefinedNetwork(definition, path, p.batch, p.k, seed=8)
    W1c, _ = other.get_weights("Input", "Hidden", N, 128)
    other.close()
    assert np.array_equal(W1, W1b)
    assert not np.array_equal(W1, W1c)


def test_definition_with_tied_weights_skip_and_two_sources(pkg, dsx, tmp_path):
    """tests/golden/ldl/tied_autoencoder.json: Enc = lrelu(X W1 + b); Mid = elu(Enc Wm + b + Enc) (skip); Side = tanh(X Ws +
    b + Enc We + b') (two sources, one of them the sparse input); Out = sigmoid(Mid W1^T + b + Side Wo + b') (first source tied to
    Input0 -> Enc, transposed).  Starting values per scheme, then random values, forward pass against fp64."""
    from amazon_dsstne_amd import host_api
    rng = np.random.default_rng(11)
    B, rows, N, H = 16, 40, 96, 32
    start, end, index = random_rows(rng, rows, N, 0, 12)        # some rows are empty
    path = str(tmp_path / "tied.nc")
    write_dataset_file(path, [("in", N, start, end, index, None), ("out", N, start, end, index, None)])
    net = host_api.DefinedNetwork(os.path.join(LDL, "tied_autoencoder.json"), path, B, 8, seed=3)
    W1, b1 = net.get_weights("Input0", "Enc", N, H)
    assert abs(W1.std() - 0.01) < 0.001 and abs(W1.mean()) < 0.001          # Gaussian, scale 0.01
    assert 3.0 < np.abs(W1).max() / 0.01 < 6.0                               # with tails, unlike a uniform law
    assert (b1 == 0.5).all()                                                 # "Bias": 0.5
    Wm, bm = net.get_weights("Enc", "Mid", H, H)
    assert (Wm == -0.03125).all() and (bm == 0).all()                        # Constant: 0 * scale - s, as the reference computes it
    Wo, _ = net.get_weights("Side", "Out", H, N)
    assert np.abs(Wo).max() <= 0.05 and np.abs(Wo).max() > 0.049             # Uniform, scale 0.05
    _, bt = net.get_weights("Mid", "Out", 0, 0, biases=N)                    # a tied connection owns biases only
    assert (bt == 0).all()

    def rnd(*shape):
        return (rng.standard_normal(shape) * 0.3).astype(np.float32)
    W1, Wm, Ws, We, Wo = rnd(N, H), rnd(H, H), rnd(N, H), rnd(H, H), rnd(H, N)
    b1, bm, bs, be, bt, bo = rnd(H), rnd(H), rnd(H), rnd(H), rnd(N), rnd(N)
    net.set_weights("Input0", "Enc", W1, b1)
    net.set_weights("Enc", "Mid", Wm, bm)
    net.set_weights("Input0", "Side", Ws, bs)
    net.set_weights("Enc", "Side", We, be)
    net.set_weights("Mid", "Out", None, bt)
    net.set_weights("Side", "Out", Wo, bo)
    X = dense(rows, N, start, end, index)
    d = np.float64
    z = X @ W1.astype(d) + b1
    enc = np.where(z > 0, z, 0.125 * z)                                      # network-wide "Slope"
    z = enc @ Wm.astype(d) + bm + enc
    mid = np.where(z > 0, z, 0.75 * (np.exp(np.minimum(z, 0)) - 1.0))        # the layer's own "ELUAlpha"
    side = np.tanh(X @ Ws.astype(d) + bs + enc @ We.astype(d) + be)
    out = sigmoid(mid @ W1.astype(d).T + bt + side @ Wo.astype(d) + bo)
    for pos in (0, 16, 32):                                                  # the last batch holds 8 rows
        n = min(B, rows - pos)
        net.predict_batch(pos)
        for layer, want, width in (("Enc", enc, H), ("Mid", mid, H), ("Side", side, H), ("Out", out, N)):
            got = net.units(layer, rows=B, width=width)[:n]
            assert np.allclose(got, want[pos:pos + n], rtol=1e-4, atol=1e-5), layer
        net.topk(8, layer="Out")
        gk, gi = net.get_topk(n, 8, layer="Out")
        order = np.argsort(-out[pos:pos + n], axis=1, kind="stable")[:, :8]
        want_k = np.take_along_axis(out[pos:pos + n], order, axis=1)
        assert np.allclose(gk, want_k, rtol=1e-4, atol=1e-6)
        mism = gi != order
        if mism.any():
            r, c = np.nonzero(mism)
            assert np.abs(out[pos + r, gi[r, c]] - want_k[r, c]).max() < 1e-5
    net.close()


def test_definition_errors_are_reported(pkg, dsx, tmp_path):
    from amazon_dsstne_amd import host_api
    rng = np.random.default_rng(5)
    start, end, index = random_rows(rng, 8, 64, 1, 4)
    path = str(tmp_path / "d.nc")
    write_dataset_file(path, [("other", 64, start, end, index, None)])
    with pytest.raises(host_api.DsxError):
        host_api.DefinedNetwork(os.path.join(LDL, "movielens_config.json"), path, 8, 4)     # "auto" names data sets that are not there
    bad = tmp_path / "bad.json"
    bad.write_text('{"Layers": [{"N": 4}, {"N": 4, "Colour": 1}]}')
    with pytest.raises(host_api.DsxError):
        host_api.DefinedNetwork(str(bad), path, 8, 4)
