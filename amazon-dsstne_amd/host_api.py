"""ctypes binding of libdsstne_amd.so (include/dsstne_capi.h): the C++ inference classes behind a C ABI.

Plumbing only, like the JNI layer of the reference: it marshals numpy arrays into the calls of dsstne_capi.h.
"""
import ctypes as C
import os

import numpy as np

from . import HOST_LIB_PATH, NP_TO_DSX, DsxError, load_library

_u32, _u64, _f32, _vp, _int, _sz, _cp = C.c_uint32, C.c_uint64, C.c_float, C.c_void_p, C.c_int, C.c_size_t, C.c_char_p
_lib = None

SIGNATURES = {
    "dsstne_load": ([_cp, _u32, _int], _vp),
    "dsstne_create": ([_cp, _u32, _int, _u32, C.POINTER(_cp), _vp, _vp, _vp, _vp, C.POINTER(_cp), _u32, _vp, _vp, C.POINTER(_vp),
                       C.POINTER(_vp)], _vp),
    "dsstne_shutdown": ([_vp], None),
    "dsstne_save_network": ([_vp, _cp], _int),
    "dsstne_load_datasets": ([_vp, _u32, C.POINTER(_cp), _vp, _vp, _vp, _vp, _vp], _int),
    "dsstne_add_sparse_dataset": ([_vp, _cp, _u32, _u32, _u32, _u32, _u64, _int, _int, _int, _int], _int),
    "dsstne_load_sparse_data": ([_vp, _cp, _vp, _vp, _vp, _vp], _int),
    "dsstne_load_indexed_data": ([_vp, _cp, _vp], _int),
    "dsstne_load_data_weight": ([_vp, _cp, _vp], _int),
    "dsstne_load_dense_data": ([_vp, _cp, _vp], _int),
    "dsstne_predict_batch": ([_vp, _u32], _int),
    "dsstne_topk": ([_vp, _cp, _u32, _cp], _int),
    "dsstne_get_topk": ([_vp, _cp, _u32, _u32, _vp, _vp], _int),
    "dsstne_predict": ([_vp, _cp, _u32, _cp, _vp, _vp], _int),
    "dsstne_get_units": ([_vp, _cp, _vp, _sz], _int),
    "dsstne_get_unit_buffer": ([_vp, _cp], _vp),
    "dsstne_set_units": ([_vp, _cp, _vp, _sz], _int),
    "dsstne_sync": ([], _int),
    "dsstne_timer_start": ([], _int),
    "dsstne_timer_stop": ([C.POINTER(_f32)], _int),
    "dsstne_last_error": ([], _cp),
    "dsstne_knn_create": ([_u32, _u32], _vp),
    "dsstne_knn_load": ([_vp, _vp, _u32, _u32, C.POINTER(_cp)], _int),
    "dsstne_knn_load_file": ([_vp, _cp, C.c_char, C.c_char], _int),
    "dsstne_load_definition": ([_cp, _cp, _u32, _int, C.c_uint64], _vp),
    "dsstne_get_weights": ([_vp, _cp, _cp, _vp, C.c_size_t, _vp, C.c_size_t], _int),
    "dsstne_set_weights": ([_vp, _cp, _cp, _vp, C.c_size_t, _vp, C.c_size_t], _int),
    "dsstne_get_topk_previous": ([_vp, _cp, _u32, _u32, _vp, _vp], _int),
    "dsstne_set_lanes": ([_vp, _u32], _int),
    "dsstne_set_deferred_output": ([_vp, _int], _int),
    "dsstne_set_split_products": ([_vp, _int], _int),
    "dsstne_knn_create_typed": ([_u32, _u32, _cp], _vp),
    "dsstne_knn_search": ([_vp, _u32, _vp, _u32, _vp, _vp], _int),
    "dsstne_knn_elapsed": ([_vp, C.POINTER(_f32), C.POINTER(_f32)], _int),
    "dsstne_knn_destroy": ([_vp], None),
}


def load_host_library():
    global _lib
    if _lib is not None:
        return _lib
    load_library()   # libdsx_hip.so first (RTLD_GLOBAL), then the host library that links against it
    if not os.path.exists(HOST_LIB_PATH):
        raise DsxError("host library %s is missing: build it with __graft_entry__.build()" % HOST_LIB_PATH)
    lib = C.CDLL(HOST_LIB_PATH)
    for name, (args, res) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = res
    _lib = lib
    return lib


def _check(rc):
    if rc != 0:
        raise DsxError("dsstne call failed: %s" % load_host_library().dsstne_last_error().decode())


def _strs(items):
    arr = (_cp * len(items))(*[(s.encode() if s is not None else None) for s in items])
    return arr


class Network:
    """One in-memory chain network (synth.Problem) behind the C++ NNNetwork API."""

    def __init__(self, problem, max_k=None, dataset="input", filter_dataset=None):
        self.lib = load_host_library()
        p = self.p = problem
        self.dataset = dataset
        n = len(p.widths)
        names = ["Input"] + ["Hidden%d" % i for i in range(1, n - 1)] + ["Output"]
        kinds = np.array([0] + [1] * (n - 2) + [2], dtype=np.uint32)
        widths = np.array(p.widths, dtype=np.uint32)
        acts = np.array([3] + list(p.acts), dtype=np.uint32)
        sparse = np.array([1] + [0] * (n - 1), dtype=np.uint32)
        dsets = [dataset] + [None] * (n - 1)
        nw = n - 1
        w_in = np.arange(0, nw, dtype=np.uint32)
        w_out = np.arange(1, nw + 1, dtype=np.uint32)
        self._keep = [np.ascontiguousarray(w, dtype=np.float32) for w in p.weights] + [np.ascontiguousarray(b, dtype=np.float32) for b in p.biases]
        W = (_vp * nw)(*[w.ctypes.data for w in self._keep[:nw]])
        B = (_vp * nw)(*[b.ctypes.data for b in self._keep[nw:]])
        self.max_k = max_k or p.k
        self.ctx = self.lib.dsstne_create(p.name.encode(), p.batch, self.max_k, n, _strs(names), kinds.ctypes.data, widths.ctypes.data,
                                          acts.ctypes.data, sparse.ctypes.data, _strs(dsets), nw, w_in.ctypes.data, w_out.ctypes.data, W, B)
        if not self.ctx:
            raise DsxError("dsstne_create failed: %s" % self.lib.dsstne_last_error().decode())

    def bind_input(self, boolean=None):
        """Creates the input dataset with the problem's shape (all rows resident) and loads it."""
        p = self.p
        from . import ATTR_BOOLEAN, ATTR_INDEXED, ATTR_WEIGHTED, T_FLOAT
        is_bool = bool(p.attributes & ATTR_BOOLEAN) if boolean is None else boolean
        dtype = p.data_type if p.sparse_data is not None else T_FLOAT
        _check(self.lib.dsstne_add_sparse_dataset(self.ctx, self.dataset.encode(), dtype, p.widths[0], p.examples, p.unique_examples,
                                                  max(p.nnz, 1), 1 if (p.attributes & ATTR_INDEXED) else 0,
                                                  1 if (p.attributes & ATTR_WEIGHTED) else 0, 1 if is_bool else 0, 1))
        data = p.sparse_data
        if data is None and not is_bool:
            data = np.ones(p.nnz, dtype=np.float32)   # API-fed 0/1 data that is not marked Boolean runs the analog kernel with 1.0
        self.load_sparse(p.start, p.end, data, p.sparse_index)
        if p.index is not None:
            _check(self.lib.dsstne_load_indexed_data(self.ctx, self.dataset.encode(), np.ascontiguousarray(p.index, np.uint32).ctypes.data))
        if p.data_weight is not None:
            _check(self.lib.dsstne_load_data_weight(self.ctx, self.dataset.encode(), np.ascontiguousarray(p.data_weight, np.float32).ctypes.data))

    def load_sparse(self, start, end, data, index, name=None):
        start = np.ascontiguousarray(start, np.uint64)
        end = np.ascontiguousarray(end, np.uint64)
        index = np.ascontiguousarray(index, np.uint32)
        dptr = None if data is None else np.ascontiguousarray(data).ctypes.data
        keep = data
        _check(self.lib.dsstne_load_sparse_data(self.ctx, (name or self.dataset).encode(), start.ctypes.data, end.ctypes.data, dptr,
                                                index.ctypes.data))
        del keep

    def predict_batch(self, position=0):
        _check(self.lib.dsstne_predict_batch(self.ctx, position))

    def topk(self, k=None, filter_dataset=None, layer="Output"):
        _check(self.lib.dsstne_topk(self.ctx, layer.encode(), k or self.p.k, filter_dataset.encode() if filter_dataset else None))

    def get_topk(self, rows, k=None, layer="Output"):
        k = k or self.p.k
        scores = np.empty((rows, k), dtype=np.float32)
        idx = np.empty((rows, k), dtype=np.uint32)
        _check(self.lib.dsstne_get_topk(self.ctx, layer.encode(), rows, k, scores.ctypes.data, idx.ctypes.data))
        return scores, idx

    def get_topk_previous(self, rows, k=None, layer="Output"):
        """Results of the batch before the current one (two or more lanes): waits for that batch only."""
        k = k or self.p.k
        scores = np.empty((rows, k), dtype=np.float32)
        idx = np.empty((rows, k), dtype=np.uint32)
        _check(self.lib.dsstne_get_topk_previous(self.ctx, layer.encode(), rows, k, scores.ctypes.data, idx.ctypes.data))
        return scores, idx

    def set_lanes(self, lanes):
        _check(self.lib.dsstne_set_lanes(self.ctx, lanes))

    def set_deferred_output(self, defer):
        """NNNetwork::SetDeferredOutput: False stores the output layer in predict_batch, as the reference does."""
        _check(self.lib.dsstne_set_deferred_output(self.ctx, 1 if defer else 0))

    def set_split_products(self, split):
        """NNNetwork::SetSplitProducts: True forms the wide dense layers' fp32 products from bf16 matrix instructions."""
        _check(self.lib.dsstne_set_split_products(self.ctx, 1 if split else 0))

    def units(self, layer="Output", rows=None, width=None):
        width = width or self.p.widths[-1]
        rows = rows or self.p.batch
        out = np.empty((rows, width), dtype=np.float32)
        _check(self.lib.dsstne_get_units(self.ctx, layer.encode(), out.ctypes.data, out.size))
        return out

    def unit_buffer(self, layer="Output"):
        """Device address of the layer's activations of the batch predicted last (NNNetwork::GetUnitBuffer)."""
        ptr = self.lib.dsstne_get_unit_buffer(self.ctx, layer.encode())
        if not ptr:
            raise DsxError("dsstne_get_unit_buffer failed: %s" % self.lib.dsstne_last_error().decode())
        return ptr

    def set_units(self, values, layer="Output"):
        values = np.ascontiguousarray(values, dtype=np.float32)
        _check(self.lib.dsstne_set_units(self.ctx, layer.encode(), values.ctypes.data, values.size))

    def save(self, path):
        _check(self.lib.dsstne_save_network(self.ctx, path.encode()))

    def get_weights(self, input_layer, output_layer, rows, cols, biases=None):
        """Weights [rows = input width][cols = output width] and the connection's biases (`biases` of them, default cols).
        A tied connection has no matrix of its own (NNWeight::GetWeights hands back nothing): ask with rows = cols = 0."""
        w = np.empty((rows, cols), dtype=np.float32)
        b = np.empty(biases or cols, dtype=np.float32)
        _check(self.lib.dsstne_get_weights(self.ctx, input_layer.encode(), output_layer.encode(), w.ctypes.data, w.size, b.ctypes.data, b.size))
        return w, b

    def set_weights(self, input_layer, output_layer, weights=None, biases=None):
        w = None if weights is None else np.ascontiguousarray(weights, dtype=np.float32)
        b = None if biases is None else np.ascontiguousarray(biases, dtype=np.float32)
        _check(self.lib.dsstne_set_weights(self.ctx, input_layer.encode(), output_layer.encode(), None if w is None else w.ctypes.data,
                                           0 if w is None else w.size, None if b is None else b.ctypes.data, 0 if b is None else b.size))

    def sync(self):
        _check(self.lib.dsstne_sync())

    def close(self):
        if self.ctx:
            self.lib.dsstne_shutdown(self.ctx)
            self.ctx = None


class DefinedNetwork(Network):
    """A network built from a JSON definition file and a dataset file (the training tool's start-up: LoadNetCDF,
    LoadNeuralNetworkJSON, LoadDataSets); weights start from the definition's initialisation schemes and `seed`."""

    def __init__(self, definition_file, dataset_file, batch, max_k, seed=12134, k=None):
        self.lib = load_host_library()
        self.dataset = None

        class _Shape:
            pass
        self.p = _Shape()
        self.p.batch, self.p.k, self.p.widths = batch, (k or max_k), [None]
        self.max_k = max_k
        self.ctx = self.lib.dsstne_load_definition(definition_file.encode(), dataset_file.encode(), batch, max_k, seed)
        if not self.ctx:
            raise DsxError("dsstne_load_definition failed: %s" % self.lib.dsstne_last_error().decode())
