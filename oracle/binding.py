"""ctypes binding of the CPU oracle (oracle/liboracle.so) and of the reference's own topKsort (oracle/_ref).

TEST INFRASTRUCTURE: imported only by tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_LIB = os.path.join(_HERE, "liboracle.so")
REF_LIB = os.path.join(_HERE, "_ref", "libref_utils.so")

_u32, _u64, _f32, _vp, _int = C.c_uint32, C.c_uint64, C.c_float, C.c_void_p, C.c_int
_lib = None
_ref = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(ORACLE_LIB):
            raise RuntimeError("oracle library %s missing: run `make -C oracle`" % ORACLE_LIB)
        L = C.CDLL(ORACLE_LIB)
        L.orc_num_threads.restype = _int
        L.orc_clear_unit.argtypes = [_vp, C.POINTER(_vp), _u32, _u32, _u32]
        L.orc_sparse_z.argtypes = [_u32, _u32, _u32, _u32, _u32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _f32]
        L.orc_sparse_z.restype = _int
        L.orc_load_sparse_input_unit.argtypes = [_u32, _u32, _u32, _u32, _u32, _vp, _vp, _vp, _vp, _vp, _vp, _vp]
        L.orc_load_input_unit.argtypes = [_u32, _u32, _u32, _u32, _vp, _vp, _vp]
        L.orc_sgemm.argtypes = [_vp, _vp, _vp, _u32, _u32, _u32, _int]
        L.orc_add_buffers.argtypes = [_vp, _vp, _u64]
        L.orc_activation.argtypes = [_vp, _u64, _u32, _f32, _f32, _f32]
        L.orc_softmax.argtypes = [_vp, _u32, _u32]
        L.orc_topk.argtypes = [_vp, _u32, _u32, _u32, _vp, _vp]
        L.orc_knn_topk.argtypes = [_vp, _u32, _u32, _u32, _u32, _vp, _vp]
        L.orc_topk_kv.argtypes = [_vp, _vp, _u32, _u32, _u32, _vp, _vp, _int]
        L.orc_apply_filter.argtypes = [_vp, _u32, _u32, _u32, _u32, _vp, _vp, _vp, _vp, _vp]
        L.orc_topk_filtered.argtypes = [_vp, _u32, _u32, _u32, _u32, _vp, _vp, _vp, _vp, _vp, _vp, _vp]
        L.orc_knn_search.argtypes = [_vp, _u32, _u32, _u32, _vp, _u32, _u32, _vp, _vp]
        L.orc_merge_knn.argtypes = [_u32, _u32, _u32, _u32, C.POINTER(_vp), C.POINTER(_vp), _vp, _vp, _vp]
        L.orc_forward.argtypes = [_u32, _vp, C.POINTER(_vp), C.POINTER(_vp), _vp, _u32, _u32, _u32, _u32, _vp, _vp, _vp, _vp, _vp, _vp,
                                  _u32, _int, _vp, _vp, _vp]
        L.orc_forward.restype = C.c_double
        _lib = L
    return _lib


def ref_lib():
    """The reference's utils/Utils.cpp compiled as is (only where /root/reference was present at build time)."""
    global _ref
    if _ref is None:
        if not os.path.exists(REF_LIB):
            return None
        R = C.CDLL(REF_LIB)
        R.ref_topksort_f32_u32.argtypes = [_vp, _int, _vp, _vp, _int]
        R.ref_topksort_f32_f32.argtypes = [_vp, _vp, _int, _vp, _vp, _int]
        _ref = R
    return _ref


def _p(a):
    return None if a is None else a.ctypes.data


def _c(a, dt):
    return None if a is None else np.ascontiguousarray(a, dtype=dt)


def clear_unit(biases, stride, batch):
    unit = np.empty((batch, stride), dtype=np.float32)
    bs = [_c(b, np.float32) for b in biases]
    arr = (_vp * max(1, len(bs)))(*[b.ctypes.data for b in bs])
    lib().orc_clear_unit(unit.ctypes.data, arr, len(bs), stride, batch)
    return unit


def sparse_z(attributes, data_type, position, batch, stride, W, index, start, end, sidx, dw, sdata, unit, beta):
    unit = np.ascontiguousarray(unit, dtype=np.float32).copy()
    rc = lib().orc_sparse_z(attributes, data_type, position, batch, stride, _p(W), _p(index), _p(start), _p(end), _p(sidx), _p(dw),
                            _p(sdata), unit.ctypes.data, beta)
    assert rc == 0
    return unit


def load_sparse_input_unit(attributes, data_type, position, batch, stride, index, start, end, sidx, dw, sdata):
    unit = np.empty((batch, stride), dtype=np.float32)
    rc = lib().orc_load_sparse_input_unit(attributes, data_type, position, batch, stride, unit.ctypes.data, _p(index), _p(start), _p(end),
                                          _p(sidx), _p(dw), _p(sdata))
    assert rc == 0
    return unit


def load_input_unit(data_type, position, batch, stride, index, data):
    unit = np.empty((batch, stride), dtype=np.float32)
    rc = lib().orc_load_input_unit(data_type, position, batch, stride, unit.ctypes.data, _p(index), _p(data))
    assert rc == 0
    return unit


def sgemm_acc(X, W, Z, transposed=False):
    """Z += X.W, returns the new Z."""
    X = _c(X, np.float32)
    W = _c(W, np.float32)
    Z = np.ascontiguousarray(Z, dtype=np.float32).copy()
    B, k = X.shape
    n = Z.shape[1]
    lib().orc_sgemm(X.ctypes.data, W.ctypes.data, Z.ctypes.data, B, k, n, 1 if transposed else 0)
    return Z


def activation(z, act, slope=0.01, alpha=1.0, lam=1.0):
    z = np.ascontiguousarray(z, dtype=np.float32).copy()
    lib().orc_activation(z.ctypes.data, z.size, act, slope, alpha, lam)
    return z


def softmax(z):
    z = np.ascontiguousarray(z, dtype=np.float32).copy()
    lib().orc_softmax(z.ctypes.data, z.shape[0], z.shape[1])
    return z


def topk(scores, k, width=None):
    scores = _c(scores, np.float32)
    batch, pitch = scores.shape
    width = pitch if width is None else width
    keys = np.empty((batch, k), dtype=np.float32)
    idx = np.empty((batch, k), dtype=np.uint32)
    if width == pitch:
        lib().orc_topk(scores.ctypes.data, batch, width, k, keys.ctypes.data, idx.ctypes.data)
    else:
        lib().orc_knn_topk(scores.ctypes.data, batch, pitch, pitch - width, k, keys.ctypes.data, idx.ctypes.data)
    return keys, idx


def topk_kv(in_keys, in_vals, k):
    in_keys = _c(in_keys, np.float32)
    batch, width = in_keys.shape
    is_u32 = in_vals.dtype == np.uint32
    in_vals = np.ascontiguousarray(in_vals)
    keys = np.empty((batch, k), dtype=np.float32)
    vals = np.empty((batch, k), dtype=in_vals.dtype)
    lib().orc_topk_kv(in_keys.ctypes.data, in_vals.ctypes.data, batch, width, k, keys.ctypes.data, vals.ctypes.data, 1 if is_u32 else 0)
    return keys, vals


def topk_filtered(scores, k, position, index, fstart, fend, fidx, fmul):
    scores = _c(scores, np.float32)
    batch, width = scores.shape
    keys = np.empty((batch, k), dtype=np.float32)
    idx = np.empty((batch, k), dtype=np.uint32)
    lib().orc_topk_filtered(scores.ctypes.data, batch, width, k, position, _p(index), _p(fstart), _p(fend), _p(fidx), _p(fmul),
                            keys.ctypes.data, idx.ctypes.data)
    return keys, idx


def knn_search(items_cm, rows_padded, padding, dim, queries, k):
    queries = _c(queries, np.float32)
    Q = queries.shape[0]
    scores = np.empty((Q, k), dtype=np.float32)
    idx = np.empty((Q, k), dtype=np.uint32)
    lib().orc_knn_search(items_cm.ctypes.data, rows_padded, padding, dim, queries.ctypes.data, Q, k, scores.ctypes.data, idx.ctypes.data)
    return scores, idx


def forward(problem, position=0, batch=None, k=None, filtered=True, want_unit=False, want_topk=True):
    """Whole chain forward + (filtered) top-K of a synth.Problem.  Returns (seconds, unit or None, keys, idx)."""
    p = problem
    batch = p.batch if batch is None else batch
    k = p.k if k is None else k
    nl = len(p.weights)
    widths = np.asarray(p.widths, dtype=np.uint32)
    acts = np.asarray(p.acts, dtype=np.uint32)
    Ws = (_vp * nl)(*[w.ctypes.data for w in p.weights])
    Bs = (_vp * nl)(*[b.ctypes.data for b in p.biases])
    N = p.widths[-1]
    unit = np.empty((batch, N), dtype=np.float32) if want_unit else None
    keys = np.empty((batch, k), dtype=np.float32) if want_topk else None
    idx = np.empty((batch, k), dtype=np.uint32) if want_topk else None
    secs = lib().orc_forward(nl, widths.ctypes.data, Ws, Bs, acts.ctypes.data, p.attributes, p.data_type, position, batch, _p(p.index),
                             _p(p.start), _p(p.end), _p(p.sparse_index), _p(p.data_weight), _p(p.sparse_data), k, 1 if filtered else 0,
                             _p(unit), _p(keys), _p(idx))
    return secs, unit, keys, idx


def ref_topksort(keys_row, k):
    """Reference topKsort<float, unsigned int> on one row (values = positions).  None when oracle/_ref is not built."""
    R = ref_lib()
    if R is None:
        return None
    row = np.ascontiguousarray(keys_row, dtype=np.float32).copy()
    tk = np.empty(k, dtype=np.float32)
    tv = np.empty(k, dtype=np.uint32)
    R.ref_topksort_f32_u32(row.ctypes.data, row.shape[0], tk.ctypes.data, tv.ctypes.data, k)
    return tk, tv
