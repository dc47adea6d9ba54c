"""Python plumbing over the C ABI of libdsx_hip.so (include/dsx.h).

This module only loads the in-tree shared library with ctypes, declares the argument types of every entry point of
include/dsx.h, and offers a small device-array helper for tests and the benchmark.  There is no Python or CPU
implementation behind it: if the HIP library has not been built, or no MI355X is visible, the calls fail loudly.

The directory name contains a hyphen, so the package is loaded by path (see load_package() in __graft_entry__.py);
inside Python it is known as ``amazon_dsstne_amd``.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libdsx_hip.so")
HOST_LIB_PATH = os.path.join(_HERE, "libdsstne_amd.so")

# NNDataSetEnums::Attributes (engine/NNEnum.h:9-19)
ATTR_SPARSE, ATTR_BOOLEAN, ATTR_INDEXED, ATTR_WEIGHTED = 1, 2, 64, 128
# NNDataSetEnums::DataType (engine/NNEnum.h:35-47)
T_UINT, T_INT, T_LLINT, T_ULLINT, T_FLOAT, T_DOUBLE, T_RGB8, T_RGB16, T_UCHAR, T_CHAR = range(10)
# Activation (engine/NNTypes.h:91-105)
(ACT_SIGMOID, ACT_TANH, ACT_RELU, ACT_LINEAR, ACT_PRELU, ACT_SOFTPLUS, ACT_SOFTSIGN, ACT_SOFTMAX, ACT_RELUMAX,
 ACT_LINEARMAX, ACT_ELU, ACT_LRELU, ACT_SELU) = range(13)

NP_TO_DSX = {
    np.dtype(np.uint32): T_UINT, np.dtype(np.int32): T_INT, np.dtype(np.int64): T_LLINT, np.dtype(np.uint64): T_ULLINT,
    np.dtype(np.float32): T_FLOAT, np.dtype(np.float64): T_DOUBLE, np.dtype(np.uint8): T_UCHAR, np.dtype(np.int8): T_CHAR,
}

MAX_VALUE = np.float32(999999999999999.0)  # engine/NNTypes.h:49


class ActParams(C.Structure):
    _fields_ = [("slope", C.c_float), ("alpha", C.c_float), ("lambda_", C.c_float)]


class DeviceInfo(C.Structure):
    _fields_ = [("name", C.c_char * 256), ("arch", C.c_char * 64), ("compute_units", C.c_int), ("wavefront_size", C.c_int),
                ("lds_bytes_per_cu", C.c_int), ("hbm_bytes", C.c_size_t), ("hbm_free_bytes", C.c_size_t), ("clock_khz", C.c_int),
                ("memory_clock_khz", C.c_int)]


_u32, _u64, _f32, _vp, _int, _sz = C.c_uint32, C.c_uint64, C.c_float, C.c_void_p, C.c_int, C.c_size_t

# name -> argtypes; every function returns int except where noted below.  Mirrors include/dsx.h one to one.
SIGNATURES = {
    "dsx_init": [_int],
    "dsx_shutdown": [],
    "dsx_is_initialized": [],
    "dsx_get_device_info": [C.POINTER(DeviceInfo)],
    "dsx_get_memory_usage": [C.POINTER(_int), C.POINTER(_int)],
    "dsx_malloc": [C.POINTER(_vp), _sz],
    "dsx_malloc_managed": [C.POINTER(_vp), _sz],
    "dsx_malloc_host": [C.POINTER(_vp), _sz],
    "dsx_free": [_vp],
    "dsx_free_host": [_vp],
    "dsx_memset": [_vp, _int, _sz],
    "dsx_memcpy_h2d": [_vp, _vp, _sz],
    "dsx_memcpy_d2h": [_vp, _vp, _sz],
    "dsx_memcpy_d2d": [_vp, _vp, _sz],
    "dsx_sync": [],
    "dsx_set_lane": [_int],
    "dsx_get_lane": [],
    "dsx_sync_lane": [_int],
    "dsx_memcpy_d2h_lane": [_int, _vp, _vp, _sz],
    "dsx_memcpy_d2h_pair": [_vp, _vp, _sz, _vp, _vp, _sz],
    "dsx_memcpy_h2d_unordered": [_vp, _vp, _sz],
    "dsx_memcpy_h2d_unordered_many": [C.c_int, _vp, _vp, _vp],
    "dsx_lane_wait_other": [],
    "dsx_marker_create": [C.POINTER(C.c_void_p)],
    "dsx_marker_record": [_vp],
    "dsx_marker_wait": [_vp],
    "dsx_marker_destroy": [_vp],
    "dsx_timer_start": [],
    "dsx_timer_stop": [C.POINTER(_f32)],
    "dsx_clear_unit": [_vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32],
    "dsx_load_input_unit": [_u32, _u32, _u32, _u32, _vp, _vp, _vp],
    "dsx_load_sparse_input_unit": [_u32, _u32, _u32, _u32, _u32, _vp, _vp, _vp, _vp, _vp, _vp, _vp],
    "dsx_sparse_z": [_u32, _u32, _u32, _u32, _u32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _f32],
    "dsx_sparse_layer_forward": [_u32, _u32, _u32, _u32, _u32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _u32,
                                 C.POINTER(ActParams), _vp],
    "dsx_fc_forward": [_vp, _u32, _vp, _int, _vp, _vp, _u32, _u32, _u32, _u32, _int, _u32, C.POINTER(ActParams)],
    "dsx_fc_forward_segmax": [_vp, _u32, _vp, _int, _vp, _vp, _u32, _u32, _u32, _u32, _u32, C.POINTER(ActParams), _vp, C.POINTER(_u32)],
    "dsx_fc_split": [_vp, _u32, _int, _u32, _u32, _vp],
    "dsx_fc_forward_planes": [_vp, _u32, _vp, _int, _vp, _vp, _u32, _u32, _u32, _u32, _u32, C.POINTER(ActParams), _vp],
    "dsx_testing_set_split_tile_rows": [_u32],
    "dsx_fc_forward_split": [_vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _int, _u32, C.POINTER(ActParams), _vp, C.POINTER(_u32)],
    "dsx_activation": [_vp, _u32, _u32, _u32, C.POINTER(ActParams)],
    "dsx_add_buffers": [_vp, _vp, _u64],
    "dsx_topk": [_vp, _vp, _vp, _u32, _u32, _u32],
    "dsx_topk_kv_f32": [_vp, _vp, _vp, _vp, _u32, _u32, _u32],
    "dsx_topk_kv_u32": [_vp, _vp, _vp, _vp, _u32, _u32, _u32],
    "dsx_knn_topk": [_vp, _vp, _vp, _u32, _u32, _u32, _u32],
    "dsx_topk_filtered": [_vp, _vp, _vp, _u32, _u32, _u32, _u32, _vp, _vp, _vp, _vp, _vp],
    "dsx_topk_filtered_static": [_vp, _vp, _vp, _u32, _u32, _u32, _u32, _vp, _vp, _vp, _vp, _vp],
    "dsx_topk_guided": [_vp, _vp, _vp, _u32, _u32, _u32, _vp, _u32, _u32, _vp, _vp, _vp, _vp, _vp],
    "dsx_fc_topk": [_vp, _u32, _vp, _vp, _u32, _u32, _u32, _u32, C.POINTER(ActParams), _u32, _vp, _vp, _u32, _vp, _vp, _vp, _vp],
    "dsx_fc_topk_split": [_vp, _u32, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, C.POINTER(ActParams), _u32, _vp, _vp, _u32, _vp, _vp, _vp, _vp],
    "dsx_fc_topk_supported": [_u32, _vp, _u32, C.POINTER(ActParams), _vp],
    "dsx_fc_topk_flagged": [_int],
    "dsx_fc_topk_flagged_for": [_vp, _int],
    "dsx_testing_reset": [],
    "dsx_testing_occupy": [_u32, _u32, _u32],
    "dsx_testing_set_fc_topk_first_columns": [_u32],
    "dsx_testing_set_fc_topk_candidate_capacity": [_u32],
    "dsx_knn_search": [_vp, _u32, _u32, _u32, _vp, _u32, _u32, _vp, _vp, _vp, _sz, C.POINTER(_f32)],
    "dsx_testing_set_knn_block_columns": [_u32],
    "dsx_knn_f16_convert_items": [_vp, _u32, _u32, _u32, _vp],
    "dsx_knn_search_f16": [_vp, _u32, _u32, _u32, _vp, _u32, _u32, _vp, _vp, _vp, _sz, C.POINTER(_f32)],
    "dsx_knn_search_split": [_vp, _u32, _u32, _u32, _vp, _u32, _u32, _vp, _vp, _vp, _sz, C.POINTER(_f32)],
    "dsx_knn_last_search_path": [],
    "dsx_testing_set_knn_f16_sweep": [_int],
}
SPECIAL_RESTYPES = {"dsx_last_error": C.c_char_p, "dsx_stream": C.c_void_p, "dsx_knn_workspace_bytes": C.c_size_t,
                    "dsx_knn_workspace_bytes_f16": C.c_size_t, "dsx_knn_f16_table_bytes": C.c_size_t, "dsx_fc_split_bytes": _u64,
                    "dsx_knn_workspace_bytes_split": C.c_size_t}
SPECIAL_ARGTYPES = {"dsx_last_error": [], "dsx_stream": [], "dsx_knn_workspace_bytes": [_u32, _u32, _u32, _u32],
                    "dsx_knn_workspace_bytes_f16": [_u32, _u32, _u32, _u32], "dsx_knn_f16_table_bytes": [_u32, _u32],
                    "dsx_fc_split_bytes": [_u32, _u32], "dsx_knn_workspace_bytes_split": [_u32, _u32, _u32, _u32]}

_lib = None


class DsxError(RuntimeError):
    pass


def library_exists():
    return os.path.exists(LIB_PATH)


def load_library():
    """Load libdsx_hip.so and declare its signatures.  Raises if the library has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise DsxError("HIP library %s is missing: build it with __graft_entry__.build() (there is no CPU fallback)" % LIB_PATH)
    lib = C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)
    for name, args in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = C.c_int
    for name, res in SPECIAL_RESTYPES.items():
        fn = getattr(lib, name)
        fn.argtypes = SPECIAL_ARGTYPES[name]
        fn.restype = res
    _lib = lib
    return lib


def check(rc):
    if rc != 0:
        raise DsxError("dsx call failed (%d): %s" % (rc, load_library().dsx_last_error().decode()))


def init(device=0):
    lib = load_library()
    check(lib.dsx_init(device))
    return lib


class DeviceArray:
    """A typed block of HBM obtained through dsx_malloc."""

    def __init__(self, shape, dtype, lib=None):
        self.lib = lib or load_library()
        self.shape = tuple(int(s) for s in (shape if isinstance(shape, (tuple, list)) else (shape,)))
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        p = C.c_void_p()
        check(self.lib.dsx_malloc(C.byref(p), max(self.nbytes, 4)))
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, a, lib=None):
        a = np.ascontiguousarray(a)
        d = cls(a.shape, a.dtype, lib)
        d.upload(a)
        return d

    def upload(self, a):
        a = np.ascontiguousarray(a, dtype=self.dtype)
        assert a.nbytes == self.nbytes, (a.nbytes, self.nbytes)
        if self.nbytes:
            check(self.lib.dsx_memcpy_h2d(self.ptr, a.ctypes.data, self.nbytes))

    def numpy(self):
        out = np.empty(self.shape, dtype=self.dtype)
        if self.nbytes:
            check(self.lib.dsx_memcpy_d2h(out.ctypes.data, self.ptr, self.nbytes))
        return out

    def free(self):
        if self.ptr:
            check(self.lib.dsx_free(self.ptr))
            self.ptr = None

    def __del__(self):
        try:
            if self.ptr and self.lib.dsx_is_initialized():
                self.lib.dsx_free(self.ptr)
        except Exception:
            pass


def ptr(x):
    """Device address of a DeviceArray (or None)."""
    if x is None:
        return None
    return x.ptr if isinstance(x, DeviceArray) else x
