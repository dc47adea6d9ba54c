"""Parity of every C-ABI kernel entry point against the CPU oracle on the same seeded inputs (needs an MI355X)."""
import ctypes as C

import numpy as np
import pytest

from parity import assert_close, assert_topk_exact, check_topk_invariants
from test_oracle import random_csr

pytestmark = pytest.mark.gpu

A_SPARSE, A_BOOLEAN, A_INDEXED, A_WEIGHTED = 1, 2, 64, 128
T_UINT, T_INT, T_LLINT, T_ULLINT, T_FLOAT, T_DOUBLE, _, _, T_UCHAR, T_CHAR = range(10)


def say(msg):
    print("[case] " + msg, flush=True)


def dev(pkg, a):
    return None if a is None else pkg.DeviceArray.from_numpy(a)


# ------------------------------------------------------------------------------------------------------------- plumbing

def test_device_is_gfx950(pkg, dsx):
    info = pkg.DeviceInfo()
    pkg.check(dsx.dsx_get_device_info(info))
    say("device %s %s CUs=%d" % (info.name.decode(), info.arch.decode(), info.compute_units))
    assert info.arch.decode().startswith("gfx950") and info.wavefront_size == 64


def test_malloc_zero_fills_and_copies(pkg, dsx, rng):
    a = pkg.DeviceArray((1000,), np.float32)
    assert not a.numpy().any()                      # GpuBuffer constructor zero-fills (engine/GpuTypes.h:523)
    x = rng.standard_normal(1000).astype(np.float32)
    a.upload(x)
    b = pkg.DeviceArray((1000,), np.float32)
    pkg.check(dsx.dsx_memcpy_d2d(b.ptr, a.ptr, a.nbytes))
    assert np.array_equal(b.numpy(), x)
    pkg.check(dsx.dsx_memset(b.ptr, 0, b.nbytes))
    assert not b.numpy().any()
    p = C.c_void_p()
    pkg.check(dsx.dsx_malloc_managed(C.byref(p), 64))   # host-dereferenceable (tst/amazon/dsstne/engine/TestGpuBuffer.cpp:31-68)
    host = (C.c_float * 16).from_address(p.value)
    host[3] = 2.5
    assert host[3] == 2.5 and host[0] == 0.0
    pkg.check(dsx.dsx_free(p))
    g = C.c_int()
    h = C.c_int()
    pkg.check(dsx.dsx_get_memory_usage(C.byref(g), C.byref(h)))
    assert g.value > 0


def test_lanes_unordered_upload_and_explicit_wait(pkg, dsx, rng):
    """dsx_memcpy_h2d_unordered queues on the selected lane only; dsx_lane_wait_other makes the selected lane run after what
    the other lane holds.  A kernel over 256 MiB keeps lane 1 busy ahead of the upload, lane 0 reads the buffer after the wait, and
    dsx_memcpy_d2h_lane waits for lane 0 alone: it can only return the uploaded data if the wait ordered the lanes."""
    n = 1 << 16
    big = pkg.DeviceArray((64 << 20,), np.float32)          # 256 MiB
    buf = pkg.DeviceArray((n,), np.float32)
    out = pkg.DeviceArray((n,), np.float32)
    try:
        for rep in range(4):
            x = rng.standard_normal(n).astype(np.float32)
            pkg.check(dsx.dsx_set_lane(1))
            assert dsx.dsx_get_lane() == 1
            pkg.check(dsx.dsx_add_buffers(big.ptr, big.ptr, 64 << 20))    # a kernel (kernels order nothing between the lanes)
            pkg.check(dsx.dsx_memcpy_h2d_unordered(buf.ptr, x.ctypes.data, x.nbytes))
            pkg.check(dsx.dsx_set_lane(0))
            pkg.check(dsx.dsx_lane_wait_other())
            pkg.check(dsx.dsx_add_buffers(out.ptr, buf.ptr, n))           # out += buf on lane 0
            got = np.empty(n, np.float32)
            pkg.check(dsx.dsx_memcpy_d2h_lane(0, got.ctypes.data, out.ptr, got.nbytes))
            want = x if rep == 0 else want + x
            assert np.array_equal(got, want), "repetition %d" % rep
        pkg.check(dsx.dsx_lane_wait_other())                              # harmless when nothing is pending
    finally:
        pkg.check(dsx.dsx_set_lane(0))
        pkg.check(dsx.dsx_sync())


def test_uploads_of_every_size_and_alignment_arrive_byte_for_byte(pkg, dsx, rng):
    """Uploads go through pinned staging memory and a copy kernel in pieces of 128 KiB (16 bytes per lane, a byte tail), through
    the copy engine when the destination is not 16-byte aligned or the array exceeds a staging slot (4 MiB).  Sizes on both
    sides of every such boundary, destinations at odd offsets, and the several-arrays form: each byte must arrive, and the
    bytes around a destination must stay as they were."""
    room = (5 << 20) + 4096
    dev = pkg.DeviceArray((room,), np.uint8)
    sizes = [1, 3, 15, 16, 17, 255, 4096, (128 << 10) - 16, (128 << 10) - 1, 128 << 10, (128 << 10) + 1, (128 << 10) + 17,
             (256 << 10) + 5, (1 << 20) + 123, 4 << 20, (4 << 20) + 1, (5 << 20) + 7]
    for size in sizes:
        for off in (0, 16, 4, 1):
            say("upload size=%d offset=%d" % (size, off))
            pkg.check(dsx.dsx_memset(dev.ptr, 0xA5, room))
            x = rng.integers(0, 256, size=size, dtype=np.uint8)
            pkg.check(dsx.dsx_memcpy_h2d(dev.ptr + 256 + off, x.ctypes.data, size))
            got = dev.numpy()
            assert np.array_equal(got[256 + off:256 + off + size], x), (size, off)
            assert (got[:256 + off] == 0xA5).all() and (got[256 + off + size:] == 0xA5).all(), (size, off)
    # several arrays in one call: sizes that share launches, cross piece boundaries, are empty, or are not multiples of 16
    for lens in [(8192, 8192, 400000), (8, 0, 131072 - 8, 40), (100, 131000, 131072, 7), (300000, 4, 4, 300001)]:
        say("upload many %s" % (lens,))
        pkg.check(dsx.dsx_memset(dev.ptr, 0x5A, room))
        xs = [rng.integers(0, 256, size=n, dtype=np.uint8) for n in lens]
        at, offs = 512, []
        for n in lens:
            offs.append(at)
            at += (n + 255) // 256 * 256 + 256
        dst = (C.c_void_p * len(lens))(*[dev.ptr + o for o in offs])
        src = (C.c_void_p * len(lens))(*[x.ctypes.data if x.size else None for x in xs])
        nb = (C.c_size_t * len(lens))(*lens)
        pkg.check(dsx.dsx_memcpy_h2d_unordered_many(len(lens), dst, src, nb))
        got = dev.numpy()
        want = np.full(room, 0x5A, np.uint8)
        for o, x in zip(offs, xs):
            want[o:o + x.size] = x
        assert np.array_equal(got, want), lens
    assert dsx.dsx_memcpy_h2d_unordered_many(2, dst, None, nb) == -1


def test_bad_arguments_are_rejected(pkg, dsx):
    a = pkg.DeviceArray((4, 8), np.float32)
    k = pkg.DeviceArray((4, 8), np.float32)
    v = pkg.DeviceArray((4, 8), np.uint32)
    assert dsx.dsx_topk(a.ptr, k.ptr, v.ptr, 4, 8, 0) == -1
    assert dsx.dsx_topk(a.ptr, k.ptr, v.ptr, 4, 8, 257) == -1
    assert b"1..256" in dsx.dsx_last_error()
    assert dsx.dsx_topk(None, k.ptr, v.ptr, 4, 8, 2) == -1
    assert dsx.dsx_knn_topk(a.ptr, k.ptr, v.ptr, 4, 8, 8, 2) == -1
    assert dsx.dsx_clear_unit(a.ptr, None, None, None, None, 1, 8, 4) == -1
    assert dsx.dsx_fc_forward(a.ptr, 8, a.ptr, 0, None, a.ptr, 4, 4, 8, 8, 0, 3, None) == -1     # ldz < n
    assert dsx.dsx_fc_forward(a.ptr, 8, a.ptr, 0, None, a.ptr, 8, 4, 8, 8, 0, 7, None) == -1     # softmax cannot be fused
    assert dsx.dsx_sparse_z(A_SPARSE, 6, 0, 1, 8, a.ptr, None, a.ptr, a.ptr, a.ptr, None, a.ptr, a.ptr, 1.0) == -5


# ------------------------------------------------------------------------------------------------- bias, loaders, misc

@pytest.mark.parametrize("nbias", [0, 1, 2, 3, 4])
def test_clear_unit(pkg, dsx, orc, rng, nbias):
    stride, batch = 77, 9
    bs = [rng.standard_normal(stride).astype(np.float32) for _ in range(4)]
    d = [dev(pkg, b) for b in bs]
    unit = pkg.DeviceArray.from_numpy(np.full((batch, stride), 7.0, dtype=np.float32))
    ptrs = [d[i].ptr if i < nbias else None for i in range(4)]
    pkg.check(dsx.dsx_clear_unit(unit.ptr, ptrs[0], ptrs[1], ptrs[2], ptrs[3], nbias, stride, batch))
    assert np.array_equal(unit.numpy(), orc.clear_unit(bs[:nbias], stride, batch))


@pytest.mark.parametrize("dtype,tag", [(np.float32, T_FLOAT), (np.float64, T_DOUBLE), (np.int32, T_INT), (np.uint32, T_UINT),
                                       (np.int64, T_LLINT), (np.uint64, T_ULLINT), (np.uint8, T_UCHAR), (np.int8, T_CHAR)])
@pytest.mark.parametrize("indexed", [False, True])
def test_load_input_unit(pkg, dsx, orc, rng, dtype, tag, indexed):
    rows, stride, position, batch = 20, 1500, 3, 11
    if np.issubdtype(dtype, np.floating):
        data = rng.standard_normal((rows, stride)).astype(dtype)
    else:
        info = np.iinfo(dtype)
        data = rng.integers(max(info.min, -1000), min(info.max, 1000), size=(rows, stride)).astype(dtype)
    index = rng.permutation(rows).astype(np.uint32) if indexed else None
    unit = pkg.DeviceArray((batch, stride), np.float32)
    dd, di = dev(pkg, data), dev(pkg, index)
    pkg.check(dsx.dsx_load_input_unit(tag, position, batch, stride, unit.ptr, pkg.ptr(di), dd.ptr))
    assert np.array_equal(unit.numpy(), orc.load_input_unit(tag, position, batch, stride, index, data))


@pytest.mark.parametrize("boolean,dtype,tag", [(True, None, T_FLOAT), (False, np.float32, T_FLOAT), (False, np.uint8, T_UCHAR),
                                               (False, np.int32, T_INT)])
@pytest.mark.parametrize("indexed,weighted", [(False, False), (True, True)])
def test_load_sparse_input_unit(pkg, dsx, orc, rng, boolean, dtype, tag, indexed, weighted):
    rows, width, position, batch = 30, 400, 4, 17
    start, end, idx = random_csr(rng, rows, width, 50)
    vals = None if boolean else rng.integers(1, 100, size=len(idx)).astype(dtype)
    index = rng.permutation(rows).astype(np.uint32) if indexed else None
    dw = (rng.random(rows, dtype=np.float32) + 0.5) if weighted else None
    attr = A_SPARSE | (A_BOOLEAN if boolean else 0) | (A_INDEXED if indexed else 0) | (A_WEIGHTED if weighted else 0)
    unit = pkg.DeviceArray.from_numpy(np.full((batch, width), 9.0, dtype=np.float32))
    ds, de, dx, dv, di, dwt = (dev(pkg, x) for x in (start, end, idx, vals, index, dw))
    pkg.check(dsx.dsx_load_sparse_input_unit(attr, tag, position, batch, width, unit.ptr, pkg.ptr(di), ds.ptr, de.ptr, dx.ptr,
                                             pkg.ptr(dwt), pkg.ptr(dv)))
    assert np.array_equal(unit.numpy(), orc.load_sparse_input_unit(attr, tag, position, batch, width, index, start, end, idx, dw, vals))


def test_add_buffers(pkg, dsx, rng):
    a = rng.standard_normal(100003).astype(np.float32)
    b = rng.standard_normal(100003).astype(np.float32)
    da, db = dev(pkg, a), dev(pkg, b)
    pkg.check(dsx.dsx_add_buffers(da.ptr, db.ptr, a.size))
    assert np.array_equal(da.numpy(), a + b)


# ------------------------------------------------------------------------------------------------------------- sparse Z

def run_sparse_z(pkg, dsx, attr, tag, position, batch, stride, W, index, start, end, idx, dw, vals, unit0, beta):
    dW, di, ds, de, dx, dwt, dv = (dev(pkg, x) for x in (W, index, start, end, idx, dw, vals))
    unit = pkg.DeviceArray.from_numpy(unit0)
    pkg.check(dsx.dsx_sparse_z(attr, tag, position, batch, stride, dW.ptr, pkg.ptr(di), ds.ptr, de.ptr, dx.ptr, pkg.ptr(dwt), pkg.ptr(dv),
                               unit.ptr, beta))
    return unit.numpy()


# stride 128/512/1024: 128-bit gathers with 32/128/256 lanes per weight row; 1500: two column tiles; 30: 64-bit gathers
# (row pitch 120 bytes); 37: scalar path; 4: fewer columns than the 16-lane minimum.
@pytest.mark.parametrize("stride", [128, 512, 1024, 1500, 30, 37, 4])
@pytest.mark.parametrize("beta", [0.0, 1.0, 0.5])
def test_sparse_z_boolean(pkg, dsx, orc, rng, stride, beta):
    say("sparse_z boolean stride=%d beta=%g" % (stride, beta))
    rows, width = 64, 3000
    start, end, idx = random_csr(rng, rows, width, 300, empty_rows=(5, 63))
    W = rng.standard_normal((width, stride)).astype(np.float32)
    unit0 = rng.standard_normal((rows, stride)).astype(np.float32)
    got = run_sparse_z(pkg, dsx, A_SPARSE | A_BOOLEAN, T_FLOAT, 0, rows, stride, W, None, start, end, idx, None, None, unit0, beta)
    ref = orc.sparse_z(A_SPARSE | A_BOOLEAN, T_FLOAT, 0, rows, stride, W, None, start, end, idx, None, None, unit0, beta)
    assert_close(got, ref, "sparse Z", rel=1e-4, abs_floor=1.0)   # sums of ~150 N(0,1) terms: compare on an absolute scale of 1
    assert np.array_equal(got[[5, 63]], unit0[[5, 63]])           # rows without non-zeros stay untouched


def test_sparse_z_long_rows_cross_lds_chunks(pkg, dsx, orc, rng):
    # rows longer than one LDS staging pass (the reference chunks at 4608 non-zeros, engine/GpuTypes.h:131-136)
    rows, width, stride = 6, 20000, 128
    counts = [0, 1, 2047, 2048, 2049, 9000]
    start = np.zeros(rows, dtype=np.uint64)
    end = np.zeros(rows, dtype=np.uint64)
    cols, pos = [], 0
    for r, c in enumerate(counts):
        cols.append(rng.choice(width, size=c, replace=False).astype(np.uint32))
        start[r], pos = pos, pos + c
        end[r] = pos
    idx = np.concatenate(cols)
    W = (rng.standard_normal((width, stride)) * 0.1).astype(np.float32)
    unit0 = np.zeros((rows, stride), dtype=np.float32)
    got = run_sparse_z(pkg, dsx, A_SPARSE | A_BOOLEAN, T_FLOAT, 0, rows, stride, W, None, start, end, idx, None, None, unit0, 0.0)
    ref = orc.sparse_z(A_SPARSE | A_BOOLEAN, T_FLOAT, 0, rows, stride, W, None, start, end, idx, None, None, unit0, 0.0)
    assert_close(got, ref, "sparse Z long rows", rel=1e-4, abs_floor=1.0)
    assert np.array_equal(got[1], W[idx[0]])   # a single non-zero copies the weight row exactly


@pytest.mark.parametrize("dtype,tag", [(np.float32, T_FLOAT), (np.float64, T_DOUBLE), (np.int32, T_INT), (np.uint32, T_UINT),
                                       (np.int64, T_LLINT), (np.uint64, T_ULLINT), (np.uint8, T_UCHAR), (np.int8, T_CHAR)])
@pytest.mark.parametrize("indexed,weighted", [(False, False), (True, False), (True, True)])
def test_sparse_z_analog(pkg, dsx, orc, rng, dtype, tag, indexed, weighted):
    say("sparse_z analog %s indexed=%s weighted=%s" % (dtype.__name__, indexed, weighted))
    rows, width, stride, position, batch = 80, 1000, 96, 7, 50
    start, end, idx = random_csr(rng, rows, width, 120)
    if np.issubdtype(dtype, np.floating):
        vals = (rng.integers(1, 11, size=len(idx)) * 0.5).astype(dtype)
    elif dtype == np.int8:
        vals = rng.integers(-100, 100, size=len(idx)).astype(dtype)
    else:
        vals = rng.integers(0, 200, size=len(idx)).astype(dtype)
    index = rng.permutation(rows).astype(np.uint32) if indexed else None
    dw = (rng.random(rows, dtype=np.float32) + 0.5) if weighted else None
    attr = A_SPARSE | (A_INDEXED if indexed else 0) | (A_WEIGHTED if weighted else 0)
    W = (rng.standard_normal((width, stride)) * 0.1).astype(np.float32)
    unit0 = rng.standard_normal((batch, stride)).astype(np.float32)
    got = run_sparse_z(pkg, dsx, attr, tag, position, batch, stride, W, index, start, end, idx, dw, vals, unit0, 1.0)
    ref = orc.sparse_z(attr, tag, position, batch, stride, W, index, start, end, idx, dw, vals, unit0, 1.0)
    scale = float(np.abs(ref).max())
    assert_close(got, ref, "analog sparse Z", rel=1e-4, abs_floor=max(1.0, scale * 0.05))


@pytest.mark.parametrize("act", [0, 1, 2, 3, 10, 11, 12])
def test_sparse_layer_forward_fused(pkg, dsx, orc, rng, act):
    rows, width, stride = 48, 2000, 128
    start, end, idx = random_csr(rng, rows, width, 200, empty_rows=(0,))
    W = (rng.standard_normal((width, stride)) * 0.1).astype(np.float32)
    bias = rng.standard_normal(stride).astype(np.float32)
    params = pkg.ActParams(0.2, 1.5, 1.05)
    dW, ds, de, dx, db = (dev(pkg, x) for x in (W, start, end, idx, bias))
    unit = pkg.DeviceArray.from_numpy(np.full((rows, stride), 123.0, dtype=np.float32))
    pkg.check(dsx.dsx_sparse_layer_forward(A_SPARSE | A_BOOLEAN, T_FLOAT, 0, rows, stride, dW.ptr, None, ds.ptr, de.ptr, dx.ptr, None, None,
                                           db.ptr, act, C.byref(params), unit.ptr))
    ref = orc.clear_unit([bias], stride, rows)
    ref = orc.sparse_z(A_SPARSE | A_BOOLEAN, T_FLOAT, 0, rows, stride, W, None, start, end, idx, None, None, ref, 1.0)
    ref = orc.activation(ref, act, 0.2, 1.5, 1.05)
    assert_close(unit.numpy(), ref, "fused first layer act=%d" % act, rel=1e-4, abs_floor=1e-2)


# ------------------------------------------------------------------------------------------------------------------ GEMM

# (batch, k, n): tile-aligned, ragged in every dimension, k below one k-step, n odd (scalar loads), n even but not /4
# (64-bit loads, the 27,278-wide case), small-tile and large-tile paths.
GEMM_SHAPES = [(128, 128, 128), (1024, 128, 128), (33, 17, 29), (200, 100, 270), (64, 5, 64), (1024, 128, 2730), (300, 64, 27278),
               (2048, 256, 4096), (1, 1, 1)]


@pytest.mark.parametrize("B,k,n", GEMM_SHAPES)
def test_fc_forward_vs_oracle(pkg, dsx, orc, rng, B, k, n):
    say("fc_forward B=%d k=%d n=%d" % (B, k, n))
    X = rng.standard_normal((B, k)).astype(np.float32)
    W = (rng.standard_normal((k, n)) * 0.1).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    dX, dW, db = dev(pkg, X), dev(pkg, W), dev(pkg, bias)
    Z = pkg.DeviceArray.from_numpy(np.full((B, n), 55.0, dtype=np.float32))
    pkg.check(dsx.dsx_fc_forward(dX.ptr, k, dW.ptr, 0, db.ptr, Z.ptr, n, B, k, n, 0, 3, None))
    ref = orc.sgemm_acc(X, W, orc.clear_unit([bias], n, B))
    scale = float(np.sqrt(k)) * 0.1
    assert_close(Z.numpy(), ref, "fc forward", rel=1e-4, abs_floor=max(scale, 1e-2))
    # fp64 cross-check: the GPU must be no further from the exact product than a few fp32 roundings
    exact = X.astype(np.float64) @ W.astype(np.float64) + bias
    assert_close(Z.numpy(), exact, "fc forward vs fp64", rel=1e-4, abs_floor=max(scale, 1e-2))


@pytest.mark.parametrize("act", [0, 1, 2, 10, 11, 12])
@pytest.mark.parametrize("accumulate", [0, 1])
def test_fc_forward_epilogue(pkg, dsx, orc, rng, act, accumulate):
    B, k, n = 70, 48, 150
    X = rng.standard_normal((B, k)).astype(np.float32)
    W = (rng.standard_normal((k, n)) * 0.3).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    Z0 = rng.standard_normal((B, n)).astype(np.float32)
    params = pkg.ActParams(0.2, 1.5, 1.05)
    dX, dW, db = dev(pkg, X), dev(pkg, W), dev(pkg, bias)
    Z = pkg.DeviceArray.from_numpy(Z0)
    pkg.check(dsx.dsx_fc_forward(dX.ptr, k, dW.ptr, 0, db.ptr, Z.ptr, n, B, k, n, accumulate, act, C.byref(params)))
    pre = orc.clear_unit([bias], n, B) + (Z0 if accumulate else 0)
    ref = orc.activation(orc.sgemm_acc(X, W, pre), act, 0.2, 1.5, 1.05)
    assert_close(Z.numpy(), ref, "fc epilogue", rel=1e-4, abs_floor=1e-2)


@pytest.mark.parametrize("B,k,n,act", [(1024, 128, 128, 2), (1000, 256, 100, 0), (33, 128, 31, 1), (5, 256, 1, 3), (777, 128, 1000, 12)])
def test_fc_forward_split_k_small_problems(pkg, dsx, orc, rng, B, k, n, act):
    # k = 128 / 256 with few output tiles runs the latency-oriented kernel (k split over the four wavefronts); pitched X and Z
    say("fc_forward split-k B=%d k=%d n=%d act=%d" % (B, k, n, act))
    X = rng.standard_normal((B, k + 4)).astype(np.float32)
    W = (rng.standard_normal((k, n)) * 0.1).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    dX, dW, db = dev(pkg, X), dev(pkg, W), dev(pkg, bias)
    Z = pkg.DeviceArray.from_numpy(np.full((B, n + 5), 55.0, dtype=np.float32))
    params = pkg.ActParams(0.2, 1.5, 1.05)
    pkg.check(dsx.dsx_fc_forward(dX.ptr, k + 4, dW.ptr, 0, db.ptr, Z.ptr, n + 5, B, k, n, 0, act, C.byref(params)))
    got = Z.numpy()
    ref = orc.activation(orc.sgemm_acc(np.ascontiguousarray(X[:, :k]), W, orc.clear_unit([bias], n, B)), act, 0.2, 1.5, 1.05)
    assert_close(got[:, :n], ref, "split-k fc", rel=1e-4, abs_floor=max(float(np.sqrt(k)) * 0.1, 1e-2))
    assert np.all(got[:, n:] == 55.0)                             # nothing written past n


def test_fc_forward_transposed_and_pitched(pkg, dsx, orc, rng):
    B, k, n = 90, 70, 130
    X = rng.standard_normal((B, k + 6)).astype(np.float32)       # row pitch larger than k
    Wt = (rng.standard_normal((n, k)) * 0.2).astype(np.float32)  # [n][k]: shared transposed weight (engine/NNLayer.cpp:1065-1072)
    dX, dW = dev(pkg, X), dev(pkg, Wt)
    Z = pkg.DeviceArray.from_numpy(np.zeros((B, n + 3), dtype=np.float32))
    pkg.check(dsx.dsx_fc_forward(dX.ptr, k + 6, dW.ptr, 1, None, Z.ptr, n + 3, B, k, n, 0, 3, None))
    got = Z.numpy()
    ref = orc.sgemm_acc(np.ascontiguousarray(X[:, :k]), Wt, np.zeros((B, n), dtype=np.float32), transposed=True)
    assert_close(got[:, :n], ref, "transposed fc", rel=1e-4, abs_floor=0.5)
    assert not got[:, n:].any()                                   # nothing written past n


@pytest.mark.parametrize("act", [0, 1, 2, 3, 7, 10, 11, 12, 5])
def test_activation(pkg, dsx, orc, rng, act):
    batch, stride = 37, 501
    z = (rng.standard_normal((batch, stride)) * 4).astype(np.float32)
    params = pkg.ActParams(0.2, 1.5, 1.05)
    d = dev(pkg, z)
    pkg.check(dsx.dsx_activation(d.ptr, batch, stride, act, C.byref(params)))
    ref = orc.softmax(z) if act == 7 else orc.activation(z, act, 0.2, 1.5, 1.05)
    # ELU / SELU compute exp(x) - 1, which cancels near 0 on both sides: compare those on an absolute scale of 1e-2
    floor = {7: 1e-7, 10: 1e-2, 12: 1e-2}.get(act, 1e-6)
    assert_close(d.numpy(), ref, "activation %d" % act, rel=1e-4, abs_floor=floor)


# ----------------------------------------------------------------------------------------------------------------- top-K

def run_topk(pkg, dsx, scores, k):
    batch, width = scores.shape
    d = dev(pkg, scores)
    keys = pkg.DeviceArray.from_numpy(np.full((batch, k), 7.0, dtype=np.float32))
    vals = pkg.DeviceArray.from_numpy(np.full((batch, k), 77, dtype=np.uint32))
    pkg.check(dsx.dsx_topk(d.ptr, keys.ptr, vals.ptr, batch, width, k))
    return keys.numpy(), vals.numpy()


# tst/gputests/TestSort.cpp:208-211 shapes (pitch padded to 128 with zeros, padded pitch passed as the width)
@pytest.mark.parametrize("batch,k,nfeat", [(128, 128, 1024), (128, 128, 100000), (128, 64, 1024), (128, 32, 64), (128, 1, 64)])
def test_topk_testsort_shapes(pkg, dsx, orc, rng, batch, k, nfeat):
    say("topk TestSort batch=%d k=%d n=%d" % (batch, k, nfeat))
    stride = (nfeat + 127) // 128 * 128
    scores = np.zeros((batch, stride), dtype=np.float32)
    scores[:, :nfeat] = rng.random((batch, nfeat), dtype=np.float32)
    keys, idx = run_topk(pkg, dsx, scores, k)
    rk, ri = orc.topk(scores, k)
    assert_topk_exact(keys, idx, rk, ri)


# widths around the 16-byte alignment head/tail logic, k at every list size (64/128/256 slots), rows whose start is
# misaligned (odd widths), more slots than columns, one workgroup per row and several.
@pytest.mark.parametrize("batch,width,k", [(5, 1, 1), (3, 2, 4), (9, 7, 3), (4, 64, 64), (6, 65, 65), (7, 255, 128), (3, 257, 129),
                                           (2, 1000, 256), (33, 4099, 10), (1024, 27278, 10), (3, 1000003, 100), (1, 300000, 256),
                                           (16, 50001, 200),
                                           # k on both sides of every width of the primed bound's key search (16, 32, 64, 128 keys
                                           # per lane group), rows of two full spans and more and rows shorter than one span
                                           (12, 27278, 16), (12, 27278, 17), (12, 27278, 33), (12, 27278, 65), (12, 27278, 128),
                                           (12, 27278, 129), (9, 5000, 16), (9, 5000, 17), (7, 70000, 32), (7, 70000, 64)])
def test_topk_random(pkg, dsx, orc, rng, batch, width, k):
    say("topk random batch=%d width=%d k=%d" % (batch, width, k))
    scores = rng.standard_normal((batch, width)).astype(np.float32)
    keys, idx = run_topk(pkg, dsx, scores, k)
    rk, ri = orc.topk(scores, k)
    assert_topk_exact(keys, idx, rk, ri)
    if batch * width < 3e6:
        check_topk_invariants(scores, keys, idx, k)


@pytest.mark.parametrize("batch,width,k", [(8, 5000, 10), (4, 700, 100), (2, 40000, 256), (64, 333, 64)])
def test_topk_many_ties(pkg, dsx, orc, rng, batch, width, k):
    # saturated sigmoids give long runs of identical scores: the order must be score descending, then index ascending
    scores = (rng.integers(0, 6, size=(batch, width)).astype(np.float32) - 2) / 2
    scores[0, :] = 1.0
    scores[-1, ::2] = -0.0
    keys, idx = run_topk(pkg, dsx, scores, k)
    rk, ri = orc.topk(scores, k)
    assert_topk_exact(keys, idx, rk, ri)


def test_topk_extremes(pkg, dsx, orc):
    scores = np.array([[np.inf, -np.inf, 3.4e38, -3.4e38, 1e-45, -1e-45, 0.0, -0.0, 5.0]], dtype=np.float32)
    keys, idx = run_topk(pkg, dsx, scores, 9)
    rk, ri = orc.topk(scores, 9)
    assert_topk_exact(keys, idx, rk, ri)
    assert idx[0].tolist() == [0, 2, 8, 4, 6, 7, 5, 3, 1]


def test_knn_topk_padding(pkg, dsx, orc, rng):
    batch, pitch, pad, k = 40, 10008, 5, 100
    scores = rng.standard_normal((batch, pitch)).astype(np.float32)
    scores[:, pitch - pad:] = 1e9
    d = dev(pkg, scores)
    keys = pkg.DeviceArray((batch, k), np.float32)
    vals = pkg.DeviceArray((batch, k), np.uint32)
    pkg.check(dsx.dsx_knn_topk(d.ptr, keys.ptr, vals.ptr, batch, pitch, pad, k))
    rk, ri = orc.topk(scores, k, width=pitch - pad)
    assert_topk_exact(keys.numpy(), vals.numpy(), rk, ri)


@pytest.mark.parametrize("payload", [np.float32, np.uint32])
def test_topk_kv(pkg, dsx, orc, rng, payload):
    batch, width, k = 20, 3000, 128
    in_keys = rng.standard_normal((batch, width)).astype(np.float32)
    in_vals = rng.random((batch, width), dtype=np.float32) if payload == np.float32 else rng.integers(0, 1 << 32, size=(batch, width)).astype(np.uint32)
    dk, dv = dev(pkg, in_keys), dev(pkg, in_vals)
    keys = pkg.DeviceArray((batch, k), np.float32)
    vals = pkg.DeviceArray((batch, k), payload)
    fn = dsx.dsx_topk_kv_f32 if payload == np.float32 else dsx.dsx_topk_kv_u32
    pkg.check(fn(dk.ptr, dv.ptr, keys.ptr, vals.ptr, batch, width, k))
    rk, rv = orc.topk_kv(in_keys, in_vals, k)
    assert np.array_equal(keys.numpy(), rk) and np.array_equal(vals.numpy(), rv)   # uint32 payloads are exact above 2^24 too


def run_filtered(pkg, dsx, scores, k, position, index, start, end, fidx, fmul):
    batch, width = scores.shape
    d, di, ds, de, dx, dm = (dev(pkg, x) for x in (scores, index, start, end, fidx, fmul))
    keys = pkg.DeviceArray((batch, k), np.float32)
    vals = pkg.DeviceArray((batch, k), np.uint32)
    pkg.check(dsx.dsx_topk_filtered(d.ptr, keys.ptr, vals.ptr, batch, width, k, position, pkg.ptr(di), ds.ptr, de.ptr, dx.ptr, pkg.ptr(dm)))
    assert np.array_equal(d.numpy(), scores)   # the score matrix itself is not modified
    return keys.numpy(), vals.numpy()


@pytest.mark.parametrize("batch,width,k,maxnnz", [(32, 1024, 10, 16), (64, 27278, 10, 2000), (6, 600000, 100, 1000), (8, 50, 40, 45),
                                                 (3, 9, 9, 9)])
@pytest.mark.parametrize("with_mul", [False, True])
def test_topk_filtered(pkg, dsx, orc, rng, batch, width, k, maxnnz, with_mul):
    say("topk_filtered batch=%d width=%d k=%d mul=%s" % (batch, width, k, with_mul))
    scores = rng.random((batch, width), dtype=np.float32)
    start, end, fidx = random_csr(rng, batch, width, maxnnz, empty_rows=(1,))
    fmul = (rng.random(len(fidx), dtype=np.float32) * 3).astype(np.float32) if with_mul else None   # multipliers above 1 can promote an item
    keys, idx = run_filtered(pkg, dsx, scores, k, 0, None, start, end, fidx, fmul)
    rk, ri = orc.topk_filtered(scores, k, 0, None, start, end, fidx, fmul)
    assert_topk_exact(keys, idx, rk, ri)
    if not with_mul and width - maxnnz >= k:
        for b in range(batch):   # the sample's own items never come back
            assert not set(idx[b].tolist()) & set(fidx[int(start[b]):int(end[b])].tolist())


def test_topk_filtered_indexed_duplicates_and_out_of_range(pkg, dsx, orc, rng):
    rows, batch, width, k, position = 12, 5, 300, 20, 4
    scores = rng.random((batch, width), dtype=np.float32)
    start, end, fidx = random_csr(rng, rows, width + 50, 60)     # some indexes beyond the width: ignored
    fidx = fidx.copy()
    fidx[1::7] = fidx[0::7][: len(fidx[1::7])]                   # duplicates inside rows: applied once
    index = rng.permutation(rows).astype(np.uint32)
    keys, idx = run_filtered(pkg, dsx, scores, k, position, index, start, end, fidx, None)
    rk, ri = orc.topk_filtered(scores, k, position, index, start, end, fidx, None)
    assert_topk_exact(keys, idx, rk, ri)


def segment_maxima(scores):
    batch, width = scores.shape
    nseg = (width + 63) // 64
    pad = np.full((batch, nseg * 64), -np.inf, dtype=np.float32)
    pad[:, :width] = np.where(np.isnan(scores), -np.inf, scores)   # a NaN is never a maximum
    return pad.reshape(batch, nseg, 64).max(axis=2)


def run_guided(pkg, dsx, scores, k, seg_max, position=0, index=None, start=None, end=None, fidx=None, fmul=None, seg_width=64):
    batch, width = scores.shape
    d, dsm, di, ds, de, dx, dm = (dev(pkg, x) for x in (scores, seg_max, index, start, end, fidx, fmul))
    keys = pkg.DeviceArray((batch, k), np.float32)
    vals = pkg.DeviceArray((batch, k), np.uint32)
    pkg.check(dsx.dsx_topk_guided(d.ptr, keys.ptr, vals.ptr, batch, width, k, pkg.ptr(dsm), seg_width, position, pkg.ptr(di), pkg.ptr(ds),
                                  pkg.ptr(de), pkg.ptr(dx), pkg.ptr(dm)))
    return keys.numpy(), vals.numpy()


@pytest.mark.parametrize("batch,width,k", [(16, 27278, 10), (5, 64, 8), (7, 65, 32), (9, 1000, 1), (4, 131072, 32), (3, 40, 32),
                                           (6, 5000, 64), (8, 27278, 50), (5, 5000, 100), (2, 200000, 10),
                                           (9, 27278, 16), (9, 27278, 17), (9, 27278, 33), (9, 130000, 16)])
def test_topk_guided_plain(pkg, dsx, orc, rng, batch, width, k):
    # (5, 5000, 100) and (2, 200000, 10) are outside the guided kernel's range (k > 64, more than 2048 segments): the call scans
    # instead; the shapes after them put k on both sides of the widths of the bound's key search
    say("topk_guided batch=%d width=%d k=%d" % (batch, width, k))
    scores = rng.standard_normal((batch, width), dtype=np.float32)
    keys, idx = run_guided(pkg, dsx, scores, k, segment_maxima(scores))
    rk, ri = orc.topk(scores, k)
    assert_topk_exact(keys, idx, rk, ri)


def test_topk_guided_ties_nan_and_constant_rows(pkg, dsx, orc, rng):
    batch, width, k = 12, 9000, 10
    scores = rng.integers(0, 4, (batch, width)).astype(np.float32)   # four distinct values: whole segments tie at the bound
    scores[1] = 1.0                                                   # a constant row: every segment is read
    scores[2, ::3] = np.nan
    scores[3] = -np.inf
    scores[3, 77] = 2.5
    scores[4, :] = np.nan                                              # nothing to report: sentinels
    keys, idx = run_guided(pkg, dsx, scores, k, segment_maxima(scores))
    sk, si = run_topk(pkg, dsx, scores, k)
    assert_topk_exact(keys, idx, sk, si)          # NaN never enters, in either kernel (rows of NaN give sentinels)
    clean = ~np.isnan(scores).any(axis=1)
    rk, ri = orc.topk(scores[clean], k)
    assert_topk_exact(keys[clean], idx[clean], rk, ri)
    assert np.all(keys[4] == np.float32(-999999999999999.0)) and np.all(idx[4] == 0)


@pytest.mark.parametrize("batch,width,k,maxnnz", [(32, 1024, 10, 16), (64, 27278, 10, 2000), (8, 70, 32, 60), (16, 27278, 32, 5000),
                                                 (16, 27278, 50, 3000), (4, 200, 64, 150)])
@pytest.mark.parametrize("with_mul", [False, True])
def test_topk_guided_filtered(pkg, dsx, orc, rng, batch, width, k, maxnnz, with_mul):
    say("topk_guided filtered batch=%d width=%d k=%d mul=%s" % (batch, width, k, with_mul))
    scores = rng.random((batch, width), dtype=np.float32)
    start, end, fidx = random_csr(rng, batch, width, maxnnz, empty_rows=(1,))
    # make the best scores of many segments listed ones: their maxima must not count towards the bound
    for b in range(batch):
        cols = fidx[int(start[b]):int(end[b])]
        scores[b, cols[: len(cols) // 2]] += np.float32(1.0)
    fmul = (rng.random(len(fidx), dtype=np.float32) * 3).astype(np.float32) if with_mul else None
    keys, idx = run_guided(pkg, dsx, scores, k, segment_maxima(scores), 0, None, start, end, fidx, fmul)
    rk, ri = orc.topk_filtered(scores, k, 0, None, start, end, fidx, fmul)
    assert_topk_exact(keys, idx, rk, ri)
    sk, si = run_filtered(pkg, dsx, scores, k, 0, None, start, end, fidx, fmul)
    assert_topk_exact(keys, idx, sk, si)


@pytest.mark.parametrize("batch,width,k,share", [(64, 27278, 10, 0.13), (64, 27278, 10, 0.004), (16, 27278, 50, 0.4), (3, 300000, 10, 0.13),
                                                  (9, 27278, 100, 0.13), (5, 70000, 200, 0.05), (6, 120000, 10, 0.05), (6, 60000, 16, 0.3),
                                                  (7, 3000, 5, 0.5)])
@pytest.mark.parametrize("filtered", [False, True])
def test_topk_saturated_rows_scan_and_guided(pkg, dsx, orc, rng, batch, width, k, share, filtered):
    """Saturated sigmoids: a share of every row is exactly 1.0, the top of the list is ties all the way down and the lowest
    columns win.  Some of the tied columns are listed in the filter (their zero must not displace anything), one row has
    fewer than k ones, one has a value above 1.0 late in the row.  Wide rows are split over several workgroups."""
    say("topk saturated batch=%d width=%d k=%d share=%g filtered=%s" % (batch, width, k, share, filtered))
    scores = (rng.random((batch, width), dtype=np.float32) * np.float32(0.999)).astype(np.float32)
    scores[rng.random((batch, width)) < share] = 1.0
    scores[1, :] = rng.random(width, dtype=np.float32) * np.float32(0.5)
    scores[1, rng.choice(width, size=max(1, k // 2), replace=False)] = 1.0     # fewer than k ones
    scores[2, width - 5] = 1.5                                                   # the best score comes last
    start = end = fidx = None
    if filtered:
        start, end, fidx = random_csr(rng, batch, width, 400, empty_rows=(0,))
    if filtered:
        keys, idx = run_filtered(pkg, dsx, scores, k, 0, None, start, end, fidx, None)
        rk, ri = orc.topk_filtered(scores, k, 0, None, start, end, fidx, None)
    else:
        keys, idx = run_topk(pkg, dsx, scores, k)
        rk, ri = orc.topk(scores, k)
    assert_topk_exact(keys, idx, rk, ri)
    gk, gi = run_guided(pkg, dsx, scores, k, segment_maxima(scores), 0, None, start, end, fidx, None)
    assert_topk_exact(gk, gi, rk, ri)


@pytest.mark.parametrize("batch,width,k,share", [(48, 27278, 10, 0.13), (8, 27278, 50, 0.4), (4, 120000, 32, 0.02)])
def test_topk_saturated_rows_with_multipliers(pkg, dsx, orc, rng, batch, width, k, share):
    """Tied rows whose listed columns carry multipliers: x1 keeps a listed column in the tie at its own place, x2 puts it on
    top, x0.5 and x0 take it out.  The guided form reads such rows in ascending order of columns and gives its bound a column."""
    say("topk saturated with multipliers batch=%d width=%d k=%d share=%g" % (batch, width, k, share))
    scores = (rng.random((batch, width), dtype=np.float32) * np.float32(0.999)).astype(np.float32)
    scores[rng.random((batch, width)) < share] = 1.0
    start, end, fidx = random_csr(rng, batch, width, 600, empty_rows=(1,))
    fmul = rng.choice(np.array([0.0, 0.5, 1.0, 2.0], dtype=np.float32), size=fidx.size).astype(np.float32)
    keys, idx = run_filtered(pkg, dsx, scores, k, 0, None, start, end, fidx, fmul)
    rk, ri = orc.topk_filtered(scores, k, 0, None, start, end, fidx, fmul)
    assert_topk_exact(keys, idx, rk, ri)
    gk, gi = run_guided(pkg, dsx, scores, k, segment_maxima(scores), 0, None, start, end, fidx, fmul)
    assert_topk_exact(gk, gi, rk, ri)


def test_topk_guided_indexed_filter_and_position(pkg, dsx, orc, rng):
    rows, batch, width, k, position = 40, 17, 3000, 20, 9
    scores = rng.random((batch, width), dtype=np.float32)
    start, end, fidx = random_csr(rng, rows, width + 50, 300)     # some indexes beyond the width: ignored
    fidx = fidx.copy()
    fidx[1::7] = fidx[0::7][: len(fidx[1::7])]                    # duplicates inside rows: applied once
    index = rng.permutation(rows).astype(np.uint32)
    keys, idx = run_guided(pkg, dsx, scores, k, segment_maxima(scores), position, index, start, end, fidx, None)
    rk, ri = orc.topk_filtered(scores, k, position, index, start, end, fidx, None)
    assert_topk_exact(keys, idx, rk, ri)


def test_fc_forward_segmax(pkg, dsx, orc, rng):
    # wide layer: the 128 x 128-tile kernel leaves exact segment maxima, ragged last row block and last column tile included
    B, k, n = 1000, 96, 33000 + 22
    X = rng.standard_normal((B, k), dtype=np.float32)
    W = (rng.standard_normal((k, n), dtype=np.float32) * np.float32(0.2)).astype(np.float32)
    bias = rng.standard_normal(n, dtype=np.float32)
    dX, dW, db = dev(pkg, X), dev(pkg, W), dev(pkg, bias)
    Z = pkg.DeviceArray((B, n), np.float32)
    Z2 = pkg.DeviceArray((B, n), np.float32)
    nseg = (n + 63) // 64
    sm = pkg.DeviceArray.from_numpy(np.full((B, nseg), 7.0, dtype=np.float32))
    sw = C.c_uint32(99)
    pkg.check(dsx.dsx_fc_forward_segmax(dX.ptr, k, dW.ptr, 0, db.ptr, Z.ptr, n, B, k, n, 0, None, sm.ptr, C.byref(sw)))
    pkg.check(dsx.dsx_fc_forward(dX.ptr, k, dW.ptr, 0, db.ptr, Z2.ptr, n, B, k, n, 0, 0, None))
    assert sw.value == 64
    z = Z.numpy()
    assert np.array_equal(z, Z2.numpy())
    assert np.array_equal(sm.numpy(), segment_maxima(z))
    # a narrow layer runs the small-tile kernel: no maxima, and it says so
    n2 = 300
    Zs = pkg.DeviceArray((B, n2), np.float32)
    pkg.check(dsx.dsx_fc_forward_segmax(dX.ptr, k, dW.ptr, 0, db.ptr, Zs.ptr, n2, B, k, n2, 0, None, sm.ptr, C.byref(sw)))
    assert sw.value == 0


# ------------------------------------------------------------------------------------------------------------------- KNN

@pytest.mark.parametrize("items,queries,dim,k", [(1003, 9, 24, 10), (50000, 64, 256, 100), (300007, 130, 64, 128)])
def test_knn_search(pkg, dsx, orc, synth, items, queries, dim, k):
    say("knn items=%d queries=%d dim=%d k=%d" % (items, queries, dim, k))
    p = synth.knn_config(seed=11, items=items, queries=queries, dim=dim, k=k)
    cm, rows, pad = p.column_major_padded()
    cm[:, rows - pad:] = 50.0     # pad rows are uninitialised in the reference (knn/KnnData.cpp:336-340): must never be returned
    dI, dQ = dev(pkg, cm), dev(pkg, p.queries)
    scores = pkg.DeviceArray((queries, k), np.float32)
    idx = pkg.DeviceArray((queries, k), np.uint32)
    el = (C.c_float * 2)()
    pkg.check(dsx.dsx_knn_search(dI.ptr, rows, pad, dim, dQ.ptr, queries, k, scores.ptr, idx.ptr, None, 0, el))
    got_s, got_i = scores.numpy(), idx.numpy()
    ref_s, ref_i = orc.knn_search(cm, rows, pad, dim, p.queries, k)
    full = p.queries.astype(np.float64) @ p.items.astype(np.float64).T
    assert got_i.max() < items
    mism = got_i != ref_i
    if mism.any():   # different summation order may swap neighbours whose scores differ by less than 1e-5
        r, c = np.nonzero(mism)
        assert np.abs(full[r, got_i[r, c]] - full[r, ref_i[r, c]]).max() < 1e-5
    assert_close(got_s, np.take_along_axis(full, got_i.astype(np.int64), axis=1), "knn scores", rel=1e-4, abs_floor=0.05)
    assert el[0] > 0 and el[1] > 0


def knn_case(pkg, dsx, orc, items_m, queries_m, k, pad_value=50.0):
    """Runs dsx_knn_search on row-major items/queries and returns (scores, indexes, oracle scores, oracle indexes, times)."""
    items, dim = items_m.shape
    queries = queries_m.shape[0]
    rows = (items + 7) // 8 * 8
    pad = rows - items
    cm = np.full((dim, rows), pad_value, dtype=np.float32)
    cm[:, :items] = items_m.T
    dI, dQ = dev(pkg, cm), dev(pkg, queries_m)
    scores = pkg.DeviceArray((queries, k), np.float32)
    idx = pkg.DeviceArray((queries, k), np.uint32)
    el = (C.c_float * 2)()
    pkg.check(dsx.dsx_knn_search(dI.ptr, rows, pad, dim, dQ.ptr, queries, k, scores.ptr, idx.ptr, None, 0, el))
    ref_s, ref_i = orc.knn_search(cm, rows, pad, dim, queries_m, k)
    return scores.numpy(), idx.numpy(), ref_s, ref_i, el


@pytest.fixture
def small_knn_blocks(dsx):
    """First column block of 1,024 items, so that searches of a few ten thousand items run the candidate ranges
    (1,024 scanned, then 4,096, 20,480, ... compared with the queries' bounds)."""
    dsx.dsx_testing_set_knn_block_columns(1024)
    yield
    dsx.dsx_testing_set_knn_block_columns(0)


@pytest.mark.parametrize("items,queries,dim,k", [(30011, 70, 64, 100), (9000, 130, 256, 10), (26000, 33, 32, 200), (1500, 5, 16, 64)])
def test_knn_search_candidate_ranges(pkg, dsx, orc, synth, small_knn_blocks, items, queries, dim, k):
    say("knn candidate ranges items=%d queries=%d dim=%d k=%d" % (items, queries, dim, k))
    p = synth.knn_config(seed=5, items=items, queries=queries, dim=dim, k=k)
    got_s, got_i, ref_s, ref_i, _ = knn_case(pkg, dsx, orc, p.items, p.queries, k)
    assert dsx.dsx_knn_last_search_path() == 1       # candidate lists, none of them full
    full = p.queries.astype(np.float64) @ p.items.astype(np.float64).T
    assert got_i.max() < items
    mism = got_i != ref_i
    if mism.any():
        r, c = np.nonzero(mism)
        assert np.abs(full[r, got_i[r, c]] - full[r, ref_i[r, c]]).max() < 1e-5
    assert_close(got_s, np.take_along_axis(full, got_i.astype(np.int64), axis=1), "knn scores", rel=1e-4, abs_floor=0.05)
    assert (np.diff(got_s, axis=1) <= 0).all()


def test_knn_search_candidate_ranges_exact_ties(pkg, dsx, orc, rng, small_knn_blocks):
    """Small integer vectors: every score is an exactly representable integer whatever the order of the sum, thousands of
    items tie, and the result must be the oracle's bit for bit (score descending, then the lower item number)."""
    items, queries, dim, k = 21000, 40, 16, 100
    it = rng.integers(-2, 3, size=(items, dim)).astype(np.float32)
    q = rng.integers(-2, 3, size=(queries, dim)).astype(np.float32)
    got_s, got_i, ref_s, ref_i, _ = knn_case(pkg, dsx, orc, it, q, k)
    assert dsx.dsx_knn_last_search_path() == 1
    assert np.array_equal(got_s, ref_s)
    assert np.array_equal(got_i, ref_i)
    q[3] = 0.0                                       # every item ties at 0 for this query: its candidate list fills up
    got_s, got_i, ref_s, ref_i, _ = knn_case(pkg, dsx, orc, it, q, k)
    assert dsx.dsx_knn_last_search_path() == 2
    assert np.array_equal(got_s, ref_s)
    assert np.array_equal(got_i, ref_i)
    assert np.array_equal(got_i[3], np.arange(k, dtype=np.uint32))


def test_knn_search_full_candidate_list_falls_back(pkg, dsx, orc, rng, small_knn_blocks):
    """Items sorted by rising score for some queries: every later item beats the bound, the candidate lists (4,096 words per
    query and range) fill up, and the search is redone block by block.  The result is exact all the same."""
    items, queries, dim, k = 40000, 12, 8, 50
    direction = rng.standard_normal(dim).astype(np.float32)
    direction /= np.linalg.norm(direction)
    scale = np.linspace(0.001, 1.0, items, dtype=np.float32)
    it = (scale[:, None] * direction[None, :]).astype(np.float32)
    it += (rng.standard_normal((items, dim)) * 1e-4).astype(np.float32)
    q = rng.standard_normal((queries, dim)).astype(np.float32)
    q[0] = direction                                 # scores rise with the item number
    q[1] = -direction                                # and fall: the first block already holds the answer
    got_s, got_i, ref_s, ref_i, _ = knn_case(pkg, dsx, orc, it, q, k)
    assert dsx.dsx_knn_last_search_path() == 2
    full = q.astype(np.float64) @ it.astype(np.float64).T
    mism = got_i != ref_i
    if mism.any():
        r, c = np.nonzero(mism)
        assert np.abs(full[r, got_i[r, c]] - full[r, ref_i[r, c]]).max() < 1e-5
    assert_close(got_s, np.take_along_axis(full, got_i.astype(np.int64), axis=1), "knn scores", rel=1e-4, abs_floor=0.05)
    assert got_i[0].min() >= items - 2 * k and got_i[1].max() < 2 * k


def test_knn_search_nan_scores_never_returned_on_either_path(pkg, dsx, orc, synth):
    """Items with a NaN component score NaN against every query.  The scanning top-K drops NaN; the candidate lists must do the
    same, so both ways of running the search give the same bits and never name such an item."""
    p = synth.knn_config(seed=11, items=20000, queries=24, dim=32, k=50)
    bad = np.arange(7, 20000, 13)
    p.items[bad, 5] = np.nan
    dsx.dsx_testing_set_knn_block_columns(1024)
    try:
        cs, ci, _, _, _ = knn_case(pkg, dsx, orc, p.items, p.queries, 50)
        assert dsx.dsx_knn_last_search_path() == 1
    finally:
        dsx.dsx_testing_set_knn_block_columns(0)
    bs, bi, _, _, _ = knn_case(pkg, dsx, orc, p.items, p.queries, 50)
    assert dsx.dsx_knn_last_search_path() == 0
    assert np.array_equal(ci, bi) and np.array_equal(cs.view(np.uint32), bs.view(np.uint32))
    assert not np.isin(ci, bad).any() and not np.isnan(cs).any()


def test_library_scratch_is_counted_and_released(pkg, dsx, rng):
    """Memory the library allocates for itself (here the partial lists of a split top-K) shows up in dsx_get_memory_usage."""
    g0, g1 = C.c_int(), C.c_int()
    scores = pkg.DeviceArray.from_numpy(rng.random((3, 1 << 20), dtype=np.float32))
    keys = pkg.DeviceArray((3, 256), np.float32)
    vals = pkg.DeviceArray((3, 256), np.uint32)
    pkg.check(dsx.dsx_get_memory_usage(C.byref(g0), None))
    for lane in (0, 1):
        pkg.check(dsx.dsx_set_lane(lane))
        pkg.check(dsx.dsx_topk(scores.ptr, keys.ptr, vals.ptr, 3, 1 << 20, 256))
    pkg.check(dsx.dsx_set_lane(0))
    pkg.check(dsx.dsx_sync())
    pkg.check(dsx.dsx_get_memory_usage(C.byref(g1), None))
    assert g1.value >= g0.value            # lists of this size may already exist from an earlier test; never less


def test_knn_search_unaligned_dim_takes_block_path(pkg, dsx, orc, synth, small_knn_blocks):
    p = synth.knn_config(seed=9, items=5000, queries=17, dim=30, k=20)      # 30 floats per row: no 128-bit loads
    got_s, got_i, ref_s, ref_i, _ = knn_case(pkg, dsx, orc, p.items, p.queries, 20)
    assert dsx.dsx_knn_last_search_path() == 0
    full = p.queries.astype(np.float64) @ p.items.astype(np.float64).T
    mism = got_i != ref_i
    if mism.any():
        r, c = np.nonzero(mism)
        assert np.abs(full[r, got_i[r, c]] - full[r, ref_i[r, c]]).max() < 1e-5
    assert_close(got_s, np.take_along_axis(full, got_i.astype(np.int64), axis=1), "knn scores", rel=1e-4, abs_floor=0.05)


def knn_case_f16(pkg, dsx, orc, items_m, queries_m, k):
    """fp16 storage: the fp32 column-major table is converted on the device, queries inside the search.  The oracle gets the
    same operands rounded to fp16 (numpy rounds to nearest even like __float2half) and multiplies them in fp32."""
    items, dim = items_m.shape
    queries = queries_m.shape[0]
    rows = (items + 7) // 8 * 8
    pad = rows - items
    cm = np.full((dim, rows), 50.0, dtype=np.float32)
    cm[:, :items] = items_m.T
    dI, dQ = dev(pkg, cm), dev(pkg, queries_m)
    table = pkg.DeviceArray((dsx.dsx_knn_f16_table_bytes(rows, dim),), np.uint8)
    pkg.check(dsx.dsx_knn_f16_convert_items(dI.ptr, rows, pad, dim, table.ptr))
    scores = pkg.DeviceArray((queries, k), np.float32)
    idx = pkg.DeviceArray((queries, k), np.uint32)
    el = (C.c_float * 2)()
    pkg.check(dsx.dsx_knn_search_f16(table.ptr, rows, pad, dim, dQ.ptr, queries, k, scores.ptr, idx.ptr, None, 0, el))
    it16 = items_m.astype(np.float16).astype(np.float32)
    q16 = queries_m.astype(np.float16).astype(np.float32)
    cm16 = np.zeros((dim, rows), dtype=np.float32)
    cm16[:, :items] = it16.T
    ref_s, ref_i = orc.knn_search(cm16, rows, pad, dim, q16, k)
    return scores.numpy(), idx.numpy(), ref_s, ref_i, it16, q16, table


# sweep 0: one workgroup per tile of scores; 2: column ranges with at least a tile per chunk go through knn_f16_sweep_kernel
# (with these few queries that is 64 chunks per row tile, so ranges from 8,192 columns on); 3: through knn_f16_wide_kernel
# (queries in registers; ranges from 4,096 columns on; 192 components is the one register layout the other cases leave out)
@pytest.mark.parametrize("sweep", [0, 2, 3])
@pytest.mark.parametrize("items,queries,dim,k,blocks", [(1003, 9, 24, 10, 0), (50000, 64, 256, 100, 0), (30011, 70, 64, 100, 1024),
                                                          (9000, 130, 250, 10, 1024), (26000, 33, 32, 200, 1024),
                                                          (70001, 300, 100, 100, 2048), (60000, 520, 256, 50, 2048),
                                                          (20000, 600, 180, 20, 1024)])
def test_knn_search_f16(pkg, dsx, orc, synth, items, queries, dim, k, blocks, sweep):
    say("knn fp16 items=%d queries=%d dim=%d k=%d first block=%d sweep=%d" % (items, queries, dim, k, blocks, sweep))
    p = synth.knn_config(seed=21, items=items, queries=queries, dim=dim, k=k)
    dsx.dsx_testing_set_knn_block_columns(blocks)
    pkg.check(dsx.dsx_testing_set_knn_f16_sweep(sweep))
    try:
        got_s, got_i, ref_s, ref_i, it16, q16, _ = knn_case_f16(pkg, dsx, orc, p.items, p.queries, k)
        assert dsx.dsx_knn_last_search_path() == (1 if blocks else 0)
    finally:
        dsx.dsx_testing_set_knn_block_columns(0)
        pkg.check(dsx.dsx_testing_set_knn_f16_sweep(1))
    full = q16.astype(np.float64) @ it16.astype(np.float64).T
    assert got_i.max() < items
    mism = got_i != ref_i
    if mism.any():
        r, c = np.nonzero(mism)
        assert np.abs(full[r, got_i[r, c]] - full[r, ref_i[r, c]]).max() < 1e-5
    assert_close(got_s, np.take_along_axis(full, got_i.astype(np.int64), axis=1), "knn fp16 scores", rel=1e-4, abs_floor=0.05)
    assert (np.diff(got_s, axis=1) <= 0).all()


@pytest.mark.parametrize("sweep", [2, 3])
@pytest.mark.parametrize("dim", [64, 128])
def test_knn_search_f16_sweep_spills_clustered_items(pkg, dsx, orc, rng, dim, sweep):
    """300 neighbouring items that all beat a query's bound land in two or three chunks of a sweep, whose lists hold 64 words
    each: the rest goes to the query's shared list, nothing is lost and the search is not redone."""
    items, queries, k = 40000, 70, 100
    it = rng.standard_normal((items, dim)).astype(np.float32)
    q = rng.standard_normal((queries, dim)).astype(np.float32)
    u = q[5] / np.linalg.norm(q[5])
    for j in range(300):
        it[21000 + j] = u * (40.0 + 0.25 * j)   # far above anything else for query 5, all different
    dsx.dsx_testing_set_knn_block_columns(1024)
    pkg.check(dsx.dsx_testing_set_knn_f16_sweep(sweep))
    try:
        got_s, got_i, ref_s, ref_i, it16, q16, _ = knn_case_f16(pkg, dsx, orc, it, q, k)
        assert dsx.dsx_knn_last_search_path() == 1
    finally:
        dsx.dsx_testing_set_knn_block_columns(0)
        pkg.check(dsx.dsx_testing_set_knn_f16_sweep(1))
    assert set(got_i[5]) <= set(range(21000, 21300))
    full = q16.astype(np.float64) @ it16.astype(np.float64).T
    mism = got_i != ref_i
    if mism.any():
        r, c = np.nonzero(mism)
        assert np.abs(full[r, got_i[r, c]] - full[r, ref_i[r, c]]).max() < 1e-5
    assert_close(got_s, np.take_along_axis(full, got_i.astype(np.int64), axis=1), "knn fp16 scores", rel=1e-4, abs_floor=0.05)


def test_knn_f16_table_layout_and_rounding(pkg, dsx, rng):
    """The converted table: item-major rows of ld = dim rounded up to 64 halves, rows rounded up to 256, values rounded to
    nearest even, padding rows and components zero."""
    items, dim = 1003, 24
    rows = (items + 7) // 8 * 8
    it = (rng.standard_normal((items, dim)) * 3).astype(np.float32)
    it[0, :4] = [65504.0, 1e-8, -0.0, 2049.0]          # largest half, flushes towards zero (a subnormal half or 0), -0, a tie (-> 2048)
    cm = np.full((dim, rows), 7.0, dtype=np.float32)
    cm[:, :items] = it.T
    table = pkg.DeviceArray((dsx.dsx_knn_f16_table_bytes(rows, dim),), np.uint8)
    pkg.check(dsx.dsx_knn_f16_convert_items(dev(pkg, cm).ptr, rows, rows - items, dim, table.ptr))
    t = table.numpy().view(np.float16).reshape(-1, 64)
    assert t.shape[0] == 1024
    assert np.array_equal(t[:items, :dim].view(np.uint16), it.astype(np.float16).view(np.uint16))
    assert (t[items:] == 0).all() and (t[:, dim:] == 0).all()


@pytest.mark.parametrize("sweep,dim", [(0, 16), (2, 16), (2, 128), (3, 16), (3, 128), (3, 250)])
def test_knn_search_f16_exact_ties_and_full_lists(pkg, dsx, orc, rng, sweep, dim):
    """Small integers are exact in fp16 too: bit-identical to the oracle, including the query whose candidates all tie (with
    the sweep: its 64-word lists per chunk fill up and spill into the shared list, which fills up as well)."""
    items, queries, k = 21000, 40, 100
    it = rng.integers(-2, 3, size=(items, dim)).astype(np.float32)
    q = rng.integers(-2, 3, size=(queries, dim)).astype(np.float32)
    dsx.dsx_testing_set_knn_block_columns(1024)
    pkg.check(dsx.dsx_testing_set_knn_f16_sweep(sweep))
    try:
        got_s, got_i, ref_s, ref_i, _, _, _ = knn_case_f16(pkg, dsx, orc, it, q, k)
        assert dsx.dsx_knn_last_search_path() == 1
        assert np.array_equal(got_s, ref_s) and np.array_equal(got_i, ref_i)
        q[3] = 0.0
        got_s, got_i, ref_s, ref_i, _, _, _ = knn_case_f16(pkg, dsx, orc, it, q, k)
        assert dsx.dsx_knn_last_search_path() == 2
        assert np.array_equal(got_s, ref_s) and np.array_equal(got_i, ref_i)
    finally:
        dsx.dsx_testing_set_knn_block_columns(0)
        pkg.check(dsx.dsx_testing_set_knn_f16_sweep(1))
