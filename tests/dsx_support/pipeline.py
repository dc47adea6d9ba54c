"""Chain-network driver over the C ABI: sparse input -> fully connected stack -> (filtered) top-K on device-resident data.

Mirrors the call sequence of NNNetwork::PredictBatch (engine/NNNetwork.cpp:1376-1429) followed by the filtered
recommendations of NNRecsGenerator::generateRecs (utils/NNRecsGenerator.cpp:132-150) for a synth.Problem.  Used by the
benchmark, the smoke check and the parity tests; every numeric step runs in libdsx_hip.so.
"""
import ctypes as C

import numpy as np

from amazon_dsstne_amd import ACT_SOFTMAX, ActParams, DeviceArray, check, load_library, ptr


class DevicePipeline:
    def __init__(self, problem, lib=None, guided=False, split=False):
        """guided: the output layer also leaves segment maxima (dsx_fc_forward_segmax) and the top-K uses them.
        split: the output layer forms its fp32 products from bf16 matrix instructions (dsx_fc_split / dsx_fc_forward_split)."""
        self.lib = lib or load_library()
        p = self.p = problem
        self.guided = guided
        self.seg_max = DeviceArray((p.batch, (p.widths[-1] + 63) // 64), np.float32, self.lib) if guided else None
        self.seg_width = C.c_uint32(0)
        self.W = [DeviceArray.from_numpy(w, self.lib) for w in p.weights]
        self.b = [DeviceArray.from_numpy(b, self.lib) for b in p.biases]
        self.start = DeviceArray.from_numpy(p.start, self.lib)
        self.end = DeviceArray.from_numpy(p.end, self.lib)
        self.sidx = DeviceArray.from_numpy(p.sparse_index, self.lib)
        self.sdata = DeviceArray.from_numpy(p.sparse_data, self.lib) if p.sparse_data is not None else None
        self.index = DeviceArray.from_numpy(p.index, self.lib) if p.index is not None else None
        self.dw = DeviceArray.from_numpy(p.data_weight, self.lib) if p.data_weight is not None else None
        self.units = [DeviceArray((p.batch, w), np.float32, self.lib) for w in p.widths[1:]]
        self.keys = DeviceArray((p.batch, 256), np.float32, self.lib)
        self.vals = DeviceArray((p.batch, 256), np.uint32, self.lib)
        self.params = ActParams(0.01, 1.0, 1.0)
        self.split = split
        if split:
            k, n = p.widths[-2], p.widths[-1]
            self.w_planes = DeviceArray((self.lib.dsx_fc_split_bytes(n, k) // 4,), np.uint32, self.lib)
            self.x_planes = DeviceArray((self.lib.dsx_fc_split_bytes(p.batch, k) // 4,), np.uint32, self.lib)
            check(self.lib.dsx_fc_split(ptr(self.W[-1]), n, 1, n, k, ptr(self.w_planes)))   # weights: once

    def forward(self, position=0, batch=None):
        """All layers; returns nothing (activations stay in self.units)."""
        p, lib = self.p, self.lib
        batch = p.batch if batch is None else batch
        act0 = p.acts[0]
        if act0 == ACT_SOFTMAX:
            raise NotImplementedError("softmax first layer")
        check(lib.dsx_sparse_layer_forward(p.attributes, p.data_type, position, batch, p.widths[1], ptr(self.W[0]), ptr(self.index),
                                           ptr(self.start), ptr(self.end), ptr(self.sidx), ptr(self.dw), ptr(self.sdata),
                                           ptr(self.b[0]), act0, C.byref(self.params), ptr(self.units[0])))
        for l in range(1, len(self.W)):
            k, n = p.widths[l], p.widths[l + 1]
            act = p.acts[l]
            fused = act if act != ACT_SOFTMAX else 3
            if self.split and l == len(self.W) - 1:
                check(lib.dsx_fc_split(ptr(self.units[l - 1]), k, 0, batch, k, ptr(self.x_planes)))
                g = self.guided and act != ACT_SOFTMAX
                check(lib.dsx_fc_forward_split(ptr(self.x_planes), ptr(self.w_planes), ptr(self.b[l]), ptr(self.units[l]), n, batch, k, n, 0,
                                               fused, C.byref(self.params), ptr(self.seg_max) if g else None,
                                               C.byref(self.seg_width) if g else None))
                if act == ACT_SOFTMAX:
                    check(lib.dsx_activation(ptr(self.units[l]), batch, n, act, C.byref(self.params)))
                continue
            if self.guided and l == len(self.W) - 1 and act != ACT_SOFTMAX:
                check(lib.dsx_fc_forward_segmax(ptr(self.units[l - 1]), k, ptr(self.W[l]), 0, ptr(self.b[l]), ptr(self.units[l]), n, batch, k,
                                                n, fused, C.byref(self.params), ptr(self.seg_max), C.byref(self.seg_width)))
                continue
            check(lib.dsx_fc_forward(ptr(self.units[l - 1]), k, ptr(self.W[l]), 0, ptr(self.b[l]), ptr(self.units[l]), n, batch, k, n, 0,
                                     fused, C.byref(self.params)))
            if act == ACT_SOFTMAX:
                check(lib.dsx_activation(ptr(self.units[l]), batch, n, act, C.byref(self.params)))

    def topk(self, position=0, batch=None, k=None, filtered=True):
        p, lib = self.p, self.lib
        batch = p.batch if batch is None else batch
        k = p.k if k is None else k
        N = p.widths[-1]
        if self.guided:
            f = filtered
            check(lib.dsx_topk_guided(ptr(self.units[-1]), ptr(self.keys), ptr(self.vals), batch, N, k, ptr(self.seg_max),
                                      self.seg_width.value, position, ptr(self.index) if f else None, ptr(self.start) if f else None,
                                      ptr(self.end) if f else None, ptr(self.sidx) if f else None, None))
        elif filtered:
            check(lib.dsx_topk_filtered(ptr(self.units[-1]), ptr(self.keys), ptr(self.vals), batch, N, k, position, ptr(self.index),
                                        ptr(self.start), ptr(self.end), ptr(self.sidx), None))
        else:
            check(lib.dsx_topk(ptr(self.units[-1]), ptr(self.keys), ptr(self.vals), batch, N, k))

    def step(self, position=0, batch=None, k=None, filtered=True):
        self.forward(position, batch)
        self.topk(position, batch, k, filtered)

    def results(self, batch=None, k=None):
        p = self.p
        batch = p.batch if batch is None else batch
        k = p.k if k is None else k
        keys = self.keys.numpy().reshape(-1)[: batch * k].reshape(batch, k)
        vals = self.vals.numpy().reshape(-1)[: batch * k].reshape(batch, k)
        return keys, vals

    def output_unit(self, batch=None):
        batch = self.p.batch if batch is None else batch
        return self.units[-1].numpy()[:batch]
