#!/usr/bin/env python3
"""Benchmark of the sparse-recommendation inference path on one MI355X.

A step = one pass of the hot path over one batch of synthetic input already resident in HBM:
sparse input layer (SpMM + bias + ReLU) -> hidden FC layers -> output FC (sigmoid) -> filtered top-K.
Default workload: the 27,278-item recommender autoencoder at batch 1024 (configs[1] of the benchmark definition).

Prints ONE JSON line: whole-job predicted samples/s, the roofline figure of the dominant kernel (timed live with HIP
events on the library's stream), every kernel's own figure, and a CPU baseline (the scalar OpenMP oracle) on a bounded
sample of the same workload.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

import numpy as np  # noqa: E402

import __graft_entry__ as entry  # noqa: E402

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
FP32_MFMA_PEAK_TF = 157.3    # MI355X dense fp32 matrix, published

# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (KiB per dispatch), scaled by what the same counters
# read for a plain 256 MiB device-to-device copy (FETCH_SIZE reads half of the bytes, factor 2.0; WRITE_SIZE factor 1.0).
# Measured on the cfg2 workload; the summary with the commands is profiles/pmc_cfg2_hbm_traffic.md.
MEASURED_TRAFFIC = {
    "cfg2-catalogue-27278": {
        "sparse_z_kernel": {"fetch": 15080 * 1024 * 2.0, "write": 512 * 1024 * 1.0},
        "fc_small_kernel[1024x128x128]": {"fetch": 1107 * 1024 * 2.0, "write": 512 * 1024 * 1.0},
        "fc_gemm_kernel[1024x128x27278]": {"fetch": 11470 * 1024 * 2.0, "write": 147200 * 1024 * 1.0},
        "topk_scan_kernel": {"fetch": 58540 * 1024 * 2.0, "write": 128 * 1024 * 1.0},
        "topk_guided_kernel": {"fetch": 10610 * 1024 * 2.0, "write": 128 * 1024 * 1.0},
    },
}


class StdoutToStderr:
    """Sends everything written to file descriptor 1 (the C++ host layer logs there, like the reference) to stderr, so that
    the JSON line is the only thing on stdout."""

    def __enter__(self):
        sys.stdout.flush()
        self.saved = os.dup(1)
        os.dup2(2, 1)
        return self

    def __exit__(self, *exc):
        sys.stdout.flush()
        os.dup2(self.saved, 1)
        os.close(self.saved)
        return False


SETTLE_SECONDS = 0.06


def settle(pkg, lib, fn, seconds=SETTLE_SECONDS):
    """Untimed: keeps the device busy with fn() for `seconds`.  From idle the clocks of this part ramp up over about 30 ms of
    sustained load (the same launch takes 85 us at the start of a burst and 73 us from then on), so a timed region that
    starts cold measures the ramp, not the kernel."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(20):
            fn()
        pkg.check(lib.dsx_sync())


def time_launches(pkg, lib, fn, reps):
    """Average milliseconds of one call of fn(), measured with HIP events on the library stream over `reps` launches."""
    settle(pkg, lib, fn)
    pkg.check(lib.dsx_timer_start())
    for _ in range(reps):
        fn()
    ms = C.c_float()
    pkg.check(lib.dsx_timer_stop(C.byref(ms)))
    return ms.value / reps


def network_bench(args, pkg, lib):
    from amazon_dsstne_amd import ATTR_BOOLEAN, ATTR_INDEXED, synth
    from amazon_dsstne_amd.pipeline import DevicePipeline

    from amazon_dsstne_amd.host_api import Network

    p = synth.config(args.config)
    B, H, N, K = p.batch, p.widths[1], p.widths[-1], p.k
    nnzB = p.batch_nnz()

    # The timed step goes through the C++ host layer, as a DSSTNE caller would: NNNetwork::PredictBatch on the resident input
    # dataset, then NNNetwork::CalculateFilteredTopK with the sample's own items as the filter.  Inputs, weights and
    # results stay in HBM.
    net = Network(p)
    net.bind_input()

    def step():
        net.predict_batch(0)
        net.topk(K, filter_dataset=net.dataset)
    settle(pkg, lib, step)
    for _ in range(args.warmup):
        step()
    net.sync()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    net.sync()
    t1 = time.perf_counter()
    ms_step = (t1 - t0) * 1e3 / args.steps

    # The step above runs as NNNetwork does by default: consecutive batches alternate between two lanes (two sets of unit
    # buffers on two streams), so one batch's input layers and top-K overlap with the next one's GEMM.  The same on one
    # lane — the reference's single set of buffers, one batch's kernels strictly after the other's — for comparison.
    net.set_lanes(1)
    settle(pkg, lib, step)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    net.sync()
    ms_one_lane = (time.perf_counter() - t0) * 1e3 / args.steps
    net.set_lanes(2)
    step()
    net.sync()

    # The same step when the batch's CSR arrays are handed over as host buffers every time (NNDataSet::LoadSparseData, as the
    # reference's JNI predict does): never `value`, reported beside it.
    up_steps = max(5, min(200, args.steps))
    def upload_step():
        net.load_sparse(p.start, p.end, p.sparse_data, p.sparse_index)
        step()
    # untimed: the first uploads allocate the pinned staging buffers
    settle(pkg, lib, upload_step)
    # (median of four runs of up_steps: somewhere in its first thousand queued copies the HIP runtime grows its pools once, a
    # stall of 6-10 ms that is no part of the steady state and would otherwise land in one run in three)
    runs = []
    for _ in range(4):
        t0 = time.perf_counter()
        for _ in range(up_steps):
            upload_step()
        net.sync()
        runs.append((time.perf_counter() - t0) * 1e3 / up_steps)
    ms_upload = float(np.median(runs))

    # One request at a time, as the reference's JNI predict serves them: upload the batch, predict, top-K, read the results
    # back, and only then the next one.
    rt = []
    for n in range(up_steps + 5):
        t0 = time.perf_counter()
        net.load_sparse(p.start, p.end, p.sparse_data, p.sparse_index)
        step()
        net.get_topk(B)
        if n >= 5:
            rt.append(time.perf_counter() - t0)
    ms_request = float(np.median(rt)) * 1e3

    # The same kernels one at a time on the same shapes (raw C ABI of the kernel library, same stream).
    pipe = DevicePipeline(p, lib)
    pipe.step()
    pkg.check(lib.dsx_sync())

    # per-kernel figures (HIP events around back-to-back launches of one kernel)
    reps = max(10, min(100, args.steps))
    params = C.byref(pipe.params)
    ptr = pkg.ptr
    kernels = {}

    def k_sparse():
        pkg.check(lib.dsx_sparse_layer_forward(p.attributes, p.data_type, 0, B, H, ptr(pipe.W[0]), ptr(pipe.index), ptr(pipe.start),
                                               ptr(pipe.end), ptr(pipe.sidx), ptr(pipe.dw), ptr(pipe.sdata), ptr(pipe.b[0]),
                                               p.acts[0], params, ptr(pipe.units[0])))
    val_bytes = 0 if (p.attributes & ATTR_BOOLEAN) else p.sparse_data.dtype.itemsize
    spmm_bytes = nnzB * (4 * H + 4 + val_bytes) + B * (16 + (4 if (p.attributes & ATTR_INDEXED) else 0)) + 4 * H + 4 * B * H
    ms = time_launches(pkg, lib, k_sparse, reps)
    kernels["sparse_z_kernel"] = {"bound": "hbm", "ms": ms, "achieved": spmm_bytes / ms / 1e6, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                  "algorithmic_bytes": spmm_bytes}

    # the dense layers as the timed step runs them: the last one also leaves segment maxima for the guided top-K
    gp = DevicePipeline(p, lib, guided=True)
    gp.step()
    pkg.check(lib.dsx_sync())
    last = len(pipe.W) - 1
    for l in range(1, len(pipe.W)):
        kk, n = p.widths[l], p.widths[l + 1]

        def k_fc(l=l, kk=kk, n=n):
            if l == last:
                pkg.check(lib.dsx_fc_forward_segmax(ptr(gp.units[l - 1]), kk, ptr(gp.W[l]), 0, ptr(gp.b[l]), ptr(gp.units[l]), n, B, kk, n,
                                                    p.acts[l], params, ptr(gp.seg_max), C.byref(gp.seg_width)))
            else:
                pkg.check(lib.dsx_fc_forward(ptr(pipe.units[l - 1]), kk, ptr(pipe.W[l]), 0, ptr(pipe.b[l]), ptr(pipe.units[l]), n, B, kk, n, 0,
                                             p.acts[l], params))
        flops = 2.0 * B * kk * n
        ms = time_launches(pkg, lib, k_fc, reps)
        small = (kk in (128, 256)) and B * n <= (1 << 20)
        name = "%s[%dx%dx%d]" % ("fc_small_kernel" if small else "fc_gemm_kernel", B, kk, n)
        kernels[name] = {"bound": "mfma", "ms": ms, "achieved": flops / ms / 1e9, "peak": FP32_MFMA_PEAK_TF, "unit": "TFLOP/s",
                         "algorithmic_flops": flops}

    def k_topk():
        pipe.topk()
    topk_bytes = 4 * B * N + 4 * nnzB + 8 * B * K
    ms = time_launches(pkg, lib, k_topk, reps)
    kernels["topk_scan_kernel"] = {"bound": "hbm", "ms": ms, "achieved": topk_bytes / ms / 1e6, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                   "algorithmic_bytes": topk_bytes}
    if gp.seg_width.value:
        # what the timed step runs when the output layer left segment maxima; priced with the scan's algorithmic bytes (it reads
        # a fraction of them, so the figure can exceed the roofline: it measures the work avoided, not bandwidth)
        ms = time_launches(pkg, lib, lambda: gp.topk(), reps)
        kernels["topk_guided_kernel"] = {"bound": "hbm", "ms": ms, "achieved": topk_bytes / ms / 1e6, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                         "algorithmic_bytes": topk_bytes, "note": "reads only the segments that can hold a result"}
    for v in kernels.values():
        v["frac"] = v["achieved"] / v["peak"]

    for n, t in MEASURED_TRAFFIC.get(p.name, {}).items():
        if n in kernels:
            kernels[n]["traffic"] = int(t["fetch"] + t["write"])

    dominant = max(kernels, key=lambda n: kernels[n]["ms"])
    d = kernels[dominant]
    roofline = {"kernel": dominant, "bound": d["bound"], "achieved": round(d["achieved"], 3), "peak": d["peak"], "unit": d["unit"],
                "frac": round(d["frac"], 4), "traffic": d.get("traffic"), "avg_launch_ms": round(d["ms"], 5)}
    if args.calibrate_copy:
        # plain device-to-device copy of known size: what FETCH_SIZE / WRITE_SIZE read for it calibrates the counters
        nbytes = args.calibrate_copy << 20
        src = pkg.DeviceArray((nbytes // 4,), np.float32)
        dst = pkg.DeviceArray((nbytes // 4,), np.float32)
        for _ in range(3):
            pkg.check(lib.dsx_memcpy_d2d(dst.ptr, src.ptr, nbytes))
        pkg.check(lib.dsx_sync())

    # CPU baseline: the oracle (scalar C++ restatement of the reference kernels, OpenMP over rows) on whole batches of the
    # same workload, bounded to about 10-20 s.
    cpu = None
    if args.cpu_seconds > 0:
        orc = entry.load_oracle()
        cores = orc.lib().orc_num_threads()
        # rows per pass sized so that one pass takes a few seconds (about 1.5 GFLOP/s per core for the scalar triple loop)
        row_flops = 2.0 * sum(p.widths[i] * p.widths[i + 1] for i in range(1, len(p.widths) - 1)) + 2.0 * nnzB / B * H
        rows = int(max(8, min(B, 4.0 * 1.5e9 * cores / row_flops)))
        secs, nb = 0.0, 0
        while secs < args.cpu_seconds and nb < 4096:
            s, _, _, _ = orc.forward(p, 0, rows, K, filtered=True)
            secs += s
            nb += 1
        cpu = {"value": round(rows * nb / secs, 1), "unit": "samples/s", "cores": cores, "kind": "port",
               "sample": "%d passes over the first %d rows of one batch of %d of the same workload (%s), %.1f s" % (nb, rows, B, p.name, secs)}

    out = {
        "metric": "predicted samples/sec (sparse-in -> filtered top-K) at batch %d" % B,
        "value": round(B / (ms_step / 1e3), 1),
        "unit": "samples/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": p.name, "batch": B, "input_width": p.widths[0], "layers": p.widths[1:], "top_k": K, "filtered": True,
                   "batch_nnz": nnzB},
        "roofline": roofline,
        "kernels": {n: {k: (round(v, 5) if isinstance(v, float) else v) for k, v in kv.items()} for n, kv in kernels.items()},
        "cpu_baseline": cpu,
        "clock_settle_ms": SETTLE_SECONDS * 1e3,
        "one_lane": {"ms_per_step": round(ms_one_lane, 5), "value": round(B / (ms_one_lane / 1e3), 1), "unit": "samples/s",
                     "note": "NNNetwork::SetLanes(1): one set of buffers, one stream, batches strictly one after the other"},
        "with_input_upload": {"ms_per_step": round(ms_upload, 5), "value": round(B / (ms_upload / 1e3), 1), "unit": "samples/s",
                              "note": "the batch's CSR arrays handed over as host memory before every step (NNDataSet::LoadSparseData; PCIe-inclusive): uploads go to alternating sets of device arrays on the lane of the batch they belong to"},
        "request_round_trip": {"ms": round(ms_request, 5), "value": round(B / (ms_request / 1e3), 1), "unit": "samples/s",
                               "note": "median over requests served one at a time: upload, predict, filtered top-K, results read back"},
    }
    return out


def knn_bench(args, pkg, lib):
    from amazon_dsstne_amd import synth

    p = synth.knn_config(items=args.knn_items)
    cm, rows, pad = p.column_major_padded()
    Q, D, K = p.queries.shape[0], p.queries.shape[1], p.k
    dI = pkg.DeviceArray.from_numpy(cm, lib)
    dQ = pkg.DeviceArray.from_numpy(p.queries, lib)
    scores = pkg.DeviceArray((Q, K), np.float32, lib)
    idx = pkg.DeviceArray((Q, K), np.uint32, lib)
    el = (C.c_float * 2)()

    def step(timing=None):
        pkg.check(lib.dsx_knn_search(dI.ptr, rows, pad, D, dQ.ptr, Q, K, scores.ptr, idx.ptr, None, 0, timing))
    for _ in range(args.warmup):
        step()
    pkg.check(lib.dsx_sync())
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    pkg.check(lib.dsx_sync())
    ms_step = (time.perf_counter() - t0) * 1e3 / args.steps
    step(el)
    flops = 2.0 * Q * D * (rows - pad)
    roofline = {"kernel": "fc_gemm_kernel (knn scores)", "bound": "mfma", "achieved": round(flops / el[0] / 1e9, 3), "peak": FP32_MFMA_PEAK_TF,
                "unit": "TFLOP/s", "frac": round(flops / el[0] / 1e9 / FP32_MFMA_PEAK_TF, 4), "traffic": None, "avg_launch_ms": round(el[0], 4),
                "topk_ms": round(el[1], 4),
                "path": {0: "blocks", 1: "candidate lists", 2: "candidate lists, redone block by block"}[lib.dsx_knn_last_search_path()]}
    # the same search with fp16 storage of items and queries (the reference's DataType::FP16): reported beside the fp32 figure
    table = pkg.DeviceArray((lib.dsx_knn_f16_table_bytes(rows, D),), np.uint8, lib)
    pkg.check(lib.dsx_knn_f16_convert_items(dI.ptr, rows, pad, D, table.ptr))

    def step16(timing=None):
        pkg.check(lib.dsx_knn_search_f16(table.ptr, rows, pad, D, dQ.ptr, Q, K, scores.ptr, idx.ptr, None, 0, timing))
    for _ in range(max(1, args.warmup)):
        step16()
    pkg.check(lib.dsx_sync())
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step16()
    pkg.check(lib.dsx_sync())
    ms16 = (time.perf_counter() - t0) * 1e3 / args.steps
    step16(el)
    f16 = {"ms_per_step": round(ms16, 4), "value": round(Q / (ms16 / 1e3), 1), "unit": "queries/s", "dtype": "f16 operands, f32 sums",
           "kernel": "knn_f16_kernel", "bound": "mfma", "achieved": round(flops / el[0] / 1e9, 3), "peak": 2500.0, "unit_roofline": "TFLOP/s",
           "frac": round(flops / el[0] / 1e9 / 2500.0, 4), "scores_ms": round(el[0], 4), "topk_ms": round(el[1], 4),
           "path": {0: "blocks", 1: "candidate lists", 2: "candidate lists, redone block by block"}[lib.dsx_knn_last_search_path()]}
    cpu = None
    if args.cpu_seconds > 0:
        orc = entry.load_oracle()
        nq, secs, done = 32, 0.0, 0
        while secs < args.cpu_seconds and done + nq <= Q:
            t0 = time.perf_counter()
            orc.knn_search(cm, rows, pad, D, p.queries[done:done + nq], K)
            secs += time.perf_counter() - t0
            done += nq
        cpu = {"value": round(done / secs, 2), "unit": "queries/s", "cores": orc.lib().orc_num_threads(), "kind": "port",
               "sample": "the first %d of the %d queries against the full item table, %.1f s" % (done, Q, secs)}
    return {"metric": "KNN queries/sec (exact top-%d over %d items)" % (K, rows - pad), "value": round(Q / (ms_step / 1e3), 1),
            "unit": "queries/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_step, 4),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
            "config": {"workload": p.name, "queries": Q, "dim": D, "items": rows - pad, "top_k": K}, "roofline": roofline,
            "cpu_baseline": cpu, "f16_storage": f16}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", type=int, default=2, help="1..4 = networks of the benchmark definition, 5 = KNN")
    ap.add_argument("--knn-items", type=int, default=2000000)
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="CPU baseline budget; 0 skips it")
    ap.add_argument("--calibrate-copy", type=int, default=0, help="also run a plain d2d copy of this many MiB (counter calibration)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (the whole model lives in one MI355X's HBM); --gpus %d is not supported"
                 % args.gpus)
    with StdoutToStderr():
        pkg = entry.load_package()
        lib = pkg.init(0)
        out = knn_bench(args, pkg, lib) if args.config == 5 else network_bench(args, pkg, lib)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
