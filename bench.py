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
BF16_MFMA_PEAK_TF = 2500.0       # dense bf16 MFMA, the published figure

# HBM bytes per launch, measured: profiles/pmc_hbm_traffic.json holds, per workload and kernel, what rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE read (KiB per dispatch) and the calibration factors from a plain 256 MiB device-to-device copy in the same runs; the
# summary beside it (profiles/pmc_cfg2_hbm_traffic.md) is made from the same file and gives the commands.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "pmc_hbm_traffic.json")
BATCHES = 8                  # distinct batches resident in HBM that the timed loop cycles over
WINDOWS = 5                  # timed windows of --steps steps each; the median is reported


def measured_traffic(workload):
    try:
        with open(TRAFFIC_FILE) as f:
            t = json.load(f)
    except OSError:
        return {}
    w = t.get("workloads", {}).get(workload, {})
    ff, wf = t.get("fetch_factor", 1.0), t.get("write_factor", 1.0)
    out = {}
    for k, v in w.items():
        out[k] = {"read": int(v["fetch_kib"] * 1024 * ff), "write": int(v["write_kib"] * 1024 * wf)}
        if "l2_hit" in v and "l2_miss" in v and v["l2_hit"] + v["l2_miss"] > 0:
            out[k]["l2_hit_rate"] = round(v["l2_hit"] / (v["l2_hit"] + v["l2_miss"]), 4)
    return out


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


def timed_windows(step, sync, steps, windows):
    """`windows` regions of exactly `steps` calls of step(i), each bracketed by sync(); milliseconds per step of every region."""
    out = []
    n = 0
    for _ in range(windows):
        sync()
        t0 = time.perf_counter()
        for _ in range(steps):
            step(n)
            n += 1
        sync()
        out.append((time.perf_counter() - t0) * 1e3 / steps)
    return out


def calibration_copy(args, pkg, lib):
    """--calibrate-copy N: a plain device-to-device copy of N MiB; what FETCH_SIZE / WRITE_SIZE read for it calibrates the counters."""
    if not args.calibrate_copy:
        return
    nbytes = args.calibrate_copy << 20
    src = pkg.DeviceArray((nbytes // 4,), np.float32)
    dst = pkg.DeviceArray((nbytes // 4,), np.float32)
    for _ in range(3):
        pkg.check(lib.dsx_memcpy_d2d(dst.ptr, src.ptr, nbytes))
    pkg.check(lib.dsx_sync())


def interference_block(pkg, lib, p, steps):
    """What each kernel of a batch costs the output layer's GEMM when it runs beside it: the GEMMs back to back on lane 0, the
    other kernel back to back on lane 1, nothing ordering the two (no step can do better than that with these kernels), and the
    same with a probe that only holds its workgroups' places (dsx_testing_occupy).  Microseconds per GEMM."""
    from dsx_support.pipeline import DevicePipeline
    ptr = pkg.ptr
    pipes = [DevicePipeline(p, lib, guided=True) for _ in range(2)]
    for q in pipes:
        q.step()
    pkg.check(lib.dsx_sync())
    B, last = p.batch, len(p.weights) - 1

    def gemm(q):
        kk, n = p.widths[last], p.widths[last + 1]
        pkg.check(lib.dsx_fc_forward_segmax(ptr(q.units[last - 1]), kk, ptr(q.W[last]), 0, ptr(q.b[last]), ptr(q.units[last]), n, B, kk, n,
                                            p.acts[last], C.byref(q.params), ptr(q.seg_max), C.byref(q.seg_width)))

    def sparse(q):
        pkg.check(lib.dsx_sparse_layer_forward(p.attributes, p.data_type, 0, B, p.widths[1], ptr(q.W[0]), ptr(q.index), ptr(q.start), ptr(q.end),
                                               ptr(q.sidx), ptr(q.dw), ptr(q.sdata), ptr(q.b[0]), p.acts[0], C.byref(q.params), ptr(q.units[0])))

    def hidden(q):
        for l in range(1, last):
            kk, n = p.widths[l], p.widths[l + 1]
            pkg.check(lib.dsx_fc_forward(ptr(q.units[l - 1]), kk, ptr(q.W[l]), 0, ptr(q.b[l]), ptr(q.units[l]), n, B, kk, n, 0, p.acts[l],
                                         C.byref(q.params)))

    def us(step):
        def run(i):
            step(i)
        settle(pkg, lib, lambda: run(0))
        w = timed_windows(run, lambda: pkg.check(lib.dsx_sync()), steps, 3)
        pkg.check(lib.dsx_set_lane(0))
        return round(float(np.median(w)) * 1e3, 2)

    def beside(other):
        def step(i):
            pkg.check(lib.dsx_set_lane(0))
            gemm(pipes[0])
            pkg.check(lib.dsx_set_lane(1))
            other(pipes[1])
        return step

    def two_lanes(i):
        pkg.check(lib.dsx_set_lane(i % 2))
        gemm(pipes[i % 2])

    def everything(q):
        q.topk()
        sparse(q)
        hidden(q)
    out = {"unit": "us per output-layer GEMM",
           "gemm_alone": us(lambda i: gemm(pipes[0])),
           "gemm_two_lanes": us(two_lanes),
           "beside_sparse_layer": us(beside(sparse)),
           "beside_hidden_layers": us(beside(hidden)),
           "beside_guided_topk": us(beside(lambda q: q.topk())),
           "beside_all_of_them": us(beside(everything)),
           "beside_probe": {}}
    for wgs, cycles, regs in ((1024, 20000, 128), (1024, 20000, 64), (1024, 20000, 0), (2048, 20000, 64), (256, 80000, 64), (256, 80000, 128),
                              (1024, 10, 0)):
        out["beside_probe"]["%d workgroups x %d cycles, %d registers" % (wgs, cycles, regs)] = us(
            beside(lambda q, wgs=wgs, cycles=cycles, regs=regs: pkg.check(lib.dsx_testing_occupy(wgs, cycles, regs))))
    out["note"] = ("lane 0: the GEMMs back to back; lane 1: the named kernel(s) back to back, unordered against lane 0.  The probe issues no "
                   "vector or memory instruction: what it costs is the place its workgroups take (20,000 cycles are about 8 us)")
    return out


def network_bench(args, pkg, lib):
    from amazon_dsstne_amd import ATTR_BOOLEAN, ATTR_INDEXED
    from dsx_support import synth
    from dsx_support.pipeline import DevicePipeline

    from amazon_dsstne_amd.host_api import Network

    batches = 1 if args.config == 4 else BATCHES      # config 4's generator takes seconds per batch; its step is 33 ms of GEMM
    p = synth.config(args.config, batches=batches)
    B, H, N, K = p.batch, p.widths[1], p.widths[-1], p.k
    nnzB = p.batch_nnz()
    nnz_mean = p.nnz / batches

    # The timed step goes through the C++ host layer, as a DSSTNE caller would: NNNetwork::PredictBatch on the resident input
    # dataset, then NNNetwork::CalculateFilteredTopK with the sample's own items as the filter.  Inputs, weights and
    # results stay in HBM; consecutive steps take consecutive batches of the resident dataset.
    net = Network(p)
    net.bind_input()
    if args.lanes != 2:
        net.set_lanes(args.lanes)   # NNNetwork's default is two

    def step(i=0):
        net.predict_batch((i % batches) * B)
        net.topk(K, filter_dataset=net.dataset)

    # From idle the clocks of this part ramp up over tens of milliseconds: what a caller sees who sends a burst after a pause.
    net.sync()
    time.sleep(2.5)
    for i in range(args.warmup):
        step(i)
    ms_cold = timed_windows(step, net.sync, args.steps, 1)[0]

    settle(pkg, lib, step)
    for i in range(args.warmup):
        step(i)
    windows = timed_windows(step, net.sync, args.steps, WINDOWS)
    ms_step = float(np.median(windows))

    # The step above runs as NNNetwork does by default: consecutive batches alternate between two lanes (two sets of unit
    # buffers on two streams), so one batch's input layers and top-K overlap with the next one's GEMM.  The same on one
    # lane — the reference's single set of buffers, one batch's kernels strictly after the other's — for comparison.
    net.set_lanes(1)
    settle(pkg, lib, step)
    ms_one_lane = float(np.median(timed_windows(step, net.sync, args.steps, 3)))
    net.set_lanes(args.lanes)
    # ... and with the output layer stored by PredictBatch as the reference does, instead of computed together with the top-K
    # (NNNetwork::SetDeferredOutput; only layers of 131,072 units or more are deferred, so this differs for config 4 alone)
    net.set_deferred_output(False)
    settle(pkg, lib, step)
    ms_stored = float(np.median(timed_windows(step, net.sync, args.steps, 3)))
    net.set_deferred_output(True)
    # ... and with the wide dense layers' fp32 products formed from bf16 matrix instructions (NNNetwork::SetSplitProducts: three
    # bf16 planes per operand, six MFMA terms per product, fp32 sums; as close to fp64 as the fp32 kernel, not bit-identical to
    # it).  A mode the caller asks for: reported beside `value`, never as `value`.
    net.set_split_products(True)
    settle(pkg, lib, step)
    ms_split = float(np.median(timed_windows(step, net.sync, args.steps, 3)))
    net.set_split_products(False)
    net.sync()
    net.close()

    # The same step when the batch's CSR arrays are handed over as host buffers every time (NNDataSet::LoadSparseData, as the
    # reference's JNI predict does): never `value`, reported beside it.  (A second network whose dataset holds one batch.)
    p1 = synth.config(args.config)
    net = Network(p1)
    net.bind_input()

    def step1():
        net.predict_batch(0)
        net.topk(K, filter_dataset=net.dataset)
    up_steps = max(5, min(200, args.steps))
    def upload_step():
        net.load_sparse(p1.start, p1.end, p1.sparse_data, p1.sparse_index)
        step1()
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
        net.load_sparse(p1.start, p1.end, p1.sparse_data, p1.sparse_index)
        step1()
        net.get_topk(B)
        if n >= 5:
            rt.append(time.perf_counter() - t0)
    ms_request = float(np.median(rt)) * 1e3
    net.close()

    # The same kernels one at a time on the first batch (raw C ABI of the kernel library, same stream): HIP events around
    # back-to-back launches of one kernel, clocks settled.
    pipe = DevicePipeline(p, lib)
    pipe.step()
    pkg.check(lib.dsx_sync())
    reps = max(10, min(100, args.steps))
    params = C.byref(pipe.params)
    ptr = pkg.ptr
    kernels = {}
    traffic = measured_traffic(p.name)

    def k_sparse():
        pkg.check(lib.dsx_sparse_layer_forward(p.attributes, p.data_type, 0, B, H, ptr(pipe.W[0]), ptr(pipe.index), ptr(pipe.start),
                                               ptr(pipe.end), ptr(pipe.sidx), ptr(pipe.dw), ptr(pipe.sdata), ptr(pipe.b[0]),
                                               p.acts[0], params, ptr(pipe.units[0])))
    val_bytes = 0 if (p.attributes & ATTR_BOOLEAN) else p.sparse_data.dtype.itemsize
    fixed = B * (16 + (4 if (p.attributes & ATTR_INDEXED) else 0)) + 4 * H + 4 * B * H
    spmm_bytes = nnzB * (4 * H + 4 + val_bytes) + fixed
    rows0 = np.arange(B) if p.index is None else p.index[:B]
    touched = np.unique(np.concatenate([p.sparse_index[int(p.start[r]):int(p.end[r])] for r in rows0])).size
    compulsory = touched * 4 * H + nnzB * (4 + val_bytes) + fixed     # every distinct weight row once
    ms = time_launches(pkg, lib, k_sparse, reps)
    # The sparse layer gathers weight rows that other rows of the batch (and the L2 / last-level cache) mostly already hold: the
    # bytes it moves to and from HBM are the counters' (profiles/pmc_hbm_traffic.json), and its roofline fraction is those over the
    # launch time.  The rate at which it consumes gathered bytes (every non-zero's weight row, no reuse) is reported beside it
    # with the L2 hit rate: a figure of the gather machinery, not of HBM.
    sp_traffic = traffic.get("sparse_z_kernel")
    sp = {"bound": "hbm", "ms": ms, "peak": HBM_PEAK_GBS, "unit": "GB/s", "compulsory_bytes": compulsory,
          "gather": {"bytes": spmm_bytes, "rate_gbs": round(spmm_bytes / ms / 1e6, 1),
                     "note": "every non-zero gathers its weight row (no reuse): served by L2 and the last-level cache, not a bandwidth of HBM"},
          "note": "achieved = HBM bytes per launch as FETCH_SIZE / WRITE_SIZE count them over the launch time; compulsory_bytes = every distinct weight row of the batch once"}
    if sp_traffic:
        sp["achieved"] = (sp_traffic["read"] + sp_traffic["write"]) / ms / 1e6
        if sp_traffic.get("l2_hit_rate") is not None:
            sp["gather"]["l2_hit_rate"] = sp_traffic["l2_hit_rate"]
    kernels["sparse_z_kernel"] = sp

    # the dense layers as the stored-output step runs them: the last one also leaves segment maxima for the guided top-K
    gp = DevicePipeline(p, lib, guided=True)
    gp.step()
    pkg.check(lib.dsx_sync())
    last = len(pipe.W) - 1
    flops_step = 0.0
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
        flops_step += flops
        ms = time_launches(pkg, lib, k_fc, reps)
        small = (kk in (128, 256)) and B * n <= (1 << 20)
        name = "%s[%dx%dx%d]" % ("fc_small_kernel" if small else "fc_gemm_kernel", B, kk, n)
        kernels[name] = {"bound": "mfma", "ms": ms, "achieved": flops / ms / 1e9, "peak": FP32_MFMA_PEAK_TF, "unit": "TFLOP/s",
                         "algorithmic_flops": flops}
    gemm_name = name

    def k_topk():
        pipe.topk()
    topk_bytes = 4 * B * N + 4 * nnzB + 8 * B * K
    ms = time_launches(pkg, lib, k_topk, reps)
    kernels["topk_scan_kernel"] = {"bound": "hbm", "ms": ms, "achieved": topk_bytes / ms / 1e6, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                   "algorithmic_bytes": topk_bytes}
    for v in kernels.values():
        if "achieved" in v:
            v["frac"] = v["achieved"] / v["peak"]
    if gp.seg_width.value:
        # what the step runs when the output layer left segment maxima: it reads the maxima and the few segments that can hold a
        # result, so it is a chain of dependent loads, not a stream.  Its figure is the bandwidth of what it really moves.
        ms = time_launches(pkg, lib, lambda: gp.topk(), reps)
        moved = traffic.get("topk_guided_kernel")
        g = {"bound": "latency", "ms": ms, "replaces_scan_of_bytes": topk_bytes,
             "note": "reads the segment maxima and the segments that can hold a result instead of scanning the row"}
        if moved:
            g.update({"achieved": (moved["read"] + moved["write"]) / ms / 1e6, "peak": HBM_PEAK_GBS, "unit": "GB/s"})
            g["frac"] = g["achieved"] / g["peak"]
        kernels["topk_guided_kernel"] = g
    deferred = N >= 131072      # NNLayer defers output layers from this width on
    if deferred:
        keys = pkg.DeviceArray((B, K), np.float32)
        vals = pkg.DeviceArray((B, K), np.uint32)

        def k_fused():
            pkg.check(lib.dsx_fc_topk(ptr(pipe.units[last - 1]), p.widths[last], ptr(pipe.W[last]), ptr(pipe.b[last]), B, p.widths[last], N,
                                      p.acts[last], params, K, keys.ptr, vals.ptr, 0, ptr(pipe.index), ptr(pipe.start), ptr(pipe.end),
                                      ptr(pipe.sidx)))
        flops = 2.0 * B * p.widths[last] * N
        ms = time_launches(pkg, lib, k_fused, max(5, reps // 4))
        kernels["dsx_fc_topk (output layer + filtered top-K, nothing stored)"] = {
            "bound": "mfma", "ms": ms, "achieved": flops / ms / 1e9, "peak": FP32_MFMA_PEAK_TF, "unit": "TFLOP/s",
            "algorithmic_flops": flops, "frac": flops / ms / 1e9 / FP32_MFMA_PEAK_TF,
            "note": "what the timed step runs for this layer: first column block stored and scanned, the rest compared in registers"}

    # The output layer's kernel of the split-products mode (off by default, so never the dominant kernel of `roofline`): priced as the
    # bf16 matrix work it executes, six products per fp32 product, against the bf16 peak.
    split_name = None
    info = pkg.DeviceInfo()
    pkg.check(lib.dsx_get_device_info(info))
    if ((B + 127) // 128) * ((N + 127) // 128) >= 2 * info.compute_units:
        kk = p.widths[last]
        xs = pkg.DeviceArray((lib.dsx_fc_split_bytes(B, kk) // 4,), np.uint32, lib)
        ws = pkg.DeviceArray((lib.dsx_fc_split_bytes(N, kk) // 4,), np.uint32, lib)
        pkg.check(lib.dsx_fc_split(ptr(gp.W[last]), N, 1, N, kk, ws.ptr))
        pkg.check(lib.dsx_fc_split(ptr(gp.units[last - 1]), kk, 0, B, kk, xs.ptr))

        def k_split():
            pkg.check(lib.dsx_fc_forward_split(xs.ptr, ws.ptr, ptr(gp.b[last]), ptr(gp.units[last]), N, B, kk, N, 0, p.acts[last], params,
                                               ptr(gp.seg_max), C.byref(gp.seg_width)))
        flops = 2.0 * B * kk * N
        ms = time_launches(pkg, lib, k_split, reps)
        split_name = "fc_gemm_split_kernel[%dx%dx%d]" % (B, kk, N)
        kernels[split_name] = {"bound": "mfma", "ms": ms, "achieved": 6 * flops / ms / 1e9, "peak": BF16_MFMA_PEAK_TF, "unit": "TFLOP/s",
                               "frac": 6 * flops / ms / 1e9 / BF16_MFMA_PEAK_TF, "algorithmic_flops": flops,
                               "fp32_equivalent_tflops": flops / ms / 1e9,
                               "note": "split-products mode only: six bf16 x bf16 products per fp32 product, priced as executed bf16 work against the bf16 peak"}
        del xs, ws

    for n, t in traffic.items():
        if n in kernels:
            kernels[n]["traffic"] = t["read"] + t["write"]
            kernels[n]["traffic_read"] = t["read"]
            kernels[n]["traffic_write"] = t["write"]
            if "l2_hit_rate" in t:
                kernels[n]["l2_hit_rate"] = t["l2_hit_rate"]

    candidates = [n for n in kernels if "frac" in kernels[n] and n != split_name and not (deferred and n in (gemm_name, "topk_scan_kernel"))]
    dominant = max(candidates, key=lambda n: kernels[n]["ms"])
    d = kernels[dominant]
    roofline = {"kernel": dominant, "bound": d["bound"], "achieved": round(d["achieved"], 3), "peak": d["peak"], "unit": d["unit"],
                "frac": round(d["frac"], 4), "traffic": d.get("traffic"), "avg_launch_ms": round(d["ms"], 5),
                "note": "isolated back-to-back launches, clocks settled; `pipeline` below prices the whole timed step"}
    calibration_copy(args, pkg, lib)

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

    interference = None
    if args.interference and gp.seg_width.value and not deferred:
        del pipe, gp
        interference = interference_block(pkg, lib, p, max(50, min(300, args.steps)))

    def rate(ms):
        return round(B / (ms / 1e3), 1)
    out = {
        "metric": "predicted samples/sec (sparse-in -> filtered top-K) at batch %d" % B,
        "value": rate(ms_step),
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
                   "resident_batches": batches, "batch_nnz": nnzB, "mean_batch_nnz": round(nnz_mean, 1), "lanes": args.lanes,
                   "weights": "N(0, std %g) (the definition's N(0, 0.01) read as a variance), biases %s" % (
                       p.law["weight_std"], "0" if not p.law["bias_std"] else "N(0, std %g)" % p.law["bias_std"]),
                   "index_law": p.law["index_law"], "nnz_per_row": p.law["nnz_per_row"], "values": p.law["values"],
                   "indexed_rows": p.law["indexed_rows"], "seed": p.law["seed"]},
        "windows": {"count": WINDOWS, "steps_each": args.steps, "ms_per_step": [round(w, 5) for w in windows],
                    "min": round(min(windows), 5), "median": round(ms_step, 5), "max": round(max(windows), 5),
                    "note": "value is the median window; the timed steps cycle over the resident batches"},
        "roofline": roofline,
        "pipeline": {"gemm_flops_per_step": flops_step, "achieved": round(flops_step / ms_step / 1e9, 3), "peak": FP32_MFMA_PEAK_TF,
                     "unit": "TFLOP/s", "frac": round(flops_step / ms_step / 1e9 / FP32_MFMA_PEAK_TF, 4),
                     "note": "all dense-layer flops of a step over the timed step itself (every kernel of the step included, batches on %d lanes)" % args.lanes + ": the fraction of the fp32 MFMA peak the whole path sustains"},
        "kernels": {n: {k: (round(v, 5) if isinstance(v, float) else v) for k, v in kv.items()} for n, kv in kernels.items()},
        "cpu_baseline": cpu,
        "clock_settle_ms": SETTLE_SECONDS * 1e3,
        "cold_clock": {"ms_per_step": round(ms_cold, 5), "value": rate(ms_cold), "unit": "samples/s",
                       "note": "the same %d steps started after 2.5 s of idling, no settling load: the clocks are still ramping up" % args.steps},
        "one_lane": {"ms_per_step": round(ms_one_lane, 5), "value": rate(ms_one_lane), "unit": "samples/s",
                     "note": "NNNetwork::SetLanes(1): one set of buffers, one stream, batches strictly one after the other"},
        "stored_output": {"ms_per_step": round(ms_stored, 5), "value": rate(ms_stored), "unit": "samples/s",
                          "note": "NNNetwork::SetDeferredOutput(false): PredictBatch stores the output layer, the top-K reads it back (the same as the default below 131,072 output units)"},
        "split_products": {"ms_per_step": round(ms_split, 5), "value": rate(ms_split), "unit": "samples/s",
                           "dtype": "f32 products as six bf16 x bf16 MFMA terms, f32 sums",
                           "note": "NNNetwork::SetSplitProducts(true), off by default: dense layers of at least two 128 x 128 tiles per compute unit run fc_gemm_split_kernel (a deferred output layer: dsx_fc_topk_split); results within the same tolerance of the oracle, as close to fp64 as the fp32 kernel's"},
        "with_input_upload": {"ms_per_step": round(ms_upload, 5), "value": rate(ms_upload), "unit": "samples/s",
                              "note": "the batch's CSR arrays handed over as host memory before every step (NNDataSet::LoadSparseData; PCIe-inclusive): uploads go to alternating sets of device arrays on the lane of the batch they belong to"},
        "request_round_trip": {"ms": round(ms_request, 5), "value": rate(ms_request), "unit": "samples/s",
                               "note": "median over requests served one at a time: upload, predict, filtered top-K, results read back"},
    }
    if interference:
        out["interference"] = interference
    return out


def knn_bench(args, pkg, lib):
    from dsx_support import synth

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
                "unit": "TFLOP/s", "frac": round(flops / el[0] / 1e9 / FP32_MFMA_PEAK_TF, 4), "traffic": (lambda t: (t["read"] + t["write"]) if t else None)(
                    measured_traffic(p.name).get("fc_gemm_kernel (knn scores)")), "avg_launch_ms": round(el[0], 4),
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
           "kernel": "knn_f16_wide_kernel (+ knn_f16_kernel for the first block)", "bound": "mfma", "achieved": round(flops / el[0] / 1e9, 3), "peak": 2500.0, "unit_roofline": "TFLOP/s",
           "frac": round(flops / el[0] / 1e9 / 2500.0, 4), "scores_ms": round(el[0], 4), "topk_ms": round(el[1], 4),
           "path": {0: "blocks", 1: "candidate lists", 2: "candidate lists, redone block by block"}[lib.dsx_knn_last_search_path()]}
    del table
    # ... and with the fp32 table's products formed from bf16 matrix instructions (dsx_knn_search_split: fp32-accurate, a mode the
    # caller asks for; reported beside the fp32 figure)
    planes = pkg.DeviceArray((lib.dsx_fc_split_bytes(rows, D) // 4,), np.uint32, lib)
    pkg.check(lib.dsx_fc_split(dI.ptr, rows, 1, rows, D, planes.ptr))

    def step_split(timing=None):
        pkg.check(lib.dsx_knn_search_split(planes.ptr, rows, pad, D, dQ.ptr, Q, K, scores.ptr, idx.ptr, None, 0, timing))
    for _ in range(max(1, args.warmup)):
        step_split()
    pkg.check(lib.dsx_sync())
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step_split()
    pkg.check(lib.dsx_sync())
    ms_split = (time.perf_counter() - t0) * 1e3 / args.steps
    step_split(el)
    split = {"ms_per_step": round(ms_split, 4), "value": round(Q / (ms_split / 1e3), 1), "unit": "queries/s",
             "dtype": "f32 products as six bf16 x bf16 MFMA terms, f32 sums", "kernel": "fc_gemm_split_kernel (candidate mode)",
             "scores_ms": round(el[0], 4), "topk_ms": round(el[1], 4),
             "path": {0: "blocks", 1: "candidate lists", 2: "candidate lists, redone block by block"}[lib.dsx_knn_last_search_path()]}
    del planes
    calibration_copy(args, pkg, lib)
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
            "config": {"workload": p.name, "queries": Q, "dim": D, "items": rows - pad, "top_k": K,
                       "vectors": "N(0, 1) components, rows L2-normalised, seed 1005"}, "roofline": roofline,
            "cpu_baseline": cpu, "f16_storage": f16, "split_products": split}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", type=int, default=2, help="1..4 = networks of the benchmark definition, 5 = KNN")
    ap.add_argument("--lanes", type=int, default=2, help="NNNetwork::SetLanes for the timed step: batches in flight (1..4, the library's default is 2)")
    ap.add_argument("--knn-items", type=int, default=2000000)
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="CPU baseline budget; 0 skips it")
    ap.add_argument("--interference", action="store_true", help="also measure what each kernel of a batch costs the output GEMM beside it")
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
