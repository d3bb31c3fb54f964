#!/usr/bin/env python3
"""Benchmark of the MI355X operator layer on BASELINE.json's metric:
"AlexNet-shape fp32 train images/s at b=256; SGEMM TFLOP/s; eltwise HBM GB/s".

One step = one forward + backward + SGD pass of the AlexNet-shaped network
(BASELINE.json configs[4]) at batch 256 on one GPU, every operator issued separately
through the C++ host layer (Task -> HipDevice -> hip::<Op> -> C ABI -> HIP kernel),
synthetic seeded inputs already resident in HBM.  `value` is images/s with one stream
synchronisation per step; the same step with the reference device's per-operator
synchronisation is reported beside it.  The dominant kernel (the MFMA matrix products of the
minimal-filtering convolution passes) is timed with HIP events on its own stream inside the
timed steps and priced against the fp32 MFMA peak.  SGEMM 4096^3 and the 8192^2 elementwise add
are measured the same way and reported in the same JSON line, and the CPU oracle is
timed on a bounded sample of the same workload on the host cores.

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W]
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0
BATCH = 256

# 2*N*Ho*Wo*K*C*R*S per convolution pass at batch 256, in GFLOP (conv1..conv5)
CONV_GFLOP = [53.97, 229.32, 76.55, 114.83, 76.55]
STEP_GFLOP = 1689.8  # convolutions (fwd, bwd-filter, bwd-data except conv1) + three FC layers
# What the matrix pipe executes: the three passes of conv2..conv5 run by minimal filtering.
# conv2 (5 x 5): 64 multiplies per 4 x 4 outputs of a channel pair on 7 x 7 tiles per 27 x 27
# plane; conv3..5 (3 x 3): 49 per 5 x 5 outputs on 3 x 3 tiles per 13 x 13 plane; the filter
# gradients the same counts with the tiles of top_diff in the filter's place.
WINOGRAD_GFLOP = [2 * 64 * 256 * 96 * 256 * 49 / 1e9] + \
                 [2 * 49 * k * c * 256 * 9 / 1e9 for (c, k) in ((256, 384), (384, 384), (384, 256))]
STEP_EXECUTED_GFLOP = round(STEP_GFLOP - 3 * sum(CONV_GFLOP[1:]) + 3 * sum(WINOGRAD_GFLOP), 1)


def capi_check(rc):
    from minerva_amd import capi
    capi.check(rc, "benchmark set-up call")


def log(*a):
    print(*a, file=sys.stderr)
    sys.stderr.flush()


def graph_replay(rt, net, steps, warmup):
    """The same step recorded once into a HIP graph and replayed, one sync per replay.  The
    replay runs the same kernels on the same buffers plus one copy kernel per parameter
    (new weights back over the old ones); reported beside the operator-by-operator figure,
    never as `value`."""
    nodes = net.capture_step(0.01)
    net.replay(warmup)
    t0 = time.perf_counter()
    net.replay(steps, sync_each_step=True)
    ms = (time.perf_counter() - t0) * 1e3 / steps
    net.release_graph()
    return {"nodes": nodes, "ms_per_step": round(ms, 4), "images_per_s": round(BATCH / ms * 1e3, 1)}


# The kernel with the largest share of the step is the matrix product of the minimal-filtering
# passes (mnv_gemm_kernel<128x128x16, WinoGemm>: forward and data gradient of conv2..conv5, eight
# launches per step); the filter gradients' products (WinoGradGemm, a stream-k launch each) come
# second.  The library brackets every such launch with an event pair on its stream while
# mnv_conv_winograd_profile is on, which is how the timed steps measure them apart from the
# transform kernels of the same operator.


def alexnet_bench(steps, warmup, dataflow=True):
    from minerva_amd import capi
    from minerva_amd import hostapi
    from minerva_amd import configs
    params, data, label = configs.make_inputs("alexnet", BATCH)
    out = {}
    # "fused": the same step with the opt-in fused operators (bit-identical results, fewer
    # launches): reported beside `value`, which stays the operator-by-operator step
    # "fused_updates": the fused step with the weight updates applied in the stores of the
    # kernels that produce the weight gradients (same parameters, no gradient tensors)
    modes = [("per_step_sync", False), ("per_op_sync", True), ("fused", False), ("fused_updates", False)]
    if dataflow:  # kernels of different streams overlap: a kernel trace that wants undisturbed
        modes.append(("dataflow", False))  # durations runs with --no-dataflow
    for mode, sync_each in modes:
        rt = hostapi.Runtime(0, sync_each_op=sync_each, dataflow=(mode == "dataflow"))
        net = hostapi.Net(rt, "alexnet", BATCH)
        if mode in ("fused", "fused_updates"):
            net.set_fused(updates=(mode == "fused_updates"))
        for k, v in params.items():
            net.set_param(k, v)
        t_h2d = time.perf_counter()
        net.load_batch(data, label)  # ArrayLoader: pageable host memory -> HBM, synchronous
        t_h2d = (time.perf_counter() - t_h2d) * 1e3
        for _ in range(warmup):
            net.step(0.01)
        rt.sync()
        ops0 = rt.ops_issued()
        # Inside the timed steps only the launches of the dominant kernels carry event pairs
        # (twelve per step, on their own stream): timing all ~100 operators costs ~5% of the
        # step in idle gaps.
        plain = mode == "per_step_sync"
        if plain:
            capi.lib().mnv_conv_winograd_profile(1)
        rt.sync()
        per_step = []
        t0 = time.perf_counter()
        for _ in range(steps):
            ts = time.perf_counter()
            net.step(0.01)
            rt.sync()
            per_step.append((time.perf_counter() - ts) * 1e3)
        t1 = time.perf_counter()
        prof = product_profile() if plain else {}
        prob = net.read("prob", 1000 * BATCH)
        ms = (t1 - t0) * 1e3 / steps
        ops_per_step = (rt.ops_issued() - ops0) // steps
        all_ops = {}
        if plain:  # the per-operator table comes from extra, untimed steps
            rt.profile(True)
            for _ in range(steps):
                net.step(0.01)
                rt.sync()
            all_ops = rt.profile_read()
            rt.profile(False)
        fed = None
        if plain:
            # The same step with a NEW batch from pageable host memory every step, loaded on a
            # second stream while the step before it runs (the reference's published figure
            # includes feeding the batch): step N is queued, the host then feeds batch N+1
            # through pinned staging, and the step's sync closes the iteration.
            feed = [(np.roll(data, i + 1), np.roll(label, 1000 * (i + 1))) for i in range(2)]
            for i in range(warmup):
                net.step(0.01)
                net.prefetch_batch(*feed[i % 2])
                rt.sync()
            t0f = time.perf_counter()
            for i in range(steps):
                net.step(0.01)
                net.prefetch_batch(*feed[i % 2])
                rt.sync()
            fed = (time.perf_counter() - t0f) * 1e3 / steps
            log("alexnet b=%d with the next batch fed under every step: %.3f ms/step" % (BATCH, fed))
        graph = None
        if plain or mode == "fused":
            graph = graph_replay(rt, net, steps, warmup)
            log("alexnet b=%d %s recorded step: %d nodes, %.3f ms/replay" %
                (BATCH, mode, graph["nodes"], graph["ms_per_step"]))
        out[mode] = {"graph_replay": graph, "ms_per_step": ms, "images_per_s": BATCH / (ms / 1e3),
                     "median_ms_per_step": float(np.median(per_step)),
                     "ops_per_step": ops_per_step,
                     "finite": bool(np.isfinite(prob).all()), "profile": prof, "all_ops": all_ops,
                     "h2d_batch_ms": t_h2d, "fed_ms_per_step": fed}
        log("alexnet b=%d %s: %.3f ms/step, %.1f img/s, %d ops/step" %
            (BATCH, mode, ms, out[mode]["images_per_s"], out[mode]["ops_per_step"]))
        net.close()
        rt.close()
    return out


def owl_front_end_bench(steps, warmup):
    """The same step issued operator by operator from Python through the NArray front end
    (minerva_amd.owl, the interface of the reference's owl binding): what a Python
    application sees.  Reported beside `value`, not as it."""
    from minerva_amd import configs, owl
    from minerva_amd.owl import models
    params, data, label = configs.make_inputs("alexnet", BATCH)
    owl.set_device(owl.create_gpu_device(0))
    net = models.AlexNet()
    net.load([params["w%d" % k] for k in range(8)], [params["b%d" % k] for k in range(8)])
    x = owl.from_numpy(np.asarray(data, np.float32).reshape(BATCH, 3, 227, 227))
    y = owl.from_numpy(np.asarray(label, np.float32).reshape(BATCH, 1000))
    rt = owl._runtime()

    def step():
        out, wgrad, bgrad = net.train_one_mb(x, y)
        net.sgd(wgrad, bgrad, BATCH, 0.01)
        owl.wait_for_all()
        return out

    for _ in range(warmup):
        step()
    ops0 = rt.ops_issued()
    t0 = time.perf_counter()
    for _ in range(steps):
        out = step()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    ops = (rt.ops_issued() - ops0) // steps
    finite = bool(np.isfinite(out.to_numpy()).all())
    del out, net, x, y
    owl.close_devices()
    log("alexnet b=%d through the owl front end: %.3f ms/step, %d ops/step" % (BATCH, ms, ops))
    return {"ms_per_step": round(ms, 3), "images_per_s": round(BATCH / (ms / 1e3), 1),
            "ops_per_step": int(ops), "finite": finite}


def owl_net_bench(steps, warmup):
    """Caffe's reference AlexNet (norm1 / norm2 LRN, drop6 / drop7, momentum 0.9, weight decay
    5e-4; every convolution in one group) trained through owl.net, the reference's Caffe-like
    layer package, at batch 256 on one synthetic batch resident in HBM.  This is the network
    behind the one number the reference publishes (189.63 images/s on a GTX Titan with
    cuDNN): context only, it is neither the metric's configuration nor `value`."""
    from minerva_amd import owl
    from minerva_amd.owl import net as onet
    from minerva_amd.owl.net import models
    owl.set_device(owl.create_gpu_device(0))
    tr = onet.NetTrainer(models.ALEXNET_SOLVER, models.alexnet_prototxt(BATCH), seed=1)
    rng = np.random.default_rng(2)
    tr.owl_net.get_data_unit().set_batch(rng.standard_normal(BATCH * 3 * 227 * 227, dtype=np.float32),
                                         rng.integers(0, 1000, BATCH))
    rt = owl._runtime()
    tr.run(warmup)
    ops0 = rt.ops_issued()
    t0 = time.perf_counter()
    tr.run(steps)
    ms = (time.perf_counter() - t0) * 1e3 / steps
    ops = (rt.ops_issued() - ops0) // steps
    loss = tr.owl_net.get_loss_units()[0].getloss()
    del tr
    owl.close_devices()
    log("caffe-style alexnet b=%d through owl.net: %.3f ms/step, %d ops/step" % (BATCH, ms, ops))
    return {"network": "Caffe reference AlexNet, single group, LRN + dropout, momentum SGD",
            "ms_per_step": round(ms, 3), "images_per_s": round(BATCH / (ms / 1e3), 1),
            "ops_per_step": int(ops), "loss_finite": bool(np.isfinite(loss)),
            "reference_published_images_per_s": 189.63,
            "reference_published_on": "GTX Titan, cuDNN, full Caffe AlexNet (README.md:76-82)"}


TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "bench_gemm_kernels_hbm_traffic_pmc.txt")


def dominant_kernel_traffic(tag):
    """HBM-side bytes per launch of a kernel, from two rocprofv3 --pmc runs of this script
    (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch, each scaled by what the same counter reads
    for the 8192^2 add kernel).  The figure is the one recorded in the committed summary of
    those runs (its line "traffic bytes per launch, <tag>: X"), so that the two cannot drift
    apart; None when the summary is absent."""
    try:
        for line in open(TRAFFIC_PROFILE):
            if "traffic bytes per launch, %s:" % tag in line:
                return float(line.split(":")[1].split()[0])
    except (OSError, ValueError, IndexError):
        pass
    return None


def product_profile():
    """{kind: (launches, device ms, GFLOP)} of the minimal-filtering products since the profile
    was switched on; switches it off."""
    from minerva_amd import capi
    L = capi.lib()
    out = {}
    for kind in (0, 1):
        n, ms, gf = ctypes.c_int(), ctypes.c_double(), ctypes.c_double()
        capi.check(L.mnv_conv_winograd_profile_read(kind, ctypes.byref(n), ctypes.byref(ms), ctypes.byref(gf)),
                   "mnv_conv_winograd_profile_read")
        out[kind] = (n.value, ms.value, gf.value)
    L.mnv_conv_winograd_profile(0)
    return out


PRODUCT_KERNELS = {
    0: ("minimal-filtering products", "mnv_gemm_kernel<128x128x16,WinoGemm> (the 16 / 36 / 64 matrix products of "
        "the forward and data-gradient passes of conv2..conv5, one launch per pass)"),
    1: ("minimal-filtering filter-gradient products", "mnv_gemm_kernel<128x128x16,WinoGradGemm,stream-k> (the "
        "products of the filter gradients of conv2..conv5, one launch per pass) + the reduction of its shares"),
}


def dominant_kernel_roofline(prof, steps):
    """The products' flops are those of the transformed problem (2 x points x channels x channels
    x tiles), i.e. what the kernel itself multiplies, not the direct sum's."""
    rows = []
    for kind, (launches, ms, gflop) in prof.items():
        if not launches:
            continue
        tag, kernel = PRODUCT_KERNELS[kind]
        achieved = gflop / ms
        rows.append({"bound": "mfma", "kernel": kernel, "achieved": round(achieved, 2),
                     "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_FP32_MFMA_TFLOPS, 4),
                     "traffic": dominant_kernel_traffic(tag),
                     "avg_launch_ms": round(ms / launches, 4), "launches": launches,
                     "ms_per_step": round(ms / steps, 4),
                     "algorithmic_gflop_per_launch": round(gflop / launches, 2)})
    if not rows:
        return None
    rows.sort(key=lambda r: -r["ms_per_step"])
    top = rows[0]
    top["other_kernels"] = rows[1:]
    return top


def op_table(prof, steps):
    rows = sorted(prof.items(), key=lambda kv: -kv[1][1])
    return [{"op": n, "launches_per_step": c // steps, "ms_per_step": round(ms / steps, 4)}
            for n, (c, ms) in rows]


def sgemm_bench():
    """SGEMM at the four shapes of BASELINE.json configs[2] (N(0,1) inputs), events on the
    stream, median of five batches of ten calls; every call's status is checked."""
    from minerva_amd import capi
    L = capi.lib()
    dev = capi.Device(0)
    rng = np.random.default_rng(7)
    m = n = k = 4096
    a = dev.upload(rng.standard_normal(m * k, dtype=np.float32))
    b = dev.upload(rng.standard_normal(k * n, dtype=np.float32))
    c = dev.empty(m * n)
    ms = dev.time_ms(lambda: L.mnv_sgemm_nn(a.p, b.p, c.p, m, n, k, None, 0, dev.stream),
                     iters=10, warmup=5, reps=5)
    tf = 2.0 * m * n * k / (ms * 1e-3) / 1e12
    sgemm = {"shape": "4096x4096x4096", "ms": round(ms, 4), "tflops": round(tf, 2),
             "roofline": {"bound": "mfma", "achieved": round(tf, 2), "peak": PEAK_FP32_MFMA_TFLOPS,
                          "unit": "TFLOP/s", "frac": round(tf / PEAK_FP32_MFMA_TFLOPS, 4)}}
    log("sgemm 4096^3: %.3f ms, %.1f TFLOP/s" % (ms, tf))
    # the same product back to back for more than a second: the clock the chip sustains under
    # this load, beside the burst figure above (50 calls spread over five batches)
    calls = 1200
    t_sus = dev.time_ms(lambda: L.mnv_sgemm_nn(a.p, b.p, c.p, m, n, k, None, 0, dev.stream),
                        iters=calls, warmup=20, reps=1)
    tf_sus = 2.0 * m * n * k / (t_sus * 1e-3) / 1e12
    sgemm["sustained"] = {"calls_back_to_back": calls, "seconds": round(calls * t_sus * 1e-3, 2),
                          "ms": round(t_sus, 4), "tflops": round(tf_sus, 2),
                          "frac": round(tf_sus / PEAK_FP32_MFMA_TFLOPS, 4)}
    log("sgemm 4096^3 sustained over %d calls: %.3f ms, %.1f TFLOP/s" % (calls, t_sus, tf_sus))
    # the same product with one operand given transposed (the operand is read in place: what
    # the reference writes as Trans + MatMult); the values differ, the timing does not care
    t_tn = dev.time_ms(lambda: L.mnv_sgemm_tn(a.p, b.p, None, c.p, m, n, k, None, 0, dev.stream),
                       iters=10, warmup=5, reps=5)
    t_nt = dev.time_ms(lambda: L.mnv_sgemm_nt(a.p, b.p, c.p, m, n, k, None, 0, dev.stream),
                       iters=10, warmup=5, reps=5)
    sgemm["transposed_operands"] = {
        "A^T*B": {"ms": round(t_tn, 4), "tflops": round(2.0 * m * n * k / (t_tn * 1e-3) / 1e12, 2)},
        "A*B^T": {"ms": round(t_nt, 4), "tflops": round(2.0 * m * n * k / (t_nt * 1e-3) / 1e12, 2)}}
    log("sgemm 4096^3 with A / B transposed: %.3f / %.3f ms" % (t_tn, t_nt))
    # the other shapes of BASELINE.json configs[2], with the split-k workspace the host layer lends
    shapes = []
    for (mm, kk, nn) in ((256, 9216, 4096), (4096, 4096, 256), (1000, 4096, 256)):
        aa = dev.upload(rng.standard_normal(mm * kk, dtype=np.float32))
        bb = dev.upload(rng.standard_normal(kk * nn, dtype=np.float32))
        cc = dev.empty(mm * nn)
        wsb = L.mnv_sgemm_nn_workspace_bytes(mm, nn, kk)
        ws = dev.empty(wsb // 4 + 1)
        t = dev.time_ms(lambda: L.mnv_sgemm_nn(aa.p, bb.p, cc.p, mm, nn, kk, ws.p,
                                               ctypes.c_size_t(wsb), dev.stream),
                        iters=10, warmup=5, reps=5)
        tfl = 2.0 * mm * nn * kk / (t * 1e-3) / 1e12
        shapes.append({"MxKxN": "%dx%dx%d" % (mm, kk, nn), "ms": round(t, 4), "tflops": round(tfl, 2),
                       "frac": round(tfl / PEAK_FP32_MFMA_TFLOPS, 4)})
        log("sgemm %dx%dx%d: %.4f ms, %.1f TFLOP/s" % (mm, kk, nn, t, tfl))
    sgemm["other_shapes"] = shapes
    return sgemm


def eltwise_bench():
    from minerva_amd import capi
    dev = capi.Device(0)
    elt = bandwidth_table(capi.lib(), dev, np.random.default_rng(7), 8192 * 8192)
    log("add 8192^2: %.4f ms, %.0f GB/s" % (elt["ms"], elt["gbs"]))
    return elt


ROTATE = 4  # buffer sets an HBM-bound operator cycles through, so that no pass finds its
            # operands in the 256 MB last-level cache left there by the previous pass


def rotating(dev, make_call, sets):
    """ms per call of an operator that takes the next of `sets` on every call: the median of
    five batches, each two rounds through the sets."""
    import itertools
    count = itertools.count()
    calls = [make_call(*s) for s in sets]
    return dev.time_ms(lambda: calls[next(count) % len(calls)](), iters=2 * len(calls),
                       warmup=2 * len(calls), reps=5)


def bandwidth_table(L, dev, rng, ne):
    """The 8192^2 bandwidth microbenchmark (BASELINE.json configs[1]): GB/s from the
    algorithmic bytes per element of each operator, every operator cycling through ROTATE
    sets of operands (with one set, 30-40% of a 268 MB operand is still in the last-level
    cache when the next pass starts, and the same kernels read 87-92% of peak instead of
    75-80%: reported as `gbs_one_set`)."""
    m = n = 8192
    S = dev.stream
    host_x = rng.standard_normal(ne, dtype=np.float32)
    host_y = rng.standard_normal(ne, dtype=np.float32)
    sets = [(dev.upload(host_x), dev.upload(host_y), dev.empty(ne)) for _ in range(ROTATE)]
    vec = dev.upload(np.random.default_rng(8).standard_normal(m, dtype=np.float32))
    small = dev.empty(m)
    f = ctypes.c_float
    ops = [
        ("add", 12, lambda x, y, z: lambda: L.mnv_add(x.p, y.p, z.p, ne, S)),
        ("copy", 8, lambda x, y, z: lambda: L.mnv_copy(x.p, z.p, ne, S)),
        ("mul", 12, lambda x, y, z: lambda: L.mnv_mul(x.p, y.p, z.p, ne, S)),
        ("sub", 12, lambda x, y, z: lambda: L.mnv_sub(x.p, y.p, z.p, ne, S)),
        ("scalar mul", 8, lambda x, y, z: lambda: L.mnv_const_mul(x.p, z.p, f(3.291), ne, S)),
        ("broadcast add {1,n}", 8, lambda x, y, z: lambda: L.mnv_norm_add_col(x.p, vec.p, z.p, m, n, S)),
        ("broadcast add {m,1}", 8, lambda x, y, z: lambda: L.mnv_norm_add_row(x.p, vec.p, z.p, m, n, S)),
        ("sigmoid fwd", 8, lambda x, y, z: lambda: L.mnv_sigmoid_fwd(x.p, z.p, ne, S)),
        ("relu fwd", 8, lambda x, y, z: lambda: L.mnv_relu_fwd(x.p, z.p, ne, S)),
        ("tanh fwd", 8, lambda x, y, z: lambda: L.mnv_tanh_fwd(x.p, z.p, ne, S)),
        ("sigmoid bwd", 12, lambda x, y, z: lambda: L.mnv_sigmoid_bwd(x.p, x.p, y.p, z.p, ne, S)),
        ("relu bwd", 12, lambda x, y, z: lambda: L.mnv_relu_bwd(x.p, x.p, y.p, z.p, ne, S)),
        ("tanh bwd", 12, lambda x, y, z: lambda: L.mnv_tanh_bwd(x.p, x.p, y.p, z.p, ne, S)),
        ("sum dim 0", 4, lambda x, y, z: lambda: L.mnv_reduce_sum_col(x.p, small.p, m, n, S)),
        ("sum dim 1", 4, lambda x, y, z: lambda: L.mnv_reduce_sum_row(x.p, small.p, m, n, S)),
        ("max dim 0", 4, lambda x, y, z: lambda: L.mnv_reduce_max_col(x.p, small.p, m, n, S)),
        ("max dim 1", 4, lambda x, y, z: lambda: L.mnv_reduce_max_row(x.p, small.p, m, n, S)),
        ("maxindex dim 0", 4, lambda x, y, z: lambda: L.mnv_maxindex_col(x.p, small.p, m, n, S)),
        ("maxindex dim 1", 4, lambda x, y, z: lambda: L.mnv_maxindex_row(x.p, small.p, m, n, S)),
        ("softmax rows", 8, lambda x, y, z: lambda: L.mnv_softmax_instance_fwd(x.p, z.p, n, m, 1, 1, S)),
        ("softmax rows bwd", 12, lambda x, y, z: lambda: L.mnv_softmax_instance_bwd(x.p, y.p, z.p, n, m, 1, 1, S)),
        # channel mode (cuda_perform.cu:355-369): 1024 channels over 256 x 256 positions
        ("softmax over channels", 8, lambda x, y, z: lambda: L.mnv_softmax_channel_fwd(x.p, z.p, 1, 1024, 256, 256, S)),
        ("softmax over channels bwd", 12, lambda x, y, z: lambda: L.mnv_softmax_channel_bwd(x.p, y.p, z.p, 1, 1024, 256, 256, S)),
        ("transpose", 8, lambda x, y, z: lambda: L.mnv_transpose(x.p, z.p, m, n, S)),
    ]
    table = []
    for name, bpe, make in ops:
        ms = rotating(dev, make, sets)
        ms_one = dev.time_ms(make(*sets[0]), iters=6, warmup=3, reps=3)
        gbs = bpe * ne / (ms * 1e-3) / 1e9
        table.append({"op": name, "ms": round(ms, 4), "gbs": round(gbs, 1),
                      "frac": round(gbs / PEAK_HBM_GBS, 4),
                      "gbs_one_set": round(bpe * ne / (ms_one * 1e-3) / 1e9, 1)})
    # a ragged transpose in the same operands (8000 x 8200 floats fit an 8192^2 buffer): rows of
    # the result off the 64-byte grid, partial tiles on both edges
    rm, rn = 8000, 8200
    ms = rotating(dev, lambda x, y, z: lambda: L.mnv_transpose(x.p, z.p, rm, rn, S), sets)
    gbs = 8 * rm * rn / (ms * 1e-3) / 1e9
    table.append({"op": "transpose 8000x8200", "ms": round(ms, 4), "gbs": round(gbs, 1),
                  "frac": round(gbs / PEAK_HBM_GBS, 4)})
    add = table[0]
    elt = {"op": "add 8192x8192", "ms": add["ms"], "gbs": add["gbs"],
           "roofline": {"bound": "hbm", "achieved": add["gbs"], "peak": PEAK_HBM_GBS,
                        "unit": "GB/s", "frac": add["frac"]},
           "buffer_sets": ROTATE}
    del sets
    # AlexNet pool1 at batch 256 ({55,55,96,256} -> {27,27,96,256}, 3x3 stride 2), the conv1
    # bias gradient and LRN over the same tensor (Caffe-style norm1: local_size 5, alpha 1e-4,
    # beta 0.75), two sets of 297 MB tensors each: bytes = every tensor once
    geo = (256, 96, 55, 55, 2, 2, 3, 3, 0, 0)
    lrn = (5, f(1e-4), f(0.75), 256, 96, 55, 55)
    nin, nout = 256 * 96 * 55 * 55, 256 * 96 * 27 * 27
    host_p = np.random.default_rng(9).standard_normal(nin, dtype=np.float32)
    big = []
    for _ in range(2):
        px, py, pdy = dev.upload(host_p), dev.empty(nout), dev.empty(nout)
        o1, o2, o3, o4 = dev.empty(nin), dev.empty(nin), dev.empty(nin), dev.empty(nin)
        capi_check(L.mnv_fill(o4.p, nin, f(0.25), S))  # a top_diff of its own for the LRN gradient
        capi_check(L.mnv_fill(pdy.p, nout, f(0.5), S))
        capi_check(L.mnv_maxpool_fwd(px.p, py.p, *geo, S))
        capi_check(L.mnv_lrn_fwd(px.p, o1.p, o2.p, *lrn, S))  # o1 = scale, o2 = top (backward row)
        assert px.n == nin and o1.n == nin and py.n == nout and pdy.n == nout
        big.append((px, py, pdy, o1, o2, o3, o4))
    bias_ws = dev.empty(1 << 18)  # 1 MiB
    extra = [
        ("maxpool 3x3/2 fwd (pool1)", 4 * (nin + nout),
         lambda px, py, pdy, o1, o2, o3, o4: lambda: L.mnv_maxpool_fwd(px.p, py.p, *geo, S)),
        ("maxpool 3x3/2 bwd (pool1)", 4 * (2 * nin + nout),
         lambda px, py, pdy, o1, o2, o3, o4: lambda: L.mnv_maxpool_bwd(px.p, py.p, pdy.p, o3.p, *geo, S)),
        ("avgpool 3x3/2 fwd (pool1 shape)", 4 * (nin + nout),
         lambda px, py, pdy, o1, o2, o3, o4: lambda: L.mnv_avgpool_fwd(px.p, py.p, *geo, S)),
        ("avgpool 3x3/2 bwd (pool1 shape)", 4 * (nin + nout),
         lambda px, py, pdy, o1, o2, o3, o4: lambda: L.mnv_avgpool_bwd(px.p, py.p, pdy.p, o3.p, *geo, S)),
        ("conv bias gradient (conv1)", 4 * nin,
         lambda px, py, pdy, o1, o2, o3, o4: lambda: L.mnv_conv_bwd_bias(
             px.p, small.p, 256, 96, 55, 55, bias_ws.p, ctypes.c_size_t(1 << 20), S)),
        ("copy, 297 MB tensors", 8 * nin,
         lambda px, py, pdy, o1, o2, o3, o4: lambda: L.mnv_copy(px.p, o3.p, nin, S)),
        ("lrn bwd (norm1)", 20 * nin,
         lambda px, py, pdy, o1, o2, o3, o4: lambda: L.mnv_lrn_bwd(px.p, o2.p, o1.p, o4.p, o3.p, *lrn, S)),
        ("lrn fwd (norm1)", 12 * nin,
         lambda px, py, pdy, o1, o2, o3, o4: lambda: L.mnv_lrn_fwd(px.p, o1.p, o2.p, *lrn, S)),
    ]
    for name, nbytes, make in extra:
        ms = rotating(dev, make, big)
        gbs = nbytes / (ms * 1e-3) / 1e9
        table.append({"op": name, "ms": round(ms, 4), "gbs": round(gbs, 1),
                      "frac": round(gbs / PEAK_HBM_GBS, 4)})
    elt["ops"] = table
    return elt


def small_nets(steps=20, warmup=3):
    """BASELINE.json configs[0] (MLP) and configs[3] (CNN) at batch 256: latency-bound
    graphs, reported as ms/step and operators/step without a roofline claim.  Beside the
    one-stream order: the same step in dataflow mode (four streams ordered by events), with
    the fused operators, and recorded into a HIP graph."""
    from minerva_amd import hostapi
    from minerva_amd import configs
    out = {}
    for name in ("mlp", "cnn"):
        params, data, label = configs.make_inputs(name, BATCH)
        row = {}
        for mode in ("stream_order", "dataflow", "fused", "fused_updates"):
            rt = hostapi.Runtime(0, sync_each_op=False, dataflow=(mode == "dataflow"))
            net = hostapi.Net(rt, name, BATCH)
            if mode in ("fused", "fused_updates"):
                net.set_fused(updates=(mode == "fused_updates"))
            for k, v in params.items():
                net.set_param(k, v)
            net.load_batch(data, label)
            for _ in range(warmup):
                net.step(0.01)
            rt.sync()
            ops0 = rt.ops_issued()
            ts = []
            for _ in range(steps):
                t0 = time.perf_counter()
                net.step(0.01)
                rt.sync()
                ts.append((time.perf_counter() - t0) * 1e3)
            ms = float(np.median(ts))
            if mode == "stream_order":
                row = {"ms_per_step": round(ms, 4), "images_per_s": round(BATCH / ms * 1e3, 1),
                       "ops_per_step": (rt.ops_issued() - ops0) // steps}
                row["graph_replay"] = g = graph_replay(rt, net, steps, warmup)
            else:
                row[mode + "_ms_per_step"] = round(ms, 4)
            net.close()
            rt.close()
        out[name + "_b256"] = row
        log("%s b=%d: %.3f ms/step (dataflow %.3f, fused %.3f, with fused updates %.3f), recorded step "
            "%.3f ms/replay (%d nodes)" %
            (name, BATCH, row["ms_per_step"], row["dataflow_ms_per_step"], row["fused_ms_per_step"],
             row["fused_updates_ms_per_step"], g["ms_per_step"], g["nodes"]))
    return out


def host_cpu():
    model = "unknown"
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    try:
        usable = len(os.sched_getaffinity(0))
    except AttributeError:
        usable = os.cpu_count()
    return {"model": model, "nproc": os.cpu_count(), "usable": usable}


def _median_time(fn, reps=3):
    ts = []
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    return float(np.median(ts))


def cpu_baseline(batch=4, full=False):
    """The CPU oracle (the repository's restatement of Minerva's single-threaded basic
    implementation; `kind` "port") on the host cores, one core per operator as the reference's
    CpuDevice runs them:
      value         one AlexNet-shaped train step at batch 4 of 256 (convolution and pooling
                    have no reference CPU implementation: the oracle's naive loops);
      config2       every operator of the 8192^2 bandwidth table at full size, median of 3;
      sgemm         the reference's i,j,k loop order (basic.cpp:164-171): 1000x4096x256 and
                    1024^3 at full size; for 4096x4096x256 and 256x9216x4096 a quarter / an
                    eighth of the output columns (columns are independent and cost the same:
                    full size = sample x 4 / x 8; --cpu-full runs them whole); 4096^3 is
                    extrapolated from the 1024^3 rate; the four products run at the same time
                    on four cores;
      mlp / cnn     one train step at batch 256, median of 3."""
    import concurrent.futures as cf
    from oracle import nets
    from oracle import mnv_oracle as ora
    params, data, label = nets.make_inputs("alexnet", batch)
    t0 = time.perf_counter()
    nets.alexnet_step(params, data, label, 0.01, batch)
    dt = time.perf_counter() - t0
    log("cpu oracle alexnet b=%d: %.2f s" % (batch, dt))
    out = {"value": round(batch / dt, 4), "unit": "images/s", "cores": 1, "kind": "port",
           "sample": "one AlexNet-shaped train step at batch %d (of 256) with the naive "
                     "single-threaded CPU oracle, %.1f s" % (batch, dt),
           "host": host_cpu()}
    del params, data, label
    rng = np.random.default_rng(11)
    m = n = 8192
    ne = m * n
    x, y = rng.standard_normal(ne, dtype=np.float32), rng.standard_normal(ne, dtype=np.float32)
    row, col = rng.standard_normal(n, dtype=np.float32), rng.standard_normal(m, dtype=np.float32)
    relu = ora.activation_fwd(ora.RELU, x)
    sm = ora.softmax_instance_fwd(x, n, m, 1, 1)
    ops = [
        ("add", 12, lambda: ora.arithmetic(ora.ADD, x, y)),
        ("mul", 12, lambda: ora.arithmetic(ora.MUL, x, y)),
        ("sub", 12, lambda: ora.arithmetic(ora.SUB, x, y)),
        ("scalar mul", 8, lambda: ora.arithmetic_const(ora.MUL, 1, 3.291, x)),
        ("broadcast add {1,n}", 8, lambda: ora.norm_arithmetic(ora.ADD, x, [m, n], row, [0])),
        ("broadcast add {m,1}", 8, lambda: ora.norm_arithmetic(ora.ADD, x, [m, n], col, [1])),
        ("sigmoid fwd", 8, lambda: ora.activation_fwd(ora.SIGMOID, x)),
        ("relu fwd", 8, lambda: ora.activation_fwd(ora.RELU, x)),
        ("tanh fwd", 8, lambda: ora.activation_fwd(ora.TANH, x)),
        ("sigmoid bwd", 12, lambda: ora.activation_bwd(ora.SIGMOID, y, sm, x)),
        ("relu bwd", 12, lambda: ora.activation_bwd(ora.RELU, y, relu, x)),
        ("tanh bwd", 12, lambda: ora.activation_bwd(ora.TANH, y, sm, x)),
        ("sum dim 0", 4, lambda: ora.reduction(ora.SUM, x, [m, n], [0])),
        ("sum dim 1", 4, lambda: ora.reduction(ora.SUM, x, [m, n], [1])),
        ("max dim 0", 4, lambda: ora.reduction(ora.MAX, x, [m, n], [0])),
        ("max dim 1", 4, lambda: ora.reduction(ora.MAX, x, [m, n], [1])),
        ("maxindex dim 0", 4, lambda: ora.maxindex(x, [m, n], 0)),
        ("softmax rows", 8, lambda: ora.softmax_instance_fwd(x, n, m, 1, 1)),
        ("softmax rows bwd", 12, lambda: ora.softmax_instance_bwd(y, sm, n, m, 1, 1)),
        ("transpose", 8, lambda: ora.transpose(x, m, n)),
    ]
    table = []
    t_cfg2 = time.perf_counter()
    for name, bpe, fn in ops:
        t = _median_time(fn, 3)
        table.append({"op": name, "s": round(t, 4), "gbs": round(bpe * ne / t / 1e9, 2)})
    log("cpu oracle config-2 table: %.1f s" % (time.perf_counter() - t_cfg2))
    out["config2_8192x8192"] = {"reps": 3, "statistic": "median", "cores": 1,
                                "note": "output allocation included, as in the reference's "
                                        "CPU device (malloc per operator output)",
                                "ops": table}
    del x, y, relu, sm

    # SGEMM in the reference's loop order; (m, k, n, columns computed)
    jobs = [(1000, 4096, 256, 256), (1024, 1024, 1024, 1024),
            (4096, 4096, 256, 256 if full else 64), (256, 9216, 4096, 4096 if full else 512)]

    def gemm(job):
        mm, kk, nn, cols = job
        r = np.random.default_rng(mm + kk)
        a = r.standard_normal(mm * kk, dtype=np.float32)
        b = r.standard_normal(kk * cols, dtype=np.float32)
        t0 = time.perf_counter()
        ora.matmult(a, b, mm, cols, kk)
        t = time.perf_counter() - t0
        return {"MxKxN": "%dx%dx%d" % (mm, kk, nn), "columns_timed": cols,
                "s_timed": round(t, 3), "s_full_size": round(t * nn / cols, 3),
                "gflops": round(2.0 * mm * kk * cols / t / 1e9, 4)}

    t_g = time.perf_counter()
    with cf.ThreadPoolExecutor(len(jobs)) as pool:  # the C loops run outside the GIL
        gemms = list(pool.map(gemm, jobs))
    log("cpu oracle sgemm shapes: %.1f s" % (time.perf_counter() - t_g))
    rate = gemms[1]["gflops"]
    out["sgemm"] = {"loop_order": "i, j outer, k inner (minerva/op/impl/basic.cpp:164-171), -O2, no BLAS",
                    "cores": "1 per product, the 4 products at the same time",
                    "shapes": gemms,
                    "4096x4096x4096": {"extrapolated_from": "1024^3", "gflops": rate,
                                       "s_full_size": round(2.0 * 4096 ** 3 / (rate * 1e9), 1)}}
    steps = {}
    for kind, fn in (("mlp", nets.mlp_step), ("cnn", nets.cnn_step)):
        pm, dm, lm = nets.make_inputs(kind, BATCH)
        t = _median_time(lambda: fn(dict(pm), dm, lm, 0.01, BATCH), 3)
        steps[kind + "_b256"] = {"s_per_step": round(t, 4), "images_per_s": round(BATCH / t, 1)}
    out["small_nets"] = steps
    return out


def parity_report():
    """Part of the CPU leg: every operator family once on the GPU (through the C ABI) and once
    through the CPU oracle on the same seeded inputs at a reduced size; "bit_exact" where the
    operator is one IEEE operation or a selection per element, else the normwise error
    max|gpu - cpu| / max|cpu| against the 1e-4 bound.  The tests hold the same comparisons at
    more sizes; this puts the figures of THIS run into the line."""
    from minerva_amd import capi
    from oracle import mnv_oracle as ora
    L = capi.lib()
    dev = capi.Device(0)
    S = dev.stream
    rng = np.random.default_rng(21)
    f = ctypes.c_float
    m, n = 1024, 768
    x, y = rng.standard_normal(m * n, dtype=np.float32), rng.standard_normal(m * n, dtype=np.float32)
    dx, dy = dev.upload(x), dev.upload(y)
    out = []

    def run(fn, count):
        o = dev.empty(count)
        capi.check(fn(o), "parity call")
        dev.sync()
        return dev.download(o)

    def exact(name, got, want):
        same = bool(np.array_equal(np.asarray(got, np.float32).view(np.uint32),
                                   np.asarray(want, np.float32).view(np.uint32)))
        out.append({"op": name, "bit_exact": same})

    def close(name, got, want):
        want = np.asarray(want, np.float64)
        err = float(np.max(np.abs(np.asarray(got, np.float64) - want)) / max(np.max(np.abs(want)), 1e-30))
        out.append({"op": name, "normwise_error": float("%.3g" % err), "within_1e-4": err <= 1e-4})

    for name, typ, fn in (("add", ora.ADD, L.mnv_add), ("sub", ora.SUB, L.mnv_sub),
                          ("mul", ora.MUL, L.mnv_mul), ("div", ora.DIV, L.mnv_div)):
        exact(name, run(lambda o: fn(dx.p, dy.p, o.p, m * n, S), m * n), ora.arithmetic(typ, x, y))
    exact("scalar mul", run(lambda o: L.mnv_const_mul(dx.p, o.p, f(3.291), m * n, S), m * n),
          ora.arithmetic_const(ora.MUL, 1, 3.291, x))
    col, row = rng.standard_normal(n, dtype=np.float32), rng.standard_normal(m, dtype=np.float32)
    dcol, drow = dev.upload(col), dev.upload(row)
    exact("broadcast add {1,n}", run(lambda o: L.mnv_norm_add_col(dx.p, dcol.p, o.p, m, n, S), m * n),
          ora.norm_arithmetic(ora.ADD, x, [m, n], col, [0]))
    exact("broadcast add {m,1}", run(lambda o: L.mnv_norm_add_row(dx.p, drow.p, o.p, m, n, S), m * n),
          ora.norm_arithmetic(ora.ADD, x, [m, n], row, [1]))
    close("exp", run(lambda o: L.mnv_exp(dx.p, o.p, m * n, S), m * n), ora.elewise(ora.EXP, x))
    for name, alg, fw, bw in (("sigmoid", ora.SIGMOID, L.mnv_sigmoid_fwd, L.mnv_sigmoid_bwd),
                              ("relu", ora.RELU, L.mnv_relu_fwd, L.mnv_relu_bwd),
                              ("tanh", ora.TANH, L.mnv_tanh_fwd, L.mnv_tanh_bwd)):
        top = ora.activation_fwd(alg, x)
        dtop = dev.upload(top)
        (exact if alg == ora.RELU else close)(name + " fwd", run(lambda o: fw(dx.p, o.p, m * n, S), m * n), top)
        (exact if alg == ora.RELU else close)(
            name + " bwd", run(lambda o: bw(dx.p, dtop.p, dy.p, o.p, m * n, S), m * n),
            ora.activation_bwd(alg, y, top, x))
    close("sum dim 0", run(lambda o: L.mnv_reduce_sum_col(dx.p, o.p, m, n, S), n), ora.reduction(ora.SUM, x, [m, n], [0]))
    close("sum dim 1", run(lambda o: L.mnv_reduce_sum_row(dx.p, o.p, m, n, S), m), ora.reduction(ora.SUM, x, [m, n], [1]))
    exact("max dim 0", run(lambda o: L.mnv_reduce_max_col(dx.p, o.p, m, n, S), n), ora.reduction(ora.MAX, x, [m, n], [0]))
    exact("max dim 1", run(lambda o: L.mnv_reduce_max_row(dx.p, o.p, m, n, S), m), ora.reduction(ora.MAX, x, [m, n], [1]))
    exact("maxindex dim 0", run(lambda o: L.mnv_maxindex_col(dx.p, o.p, m, n, S), n), ora.maxindex(x, [m, n], 0))
    exact("maxindex dim 1", run(lambda o: L.mnv_maxindex_row(dx.p, o.p, m, n, S), m), ora.maxindex(x, [m, n], 1))
    sm = ora.softmax_instance_fwd(x, n, m, 1, 1)
    dsm = dev.upload(sm)
    close("softmax rows", run(lambda o: L.mnv_softmax_instance_fwd(dx.p, o.p, n, m, 1, 1, S), m * n), sm)
    close("softmax rows bwd", run(lambda o: L.mnv_softmax_instance_bwd(dy.p, dsm.p, o.p, n, m, 1, 1, S), m * n),
          ora.softmax_instance_bwd(y, sm, n, m, 1, 1))
    exact("transpose", run(lambda o: L.mnv_transpose(dx.p, o.p, m, n, S), m * n), ora.transpose(x, n, m))
    gm, gn, gk = 384, 200, 1000
    a, b = rng.standard_normal(gm * gk, dtype=np.float32), rng.standard_normal(gk * gn, dtype=np.float32)
    da, db = dev.upload(a), dev.upload(b)
    close("sgemm 384x1000x200", run(lambda o: L.mnv_sgemm_nn(da.p, db.p, o.p, gm, gn, gk, None, 0, S), gm * gn),
          ora.matmult(a, b, gm, gn, gk))
    # conv3 of the AlexNet shape at batch 4, pool1's window on a 27x27 plane
    p = (4, 256, 384, 13, 13, 1, 1, 1, 1, 3, 3)
    N, C, K, H, W = p[:5]
    cx, cw = rng.standard_normal(N * C * H * W, dtype=np.float32), rng.standard_normal(K * C * 9, dtype=np.float32) * np.float32(0.05)
    cb, cdy = rng.standard_normal(K, dtype=np.float32), rng.standard_normal(N * K * H * W, dtype=np.float32)
    dcx, dcw, dcb, dcdy = dev.upload(cx), dev.upload(cw), dev.upload(cb), dev.upload(cdy)
    wsb = 128 << 20
    ws = dev.empty(wsb // 4)
    z = ctypes.c_size_t(wsb)
    close("conv forward", run(lambda o: L.mnv_conv_fwd(dcx.p, dcw.p, dcb.p, o.p, *p, ws.p, z, S), N * K * H * W),
          ora.conv_fwd(cx, cw, cb, *p))
    close("conv backward data", run(lambda o: L.mnv_conv_bwd_data(dcdy.p, dcw.p, o.p, *p, ws.p, z, S), N * C * H * W),
          ora.conv_bwd_data(cdy, cw, *p))
    close("conv backward filter", run(lambda o: L.mnv_conv_bwd_filter(dcx.p, dcdy.p, o.p, *p, ws.p, z, S), K * C * 9),
          ora.conv_bwd_filter(cdy, cx, *p))
    close("conv backward bias", run(lambda o: L.mnv_conv_bwd_bias(dcdy.p, o.p, N, K, H, W, ws.p, z, S), K),
          ora.conv_bwd_bias(cdy, N, K, H, W))
    # the same layer by minimal filtering, the way the batch-256 step runs it (at batch 4 the
    # library would not choose it by itself)
    L.mnv_conv_winograd_mode(2)
    try:
        close("conv forward, F(5x5,3x3)", run(lambda o: L.mnv_conv_fwd(dcx.p, dcw.p, dcb.p, o.p, *p, ws.p, z, S), N * K * H * W),
              ora.conv_fwd(cx, cw, cb, *p))
        close("conv backward data, F(5x5,3x3)", run(lambda o: L.mnv_conv_bwd_data(dcdy.p, dcw.p, o.p, *p, ws.p, z, S), N * C * H * W),
              ora.conv_bwd_data(cdy, cw, *p))
        close("conv backward filter, F(3x3,5x5)", run(lambda o: L.mnv_conv_bwd_filter(dcx.p, dcdy.p, o.p, *p, ws.p, z, S), K * C * 9),
              ora.conv_bwd_filter(cdy, cx, *p))
        L.mnv_conv_winograd_mode(4)  # the smaller tiles, which planes with fewer outputs take
        close("conv forward, F(4x4,3x3)", run(lambda o: L.mnv_conv_fwd(dcx.p, dcw.p, dcb.p, o.p, *p, ws.p, z, S), N * K * H * W),
              ora.conv_fwd(cx, cw, cb, *p))
        close("conv backward data, F(4x4,3x3)", run(lambda o: L.mnv_conv_bwd_data(dcdy.p, dcw.p, o.p, *p, ws.p, z, S), N * C * H * W),
              ora.conv_bwd_data(cdy, cw, *p))
        close("conv backward filter, F(3x3,4x4)", run(lambda o: L.mnv_conv_bwd_filter(dcx.p, dcdy.p, o.p, *p, ws.p, z, S), K * C * 9),
              ora.conv_bwd_filter(cdy, cx, *p))
        L.mnv_conv_winograd_mode(3)
        close("conv forward, F(2x2,3x3)", run(lambda o: L.mnv_conv_fwd(dcx.p, dcw.p, dcb.p, o.p, *p, ws.p, z, S), N * K * H * W),
              ora.conv_fwd(cx, cw, cb, *p))
        close("conv backward data, F(2x2,3x3)", run(lambda o: L.mnv_conv_bwd_data(dcdy.p, dcw.p, o.p, *p, ws.p, z, S), N * C * H * W),
              ora.conv_bwd_data(cdy, cw, *p))
        close("conv backward filter, F(3x3,2x2)", run(lambda o: L.mnv_conv_bwd_filter(dcx.p, dcdy.p, o.p, *p, ws.p, z, S), K * C * 9),
              ora.conv_bwd_filter(cdy, cx, *p))
    finally:
        L.mnv_conv_winograd_mode(1)
    g = (8, 16, 27, 27, 2, 2, 3, 3, 0, 0)
    px = np.round(rng.standard_normal(8 * 16 * 27 * 27) * 2).astype(np.float32)  # many ties
    pt = ora.pool_fwd(ora.POOL_MAX, px, *g)
    pdy = rng.standard_normal(pt.size, dtype=np.float32)
    dpx, dpt, dpdy = dev.upload(px), dev.upload(pt), dev.upload(pdy)
    exact("max pooling forward", run(lambda o: L.mnv_maxpool_fwd(dpx.p, o.p, *g, S), pt.size), pt)
    exact("max pooling backward (ties)", run(lambda o: L.mnv_maxpool_bwd(dpx.p, dpt.p, dpdy.p, o.p, *g, S), px.size),
          ora.pool_bwd(ora.POOL_MAX, pdy, pt, px, *g))
    del dev
    # the benchmark's own step: batch 256 on the GPU, and the probabilities of its first four
    # images against the oracle's forward pass at batch 4 on the same parameters and images
    # (the forward pass treats images independently)
    from minerva_amd import hostapi
    from oracle import nets
    params, data, label = nets.make_inputs("alexnet", BATCH)
    _, want = nets.alexnet_forward(params, np.ascontiguousarray(data[:4 * 3 * 227 * 227]), 4)
    rt = hostapi.Runtime(0, sync_each_op=False)
    net = hostapi.Net(rt, "alexnet", BATCH)
    for k, v in params.items():
        net.set_param(k, v)
    net.load_batch(data, label)
    net.step(0.01)
    rt.sync()
    prob = net.read("prob", 1000 * BATCH)
    net.close()
    rt.close()
    close("alexnet step at batch 256: probabilities of the first 4 images", prob[:4000], want)
    bad = [r["op"] for r in out if not (r.get("bit_exact") or r.get("within_1e-4"))]
    return {"against": "the CPU oracle (oracle/mnv_oracle.c), same seeded inputs, reduced sizes",
            "all_within_bounds": not bad, "failed": bad, "ops": out}


SECTIONS = ("alexnet", "sgemm", "eltwise", "small", "owl", "cpu")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-full", action="store_true",
                    help="CPU baseline: run the two larger SGEMM shapes whole (minutes)")
    ap.add_argument("--no-dataflow", action="store_true",
                    help="skip the run with operators spread over four streams (their kernels "
                         "overlap, which disturbs per-kernel durations in a trace)")
    ap.add_argument("--sections", default="all",
                    help="comma-separated parts to run (for profiling one part): " + ",".join(SECTIONS))
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures the one-GPU operator path only: run with --gpus 1 "
                 "(nothing in this build uses a second GPU)")
    want = set(SECTIONS) if args.sections == "all" else set(args.sections.split(","))
    if want - set(SECTIONS):
        sys.exit("unknown section(s): %s" % ", ".join(sorted(want - set(SECTIONS))))
    if args.no_cpu:
        want.discard("cpu")
    from minerva_amd import capi
    dev_info = capi.Device(0, own_stream=False).info()
    log("device:", dev_info)
    line = {
        "metric": "AlexNet-shape fp32 train images/s at b=256; SGEMM TFLOP/s; eltwise HBM GB/s",
        "value": None, "unit": "images/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": None,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "AlexNet-shaped single-group network (BASELINE.json configs[4]): "
                               "NCHW fp32, batch 256, 3x227x227 input, forward + backward + SGD, "
                               "one operator per launch, one stream sync per step",
                   "global_batch": BATCH, "algorithmic_gflop_per_step": STEP_GFLOP},
        "timing": "value / ms_per_step: mean over exactly `steps` steps; kernels: median of 5 "
                  "batches of back-to-back calls between two events on the kernels' stream",
        "roofline": None, "cpu_baseline": None,
    }
    if "alexnet" in want:
        res = alexnet_bench(args.steps, args.warmup, not args.no_dataflow)
        main_run = res["per_step_sync"]
        line.update({
            "value": round(main_run["images_per_s"], 1),
            "ms_per_step": round(main_run["ms_per_step"], 3),
            "median_ms_per_step": round(main_run["median_ms_per_step"], 3),
            "step_mfma_frac": round(STEP_GFLOP / main_run["ms_per_step"] / PEAK_FP32_MFMA_TFLOPS, 4),
            "step_mfma_frac_note": "algorithmic (direct-sum) flops of the step / time / fp32 MFMA peak; "
                                   "conv2 executes 4/25 x (28/27)^2 of its, the 3 x 3 layers 49/225 x (15/13)^2 of theirs",
            "step_executed_gflop": STEP_EXECUTED_GFLOP,
            "step_executed_mfma_frac": round(STEP_EXECUTED_GFLOP / main_run["ms_per_step"] /
                                             PEAK_FP32_MFMA_TFLOPS, 4),
            "per_op_sync": {"images_per_s": round(res["per_op_sync"]["images_per_s"], 1),
                            "ms_per_step": round(res["per_op_sync"]["ms_per_step"], 3)},
            "graph_replay": main_run["graph_replay"],
            "fused_epilogues": {"images_per_s": round(res["fused"]["images_per_s"], 1),
                                "ms_per_step": round(res["fused"]["ms_per_step"], 3),
                                "ops_per_step": res["fused"]["ops_per_step"],
                                "graph_replay": res["fused"]["graph_replay"],
                                "weight_updates_in_gradient_kernels": {
                                    "images_per_s": round(res["fused_updates"]["images_per_s"], 1),
                                    "ms_per_step": round(res["fused_updates"]["ms_per_step"], 3),
                                    "ops_per_step": res["fused_updates"]["ops_per_step"],
                                    "note": "same parameters bit for bit; weight gradients are not stored"},
                                "note": "opt-in fused operators, results bit-identical to the "
                                        "operator-by-operator step"},
            "dataflow_4_streams": ({"images_per_s": round(res["dataflow"]["images_per_s"], 1),
                                    "ms_per_step": round(res["dataflow"]["ms_per_step"], 3)}
                                   if "dataflow" in res else None),
            "h2d_batch_ms": round(main_run["h2d_batch_ms"], 2),
            "value_with_input_feed": {
                "images_per_s": round(BATCH / main_run["fed_ms_per_step"] * 1e3, 1),
                "ms_per_step": round(main_run["fed_ms_per_step"], 3),
                "note": "a new 158 MB batch from pageable host memory every step, copied on a "
                        "second stream through pinned staging while the step before it runs "
                        "(mnvh_net_prefetch_batch); `value` is measured on a resident batch"},
            "roofline": dominant_kernel_roofline(main_run["profile"], args.steps),
            "top_ops": op_table(main_run["all_ops"], args.steps),
            "outputs_finite": main_run["finite"] and res["per_op_sync"]["finite"],
        })
        line["config"]["ops_per_step"] = main_run["ops_per_step"]
    if "owl" in want:
        line["owl_front_end"] = owl_front_end_bench(args.steps, args.warmup)
        line["owl_net_caffe_alexnet"] = owl_net_bench(args.steps, args.warmup)
    if "sgemm" in want:
        line["sgemm"] = sgemm_bench()
    if "eltwise" in want:
        line["eltwise"] = eltwise_bench()
    if "small" in want:
        line["small_nets"] = small_nets()
    line["device"] = dev_info
    if "cpu" in want:
        line["cpu_baseline"] = cpu_baseline(full=args.cpu_full)
        line["cpu_baseline"]["parity"] = parity_report()
        log("parity against the CPU oracle: %s" % ("all operators within their bounds"
            if line["cpu_baseline"]["parity"]["all_within_bounds"]
            else "FAILED: " + ", ".join(line["cpu_baseline"]["parity"]["failed"])))
    print(json.dumps(line))


if __name__ == "__main__":
    main()
