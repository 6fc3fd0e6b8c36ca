#!/usr/bin/env python3
"""Benchmark of the Shadow tensor hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-configs]

A "step" is one pass of the headline workload (BASELINE.json configs[1]): seven
launches over an fp32 [64,256,56,56] tensor -- Activate relu, sigmoid, tanh;
Unary exp, abs, sqrt(abs); Scale(per-channel gamma, beta)+ReLU in one launch.
Inputs are generated from fixed seeds, uploaded once and stay resident in HBM;
the timed region is K steps between two stream synchronisations.

Prints ONE JSON line.  `value` is algorithmic GB/s of the whole step
(compulsory reads + writes of every op / wall time).  `roofline` describes the
kernel that takes the largest share of the step, timed with HIP events on the
launch stream inside the timed region.  `cpu_baseline` is the CPU oracle (a C
port of the reference's loops, one thread) timed on this host on the same
buffers.  `configs` lists every op of the five BASELINE workloads measured the
same way (events around batches of launches that rotate over >256 MB of
buffers), so that each can be held against the 8 TB/s HBM roofline.
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

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published

# HBM bytes per launch of the headline kernels, from the FETCH_SIZE / WRITE_SIZE
# counters of `rocprofv3 --pmc` runs of `bench.py --probe`, each scaled by what
# the same counter reads for a plain copy of known size (the summary with the
# raw readings and the factors is profiles/headline_unary_chain_hbm_counters.txt).
# They cannot be collected from inside this process, so they are recorded here.
MEASURED_TRAFFIC_BYTES = {
    "activate_relu": 411.04e6, "activate_sigmoid": 411.06e6, "unary_exp": 411.01e6,
    "unary_abs": 411.04e6, "unary_sqrt_of_abs": 411.00e6, "activate_tanh": 411.02e6,
    "scale_relu_fused": 411.02e6,
}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-configs", action="store_true", help="skip the per-config table")
    ap.add_argument("--cpu-passes", type=int, default=10)
    ap.add_argument("--operand-sets", type=int, default=1,
                    help="multiplier on the number of rotating operand sets of the config table")
    ap.add_argument("--probe", action="store_true",
                    help="counter probe: 3 launches of a plain copy and of every headline op on "
                         "the 51.4M tensor, nothing timed, no JSON (run under rocprofv3 --pmc)")
    ap.add_argument("--probe-next", action="store_true",
                    help="the same for the neighbouring operators and the data movers")
    return ap.parse_args()


def normal(seed, n, sigma=1.0):
    return (np.random.default_rng(seed).standard_normal(n, dtype=np.float32) * np.float32(sigma))


def uniform(seed, n, lo, hi):
    u = np.random.default_rng(seed).random(n, dtype=np.float32)
    return (np.float32(lo) + u * np.float32(hi - lo)).astype(np.float32)


class Dev:
    """Device-side plumbing over the C ABI: one stream, events, buffers."""

    def __init__(self):
        import shadow_amd
        self.sa = shadow_amd
        self.lib = shadow_amd.hip()
        if shadow_amd.device_count() < 1:
            raise SystemExit("bench.py: no HIP device visible")
        self.ck(self.lib.shdw_hip_set_device(0))
        s = ctypes.c_void_p()
        self.ck(self.lib.shdw_hip_stream_create(ctypes.byref(s)))
        self.stream = s
        info = ctypes.create_string_buffer(256)
        self.ck(self.lib.shdw_hip_device_info(0, info, 256))
        self.info = info.value.decode()
        if self.info.startswith("|"):  # the runtime reports no marketing name on some boxes
            self.info = "gfx950 device" + self.info

    def ck(self, rc):
        self.sa.check(rc)

    def buf(self, arr=None, nbytes=None):
        if arr is not None:
            return self.sa.Buffer.from_numpy(arr)
        return self.sa.Buffer(nbytes)

    def event(self):
        e = ctypes.c_void_p()
        self.ck(self.lib.shdw_hip_event_create(ctypes.byref(e)))
        return e

    def record(self, e):
        self.ck(self.lib.shdw_hip_event_record(e, self.stream))

    def elapsed_ms(self, a, b):
        ms = ctypes.c_float(0)
        self.ck(self.lib.shdw_hip_event_elapsed_ms(a, b, ctypes.byref(ms)))
        return ms.value

    def sync(self):
        self.ck(self.lib.shdw_hip_stream_sync(self.stream))


# ------------------------------------------------------------------ headline
def headline(dev, steps, warmup):
    lib, st = dev.lib, dev.stream
    shape = (64, 256, 56, 56)
    n = int(np.prod(shape))
    C, inner = shape[1], shape[2] * shape[3]
    x_h = normal(201, n, 2.0)
    g_h, b_h = uniform(202, C, 0.5, 1.5), uniform(203, C, -0.1, 0.1)
    x, g, b = dev.buf(x_h), dev.buf(g_h), dev.buf(b_h)
    y = [dev.buf(nbytes=4 * n) for _ in range(2)]
    a = dev.buf(nbytes=4 * n)  # abs output, input of sqrt

    per_op = 8 * n
    ops = [
        ("activate_relu", per_op, lambda o: lib.shdw_hip_activate(1, 0.1, n, x.ptr, o.ptr, st)),
        ("activate_sigmoid", per_op, lambda o: lib.shdw_hip_activate(3, 0.1, n, x.ptr, o.ptr, st)),
        ("unary_exp", per_op, lambda o: lib.shdw_hip_unary(4, n, x.ptr, o.ptr, st)),
        ("unary_abs", per_op, lambda o: lib.shdw_hip_unary(0, n, x.ptr, a.ptr, st)),
        ("unary_sqrt_of_abs", per_op, lambda o: lib.shdw_hip_unary(2, n, a.ptr, o.ptr, st)),
        ("activate_tanh", per_op, lambda o: lib.shdw_hip_activate(5, 0.1, n, x.ptr, o.ptr, st)),
        ("scale_relu_fused", per_op + 8 * C,
         lambda o: lib.shdw_hip_scale_bias(n, C, inner, x.ptr, g.ptr, b.ptr, 1, o.ptr, st)),
    ]
    step_bytes = sum(nb for _, nb, _ in ops)

    def step(i, events=None, only=None):
        """events: one (start, stop) pair per op; only: record just around that op."""
        for k, (_, _, fn) in enumerate(ops):
            marked = events is not None and (only is None or only == k)
            if marked:
                dev.record(events[k][0])
            dev.ck(fn(y[(i + k) & 1]))
            if marked:
                dev.record(events[k][1])

    for i in range(warmup):
        step(i)
    dev.sync()

    # Untimed pass with events around every launch: the per-op table, and which
    # kernel dominates.  Event records between launches cost ~2.5 us each, so the
    # timed region below carries them around the dominant kernel only.
    ev = [[(dev.event(), dev.event()) for _ in ops] for _ in range(steps)]
    for i in range(steps):
        step(i, ev[i])
    dev.sync()
    kernel_ms = []
    for k in range(len(ops)):
        kernel_ms.append(sum(dev.elapsed_ms(ev[i][k][0], ev[i][k][1]) for i in range(steps)) / steps)
    detail = []
    for (name, nb, _), ms in zip(ops, kernel_ms):
        gbs = nb / (ms * 1e-3) / 1e9
        detail.append({"op": name, "bytes": nb, "us": round(ms * 1e3, 2), "GBps": round(gbs, 1),
                       "frac": round(gbs / HBM_PEAK_GBS, 4)})
    dom = int(np.argmax(kernel_ms))

    t0 = time.perf_counter()
    for i in range(steps):
        step(i, ev[i], only=dom)
    dev.sync()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / steps
    kernel_ms[dom] = sum(dev.elapsed_ms(ev[i][dom][0], ev[i][dom][1]) for i in range(steps)) / steps
    dom_gbs = ops[dom][1] / (kernel_ms[dom] * 1e-3) / 1e9
    roofline = {"bound": "hbm", "kernel": ops[dom][0], "achieved": round(dom_gbs, 1),
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(dom_gbs / HBM_PEAK_GBS, 4),
                "traffic": MEASURED_TRAFFIC_BYTES.get(ops[dom][0]), "avg_us": round(kernel_ms[dom] * 1e3, 2),
                "algorithmic_bytes": ops[dom][1]}
    host = {"x": x_h, "gamma": g_h, "beta": b_h, "shape": shape}
    return ms_per_step, step_bytes, n, roofline, detail, host


def probe(dev):
    """For `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE`: the copy kernel moves a
    known 205,520,896 B each way and calibrates the counters; the other launches
    are the headline ops on the same tensor."""
    lib, st = dev.lib, dev.stream
    n, C, inner = 64 * 256 * 56 * 56, 256, 56 * 56
    x = dev.buf(normal(201, n, 2.0))
    g, b = dev.buf(uniform(202, C, 0.5, 1.5)), dev.buf(uniform(203, C, -0.1, 0.1))
    y = dev.buf(nbytes=4 * n)
    for _ in range(3):
        dev.ck(lib.shdw_hip_copy(n, x.ptr, y.ptr, st))
        dev.ck(lib.shdw_hip_activate(1, 0.1, n, x.ptr, y.ptr, st))
        dev.ck(lib.shdw_hip_activate(3, 0.1, n, x.ptr, y.ptr, st))
        dev.ck(lib.shdw_hip_unary(4, n, x.ptr, y.ptr, st))
        dev.ck(lib.shdw_hip_unary(0, n, x.ptr, y.ptr, st))
        dev.ck(lib.shdw_hip_unary(2, n, x.ptr, y.ptr, st))
        dev.ck(lib.shdw_hip_activate(5, 0.1, n, x.ptr, y.ptr, st))
        dev.ck(lib.shdw_hip_scale_bias(n, C, inner, x.ptr, g.ptr, b.ptr, 1, y.ptr, st))
    dev.sync()


def probe_next(dev):
    """Counter probe for the operators next to the path, 3 launches each on the
    headline tensor (or the ResNet shape that feeds them); the copy calibrates."""
    lib, st = dev.lib, dev.stream
    I = dev.sa.ints
    n, C, inner = 64 * 256 * 56 * 56, 256, 56 * 56
    x, x2 = dev.buf(normal(201, n, 2.0)), dev.buf(normal(204, n))
    g, b = dev.buf(uniform(202, C, 0.5, 1.5)), dev.buf(uniform(203, C, -0.1, 0.1))
    alpha = dev.buf(uniform(205, 64 * C, 0.0, 1.0))
    ls, lb = dev.buf(uniform(206, 784, 0.5, 1.5)), dev.buf(uniform(207, 784, -0.1, 0.1))
    y = dev.buf(nbytes=4 * n)
    ssd_ws = dev.buf(nbytes=max(8, lib.shdw_hip_ssd_normalize_workspace_bytes(64, 512, 1444, 1)))
    ssd_sc = dev.buf(uniform(208, 512, 10.0, 30.0))
    stem_in, stem_out = [64, 64, 112, 112], [64, 64, 56, 56]
    for _ in range(3):
        dev.ck(lib.shdw_hip_copy(n, x.ptr, y.ptr, st))
        dev.ck(lib.shdw_hip_batch_norm(n, C, inner, x.ptr, b.ptr, g.ptr, 1.0, 1e-5, y.ptr, st))
        dev.ck(lib.shdw_hip_axpy_rows(64 * C, inner, alpha.ptr, x.ptr, x2.ptr, y.ptr, st))
        dev.ck(lib.shdw_hip_pooling2d(I(stem_in), 0, 3, 3, 2, 2, 0, 0, I(stem_out), x.ptr, y.ptr, st))
        dev.ck(lib.shdw_hip_pooling2d(I([512, 2048, 7, 7]), 1, 7, 7, 1, 1, 0, 0, I([512, 2048, 1, 1]), x.ptr,
                                      y.ptr, st))
        dev.ck(lib.shdw_hip_softmax(64, 49, 16384, x.ptr, y.ptr, st))
        dev.ck(lib.shdw_hip_normalize(64, 49, 16384, 2.0, 1e-12, x.ptr, y.ptr, st))
        dev.ck(lib.shdw_hip_group_norm(64 * C, inner, 1e-5, x.ptr, g.ptr, b.ptr, C, inner, y.ptr, st))
        dev.ck(lib.shdw_hip_group_norm(64 * 32, 8 * inner, 1e-5, x.ptr, g.ptr, b.ptr, C, inner, y.ptr, st))
        dev.ck(lib.shdw_hip_group_norm(65536, 784, 1e-5, x.ptr, ls.ptr, lb.ptr, 784, 1, y.ptr, st))
        dev.ck(lib.shdw_hip_permute(4, I([64, 256, 56, 56]), I([0, 2, 3, 1]), x.ptr, y.ptr, st))
        dev.ck(lib.shdw_hip_shuffle_channel(64, 256, inner, 2, x.ptr, y.ptr, st))
        dev.ck(lib.shdw_hip_pad(I([64, 64, 110, 110]), I([1, 1, 1, 1]), 0.0, x.ptr, y.ptr, st))
        dev.ck(lib.shdw_hip_resize(I(stem_out), I(stem_in), 1, 0, x.ptr, y.ptr, st))
        dev.ck(lib.shdw_hip_resize(I(stem_out), I(stem_in), 0, 0, x.ptr, y.ptr, st))
        dev.ck(lib.shdw_hip_reorg(I(stem_in), 1, 2, x.ptr, y.ptr, st))
        dev.ck(lib.shdw_hip_reorg(I(stem_in), 0, 2, x.ptr, y.ptr, st))
        dev.ck(lib.shdw_hip_softmax(64, 150, 5184, x.ptr, y.ptr, st))
        dev.ck(lib.shdw_hip_softmax(64, 150, 5329, x.ptr, y.ptr, st))
        dev.ck(lib.shdw_hip_ssd_normalize(64, 512, 1444, 0, 1e-5, x.ptr, ssd_sc.ptr, 0, y.ptr, None, st))
        dev.ck(lib.shdw_hip_ssd_normalize(64, 256, 3136, 0, 1e-5, x.ptr, ssd_sc.ptr, 0, y.ptr, None, st))
        dev.ck(lib.shdw_hip_ssd_normalize(64, 512, 1444, 1, 1e-5, x.ptr, ssd_sc.ptr, 0, y.ptr, ssd_ws.ptr, st))
    dev.sync()


def cpu_baseline(host, step_bytes, passes):
    """The oracle on this host, one thread: the same seven results, with
    Scale and ReLU as the two separate operators the reference runs."""
    import oracle
    x, g, b = host["x"], host["gamma"], host["beta"]
    C, inner = host["shape"][1], host["shape"][2] * host["shape"][3]
    oracle.lib()
    best = None
    for _ in range(passes):
        t0 = time.perf_counter()
        oracle.activate(x, 1)
        oracle.activate(x, 3)
        oracle.unary(4, x)
        a = oracle.unary(0, x)
        oracle.unary(2, a)
        oracle.activate(x, 5)
        s = oracle.scale_bias(x, g, b, C, inner)
        oracle.activate(s, 1)
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    return {"value": round(step_bytes / best / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "%d full passes of the same step on the same buffers (51.4M elements, 8 "
                      "operator runs each), best pass %.2f s; host has %d logical CPUs" % (
                          passes, best, os.cpu_count() or 0),
            "seconds_per_step": round(best, 3)}


# ------------------------------------------------------------- config table
def time_batch(dev, launch, sets, reps=40, warm=5):
    """Average device time of one launch: events around `reps` back-to-back
    launches that rotate over `sets` operand sets."""
    for i in range(warm):
        dev.ck(launch(i % sets))
    e0, e1 = dev.event(), dev.event()
    dev.record(e0)
    for i in range(reps):
        dev.ck(launch(i % sets))
    dev.record(e1)
    dev.sync()
    return dev.elapsed_ms(e0, e1) / reps


def config_table(dev, sets_scale=1):
    lib, st = dev.lib, dev.stream
    I = dev.sa.ints
    rows = []

    def add(cfg, name, nbytes, ms, elems):
        gbs = nbytes / (ms * 1e-3) / 1e9
        rows.append({"cfg": cfg, "op": name, "bytes": nbytes, "us": round(ms * 1e3, 2),
                     "GBps": round(gbs, 1), "frac": round(gbs / HBM_PEAK_GBS, 4),
                     "Gelem_s": round(elems / (ms * 1e-3) / 1e9, 2)})

    SETS = 6 * sets_scale  # 6 x (in + out) of 51 MB each: more than the 256 MB Infinity Cache
    NBIG = 12845056  # elements of the cfg-3 and cfg-5 tensors (51.4 MB)
    A = [dev.buf(normal(301 + 10 * k, NBIG)) for k in range(SETS)]
    Y = [dev.buf(nbytes=4 * NBIG) for _ in range(SETS)]

    # cfg 1: Binary add with channel broadcast.  Its tensor is half of a set (25.7 MB):
    # both halves of every set take turns, 12 x 25.7 MB of inputs, so that no launch
    # finds its input still in the 256 MB Infinity Cache (with six inputs, 154 MB,
    # it did, and measured 8.7 us instead of 10.7).
    sa, sb = [8, 64, 112, 112], [1, 64, 1, 1]
    n = int(np.prod(sa))
    B = dev.buf(uniform(102, 64, -1, 1))
    ms = time_batch(dev, lambda k: lib.shdw_hip_broadcast_binary(
        0, 4, I(sa), I(sb), I(sa), A[k % SETS].ptr + (k // SETS) * 4 * n, B.ptr, Y[k % SETS].ptr, st), 2 * SETS)
    add(1, "binary_add_channel_broadcast", 8 * n + 256, ms, n)

    # cfg 3: reductions over [32,512,28,28]
    shp = [32, 512, 28, 28]
    for name, op, axes, outs in [("reduce_sum_hw", 1, [2, 3], 16384), ("reduce_avg_hw", 4, [2, 3], 16384),
                                 ("reduce_max_c", 2, [1], 25088), ("reduce_sum_all", 1, [0, 1, 2, 3], 1)]:
        need = lib.shdw_hip_reduce_workspace_bytes(4, I(shp), len(axes), I(axes))
        ws = dev.buf(nbytes=max(need, 16))
        ms = time_batch(dev, lambda k: lib.shdw_hip_reduce(op, 4, I(shp), len(axes), I(axes), A[k].ptr,
                                                           Y[k].ptr, ws.ptr, need, st), SETS)
        add(3, name, 4 * NBIG + 4 * outs, ms, NBIG)

    # cfg 5: ResNet bottleneck tail on [64,1024,14,14]
    n5, C5, in5 = 12845056, 1024, 196
    g5, b5 = dev.buf(uniform(502, C5, 0.5, 1.5)), dev.buf(uniform(503, C5, -0.1, 0.1))
    M = [dev.buf(nbytes=4 * 65536) for _ in range(SETS)]
    ms = time_batch(dev, lambda k: lib.shdw_hip_scale_bias(n5, C5, in5, A[k].ptr, g5.ptr, b5.ptr, 0,
                                                           Y[k].ptr, st), SETS)
    add(5, "scale", 8 * n5 + 8 * C5, ms, n5)

    def eltwise_sum(k):
        ptrs = (ctypes.c_void_p * 2)(A[k].ptr, A[(k + 1) % SETS].ptr)
        return lib.shdw_hip_eltwise(1, 2, ptrs, None, n5, Y[k].ptr, st)
    ms = time_batch(dev, eltwise_sum, SETS)
    add(5, "eltwise_sum", 12 * n5, ms, n5)
    ms = time_batch(dev, lambda k: lib.shdw_hip_activate(1, 0.1, n5, A[k].ptr, Y[k].ptr, st), SETS)
    add(5, "relu", 8 * n5, ms, n5)
    sh5, ax5 = [64, 1024, 14, 14], [2, 3]
    ms = time_batch(dev, lambda k: lib.shdw_hip_reduce(4, 4, I(sh5), 2, I(ax5), A[k].ptr, M[k].ptr,
                                                       None, 0, st), SETS)
    add(5, "reduce_avg_hw", 4 * n5 + 4 * 65536, ms, n5)
    sh7 = [128, 2048, 7, 7]  # the same reduction over 7 x 7 planes: rows of 49 floats start on odd dwords
    M7 = [dev.buf(nbytes=4 * 128 * 2048) for _ in range(SETS)]
    ms = time_batch(dev, lambda k: lib.shdw_hip_reduce(4, 4, I(sh7), 2, I(ax5), A[k].ptr, M7[k].ptr,
                                                       None, 0, st), SETS)
    add("next", "reduce_avg_hw 7x7 planes [128,2048,7,7]", 4 * n5 + 4 * 128 * 2048, ms, n5)
    # more of the same late-stage tensor, whose rows and planes are not multiples of four floats
    ws7 = dev.buf(nbytes=1 << 20)
    ms = time_batch(dev, lambda k: lib.shdw_hip_reduce(2, 4, I(sh7), 1, I([1]), A[k].ptr, M7[k].ptr,
                                                       ws7.ptr, 1 << 20, st), SETS)
    add("next", "reduce_max_c 7x7 maps [128,2048,7,7]", 4 * n5 + 4 * 128 * 49, ms, n5)
    g7, b7 = dev.buf(uniform(507, 2048, 0.5, 1.5)), dev.buf(uniform(508, 2048, -0.1, 0.1))
    ms = time_batch(dev, lambda k: lib.shdw_hip_group_norm(128 * 2048, 49, 1e-5, A[k].ptr, g7.ptr, b7.ptr,
                                                           2048, 49, Y[k].ptr, st), SETS)
    add("next", "instance_norm affine 7x7 planes [128,2048,7,7]", 8 * n5 + 8 * 2048, ms, n5)
    ms = time_batch(dev, lambda k: lib.shdw_hip_broadcast_binary(
        0, 4, I(sh7), I([1, 2048, 1, 1]), I(sh7), A[k].ptr, b7.ptr, Y[k].ptr, st), SETS)
    add("next", "binary_add_channel_broadcast 7x7 maps [128,2048,7,7]", 8 * n5 + 4 * 2048, ms, n5)
    for bb in M7 + [ws7, g7, b7]:
        bb.free()
    ms = time_batch(dev, lambda k: lib.shdw_hip_scale_residual_relu_rowmean(
        n5, C5, in5, A[k].ptr, g5.ptr, b5.ptr, A[(k + 1) % SETS].ptr, Y[k].ptr, M[k].ptr, st), SETS)
    add(5, "fused_tail", 12 * n5 + 8 * C5 + 4 * 65536, ms, n5)

    # Operators next to the path (label "next").  Global pooling, Softmax and
    # Normalize run on the 51 MB sets; BatchNorm, Axpy and the stem max pooling
    # run further down on 205 MB tensors like the headline step.
    pin, pout = [16, 64, 112, 112], [16, 64, 56, 56]
    npo = int(np.prod(pout))
    ms = time_batch(dev, lambda k: lib.shdw_hip_pooling2d(I(pin), 0, 3, 3, 2, 2, 0, 0, I(pout), A[k].ptr,
                                                          Y[k].ptr, st), SETS)
    add("next", "pooling_max_3x3s2 [16,64,112,112]", 4 * (NBIG + npo), ms, NBIG)
    gin, gout = [128, 2048, 7, 7], [128, 2048, 1, 1]
    ms = time_batch(dev, lambda k: lib.shdw_hip_pooling2d(I(gin), 1, 7, 7, 1, 1, 0, 0, I(gout), A[k].ptr,
                                                          Y[k].ptr, st), SETS)
    add("next", "pooling_global_avg_7x7", 4 * (NBIG + 128 * 2048), ms, NBIG)
    gin2, gout2 = [64, 1024, 14, 14], [64, 1024, 1, 1]
    ms = time_batch(dev, lambda k: lib.shdw_hip_pooling2d(I(gin2), 1, 14, 14, 1, 1, 0, 0, I(gout2), A[k].ptr,
                                                          Y[k].ptr, st), SETS)
    add("next", "pooling_global_avg_14x14", 4 * (NBIG + 65536), ms, NBIG)
    # [16, 49, 128, 128]: channel softmax / L2 normalize of a dense map (inner = 16384)
    ms = time_batch(dev, lambda k: lib.shdw_hip_softmax(16, 49, 16384, A[k].ptr, Y[k].ptr, st), SETS)
    add("next", "softmax_channels_dense", 8 * NBIG, ms, NBIG)
    ms = time_batch(dev, lambda k: lib.shdw_hip_normalize(16, 49, 16384, 2.0, 1e-12, A[k].ptr, Y[k].ptr, st),
                    SETS)
    add("next", "normalize_l2_channels_dense", 8 * NBIG, ms, NBIG)
    ms = time_batch(dev, lambda k: lib.shdw_hip_softmax(64, 1000, 1, A[k].ptr, Y[k].ptr, st), SETS)
    add("next", "softmax_classifier_64x1000", 8 * 64000, ms, 64000)
    ms = time_batch(dev, lambda k: lib.shdw_hip_normalize(64, 512, 1, 2.0, 1e-12, A[k].ptr, Y[k].ptr, st), SETS)
    add("next", "normalize_l2_embedding_64x512", 8 * 64 * 512, ms, 64 * 512)
    for bset in (A, Y):
        for bb in bset:
            bb.free()

    # "next" operators at the size of the headline tensor (205 MB in, 3 rotating sets)
    NH, SH = 51380224, 3 * sets_scale
    AH = [dev.buf(normal(701 + k, NH)) for k in range(SH)]
    YH = [dev.buf(nbytes=4 * NH) for _ in range(SH)]
    CH, INH = 256, 3136
    meanh, varh = dev.buf(normal(611, CH)), dev.buf(uniform(612, CH, 0.5, 2.0))
    ms = time_batch(dev, lambda k: lib.shdw_hip_batch_norm(NH, CH, INH, AH[k].ptr, meanh.ptr, varh.ptr,
                                                           1.0, 1e-5, YH[k].ptr, st), SH, reps=20)
    add("next", "batch_norm [64,256,56,56]", 8 * NH + 8 * CH, ms, NH)
    alh = dev.buf(uniform(613, 64 * CH, 0.0, 1.0))
    ms = time_batch(dev, lambda k: lib.shdw_hip_axpy_rows(64 * CH, INH, alh.ptr, AH[k].ptr,
                                                          AH[(k + 1) % SH].ptr, YH[k].ptr, st), SH, reps=20)
    add("next", "axpy_rows [64,256,56,56]", 12 * NH + 4 * 64 * CH, ms, NH)
    pinh, pouth = [64, 64, 112, 112], [64, 64, 56, 56]
    ms = time_batch(dev, lambda k: lib.shdw_hip_pooling2d(I(pinh), 0, 3, 3, 2, 2, 0, 0, I(pouth), AH[k].ptr,
                                                          YH[k].ptr, st), SH, reps=20)
    add("next", "pooling_max_3x3s2 [64,64,112,112]", 4 * (NH + NH // 4), ms, NH)
    ginh, gouth = [512, 2048, 7, 7], [512, 2048, 1, 1]
    ms = time_batch(dev, lambda k: lib.shdw_hip_pooling2d(I(ginh), 1, 7, 7, 1, 1, 0, 0, I(gouth), AH[k].ptr,
                                                          YH[k].ptr, st), SH, reps=20)
    add("next", "pooling_global_avg_7x7 [512,2048,7,7]", 4 * (NH + 512 * 2048), ms, NH)
    ms = time_batch(dev, lambda k: lib.shdw_hip_softmax(64, 49, 16384, AH[k].ptr, YH[k].ptr, st), SH, reps=20)
    add("next", "softmax_channels_dense [64,49,128,128]", 8 * NH, ms, NH)
    NSEG = 64 * 150 * 5329  # a 150-class segmentation head, 73 x 73
    ms = time_batch(dev, lambda k: lib.shdw_hip_softmax(64, 150, 5329, AH[k].ptr, YH[k].ptr, st), SH, reps=10)
    add("next", "softmax_150_classes [64,150,73,73]", 8 * NSEG, ms, NSEG)
    NSEG = 64 * 150 * 5184  # the same head on 72 x 72: rows of whole 128-bit vectors
    ms = time_batch(dev, lambda k: lib.shdw_hip_softmax(64, 150, 5184, AH[k].ptr, YH[k].ptr, st), SH, reps=10)
    add("next", "softmax_150_classes [64,150,72,72]", 8 * NSEG, ms, NSEG)
    ms = time_batch(dev, lambda k: lib.shdw_hip_normalize(64, 49, 16384, 2.0, 1e-12, AH[k].ptr, YH[k].ptr, st),
                    SH, reps=20)
    add("next", "normalize_l2_channels_dense [64,49,128,128]", 8 * NH, ms, NH)
    sch, bih = dev.buf(uniform(614, CH, 0.5, 1.5)), dev.buf(uniform(615, CH, -0.1, 0.1))
    ms = time_batch(dev, lambda k: lib.shdw_hip_group_norm(64 * CH, INH, 1e-5, AH[k].ptr, sch.ptr, bih.ptr,
                                                           CH, INH, YH[k].ptr, st), SH, reps=20)
    add("next", "instance_norm affine [64,256,56,56]", 8 * NH + 8 * CH, ms, NH)
    ms = time_batch(dev, lambda k: lib.shdw_hip_group_norm(64 * 32, 8 * INH, 1e-5, AH[k].ptr, sch.ptr, bih.ptr,
                                                           CH, INH, YH[k].ptr, st), SH, reps=20)
    add("next", "group_norm 32 groups affine [64,256,56,56]", 8 * NH + 8 * CH, ms, NH)
    lns, lnb = dev.buf(uniform(616, 784, 0.5, 1.5)), dev.buf(uniform(617, 784, -0.1, 0.1))
    ms = time_batch(dev, lambda k: lib.shdw_hip_group_norm(65536, 784, 1e-5, AH[k].ptr, lns.ptr, lnb.ptr,
                                                           784, 1, YH[k].ptr, st), SH, reps=20)
    add("next", "layer_norm affine [65536,784]", 8 * NH + 8 * 784, ms, NH)
    # SSDNormalize on the SSD conv4_3 map, batch 64: 8 bytes per element are compulsory
    # (the per-item form reads x a second time on top of that)
    NS = 64 * 512 * 1444
    ssc = dev.buf(uniform(618, 512, 10.0, 30.0))
    ms = time_batch(dev, lambda k: lib.shdw_hip_ssd_normalize(64, 512, 1444, 0, 1e-5, AH[k].ptr, ssc.ptr, 0,
                                                              YH[k].ptr, None, st), SH, reps=20)
    add("next", "ssd_normalize per position, channel scale [64,512,38,38]", 8 * NS + 4 * 512, ms, NS)
    ms = time_batch(dev, lambda k: lib.shdw_hip_ssd_normalize(64, 256, 3136, 0, 1e-5, AH[k].ptr, ssc.ptr, 0,
                                                              YH[k].ptr, None, st), SH, reps=20)
    add("next", "ssd_normalize per position, channel scale [64,256,56,56]", 8 * NH + 4 * 256, ms, NH)
    swb = dev.buf(nbytes=max(8, lib.shdw_hip_ssd_normalize_workspace_bytes(64, 512, 1444, 1)))
    ms = time_batch(dev, lambda k: lib.shdw_hip_ssd_normalize(64, 512, 1444, 1, 1e-5, AH[k].ptr, ssc.ptr, 0,
                                                              YH[k].ptr, swb.ptr, st), SH, reps=20)
    add("next", "ssd_normalize per item, channel scale [64,512,38,38] (2 launches)", 8 * NS + 4 * 512, ms, NS)
    # data movers ("movers") on the same 205 MB tensors
    half = NH // 2
    def concat2(k):
        # two [64,128,56,56] halves -> [64,256,56,56] along axis 1
        rc = lib.shdw_hip_copy_chunks(64, 128 * INH, AH[k].ptr, 128 * INH, 0, YH[k].ptr, 256 * INH, 0, st)
        return rc or lib.shdw_hip_copy_chunks(64, 128 * INH, AH[(k + 1) % SH].ptr, 128 * INH, 0, YH[k].ptr,
                                              256 * INH, 128 * INH, st)
    ms = time_batch(dev, concat2, SH, reps=20)
    add("movers", "concat 2x[64,128,56,56] axis 1 (2 launches)", 8 * NH, ms, NH)
    shp4 = [64, 256, 56, 56]
    ms = time_batch(dev, lambda k: lib.shdw_hip_permute(4, I(shp4), I([0, 2, 3, 1]), AH[k].ptr, YH[k].ptr, st),
                    SH, reps=20)
    add("movers", "permute NCHW->NHWC [64,256,56,56]", 8 * NH, ms, NH)
    ms = time_batch(dev, lambda k: lib.shdw_hip_permute(4, I(shp4), I([0, 3, 1, 2]), AH[k].ptr, YH[k].ptr, st),
                    SH, reps=20)
    add("movers", "permute [0,3,1,2] [64,256,56,56]", 8 * NH, ms, NH)
    ms = time_batch(dev, lambda k: lib.shdw_hip_shuffle_channel(64, 256, INH, 2, AH[k].ptr, YH[k].ptr, st), SH,
                    reps=20)
    add("movers", "shuffle_channel g=2 [64,256,56,56]", 8 * NH, ms, NH)
    pshape = [64, 64, 110, 110]
    npi = int(np.prod(pshape))
    ms = time_batch(dev, lambda k: lib.shdw_hip_pad(I(pshape), I([1, 1, 1, 1]), 0.0, AH[k].ptr, YH[k].ptr, st), SH,
                    reps=20)
    add("movers", "pad 1 [64,64,110,110] -> 112x112", 4 * (npi + NH), ms, NH)
    rin, rout = [64, 64, 56, 56], [64, 64, 112, 112]
    nri = int(np.prod(rin))
    # The resize input is a quarter of a set (51 MB): all four quarters of every set
    # take turns (12 inputs, 617 MB).  With three inputs the gathers found them in the
    # Infinity Cache and the kernels looked faster than they are from HBM (nearest:
    # 38 us against 64).
    def resize_in(k):
        return AH[k % SH].ptr + (k // SH) * 4 * nri
    ms = time_batch(dev, lambda k: lib.shdw_hip_resize(I(rin), I(rout), 1, 0, resize_in(k), YH[k % SH].ptr, st),
                    4 * SH, reps=24)
    add("movers", "resize bilinear x2 [64,64,56,56]", 4 * (nri + NH), ms, NH)
    ms = time_batch(dev, lambda k: lib.shdw_hip_resize(I(rin), I(rout), 0, 0, resize_in(k), YH[k % SH].ptr, st),
                    4 * SH, reps=24)
    add("movers", "resize nearest x2 [64,64,56,56]", 4 * (nri + NH), ms, NH)
    ms = time_batch(dev, lambda k: lib.shdw_hip_reorg(I(rout), 1, 2, AH[k].ptr, YH[k].ptr, st), SH, reps=20)
    add("movers", "reorg natural s2 [64,64,112,112]", 8 * NH, ms, NH)
    ms = time_batch(dev, lambda k: lib.shdw_hip_reorg(I(rout), 0, 2, AH[k].ptr, YH[k].ptr, st), SH, reps=20)
    add("movers", "reorg darknet s2 [64,64,112,112]", 8 * NH, ms, NH)
    for bset in (AH, YH):
        for bb in bset:
            bb.free()

    # cfg 4: general broadcast; outputs dominate the traffic
    for tag, sa4, sb4 in [("i", [16, 1, 128, 256], [1, 32, 128, 1]), ("ii", [4, 64, 1, 512], [1, 1, 64, 512]),
                          ("iii", [128, 1024], [1, 1])]:
        so4 = [max(p, q) for p, q in zip(sa4, sb4)]
        na, nb_, no = int(np.prod(sa4)), int(np.prod(sb4)), int(np.prod(so4))
        a4 = dev.buf(normal(401, na))
        b4 = dev.buf(uniform(402, nb_, 0.5, 2.0))
        y4 = [dev.buf(nbytes=4 * no) for _ in range(SETS)]
        for name, op in [("mul", 2), ("sub", 1), ("div", 3), ("max", 5)]:
            ms = time_batch(dev, lambda k: lib.shdw_hip_broadcast_binary(
                op, len(so4), I(sa4), I(sb4), I(so4), a4.ptr, b4.ptr, y4[k].ptr, st), SETS)
            add(4, "broadcast_%s_%s" % (name, tag), 4 * (na + nb_ + no), ms, no)
        for bb in y4:
            bb.free()
    return rows


NETWORK_TEXT = """[bottleneck_tail]
[{out_blob, v_s, [prob]}]
[{gamma, float, [1024]}; {beta, float, [1024]}]
[Input] | [in] | [0 2 2] | [] | [x; r] | [{x, v_i, [64 # 1024 # 14 # 14]}; {r, v_i, [64 # 1024 # 14 # 14]}]
[Scale] | [bn] | [3 1 3] | [x; gamma; beta] | [s] | [{axis, s_i, [1]}; {has_scale, s_i, [1]}; {has_bias, s_i, [1]}]
[Eltwise] | [add] | [2 1 1] | [s; r] | [e] | [{operation, s_i, [1]}]
[Activate] | [relu] | [1 1 1] | [e] | [e] | [{type, s_i, [1]}]
[Pooling] | [gap] | [1 1 2] | [e] | [p] | [{pool, s_i, [1]}; {global_pooling, s_i, [1]}]
[Flatten] | [flat] | [1 1 0] | [p] | [f] | []
[Softmax] | [prob] | [1 1 1] | [f] | [prob] | [{axis, s_i, [1]}]
"""


def network_forward(dev, reps=50):
    """Wall time of Network::Forward for a six-operator text model on
    [64,1024,14,14] with device inputs: two 51 MB device-to-device input copies,
    five launches, one stream synchronisation per call."""
    sa = dev.sa
    n = 64 * 1024 * 14 * 14
    x, r = dev.buf(normal(801, n)), dev.buf(normal(802, n))
    weights = [uniform(803, 1024, 0.5, 1.5), uniform(804, 1024, -0.1, 0.1)]
    with sa.Network(NETWORK_TEXT, weights, device_input=True) as net:
        for _ in range(5):
            net.forward({"x": x, "r": r})
        t0 = time.perf_counter()
        for _ in range(reps):
            net.forward({"x": x, "r": r})
        t1 = time.perf_counter()
    us = (t1 - t0) * 1e6 / reps
    moved = 4 * n * (2 * 2 + 3 + 3 + 2 + 1)  # input copies, scale, eltwise, relu, pooling read
    return {"model": "Scale -> Eltwise -> ReLU -> global avg Pooling -> Flatten -> Softmax, [64,1024,14,14]",
            "us_per_forward": round(us, 1), "operators": 6, "launches": 5, "input_copies": 2,
            "bytes_moved": moved, "GBps": round(moved / us / 1e3, 1)}


def main():
    args = parse()
    if args.gpus != 1:
        raise SystemExit("bench.py: this build measures one GPU; the path shards by batch with no "
                         "exchange, so run one process per GPU (got --gpus %d)" % args.gpus)
    dev = Dev()
    if args.probe:
        probe(dev)
        return
    if args.probe_next:
        probe_next(dev)
        return
    ms_per_step, step_bytes, n, roofline, detail, host = headline(dev, args.steps, args.warmup)
    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    out = {
        "metric": "achieved HBM GB/s (% of MI355X peak) per op; speedup vs host-CPU Shadow",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "BASELINE configs[1]: fp32 [64,256,56,56] ~N(0,2) seed 201; relu, "
                               "sigmoid, exp, abs, sqrt(abs), tanh as single ops + fused per-channel "
                               "Scale+ReLU (7 launches per step)",
                   "elements": n, "bytes_per_step": step_bytes, "device": dev.info},
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
        "elements_per_s": round(7 * n / (ms_per_step * 1e-3), 1),
        "roofline": roofline, "step_ops": detail,
        "step_ops_note": "per-op times from an untimed pass of the same K steps with events around every "
                         "launch; roofline.avg_us from events around the dominant kernel inside the timed region",
    }
    if not args.no_configs:
        out["configs"] = config_table(dev, args.operand_sets)
        out["network"] = network_forward(dev)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(host, step_bytes, args.cpu_passes)
        out["speedup_vs_cpu"] = round(value / out["cpu_baseline"]["value"], 1)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
