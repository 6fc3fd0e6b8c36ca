#!/usr/bin/env python3
"""Benchmark of the Shadow tensor hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-configs]

A "step" is one pass of the headline workload (BASELINE.json configs[1]): seven
launches over an fp32 [64,256,56,56] tensor -- Activate relu, sigmoid, tanh;
Unary exp, abs, sqrt(abs); Scale(per-channel gamma, beta)+ReLU in one launch.
Inputs are generated from fixed seeds, uploaded once and stay resident in HBM
(two copies of the input take turns, 411 MB, more than the 256 MB Infinity
Cache); the timed region is K steps between two stream synchronisations.

Prints ONE JSON line on stdout, under 4 KB (see final_record); every row of the
measurement goes to the --table file and, one short text line per row, to stderr.
`value` is algorithmic GB/s of the whole step
(compulsory reads + writes of every op / wall time).  `roofline` describes the
kernel that takes the largest share of the step, timed with HIP events on the
launch stream inside the timed region; its `bound` is "hbm" unless the kernel
takes over 10 % longer than a plain copy of the same tensor measured in the same
run, in which case it is "valu" and carries the instruction counters of the
profile summary.  `cpu_baseline` is the CPU oracle (a C port of the reference's
loops, one thread) timed on this host on the same buffers, outputs allocated
beforehand.  `configs` lists every op of the five BASELINE workloads measured
the same way (events around batches of launches that rotate over >256 MB of
buffers), each with the time of a plain copy / read / write of the same number
of bytes (`ceiling_us`, whichever matches the op's traffic) and, for the
BASELINE rows, the oracle's time on this host.
"""
import argparse
import ctypes
import itertools
import json
import os
import re
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published

# rocprofv3 summaries that `roofline` quotes (counters cannot be collected from
# inside this process): HBM bytes per launch of the headline kernels from
# FETCH_SIZE / WRITE_SIZE, and their VALU instruction counters.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "headline_unary_chain_hbm_counters.txt")
VALU_PROFILE = os.path.join(ROOT, "profiles", "headline_unary_chain_valu_counters.txt")
PROFILE_LABEL = {"activate_relu": "Activate relu", "activate_sigmoid": "Activate sigmoid",
                 "unary_exp": "Unary exp", "unary_abs": "Unary abs", "unary_sqrt_of_abs": "Unary sqrt",
                 "activate_tanh": "Activate tanh", "scale_relu_fused": "Scale+ReLU fused"}


def profile_rows(path):
    """{workload label: [columns...]} of a profiles/ table (columns two or more blanks apart)."""
    rows = {}
    if os.path.exists(path):
        for line in open(path):
            cols = re.split(r"\s{2,}", line.strip())
            if len(cols) >= 4:
                rows[cols[0]] = cols[1:]
    return rows


def measured_traffic(op):
    """HBM bytes per launch (reads + writes) from the counter summary, or None."""
    cols = profile_rows(TRAFFIC_PROFILE).get(PROFILE_LABEL.get(op, ""))
    try:
        return round((float(cols[3]) + float(cols[5])) * 1e6)  # read MB, write MB
    except (TypeError, IndexError, ValueError):
        return None


def measured_valu(op):
    """{"insts_per_element", "valu_busy"} from the VALU counter summary, or None."""
    cols = profile_rows(VALU_PROFILE).get(PROFILE_LABEL.get(op, ""))
    try:
        return {"insts_per_element": float(cols[-2]), "valu_busy": float(cols[-1])}
    except (TypeError, IndexError, ValueError):
        return None


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--no-configs", action="store_true", help="skip the per-config table")
    ap.add_argument("--cpu-passes", type=int, default=5)
    ap.add_argument("--operand-sets", type=int, default=1,
                    help="multiplier on the number of rotating operand sets of the config table")
    ap.add_argument("--single-input", action="store_true",
                    help="headline step on one input instead of two taking turns (A/B of the cache effect)")
    ap.add_argument("--probe", action="store_true",
                    help="counter probe: 3 launches of a plain copy and of every headline op on "
                         "the 51.4M tensor, nothing timed, no JSON (run under rocprofv3 --pmc)")
    ap.add_argument("--sweep", action="store_true",
                    help="time the operators over shapes off the benchmark's (short and long rows, thin and "
                         "small extents) against a plain copy of the same bytes, print a table, exit")
    ap.add_argument("--probe-next", action="store_true",
                    help="the same for the neighbouring operators and the data movers")
    ap.add_argument("--launch-shapes", action="store_true",
                    help="run tests/native/launch_shapes (alternative launch shapes of the streaming, strided-reduce "
                         "and channel-tile kernels), print its table and how the shapes in use compare, exit")
    ap.add_argument("--scaling", action="store_true",
                    help="time the BASELINE reductions, broadcasts and the bottleneck tail at 1x, 2x and 4x their batch "
                         "and fit time = fixed + bytes / rate per operator (what a launch costs before it streams), exit")
    ap.add_argument("--table", default=os.path.join(ROOT, "gpurun_out", "bench_table.json"),
                    help="file that receives every row of the measurement; the final stdout line is a short record")
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
def headline(dev, steps, warmup, single_input=False):
    lib, st = dev.lib, dev.stream
    shape = (64, 256, 56, 56)
    n = int(np.prod(shape))
    C, inner = shape[1], shape[2] * shape[3]
    x_h = normal(201, n, 2.0)
    g_h, b_h = uniform(202, C, 0.5, 1.5), uniform(203, C, -0.1, 0.1)
    g, b = dev.buf(g_h), dev.buf(b_h)
    # two resident copies of the input take turns step by step
    xs = [dev.buf(x_h)] if single_input else [dev.buf(x_h), dev.buf(x_h)]
    y = [dev.buf(nbytes=4 * n) for _ in range(2)]
    a = dev.buf(nbytes=4 * n)  # abs output, input of sqrt

    per_op = 8 * n
    ops = [
        ("activate_relu", per_op, lambda x, o: lib.shdw_hip_activate(1, 0.1, n, x.ptr, o.ptr, st)),
        ("activate_sigmoid", per_op, lambda x, o: lib.shdw_hip_activate(3, 0.1, n, x.ptr, o.ptr, st)),
        ("unary_exp", per_op, lambda x, o: lib.shdw_hip_unary(4, n, x.ptr, o.ptr, st)),
        ("unary_abs", per_op, lambda x, o: lib.shdw_hip_unary(0, n, x.ptr, a.ptr, st)),
        ("unary_sqrt_of_abs", per_op, lambda x, o: lib.shdw_hip_unary(2, n, a.ptr, o.ptr, st)),
        ("activate_tanh", per_op, lambda x, o: lib.shdw_hip_activate(5, 0.1, n, x.ptr, o.ptr, st)),
        ("scale_relu_fused", per_op + 8 * C,
         lambda x, o: lib.shdw_hip_scale_bias(n, C, inner, x.ptr, g.ptr, b.ptr, 1, o.ptr, st)),
    ]
    step_bytes = sum(nb for _, nb, _ in ops)

    def step(i, events=None, only=None):
        """events: one (start, stop) pair per op; only: record just around that op."""
        x = xs[i % len(xs)]
        for k, (_, _, fn) in enumerate(ops):
            marked = events is not None and (only is None or only == k)
            if marked:
                dev.record(events[k][0])
            dev.ck(fn(x, y[(i + k) & 1]))
            if marked:
                dev.record(events[k][1])

    for i in range(warmup):
        step(i)
    dev.sync()

    # Untimed pass with events around every launch: the per-op table, and which
    # kernel dominates.  Event records between launches cost ~2.5 us each, so the
    # timed region below carries them around the dominant kernel only.  A plain
    # copy of the same tensor, bracketed the same way, rides along as the yardstick.
    ev = [[(dev.event(), dev.event()) for _ in ops] for _ in range(steps)]
    cev = [(dev.event(), dev.event()) for _ in range(steps)]
    for i in range(steps):
        step(i, ev[i])
        dev.record(cev[i][0])
        dev.ck(lib.shdw_hip_copy(n, xs[i % len(xs)].ptr, y[i & 1].ptr, st))
        dev.record(cev[i][1])
    dev.sync()
    kernel_ms = []
    for k in range(len(ops)):
        kernel_ms.append(sum(dev.elapsed_ms(ev[i][k][0], ev[i][k][1]) for i in range(steps)) / steps)
    copy_ms = sum(dev.elapsed_ms(c0, c1) for c0, c1 in cev) / steps
    detail = []
    for (name, nb, _), ms in zip(ops, kernel_ms):
        gbs = nb / (ms * 1e-3) / 1e9
        detail.append({"op": name, "bytes": nb, "us": round(ms * 1e3, 2), "GBps": round(gbs, 1),
                       "frac": round(gbs / HBM_PEAK_GBS, 4), "vs_copy": round(ms / copy_ms, 3)})
    detail.append({"op": "plain_copy (yardstick, not part of the step)", "bytes": per_op,
                   "us": round(copy_ms * 1e3, 2), "GBps": round(per_op / (copy_ms * 1e-3) / 1e9, 1),
                   "frac": round(per_op / (copy_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "vs_copy": 1.0})
    dom = int(np.argmax(kernel_ms))

    t0 = time.perf_counter()
    for i in range(steps):
        step(i, ev[i], only=dom)
    dev.sync()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / steps
    vs_copy = kernel_ms[dom] / copy_ms  # both from the pass that brackets every launch
    kernel_ms[dom] = sum(dev.elapsed_ms(ev[i][dom][0], ev[i][dom][1]) for i in range(steps)) / steps
    dom_gbs = ops[dom][1] / (kernel_ms[dom] * 1e-3) / 1e9
    name = ops[dom][0]
    roofline = {"bound": "valu" if vs_copy > 1.10 else "hbm", "kernel": name, "achieved": round(dom_gbs, 1),
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(dom_gbs / HBM_PEAK_GBS, 4),
                "traffic": measured_traffic(name), "traffic_source": os.path.relpath(TRAFFIC_PROFILE, ROOT),
                "avg_us": round(kernel_ms[dom] * 1e3, 2), "algorithmic_bytes": ops[dom][1],
                "same_size_copy_us": round(copy_ms * 1e3, 2), "time_vs_same_size_copy": round(vs_copy, 3)}
    if roofline["bound"] == "valu":
        roofline["valu"] = measured_valu(name)
        roofline["valu_source"] = os.path.relpath(VALU_PROFILE, ROOT)
        roofline["note"] = ("achieved/peak/frac stay in HBM terms (algorithmic bytes / kernel time against 8 TB/s); "
                            "the kernel is held back by vector-ALU issue, not by memory")
    host = {"x": x_h, "gamma": g_h, "beta": b_h, "shape": shape}
    for bb in xs + y + [a, g, b]:
        bb.free()
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
    gy, gx = np.meshgrid(np.linspace(-1, 1, 56), np.linspace(-1, 1, 56), indexing="ij")
    warp = np.stack([gx, gy], -1).astype(np.float32)[None] + uniform(614, (64, 56, 56, 2), -0.05, 0.05)
    grid = dev.buf(np.ascontiguousarray(warp, np.float32).ravel())
    whole = I([64, C, 56, 56])
    for _ in range(3):
        dev.ck(lib.shdw_hip_copy(n, x.ptr, y.ptr, st))
        dev.ck(lib.shdw_hip_grid_sample(whole, whole, 1, 0, x.ptr, grid.ptr, y.ptr, st))
        dev.ck(lib.shdw_hip_batch_norm(n, C, inner, x.ptr, b.ptr, g.ptr, 1.0, 1e-5, y.ptr, st))
        dev.ck(lib.shdw_hip_batch_norm_scale(n, C, inner, x.ptr, b.ptr, g.ptr, 1.0, 1e-5, g.ptr, b.ptr, 1, y.ptr, st))
        dev.ck(lib.shdw_hip_lrn(I([64, C, 56, 56]), 5, 1e-4, 0.75, 1.0, x.ptr, y.ptr, st))
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


def sweep(dev):
    """Shapes off the benchmark's: every line is one operator on about 51 MB with the
    time of a plain copy (51 MB read + 51 MB written) scaled to the bytes the operator
    has to move, so 1.0 means the speed of a copy.  Prints the worst ratio of each
    family (operators that share a set of kernels) at the end."""
    lib, st = dev.lib, dev.stream
    I = dev.sa.ints
    SETS, N = 4, 12845056
    X = [dev.buf(normal(11 + k, N, 2.0)) for k in range(SETS)]
    Y = [dev.buf(nbytes=4 * N) for _ in range(SETS)]
    P, Q = dev.buf(uniform(5, N, 0.5, 1.5)), dev.buf(uniform(6, N, -0.5, 0.5))
    scratch = dev.buf(nbytes=64 << 20)
    tm = lambda fn: time_median(dev, fn, SETS, reps=20) * 1e3
    t_copy = tm(lambda k: lib.shdw_hip_copy(N, X[k].ptr, Y[k].ptr, st))
    print("plain copy of 12,845,056 floats (51 MB read, 51 MB written): %.2f us" % t_copy)
    worst = {}

    def show(family, name, us, nbytes):
        ratio = us / (t_copy * nbytes / (8.0 * N))
        worst[family] = max(worst.get(family, (0.0, "")), (ratio, name))
        print("%-14s %-58s %9.2f us  %6.2f x copy" % (family, name, us, ratio), flush=True)

    for L in (1, 2, 3, 4, 5, 8, 9, 12, 16, 17, 49, 64, 65, 127, 128, 129, 196, 255, 256, 257, 512, 784, 1024, 3136,
              4097, 12544, 50176, 200000, 12845056):
        rows = N // L
        for kind, shape, axes in (("reduce rows", [rows, L], [1]), ("reduce strided", [L, rows], [0])):
            need = lib.shdw_hip_reduce_workspace_bytes(2, I(shape), 1, I(axes))
            assert need <= (64 << 20)
            for op, nm in ((1, "sum"), (2, "max")):
                us = tm(lambda k: lib.shdw_hip_reduce(op, 2, I(shape), 1, I(axes), X[k].ptr, Y[k].ptr,
                                                      scratch.ptr if need else None, need, st))
                show(kind, "%s over %d of [%s]" % (nm, L, "x".join(map(str, shape))), us, 4 * (rows * L + rows))
    for shape in ([64, 256, 28, 28], [256, 1024, 7, 7], [8, 3, 732, 731]):
        n = int(np.prod(shape))
        assert n <= N
        for r in (1, 2, 3):
            for axes in itertools.combinations(range(4), r):
                axes = list(axes)
                need = lib.shdw_hip_reduce_workspace_bytes(4, I(shape), r, I(axes))
                assert need <= (64 << 20)
                outs = n // int(np.prod([shape[a] for a in axes]))
                for op, nm in ((1, "sum"), (2, "max")):
                    us = tm(lambda k: lib.shdw_hip_reduce(op, 4, I(shape), r, I(axes), X[k].ptr, Y[k].ptr,
                                                          scratch.ptr if need else None, need, st))
                    show("reduce axes", "%s of %s over axes %s" % (nm, shape, axes), us, 4 * (n + outs))
    for which in ("softmax", "normalize"):
        for dim in (2, 8, 21, 49, 64, 65, 150, 256, 512, 513, 1000, 4096):
            for inner in (1, 2, 7, 16, 49, 196, 3136):
                if dim * inner > N:
                    continue
                outer = N // (dim * inner)
                n = outer * dim * inner
                if which == "softmax":
                    us = tm(lambda k: lib.shdw_hip_softmax(outer, dim, inner, X[k].ptr, Y[k].ptr, st))
                else:
                    us = tm(lambda k: lib.shdw_hip_normalize(outer, dim, inner, 2.0, 1e-12, X[k].ptr, Y[k].ptr, st))
                show(which, "[%d,%d,%d]" % (outer, dim, inner), us, 8 * n)
    for inner in (1, 2, 4, 8, 16, 17, 49, 196, 256, 257, 784, 3136, 12544, 50176, 400000, 12845056):
        outer = N // inner
        need = lib.shdw_hip_group_norm_workspace_bytes(outer, inner)
        assert need <= (64 << 20)
        us = tm(lambda k: lib.shdw_hip_group_norm_ws(outer, inner, 1e-5, X[k].ptr, None, None, 1, 1, Y[k].ptr,
                                                     scratch.ptr if need else None, need, st))
        show("row norm", "[%d,%d]%s" % (outer, inner, " (sliced rows)" if need else ""), us, 8 * outer * inner)
    for shape, k, s, p in (([16, 64, 112, 112], 3, 2, 1), ([16, 64, 112, 112], 2, 2, 0), ([16, 64, 112, 112], 3, 1, 1),
                           ([64, 1024, 14, 14], 2, 2, 0), ([64, 1024, 14, 14], 3, 1, 1), ([128, 2048, 7, 7], 3, 1, 1),
                           ([512, 512, 7, 7], 7, 1, 3), ([64, 1024, 14, 14], 13, 1, 6), ([16, 64, 112, 112], 5, 1, 2),
                           ([64, 512, 19, 19], 9, 1, 4), ([19, 1000, 26, 26], 5, 1, 2), ([19, 1000, 26, 26], 13, 1, 6)):
        n_, c_, h_, w_ = shape
        oh, ow = (h_ + 2 * p - k) // s + 1, (w_ + 2 * p - k) // s + 1
        for pt, nm in ((0, "max"), (1, "avg")):
            us = tm(lambda kk: lib.shdw_hip_pooling2d(I(shape), pt, k, k, s, s, p, p, I([n_, c_, oh, ow]), X[kk].ptr,
                                                      Y[kk].ptr, st))
            show("pooling", "%s %dx%d s%d p%d on %s" % (nm, k, k, s, p, shape), us, 4 * (n_ * c_ * (h_ * w_ + oh * ow)))
    for side in (3, 7, 14, 28, 56):
        rows = N // (side * side)
        shape = [rows // 64, 64, side, side]
        for pt, nm in ((0, "max"), (1, "avg")):
            us = tm(lambda kk: lib.shdw_hip_pooling2d(I(shape), pt, side, side, 1, 1, 0, 0, I(shape[:2] + [1, 1]),
                                                      X[kk].ptr, Y[kk].ptr, st))
            show("global pool", "%s over %dx%d planes of %s" % (nm, side, side, shape), us,
                 4 * shape[0] * 64 * (side * side + 1))
    for a, b in (([64, 256, 28, 28], [1, 256, 1, 1]), ([64, 256, 28, 28], [64, 256, 1, 1]),
                 ([64, 256, 28, 28], [1, 1, 28, 28]), ([64, 256, 28, 28], [1, 1, 1, 28]),
                 ([64, 256, 28, 28], [64, 1, 28, 28]), ([64, 256, 28, 28], [1, 256, 28, 1]),
                 ([64, 256, 28, 28], [1, 1, 1, 1]), ([1792, 7168], [1792, 1]), ([1792, 7168], [1, 7168]),
                 ([4096, 49, 64], [4096, 1, 64]), ([4096, 49, 64], [1, 49, 1]), ([200704, 8, 8], [200704, 1, 8]),
                 ([200704, 8, 8], [200704, 8, 1]), ([262144, 7, 7], [262144, 1, 1]), ([4281685, 3], [1, 3]),
                 ([64, 256, 1, 28], [64, 1, 28, 28]), ([4, 4, 7, 8, 14, 8, 16, 7], [1, 4, 1, 8, 1, 8, 1, 7])):
        out = [max(p_, q_) for p_, q_ in zip(a, b)]
        n, na, nb = int(np.prod(out)), int(np.prod(a)), int(np.prod(b))
        assert n <= N and na <= N and nb <= N
        for op, nm in ((0, "add"), (3, "div")):
            us = tm(lambda k: lib.shdw_hip_broadcast_binary(op, len(out), I(a), I(b), I(out), X[k].ptr, P.ptr,
                                                            Y[k].ptr, st))
            show("broadcast", "%s %s with %s" % (nm, a, b), us, 4 * (na + nb + n))
    for inner in (1, 2, 3, 4):
        for num in (3, 64, 1000):
            n = (N // (num * inner)) * num * inner
            us = tm(lambda k: lib.shdw_hip_scale_bias(n, num, inner, X[k].ptr, P.ptr, Q.ptr, 0, Y[k].ptr, st))
            show("scale", "%d parameters, inner %d" % (num, inner), us, 8 * n)
    for shape, order in (([N // 3, 3], [1, 0]), ([3, N // 3], [1, 0]), ([16, 224, 224, 16], [0, 3, 1, 2]),
                         ([64, 256, 28, 28], [0, 2, 3, 1]), ([8, 3, 85, 76, 76], [0, 1, 3, 4, 2])):
        n = int(np.prod(shape))
        us = tm(lambda k: lib.shdw_hip_permute(len(shape), I(shape), I(order), X[k].ptr, Y[k].ptr, st))
        show("permute", "%s order %s" % (shape, order), us, 8 * n)
    # the channel-parameter operators at row lengths that are and are not whole vectors
    for inner in (1, 2, 3, 7, 16, 49, 196, 3136):
        for ch in (3, 64, 1000):
            n = (N // (ch * inner)) * ch * inner
            us = tm(lambda k: lib.shdw_hip_batch_norm(n, ch, inner, X[k].ptr, Q.ptr, P.ptr, 1.0, 1e-5, Y[k].ptr, st))
            show("batch norm", "%d channels, inner %d" % (ch, inner), us, 8 * n)
            us = tm(lambda k: lib.shdw_hip_prelu(n, ch, inner, 0, X[k].ptr, P.ptr, Y[k].ptr, st))
            show("prelu", "%d channels, inner %d" % (ch, inner), us, 8 * n)
    for inner in (1, 3, 16, 49, 196, 3136, 50176):
        rows = N // inner
        us = tm(lambda k: lib.shdw_hip_axpy_rows(rows, inner, P.ptr, X[k].ptr, X[(k + 1) % SETS].ptr, Y[k].ptr, st))
        show("axpy rows", "[%d,%d]" % (rows, inner), us, 12 * rows * inner + 4 * rows)
    for k_in in (2, 3, 5):
        m = N // 2
        ptrs = (ctypes.c_void_p * k_in)(*[X[j % SETS].ptr + (4 * m if j >= SETS else 0) for j in range(k_in)])
        for op, nm in ((0, "prod"), (1, "sum"), (2, "max")):
            coeff = (ctypes.c_float * k_in)(*[0.5 + 0.25 * j for j in range(k_in)]) if op == 1 else None
            us = tm(lambda k: lib.shdw_hip_eltwise(op, k_in, ptrs, coeff, m, Y[k].ptr, st))
            show("eltwise", "%s of %d inputs" % (nm, k_in), us, 4 * m * (k_in + 1))
    # Concat / Slice / Stack chunks: rows of `chunk` floats copied into rows of a different pitch
    for chunk, dst_pitch, off in ((1, 2, 1), (3, 7, 2), (49, 98, 49), (100, 300, 100), (3136, 6272, 3136), (12544, 12545, 1),
                                  (401408, 802816, 0), (200704 * 3, 200704 * 4, 200704)):
        outer = min(N // chunk, N // dst_pitch)
        us = tm(lambda k: lib.shdw_hip_copy_chunks(outer, chunk, X[k].ptr, chunk, 0, Y[k].ptr, dst_pitch, off, st))
        show("copy chunks", "%d chunks of %d into rows of %d at %d (concat)" % (outer, chunk, dst_pitch, off), us, 8 * outer * chunk)
        us = tm(lambda k: lib.shdw_hip_copy_chunks(outer, chunk, X[k].ptr, dst_pitch, off, Y[k].ptr, chunk, 0, st))
        show("copy chunks", "%d chunks of %d out of rows of %d at %d (slice)" % (outer, chunk, dst_pitch, off), us, 8 * outer * chunk)
    for shape, pads in (([64, 64, 54, 54], [1, 1, 1, 1]), ([64, 64, 50, 50], [3, 3, 3, 3]), ([256, 64, 27, 27], [0, 1, 0, 1]),
                        ([64, 64, 56, 56], [-1, -1, -1, -1]), ([2400, 64, 7, 7], [1, 1, 1, 1]), ([16, 3, 500, 501], [2, 1, 3, 0])):
        n_in = int(np.prod(shape))
        n_out = shape[0] * shape[1] * (shape[2] + pads[0] + pads[1]) * (shape[3] + pads[2] + pads[3])
        assert n_in <= N and n_out <= N
        us = tm(lambda k: lib.shdw_hip_pad(I(shape), I(pads), 0.5, X[k].ptr, Y[k].ptr, st))
        show("pad", "%s by %s" % (shape, pads), us, 4 * (min(n_in, n_out) + n_out))
    for shape, out_hw in (([64, 64, 28, 28], (56, 56)), ([64, 64, 28, 28], (55, 57)), ([64, 64, 56, 56], (28, 28)),
                          ([16, 3, 300, 300], (513, 513)), ([256, 256, 7, 7], (14, 14)), ([8, 255, 19, 19], (76, 76)),
                          ([4, 3, 720, 1280], (360, 640))):
        out = shape[:2] + list(out_hw)
        n_in, n_out = int(np.prod(shape)), int(np.prod(out))
        assert n_in <= N and n_out <= N
        for typ, nm in ((0, "nearest"), (1, "bilinear")):
            us = tm(lambda k: lib.shdw_hip_resize(I(shape), I(out), typ, 0, X[k].ptr, Y[k].ptr, st))
            show("resize", "%s %s -> %dx%d" % (nm, shape, out_hw[0], out_hw[1]), us, 4 * (min(n_in, 4 * n_out) + n_out))
    # GridSample: the grid of the cell centres warped by up to 1.4 cells, and positions drawn at random inside the input
    for shape in ([16, 256, 56, 56], [64, 64, 56, 56], [1024, 256, 7, 7], [4, 3, 1024, 1024]):
        b, c, h, w = shape
        gy, gx = np.meshgrid(np.linspace(-1, 1, h), np.linspace(-1, 1, w), indexing="ij")
        centres = np.stack([gx, gy], -1).astype(np.float32)[None]
        grids = (("warped identity", dev.buf(np.ascontiguousarray(centres + uniform(31, (b, h, w, 2), -2.8 / h, 2.8 / h)).ravel())),
                 ("random positions", dev.buf(uniform(32, b * h * w * 2, -1.0, 1.0))))
        for what, g in grids:
            for mode, nm in ((0, "nearest"), (1, "bilinear")):
                us = tm(lambda k: lib.shdw_hip_grid_sample(I(shape), I(shape), mode, 0, X[k].ptr, g.ptr, Y[k].ptr, st))
                show("grid sample", "%s %s, %s" % (nm, shape, what), us, 8 * b * c * h * w + 8 * b * h * w)
        for _, g in grids:
            g.free()
    # LRN: the window in registers (3, 5, 7) and in LDS (9, 15), few and many channels
    for shape, size in (([16, 256, 56, 56], 5), ([16, 256, 56, 56], 3), ([16, 256, 56, 56], 9), ([44, 96, 55, 55], 5),
                        ([68, 256, 27, 27], 5), ([1024, 256, 7, 7], 5), ([256, 256, 14, 14], 15), ([64, 8, 158, 158], 7)):
        n = int(np.prod(shape))
        assert n <= N
        us = tm(lambda k: lib.shdw_hip_lrn(I(shape), size, 1e-4, 0.75, 1.0, X[k].ptr, Y[k].ptr, st))
        show("lrn", "window %d on %s" % (size, shape), us, 8 * n)
    for shape, stride in (([64, 64, 56, 56], 2), ([138, 64, 38, 38], 2), ([64, 16, 112, 112], 4), ([36, 512, 26, 26], 2)):
        n = int(np.prod(shape))
        for typ, nm in ((0, "darknet"), (1, "natural")):
            us = tm(lambda k: lib.shdw_hip_reorg(I(shape), typ, stride, X[k].ptr, Y[k].ptr, st))
            show("reorg", "%s %s stride %d" % (nm, shape, stride), us, 8 * n)
    for batch, ch, sp, group in ((64, 256, 784, 2), (1120, 232, 49, 2), (15000, 116, 7, 4), (8, 480, 3136, 3), (50176, 256, 1, 8)):
        n = batch * ch * sp
        assert n <= N
        us = tm(lambda k: lib.shdw_hip_shuffle_channel(batch, ch, sp, group, X[k].ptr, Y[k].ptr, st))
        show("shuffle", "[%d,%d,%d] in %d groups" % (batch, ch, sp, group), us, 8 * n)
    idx_host = np.arange(0, 1000, 3, dtype=np.int32)
    idx = dev.buf(idx_host.view(np.float32))
    for outer, inner in ((12, 1000), (1, 12845), (12845, 1), (256, 49), (3000, 4)):
        us = tm(lambda k: lib.shdw_hip_gather(outer, 1000, inner, idx_host.size, idx.ptr, X[k].ptr, Y[k].ptr, st))
        show("gather", "%d of 1000 rows of %d, %d times" % (idx_host.size, inner, outer), us, 8 * outer * idx_host.size * inner)
    print("worst of each family:")
    for family, (ratio, name) in worst.items():
        print("  %-14s %6.2f x copy  (%s)" % (family, ratio, name))


def scaling(dev):
    """Each BASELINE operator whose tensor is 25-70 MB at 1x, 2x and 4x its batch (the leading
    extent), operands rotating through 1.2 GB pools, with a plain read / write / copy of the
    same bytes beside it.  A least-squares line time = fixed + bytes / rate through the three
    points separates what a launch costs before and after it streams (ramp, the last
    workgroups, a dependent second launch) from the rate it streams at."""
    lib, st = dev.lib, dev.stream
    I = dev.sa.ints
    POOL = 6 * 205520896
    rp, wp = dev.buf(nbytes=POOL), dev.buf(nbytes=POOL)
    seed = dev.buf(normal(999, 12845056))
    piece = 4 * 12845056
    for k in range(POOL // piece):
        dev.ck(lib.shdw_hip_memcpy_d2d(rp.ptr + k * piece, seed.ptr, piece, st))
    dev.sync()
    seed.free()
    small = dev.buf(uniform(5, 1 << 20, 0.5, 2.0))
    ws = dev.buf(nbytes=64 << 20)
    sink = dev.buf(nbytes=256)

    def reduce_case(op, shape, axes):
        def make(m):
            shp = [shape[0] * m] + shape[1:]
            n = int(np.prod(shp))
            outs = n // int(np.prod([shp[a] for a in axes]))
            need = lib.shdw_hip_reduce_workspace_bytes(len(shp), I(shp), len(axes), I(axes))
            assert need <= (64 << 20)
            sets = POOL // (4 * n)
            fn = lambda k: lib.shdw_hip_reduce(op, len(shp), I(shp), len(axes), I(axes), rp.ptr + k * 4 * n,
                                               wp.ptr + k * 4 * outs, ws.ptr if need else None, need, st)
            return fn, sets, 4 * n, 4 * outs
        return make

    def bcast_case(op, sa, sb):
        def make(m):
            a_shape, b_shape = [sa[0] * m] + sa[1:], list(sb)
            out = [max(p, q) for p, q in zip(a_shape, b_shape)]
            na, nb, no = int(np.prod(a_shape)), int(np.prod(b_shape)), int(np.prod(out))
            sets = POOL // (4 * no)
            ia, ib, io = I(a_shape), I(b_shape), I(out)
            fn = lambda k: lib.shdw_hip_broadcast_binary(op, len(out), ia, ib, io, rp.ptr, small.ptr, wp.ptr + k * 4 * no, st)
            return fn, sets, 4 * (na + nb), 4 * no
        return make

    def tail_case(m):
        n, C, inner = 12845056 * m, 1024, 196
        sets = POOL // (4 * n) - 1
        fn = lambda k: lib.shdw_hip_scale_residual_relu_rowmean(n, C, inner, rp.ptr + k * 4 * n, small.ptr, small.ptr + 4096,
                                                                 rp.ptr + (k + 1) * 4 * n, wp.ptr + k * 4 * n,
                                                                 ws.ptr, st)
        return fn, sets, 8 * n + 8 * C, 4 * n + 4 * (n // inner)

    def plain(kind):
        def make(m, nbytes):
            per_side = nbytes // 2 if kind == "copy" else nbytes
            n = per_side // 4
            sets = max(1, POOL // (4 * n))
            if kind == "copy":
                return (lambda k: lib.shdw_hip_copy(n, rp.ptr + k * 4 * n, wp.ptr + k * 4 * n, st)), sets
            if kind == "read":
                return (lambda k: lib.shdw_hip_probe_read(n, rp.ptr + k * 4 * n, 1e30, sink.ptr, st)), sets
            return (lambda k: lib.shdw_hip_set(n, 1.0, wp.ptr + k * 4 * n, st)), sets
        return make

    cases = [("cfg3 reduce sum {2,3} [32m,512,28,28]", reduce_case(1, [32, 512, 28, 28], [2, 3]), "read"),
             ("cfg3 reduce max {1} [32m,512,28,28]", reduce_case(2, [32, 512, 28, 28], [1]), "read"),
             ("cfg3 reduce sum {1} [32m,512,28,28]", reduce_case(1, [32, 512, 28, 28], [1]), "read"),
             ("cfg3 reduce sum all [32m,512,28,28] (2 launches)", reduce_case(1, [32, 512, 28, 28], [0, 1, 2, 3]), "read"),
             ("cfg5 reduce avg {2,3} [64m,1024,14,14]", reduce_case(4, [64, 1024, 14, 14], [2, 3]), "read"),
             ("cfg5 fused tail [64m,1024,14,14]", tail_case, "copy"),
             ("cfg1 add [8m,64,112,112] + [1,64,1,1]", bcast_case(0, [8, 64, 112, 112], [1, 64, 1, 1]), "copy"),
             ("cfg4(i) mul [16m,1,128,256] x [1,32,128,1]", bcast_case(2, [16, 1, 128, 256], [1, 32, 128, 1]), "write"),
             ("cfg4(i) div", bcast_case(3, [16, 1, 128, 256], [1, 32, 128, 1]), "write"),
             ("cfg4(ii) mul [4m,64,1,512] x [1,1,64,512]", bcast_case(2, [4, 64, 1, 512], [1, 1, 64, 512]), "write")]

    def fit(points):  # [(bytes, us)] -> fixed us, GB/s
        b = np.array([p[0] for p in points], np.float64)
        t = np.array([p[1] for p in points], np.float64)
        slope, fixed = np.polyfit(b, t, 1)
        return fixed, 1e-3 / slope

    print("%-52s %27s %27s %27s   %s" % ("operator (m = 1, 2, 4)", "bytes", "us", "us of a plain pass", "fit: fixed us + bytes / GB/s"))
    for name, make, kind in cases:
        mine, yard, sizes = [], [], []
        for m in (1, 2, 4):
            fn, sets, rd, wr = make(m)
            us = time_median(dev, fn, max(1, sets), reps=20) * 1e3
            pfn, psets = plain(kind)(m, rd + wr)
            pus = time_median(dev, pfn, psets, reps=20) * 1e3
            mine.append((rd + wr, us)), yard.append((rd + wr, pus)), sizes.append(rd + wr)
        f0, r0 = fit(mine)
        f1, r1 = fit(yard)
        print("%-52s %27s %27s %27s   %.2f us + bytes / %.0f GB/s   (plain %s: %.2f us + bytes / %.0f GB/s)" % (
            name, " ".join("%d" % b for b in sizes), " ".join("%7.2f" % p[1] for p in mine),
            " ".join("%7.2f" % p[1] for p in yard), f0, r0, kind, f1, r1), flush=True)
    for b in (rp, wp, small, ws, sink):
        b.free()


def launch_shapes():
    """Timing comparison of the launch shapes the library uses against their alternatives
    (tests/native/launch_shapes.hip).  A report, not a gate: each line ends in `ok` or `BEHIND`."""
    import subprocess
    exe = os.path.join(ROOT, "tests", "native", "launch_shapes")
    if not os.path.exists(exe):
        raise SystemExit("bench.py: tests/native/launch_shapes is not built; run `python -m tests.native.build`")
    out = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    print(out.stdout)
    if out.returncode != 0:
        raise SystemExit("bench.py: launch_shapes exited with %d" % out.returncode)
    table, slack = out.stdout, 1.12

    def verdict(what, mine, best, bound):
        print("%-72s %8.2f vs %8.2f  %s" % (what, mine, best, "ok" if mine <= bound * best else "BEHIND"))

    # elementwise kernels: single waves, one vector per lane; Blas::Set: 256 lanes; the read probe: 1024 lanes
    used = {"copy": "T64x1", "write": "T256x1", "read": "T1024x1"}
    for m in re.finditer(r"stream (\w+)\s+(\d+) MB:(.*)", table):
        row = {k: float(v) for k, v in re.findall(r"(\S+x\d) (\d+\.\d+)", m.group(3))}
        if m.group(1) in used and row:
            verdict("stream %s %s MB, %s against the best of %d shapes (us)" % (m.group(1), m.group(2), used[m.group(1)],
                                                                              len(row)), row[used[m.group(1)]],
                    min(row.values()), slack)
    t = {(int(l), kind): float(us) for l, kind, us, _ in re.findall(r"strided L(\d+)\s+(\S+)\s+(\d+\.\d+) (\w+)", table)}
    if (32, "xcd-contiguous") in t:
        verdict("strided reduce, 32-wide tiles numbered XCD-contiguously against the best (us)",
                t[(32, "xcd-contiguous")], min(t.values()), slack)
    flat, rows = {}, {}
    for line in table.splitlines():
        m = re.match(r"tile \[(\d+),(\d+),(\d+)\] flat (\d+\.\d+)", line)
        if m:
            flat[int(m.group(3))] = float(m.group(4))
        m = re.match(r"tile \[(\d+),(\d+),(\d+)\] (T\d+x\d+) (\w+)\s+(\w+)\s+(\d+\.\d+) (\w+)", line)
        if m:
            rows[(int(m.group(3)), m.group(4), m.group(5), m.group(6))] = float(m.group(7))
    for inner, shape in ((3136, ("T256x16", "streaming", "parked")), (1444, ("T256x16", "plain", "parked"))):
        mine = {k[1:]: v for k, v in rows.items() if k[0] == inner}
        if shape in mine:
            verdict("channel tile, rows of %d: %s against the best variant (us)" % (inner, " ".join(shape)),
                    mine[shape], min(mine.values()), slack)
            print("%-72s %8.2f vs %8.2f" % ("  the pattern against a flat copy of the same bytes (us)",
                                            min(mine.values()), flat.get(inner, float("nan"))))
    chains = {(int(w), int(c)): (float(a), float(b))
              for w, c, a, b in re.findall(r"add chain waves (\d+) chains (\d+): (\d+\.\d+) (\d+\.\d+)", table)}
    if (1, 1) in chains and (8, 1) in chains:
        print("%-72s %8.2f vs %8.2f" % ("one dependent add chain alone on a SIMD against eight waves sharing it",
                                        chains[(1, 1)][0], chains[(8, 1)][1]))


# ------------------------------------------------------------- CPU baseline
class Cpu:
    """The oracle's C functions called directly on arrays allocated beforehand, so
    that only the operator's work is timed (the reference's blobs are grow-only
    and resident), one thread.  best / median of `runs` calls."""

    def __init__(self, runs):
        import oracle
        self.o = oracle
        self.lib = oracle.lib()
        self.runs = runs
        self.f32p = ctypes.POINTER(ctypes.c_float)

    def p(self, a):
        return a.ctypes.data_as(self.f32p)

    def ints(self, v):
        return (ctypes.c_int * max(1, len(v)))(*[int(x) for x in v])

    def time(self, fn):
        fn()  # pages of the outputs are touched before anything is timed
        ts = []
        for _ in range(self.runs):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        ts.sort()
        return ts[0], ts[len(ts) // 2]

    # --- the operator bodies (reference lines in oracle/shadow_cpu.c) ---
    def activate(self, x, y, kind):
        return lambda: self.lib.orc_activate(self.p(x), self.p(y), x.size, kind, ctypes.c_float(0.1))

    def unary(self, x, y, op):
        return lambda: self.lib.orc_unary(op, x.size, self.p(x), self.p(y))

    def scale_bias(self, x, g, b, num, inner, y):
        return lambda: self.lib.orc_scale_bias(self.p(x), x.size, self.p(g), self.p(b), num, inner, self.p(y))

    def broadcast(self, op, a, sa, b, sb, so, y):
        return lambda: self.lib.orc_broadcast_binary(self.p(a), self.ints(sa), self.p(b), self.ints(sb), op,
                                                     len(so), y.size, self.ints(so), self.p(y))

    def binary_scalar(self, op, a, alpha, y):
        return lambda: self.lib.orc_binary_scalar(op, a.size, self.p(a), ctypes.c_float(alpha), self.p(y))

    def eltwise_sum(self, xs, y):
        ptrs = (self.f32p * len(xs))(*[self.p(x) for x in xs])
        co = np.ones(len(xs), np.float32)
        return lambda: self.lib.orc_eltwise(1, len(xs), ptrs, self.p(co), y.size, self.p(y))

    def reduce(self, op, x, shape, axes, y):
        """Vision::Reduce on index lists built beforehand: the reference keeps them
        while the input shape is unchanged (kernels/reduce.hpp:45)."""
        window = int(np.prod([shape[a] for a in axes])) if axes else 1
        lst, off = np.empty(window, np.int32), np.empty(y.size, np.int32)
        i32p = ctypes.POINTER(ctypes.c_int)
        num_list = self.lib.orc_reduce_lists(self.ints(shape), len(shape), self.ints(axes), len(axes),
                                             lst.ctypes.data_as(i32p), off.ctypes.data_as(i32p))
        assert num_list == window
        keep = (lst, off)
        return lambda: self.lib.orc_vision_reduce(self.p(x), keep[0].ctypes.data_as(i32p),
                                                  keep[1].ctypes.data_as(i32p), num_list, op, y.size, self.p(y))


def cpu_headline(cpu, host, step_bytes):
    """The same seven results as the step, with Scale and ReLU as the two separate
    operators the reference runs; per-op and whole-step times."""
    x, g, b = host["x"], host["gamma"], host["beta"]
    C, inner = host["shape"][1], host["shape"][2] * host["shape"][3]
    y, a = np.empty_like(x), np.empty_like(x)
    legs = [("activate_relu", [cpu.activate(x, y, 1)]), ("activate_sigmoid", [cpu.activate(x, y, 3)]),
            ("unary_exp", [cpu.unary(x, y, 4)]), ("unary_abs", [cpu.unary(x, a, 0)]),
            ("unary_sqrt_of_abs", [cpu.unary(a, y, 2)]), ("activate_tanh", [cpu.activate(x, y, 5)]),
            ("scale_relu_fused", [cpu.scale_bias(x, g, b, C, inner, y), cpu.activate(y, y, 1)])]
    for _, fns in legs:
        for fn in fns:
            fn()
    per_op = {name: [] for name, _ in legs}
    totals = []
    for _ in range(cpu.runs):
        total = 0.0
        for name, fns in legs:
            t0 = time.perf_counter()
            for fn in fns:
                fn()
            dt = time.perf_counter() - t0
            per_op[name].append(dt)
            total += dt
        totals.append(total)
    best = min(totals)
    ops = {name: {"best_us": round(min(v) * 1e6, 1), "median_us": round(sorted(v)[len(v) // 2] * 1e6, 1)}
           for name, v in per_op.items()}
    return {"value": round(step_bytes / best / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "%d full passes of the same step on the same buffers (51.4M elements, 8 operator runs "
                      "each, outputs allocated beforehand), best pass %.2f s; host: %s, %d logical CPUs" % (
                          cpu.runs, best, cpu_model(), os.cpu_count() or 0),
            "seconds_per_step": round(best, 3), "ops": ops}


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown CPU"


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


def time_median(dev, launch, sets, reps=40):
    """Median of three batches."""
    return sorted(time_batch(dev, launch, sets, reps) for _ in range(3))[1]


class Ceilings:
    """Plain copy / read-only / write-only passes over a given number of bytes, in the
    launch shape of the elementwise kernels, rotating through 1.2 GB pools."""
    POOL = 6 * 205520896

    def __init__(self, dev):
        self.dev = dev
        self.rp, self.wp = dev.buf(nbytes=self.POOL), dev.buf(nbytes=self.POOL)
        seed = dev.buf(normal(999, 12845056))
        piece = 4 * 12845056
        for k in range(self.POOL // piece):
            dev.ck(dev.lib.shdw_hip_memcpy_d2d(self.rp.ptr + k * piece, seed.ptr, piece, dev.stream))
        dev.sync()
        seed.free()
        self.sink = dev.buf(nbytes=256)
        self.cache = {}

    def us(self, kind, nbytes):
        key = (kind, nbytes)
        if key in self.cache:
            return self.cache[key]
        dev, lib, st = self.dev, self.dev.lib, self.dev.stream
        per_side = nbytes // 2 if kind == "copy" else nbytes
        n = max(4, per_side // 4)
        m = max(1, min(64, self.POOL // (4 * n)))
        rp, wp, sink = self.rp.ptr, self.wp.ptr, self.sink.ptr
        if kind == "copy":
            fn = lambda k: lib.shdw_hip_copy(n, rp + k * 4 * n, wp + k * 4 * n, st)
        elif kind == "read":
            fn = lambda k: lib.shdw_hip_probe_read(n, rp + k * 4 * n, 1e30, sink, st)
        else:
            fn = lambda k: lib.shdw_hip_set(n, 1.0, wp + k * 4 * n, st)
        self.cache[key] = time_median(dev, fn, m) * 1e3
        return self.cache[key]

    def free(self):
        for b in (self.rp, self.wp, self.sink):
            b.free()


def traffic_kind(read_bytes, write_bytes):
    if read_bytes >= 4 * write_bytes:
        return "read"
    if write_bytes >= 4 * read_bytes:
        return "write"
    return "copy"


def config_table(dev, sets_scale=1, cpu=None):
    lib, st = dev.lib, dev.stream
    I = dev.sa.ints
    rows = []
    ceil = Ceilings(dev)

    def add(cfg, name, rd, wr, ms, elems, cpu_fn=None):
        nbytes = rd + wr
        gbs = nbytes / (ms * 1e-3) / 1e9
        kind = traffic_kind(rd, wr)
        cus = ceil.us(kind, nbytes)
        row = {"cfg": cfg, "op": name, "bytes": nbytes, "us": round(ms * 1e3, 2),
               "GBps": round(gbs, 1), "frac": round(gbs / HBM_PEAK_GBS, 4),
               "Gelem_s": round(elems / (ms * 1e-3) / 1e9, 2),
               "ceiling": kind, "ceiling_us": round(cus, 2), "frac_of_ceiling": round(cus / (ms * 1e3), 3)}
        if cpu is not None and cpu_fn is not None:
            best, med = cpu.time(cpu_fn)
            row.update({"cpu_us": round(best * 1e6, 1), "cpu_median_us": round(med * 1e6, 1),
                        "cpu_GBps": round(nbytes / best / 1e9, 3), "speedup_vs_cpu": round(best * 1e3 / ms, 1)})
        rows.append(row)

    SETS = 6 * sets_scale  # 6 x (in + out) of 51 MB each: more than the 256 MB Infinity Cache
    NBIG = 12845056  # elements of the cfg-3 and cfg-5 tensors (51.4 MB)
    A = [dev.buf(normal(301 + 10 * k, NBIG)) for k in range(SETS)]
    Y = [dev.buf(nbytes=4 * NBIG) for _ in range(SETS)]
    hx = normal(301, NBIG) if cpu else None   # host copy of the 51 MB tensor for the oracle
    hy = np.empty(NBIG, np.float32) if cpu else None

    # cfg 1: Binary add with channel broadcast.  Its tensor is half of a set (25.7 MB):
    # both halves of every set take turns, 12 x 25.7 MB of inputs, so that no launch
    # finds its input still in the 256 MB Infinity Cache.
    sa, sb = [8, 64, 112, 112], [1, 64, 1, 1]
    n = int(np.prod(sa))
    hb = uniform(102, 64, -1, 1)
    B = dev.buf(hb)
    ms = time_median(dev, lambda k: lib.shdw_hip_broadcast_binary(
        0, 4, I(sa), I(sb), I(sa), A[k % SETS].ptr + (k // SETS) * 4 * n, B.ptr, Y[k % SETS].ptr, st), 2 * SETS)
    add(1, "binary_add_channel_broadcast", 4 * n + 256, 4 * n, ms, n,
        cpu and cpu.broadcast(0, uniform(101, n, -1, 1), sa, hb, sb, sa, hy[:n]))

    # cfg 3: reductions over [32,512,28,28]
    shp = [32, 512, 28, 28]
    for name, op, axes, outs in [("reduce_sum_hw", 1, [2, 3], 16384), ("reduce_avg_hw", 4, [2, 3], 16384),
                                 ("reduce_max_c", 2, [1], 25088), ("reduce_sum_all", 1, [0, 1, 2, 3], 1)]:
        need = lib.shdw_hip_reduce_workspace_bytes(4, I(shp), len(axes), I(axes))
        ws = dev.buf(nbytes=max(need, 16))
        ms = time_median(dev, lambda k: lib.shdw_hip_reduce(op, 4, I(shp), len(axes), I(axes), A[k].ptr,
                                                            Y[k].ptr, ws.ptr, need, st), SETS)
        add(3, name, 4 * NBIG, 4 * outs, ms, NBIG, cpu and cpu.reduce(op, hx, shp, axes, hy[:outs]))
        ws.free()

    # cfg 5: ResNet bottleneck tail on [64,1024,14,14]
    n5, C5, in5 = 12845056, 1024, 196
    hg5, hb5 = uniform(502, C5, 0.5, 1.5), uniform(503, C5, -0.1, 0.1)
    g5, b5 = dev.buf(hg5), dev.buf(hb5)
    hr = normal(504, n5) if cpu else None
    M = [dev.buf(nbytes=4 * 65536) for _ in range(SETS)]
    ms = time_median(dev, lambda k: lib.shdw_hip_scale_bias(n5, C5, in5, A[k].ptr, g5.ptr, b5.ptr, 0,
                                                            Y[k].ptr, st), SETS)
    add(5, "scale", 4 * n5 + 8 * C5, 4 * n5, ms, n5, cpu and cpu.scale_bias(hx, hg5, hb5, C5, in5, hy))

    def eltwise_sum(k):
        ptrs = (ctypes.c_void_p * 2)(A[k].ptr, A[(k + 1) % SETS].ptr)
        return lib.shdw_hip_eltwise(1, 2, ptrs, None, n5, Y[k].ptr, st)
    ms = time_median(dev, eltwise_sum, SETS)
    add(5, "eltwise_sum", 8 * n5, 4 * n5, ms, n5, cpu and cpu.eltwise_sum([hx, hr], hy))
    ms = time_median(dev, lambda k: lib.shdw_hip_activate(1, 0.1, n5, A[k].ptr, Y[k].ptr, st), SETS)
    add(5, "relu", 4 * n5, 4 * n5, ms, n5, cpu and cpu.activate(hx, hy, 1))
    sh5, ax5 = [64, 1024, 14, 14], [2, 3]
    ms = time_median(dev, lambda k: lib.shdw_hip_reduce(4, 4, I(sh5), 2, I(ax5), A[k].ptr, M[k].ptr,
                                                        None, 0, st), SETS)
    add(5, "reduce_avg_hw", 4 * n5, 4 * 65536, ms, n5, cpu and cpu.reduce(4, hx, sh5, ax5, hy[:65536]))
    ms = time_median(dev, lambda k: lib.shdw_hip_scale_residual_relu_rowmean(
        n5, C5, in5, A[k].ptr, g5.ptr, b5.ptr, A[(k + 1) % SETS].ptr, Y[k].ptr, M[k].ptr, st), SETS)
    if cpu:
        hs, hm = np.empty(n5, np.float32), np.empty(65536, np.float32)
        chain = [cpu.scale_bias(hx, hg5, hb5, C5, in5, hs), cpu.eltwise_sum([hs, hr], hy), cpu.activate(hy, hy, 1),
                 cpu.reduce(4, hy, sh5, ax5, hm)]
        tail_cpu = lambda: [f() for f in chain]
    add(5, "fused_tail (CPU: the four operators)", 8 * n5 + 8 * C5, 4 * n5 + 4 * 65536, ms, n5, cpu and tail_cpu)
    # the same tail with its BatchNorm in front, as a Caffe-style model holds it (g5 > 0 serves as the variances)
    ms = time_median(dev, lambda k: lib.shdw_hip_batch_norm_scale_residual_relu(
        n5, C5, in5, A[k].ptr, b5.ptr, g5.ptr, 1.0, 1e-5, g5.ptr, b5.ptr, A[(k + 1) % SETS].ptr, 0, Y[k].ptr,
        M[k].ptr, st), SETS)
    add("next", "batch_norm + fused_tail [64,1024,14,14]", 8 * n5 + 16 * C5, 4 * n5 + 4 * 65536, ms, n5)

    sh7 = [128, 2048, 7, 7]  # the same reduction over 7 x 7 planes: rows of 49 floats start on odd dwords
    M7 = [dev.buf(nbytes=4 * 128 * 2048) for _ in range(SETS)]
    ms = time_median(dev, lambda k: lib.shdw_hip_reduce(4, 4, I(sh7), 2, I(ax5), A[k].ptr, M7[k].ptr,
                                                        None, 0, st), SETS)
    add("next", "reduce_avg_hw 7x7 planes [128,2048,7,7]", 4 * n5, 4 * 128 * 2048, ms, n5)
    # more of the same late-stage tensor, whose rows and planes are not multiples of four floats
    ws7 = dev.buf(nbytes=1 << 20)
    ms = time_median(dev, lambda k: lib.shdw_hip_reduce(2, 4, I(sh7), 1, I([1]), A[k].ptr, M7[k].ptr,
                                                        ws7.ptr, 1 << 20, st), SETS)
    add("next", "reduce_max_c 7x7 maps [128,2048,7,7]", 4 * n5, 4 * 128 * 49, ms, n5)
    g7, b7 = dev.buf(uniform(507, 2048, 0.5, 1.5)), dev.buf(uniform(508, 2048, -0.1, 0.1))
    ms = time_median(dev, lambda k: lib.shdw_hip_group_norm(128 * 2048, 49, 1e-5, A[k].ptr, g7.ptr, b7.ptr,
                                                            2048, 49, Y[k].ptr, st), SETS)
    add("next", "instance_norm affine 7x7 planes [128,2048,7,7]", 4 * n5 + 8 * 2048, 4 * n5, ms, n5)
    ms = time_median(dev, lambda k: lib.shdw_hip_broadcast_binary(
        0, 4, I(sh7), I([1, 2048, 1, 1]), I(sh7), A[k].ptr, b7.ptr, Y[k].ptr, st), SETS)
    add("next", "binary_add_channel_broadcast 7x7 maps [128,2048,7,7]", 4 * n5 + 4 * 2048, 4 * n5, ms, n5)
    for bb in M7 + [ws7, g7, b7]:
        bb.free()

    # Operators next to the path (label "next").  Global pooling, Softmax and
    # Normalize run on the 51 MB sets; BatchNorm, Axpy and the stem max pooling
    # run further down on 205 MB tensors like the headline step.
    pin, pout = [16, 64, 112, 112], [16, 64, 56, 56]
    npo = int(np.prod(pout))
    ms = time_median(dev, lambda k: lib.shdw_hip_pooling2d(I(pin), 0, 3, 3, 2, 2, 0, 0, I(pout), A[k].ptr,
                                                           Y[k].ptr, st), SETS)
    add("next", "pooling_max_3x3s2 [16,64,112,112]", 4 * NBIG, 4 * npo, ms, NBIG)
    gin, gout = [128, 2048, 7, 7], [128, 2048, 1, 1]
    ms = time_median(dev, lambda k: lib.shdw_hip_pooling2d(I(gin), 1, 7, 7, 1, 1, 0, 0, I(gout), A[k].ptr,
                                                           Y[k].ptr, st), SETS)
    add("next", "pooling_global_avg_7x7", 4 * NBIG, 4 * 128 * 2048, ms, NBIG)
    gin2, gout2 = [64, 1024, 14, 14], [64, 1024, 1, 1]
    ms = time_median(dev, lambda k: lib.shdw_hip_pooling2d(I(gin2), 1, 14, 14, 1, 1, 0, 0, I(gout2), A[k].ptr,
                                                           Y[k].ptr, st), SETS)
    add("next", "pooling_global_avg_14x14", 4 * NBIG, 4 * 65536, ms, NBIG)
    ms = time_median(dev, lambda k: lib.shdw_hip_pooling2d(I(gin2), 0, 14, 14, 1, 1, 0, 0, I(gout2), A[k].ptr,
                                                           Y[k].ptr, st), SETS)
    add("next", "pooling_global_max_14x14 (Reduce's row kernel)", 4 * NBIG, 4 * 65536, ms, NBIG)
    for gshape in ([32, 512, 28, 28], [16, 256, 56, 56]):  # squeeze-and-excitation stages: long planes
        gside, grows = gshape[2], gshape[0] * gshape[1]
        ms = time_median(dev, lambda k: lib.shdw_hip_pooling2d(I(gshape), 1, gside, gside, 1, 1, 0, 0,
                                                               I(gshape[:2] + [1, 1]), A[k].ptr, Y[k].ptr, st), SETS)
        add("next", "pooling_global_avg_%dx%d (streamed rows)" % (gside, gside), 4 * NBIG, 4 * grows, ms, NBIG)
    # [16, 49, 128, 128]: channel softmax / L2 normalize of a dense map (inner = 16384)
    ms = time_median(dev, lambda k: lib.shdw_hip_softmax(16, 49, 16384, A[k].ptr, Y[k].ptr, st), SETS)
    add("next", "softmax_channels_dense", 4 * NBIG, 4 * NBIG, ms, NBIG)
    ms = time_median(dev, lambda k: lib.shdw_hip_normalize(16, 49, 16384, 2.0, 1e-12, A[k].ptr, Y[k].ptr, st),
                     SETS)
    add("next", "normalize_l2_channels_dense", 4 * NBIG, 4 * NBIG, ms, NBIG)
    ms = time_median(dev, lambda k: lib.shdw_hip_softmax(64, 1000, 1, A[k].ptr, Y[k].ptr, st), SETS)
    add("next", "softmax_classifier_64x1000", 4 * 64000, 4 * 64000, ms, 64000)
    ms = time_median(dev, lambda k: lib.shdw_hip_normalize(64, 512, 1, 2.0, 1e-12, A[k].ptr, Y[k].ptr, st), SETS)
    add("next", "normalize_l2_embedding_64x512", 4 * 64 * 512, 4 * 64 * 512, ms, 64 * 512)
    for bset in (A, Y, M, [B, g5, b5]):
        for bb in bset:
            bb.free()

    # "next" operators at the size of the headline tensor (205 MB in, 3 rotating sets)
    NH, SH = 51380224, 3 * sets_scale
    AH = [dev.buf(normal(701 + k, NH)) for k in range(SH)]
    YH = [dev.buf(nbytes=4 * NH) for _ in range(SH)]
    CH, INH = 256, 3136
    meanh, varh = dev.buf(normal(611, CH)), dev.buf(uniform(612, CH, 0.5, 2.0))
    ms = time_median(dev, lambda k: lib.shdw_hip_batch_norm(NH, CH, INH, AH[k].ptr, meanh.ptr, varh.ptr,
                                                            1.0, 1e-5, YH[k].ptr, st), SH, reps=20)
    add("next", "batch_norm [64,256,56,56]", 4 * NH + 8 * CH, 4 * NH, ms, NH)
    # BatchNorm -> Scale -> ReLU as the backend's fusion pass runs it: one launch, one pass over the tensor
    ms = time_median(dev, lambda k: lib.shdw_hip_batch_norm_scale(NH, CH, INH, AH[k].ptr, meanh.ptr, varh.ptr, 1.0, 1e-5,
                                                                  varh.ptr, meanh.ptr, 1, YH[k].ptr, st), SH, reps=20)
    add("next", "batch_norm_scale_relu [64,256,56,56]", 4 * NH + 16 * CH, 4 * NH, ms, NH)
    ms = time_median(dev, lambda k: lib.shdw_hip_lrn(I([64, CH, 56, 56]), 5, 1e-4, 0.75, 1.0, AH[k].ptr, YH[k].ptr, st),
                     SH, reps=20)
    add("next", "lrn across 5 channels [64,256,56,56]", 4 * NH, 4 * NH, ms, NH)
    # GridSample with a mildly warped identity grid (what a spatial transformer produces): bilinear, zeros outside
    gy, gx = np.meshgrid(np.linspace(-1, 1, 56), np.linspace(-1, 1, 56), indexing="ij")
    warp = np.stack([gx, gy], -1).astype(np.float32)[None] + uniform(614, (64, 56, 56, 2), -0.05, 0.05)
    gridh = dev.buf(np.ascontiguousarray(warp, np.float32).ravel())
    hw = I([64, CH, 56, 56])
    ms = time_median(dev, lambda k: lib.shdw_hip_grid_sample(hw, hw, 1, 0, AH[k].ptr, gridh.ptr, YH[k].ptr, st), SH, reps=20)
    add("next", "grid_sample bilinear, warped identity [64,256,56,56]", 4 * NH + 8 * 64 * 3136, 4 * NH, ms, NH)
    alh = dev.buf(uniform(613, 64 * CH, 0.0, 1.0))
    ms = time_median(dev, lambda k: lib.shdw_hip_axpy_rows(64 * CH, INH, alh.ptr, AH[k].ptr,
                                                           AH[(k + 1) % SH].ptr, YH[k].ptr, st), SH, reps=20)
    add("next", "axpy_rows [64,256,56,56]", 8 * NH + 4 * 64 * CH, 4 * NH, ms, NH)
    pinh, pouth = [64, 64, 112, 112], [64, 64, 56, 56]
    ms = time_median(dev, lambda k: lib.shdw_hip_pooling2d(I(pinh), 0, 3, 3, 2, 2, 0, 0, I(pouth), AH[k].ptr,
                                                           YH[k].ptr, st), SH, reps=20)
    add("next", "pooling_max_3x3s2 [64,64,112,112]", 4 * NH, NH, ms, NH)
    ginh, gouth = [512, 2048, 7, 7], [512, 2048, 1, 1]
    ms = time_median(dev, lambda k: lib.shdw_hip_pooling2d(I(ginh), 1, 7, 7, 1, 1, 0, 0, I(gouth), AH[k].ptr,
                                                           YH[k].ptr, st), SH, reps=20)
    add("next", "pooling_global_avg_7x7 [512,2048,7,7]", 4 * NH, 4 * 512 * 2048, ms, NH)
    ms = time_median(dev, lambda k: lib.shdw_hip_softmax(64, 49, 16384, AH[k].ptr, YH[k].ptr, st), SH, reps=20)
    add("next", "softmax_channels_dense [64,49,128,128]", 4 * NH, 4 * NH, ms, NH)
    NSEG = 64 * 150 * 5329  # a 150-class segmentation head, 73 x 73
    ms = time_median(dev, lambda k: lib.shdw_hip_softmax(64, 150, 5329, AH[k].ptr, YH[k].ptr, st), SH, reps=10)
    add("next", "softmax_150_classes [64,150,73,73]", 4 * NSEG, 4 * NSEG, ms, NSEG)
    NSEG = 64 * 150 * 5184  # the same head on 72 x 72: rows of whole 128-bit vectors
    ms = time_median(dev, lambda k: lib.shdw_hip_softmax(64, 150, 5184, AH[k].ptr, YH[k].ptr, st), SH, reps=10)
    add("next", "softmax_150_classes [64,150,72,72]", 4 * NSEG, 4 * NSEG, ms, NSEG)
    ms = time_median(dev, lambda k: lib.shdw_hip_normalize(64, 49, 16384, 2.0, 1e-12, AH[k].ptr, YH[k].ptr, st),
                     SH, reps=20)
    add("next", "normalize_l2_channels_dense [64,49,128,128]", 4 * NH, 4 * NH, ms, NH)
    sch, bih = dev.buf(uniform(614, CH, 0.5, 1.5)), dev.buf(uniform(615, CH, -0.1, 0.1))
    ms = time_median(dev, lambda k: lib.shdw_hip_group_norm(64 * CH, INH, 1e-5, AH[k].ptr, sch.ptr, bih.ptr,
                                                            CH, INH, YH[k].ptr, st), SH, reps=20)
    add("next", "instance_norm affine [64,256,56,56]", 4 * NH + 8 * CH, 4 * NH, ms, NH)
    ms = time_median(dev, lambda k: lib.shdw_hip_group_norm(64 * 32, 8 * INH, 1e-5, AH[k].ptr, sch.ptr, bih.ptr,
                                                            CH, INH, YH[k].ptr, st), SH, reps=20)
    add("next", "group_norm 32 groups affine [64,256,56,56]", 4 * NH + 8 * CH, 4 * NH, ms, NH)
    lns, lnb = dev.buf(uniform(616, 784, 0.5, 1.5)), dev.buf(uniform(617, 784, -0.1, 0.1))
    ms = time_median(dev, lambda k: lib.shdw_hip_group_norm(65536, 784, 1e-5, AH[k].ptr, lns.ptr, lnb.ptr,
                                                            784, 1, YH[k].ptr, st), SH, reps=20)
    add("next", "layer_norm affine [65536,784]", 4 * NH + 8 * 784, 4 * NH, ms, NH)
    # SSDNormalize on the SSD conv4_3 map, batch 64: 8 bytes per element are compulsory
    # (the per-item form reads x a second time on top of that)
    NS = 64 * 512 * 1444
    ssc = dev.buf(uniform(618, 512, 10.0, 30.0))
    ms = time_median(dev, lambda k: lib.shdw_hip_ssd_normalize(64, 512, 1444, 0, 1e-5, AH[k].ptr, ssc.ptr, 0,
                                                               YH[k].ptr, None, st), SH, reps=20)
    add("next", "ssd_normalize per position, channel scale [64,512,38,38]", 4 * NS + 4 * 512, 4 * NS, ms, NS)
    ms = time_median(dev, lambda k: lib.shdw_hip_ssd_normalize(64, 256, 3136, 0, 1e-5, AH[k].ptr, ssc.ptr, 0,
                                                               YH[k].ptr, None, st), SH, reps=20)
    add("next", "ssd_normalize per position, channel scale [64,256,56,56]", 4 * NH + 4 * 256, 4 * NH, ms, NH)
    swb = dev.buf(nbytes=max(8, lib.shdw_hip_ssd_normalize_workspace_bytes(64, 512, 1444, 1)))
    ms = time_median(dev, lambda k: lib.shdw_hip_ssd_normalize(64, 512, 1444, 1, 1e-5, AH[k].ptr, ssc.ptr, 0,
                                                               YH[k].ptr, swb.ptr, st), SH, reps=20)
    add("next", "ssd_normalize per item, channel scale [64,512,38,38] (3 launches)", 4 * NS + 4 * 512, 4 * NS, ms, NS)
    # data movers ("movers") on the same 205 MB tensors
    def concat2(k):
        # two [64,128,56,56] halves -> [64,256,56,56] along axis 1
        rc = lib.shdw_hip_copy_chunks(64, 128 * INH, AH[k].ptr, 128 * INH, 0, YH[k].ptr, 256 * INH, 0, st)
        return rc or lib.shdw_hip_copy_chunks(64, 128 * INH, AH[(k + 1) % SH].ptr, 128 * INH, 0, YH[k].ptr,
                                              256 * INH, 128 * INH, st)
    ms = time_median(dev, concat2, SH, reps=20)
    add("movers", "concat 2x[64,128,56,56] axis 1 (2 launches)", 4 * NH, 4 * NH, ms, NH)
    shp4 = [64, 256, 56, 56]
    ms = time_median(dev, lambda k: lib.shdw_hip_permute(4, I(shp4), I([0, 2, 3, 1]), AH[k].ptr, YH[k].ptr, st),
                     SH, reps=20)
    add("movers", "permute NCHW->NHWC [64,256,56,56]", 4 * NH, 4 * NH, ms, NH)
    ms = time_median(dev, lambda k: lib.shdw_hip_permute(4, I(shp4), I([0, 3, 1, 2]), AH[k].ptr, YH[k].ptr, st),
                     SH, reps=20)
    add("movers", "permute [0,3,1,2] [64,256,56,56]", 4 * NH, 4 * NH, ms, NH)
    ms = time_median(dev, lambda k: lib.shdw_hip_shuffle_channel(64, 256, INH, 2, AH[k].ptr, YH[k].ptr, st), SH,
                     reps=20)
    add("movers", "shuffle_channel g=2 [64,256,56,56]", 4 * NH, 4 * NH, ms, NH)
    pshape = [64, 64, 110, 110]
    npi = int(np.prod(pshape))
    ms = time_median(dev, lambda k: lib.shdw_hip_pad(I(pshape), I([1, 1, 1, 1]), 0.0, AH[k].ptr, YH[k].ptr, st), SH,
                     reps=20)
    add("movers", "pad 1 [64,64,110,110] -> 112x112", 4 * npi, 4 * NH, ms, NH)
    rin, rout = [64, 64, 56, 56], [64, 64, 112, 112]
    nri = int(np.prod(rin))
    # The resize input is a quarter of a set (51 MB): all four quarters of every set
    # take turns (12 inputs, 617 MB), so that the gathers do not find them in the
    # Infinity Cache.
    def resize_in(k):
        return AH[k % SH].ptr + (k // SH) * 4 * nri
    ms = time_median(dev, lambda k: lib.shdw_hip_resize(I(rin), I(rout), 1, 0, resize_in(k), YH[k % SH].ptr, st),
                     4 * SH, reps=24)
    add("movers", "resize bilinear x2 [64,64,56,56]", 4 * nri, 4 * NH, ms, NH)
    ms = time_median(dev, lambda k: lib.shdw_hip_resize(I(rin), I(rout), 0, 0, resize_in(k), YH[k % SH].ptr, st),
                     4 * SH, reps=24)
    add("movers", "resize nearest x2 [64,64,56,56]", 4 * nri, 4 * NH, ms, NH)
    ms = time_median(dev, lambda k: lib.shdw_hip_reorg(I(rout), 1, 2, AH[k].ptr, YH[k].ptr, st), SH, reps=20)
    add("movers", "reorg natural s2 [64,64,112,112]", 4 * NH, 4 * NH, ms, NH)
    ms = time_median(dev, lambda k: lib.shdw_hip_reorg(I(rout), 0, 2, AH[k].ptr, YH[k].ptr, st), SH, reps=20)
    add("movers", "reorg darknet s2 [64,64,112,112]", 4 * NH, 4 * NH, ms, NH)
    for bset in (AH, YH, [meanh, varh, alh, sch, bih, lns, lnb, ssc, swb]):
        for bb in bset:
            bb.free()

    # cfg 4: general broadcast; outputs dominate the traffic
    for tag, sa4, sb4 in [("i", [16, 1, 128, 256], [1, 32, 128, 1]), ("ii", [4, 64, 1, 512], [1, 1, 64, 512]),
                          ("iii", [128, 1024], [1, 1])]:
        so4 = [max(p, q) for p, q in zip(sa4, sb4)]
        na, nb_, no = int(np.prod(sa4)), int(np.prod(sb4)), int(np.prod(so4))
        ha, hb4 = normal(401, na), uniform(402, nb_, 0.5, 2.0)
        a4, b4 = dev.buf(ha), dev.buf(hb4)
        y4 = [dev.buf(nbytes=4 * no) for _ in range(SETS)]
        hy4 = np.empty(no, np.float32) if cpu else None
        isa4, isb4, iso4 = I(sa4), I(sb4), I(so4)  # built once: on 1 MB tensors the caller's own time per launch shows
        for name, op in [("mul", 2), ("sub", 1), ("div", 3), ("max", 5)]:
            ms = time_median(dev, lambda k: lib.shdw_hip_broadcast_binary(
                op, len(so4), isa4, isb4, iso4, a4.ptr, b4.ptr, y4[k].ptr, st), SETS)
            add(4, "broadcast_%s_%s" % (name, tag), 4 * (na + nb_), 4 * no, ms, no,
                cpu and cpu.broadcast(op, ha, sa4, hb4, sb4, so4, hy4))
        if tag == "iii":  # the same pair through the scalar-argument form
            alpha = float(hb4[0])
            for name, op in [("mul", 2), ("sub", 1), ("div", 3), ("max", 5)]:
                ms = time_median(dev, lambda k: lib.shdw_hip_binary_scalar(op, na, a4.ptr, alpha, y4[k].ptr, st), SETS)
                add(4, "scalar_%s_iii" % name, 4 * na, 4 * no, ms, no, cpu and cpu.binary_scalar(op, ha, alpha, hy4))
        for bb in y4 + [a4, b4]:
            bb.free()

    # The yardsticks themselves, at the byte counts of the BASELINE rows.
    for mb, nbytes in [(25.7, 25690112), (34, 34209792), (51, 51380224), (69, 69222400), (103, 102760448),
                       (154, 154140672), (411, 411041792)]:
        for kind in ("copy", "read", "write"):
            us = ceil.us(kind, nbytes)
            rows.append({"cfg": "ceiling", "op": "%s of %s MB" % (kind, mb), "bytes": nbytes, "us": round(us, 2),
                         "GBps": round(nbytes / us / 1e3, 1), "frac": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)})
    ceil.free()
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
    the launches (three with the backend's fusion pass, five without), one stream
    synchronisation per call."""
    sa = dev.sa
    n = 64 * 1024 * 14 * 14
    x, r = dev.buf(normal(801, n)), dev.buf(normal(802, n))
    weights = [uniform(803, 1024, 0.5, 1.5), uniform(804, 1024, -0.1, 0.1)]
    out = {"model": "Scale -> Eltwise -> ReLU -> global avg Pooling -> Flatten -> Softmax, [64,1024,14,14]",
           "operators": 6, "input_copies": 2}
    for fuse, key in ((True, "us_per_forward"), (False, "us_per_forward_unfused")):
        with sa.Network(NETWORK_TEXT, weights, device_input=True, fuse=fuse) as net:
            for _ in range(5):
                net.forward({"x": x, "r": r})
            t0 = time.perf_counter()
            for _ in range(reps):
                net.forward({"x": x, "r": r})
            t1 = time.perf_counter()
            if fuse:
                out["fused"] = net.fused
        out[key] = round((t1 - t0) * 1e6 / reps, 1)
    x.free(), r.free()
    return out


def tail_text(copies, batch_norm=False):
    """BASELINE configs[4] as a converted model holds it, `copies` times side by side on
    blobs of their own, so that one run walks over more than the 256 MB Infinity Cache.
    batch_norm: a BatchNorm on stored statistics in front of every Scale, as a Caffe-style
    model holds the normalisation."""
    shape = "64 # 1024 # 14 # 14"
    names = ["x%d" % k for k in range(copies)] + ["r%d" % k for k in range(copies)]
    lines = ["[bottleneck_tails]", "[{out_blob, v_s, [%s]}]" % " # ".join("pool%d" % k for k in range(copies)),
             "[{gamma, float, [1024]}; {beta, float, [1024]}]",
             "[Input] | [in] | [0 %d %d] | [] | [%s] | [%s]" % (
                 len(names), len(names), "; ".join(names), "; ".join("{%s, v_i, [%s]}" % (nm, shape) for nm in names))]
    for k in range(copies):
        if batch_norm:  # beta as the means, gamma (0.5 ... 1.5) as the variances
            lines += ["[BatchNorm] | [norm%d] | [3 1 1] | [x%d; beta; gamma] | [n%d] | [{eps, s_f, [0.001]}]" % (k, k, k)]
        lines += ["[Scale] | [bn%d] | [3 1 3] | [%s%d; gamma; beta] | [s%d] | [{axis, s_i, [1]}; {has_scale, s_i, [1]}; "
                  "{has_bias, s_i, [1]}]" % (k, "n" if batch_norm else "x", k, k),
                  "[Eltwise] | [add%d] | [2 1 1] | [s%d; r%d] | [e%d] | [{operation, s_i, [1]}]" % (k, k, k, k),
                  "[Activate] | [relu%d] | [1 1 1] | [e%d] | [e%d] | [{type, s_i, [1]}]" % (k, k, k),
                  "[Reduce] | [gap%d] | [1 1 2] | [e%d] | [pool%d] | [{operation, s_i, [4]}; {axes, v_i, [2 # 3]}]" % (
                      k, k, k)]
    return "\n".join(lines) + "\n"


def network_tail(dev, copies=6, reps=20, batch_norm=False):
    """Device time of the bottleneck tail (Scale -> Eltwise SUM -> ReLU -> Reduce AVG on
    [64,1024,14,14]) run by the Native backend from a model text, per tail: events on the
    backend's stream around `reps` runs of a network that holds `copies` such tails on
    separate blobs, nothing waited for in between.  Fused: one launch per tail.
    batch_norm: the tail with a BatchNorm in front of its Scale (five operators)."""
    sa, lib = dev.sa, dev.lib
    n = 64 * 1024 * 14 * 14
    src = [dev.buf(normal(811 + k, n)) for k in range(2)]
    weights = [uniform(803, 1024, 0.5, 1.5), uniform(804, 1024, -0.1, 0.1)]
    feed = {}
    for k in range(copies):
        feed["x%d" % k], feed["r%d" % k] = src[k & 1], src[(k + 1) & 1]
    out = {"model": "%d x (%sScale -> Eltwise SUM -> ReLU -> Reduce AVG{2,3}) on [64,1024,14,14]" % (
        copies, "BatchNorm -> " if batch_norm else "")}
    for fuse, key in ((True, "us_per_tail"), (False, "us_per_tail_unfused")):
        with sa.Network(tail_text(copies, batch_norm), weights, device_input=True, fuse=fuse) as net:
            net.forward(feed)
            st = net.stream
            e0, e1 = dev.event(), dev.event()
            best = None
            for _ in range(3):
                net.run()
                dev.ck(lib.shdw_hip_event_record(e0, st))
                for _ in range(reps):
                    net.run()
                dev.ck(lib.shdw_hip_event_record(e1, st))
                dev.ck(lib.shdw_hip_stream_sync(st))
                ms = dev.elapsed_ms(e0, e1) / (reps * copies)
                best = ms if best is None else min(best, ms)
            out[key] = round(best * 1e3, 2)
            out["launches_per_tail" if fuse else "launches_per_tail_unfused"] = 1 if net.fused else 4 + batch_norm
    for b in src:
        b.free()
    return out


SHORT_OP = {"binary_add_channel_broadcast": "add_chan_bcast", "fused_tail (CPU: the four operators)": "fused_tail"}
FINAL_LINE_LIMIT = 4096  # the driver keeps a bounded tail of stdout: the record has to fit in it whole


def final_record(full, table_path=None):
    """The one line printed last: the fields the contract names, the roofline of the
    dominant kernel, the CPU baseline and one short row per BASELINE operator
    ([cfg, op, us, frac of 8 TB/s, frac of the same-size ceiling, cpu_us]).  Everything
    else (per-op step table, neighbouring operators, movers, ceilings, notes) stays in
    the table file.  Kept free of device calls so that its size can be tested anywhere."""
    keep = ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
            "vs_baseline", "dtype", "data", "config", "frac_of_hbm_peak", "elements_per_s")
    rec = {k: full[k] for k in keep if k in full}
    roof = dict(full["roofline"])
    for k in ("note", "traffic_source", "valu_source"):
        roof.pop(k, None)
    rec["roofline"] = roof
    if "cpu_baseline" in full:
        rec["cpu_baseline"] = {k: v for k, v in full["cpu_baseline"].items() if k != "ops"}
        rec["speedup_vs_cpu"] = full.get("speedup_vs_cpu")
    rec["step_ops"] = [[d["op"], d["us"], d["frac"]] for d in full.get("step_ops", []) if "yardstick" not in d["op"]]
    rows = [r for r in full.get("configs", []) if r["cfg"] in (1, 3, 4, 5)]
    if rows:
        rec["baseline_rows_columns"] = ["cfg", "op", "us", "frac", "of_ceiling", "cpu_us"]
        rec["baseline_rows"] = [[r["cfg"], SHORT_OP.get(r["op"], r["op"]), r["us"], round(r["frac"], 3),
                                 round(r["frac_of_ceiling"], 2), r.get("cpu_us") and round(r["cpu_us"])] for r in rows]
        big = [r for r in rows if r["bytes"] >= (8 << 20)]  # cfg 4(iii) is a 1 MB tensor: launch-bound by size
        worst = min(big, key=lambda r: r["frac_of_ceiling"])
        rec["worst_of_ceiling"] = [worst["cfg"], SHORT_OP.get(worst["op"], worst["op"]), worst["frac_of_ceiling"]]
    if "network" in full:
        rec["network"] = {k: v for k, v in full["network"].items() if k not in ("model", "fused")}
    for key in ("network_tail", "network_bn_tail"):
        if key in full:
            rec[key] = {k: v for k, v in full[key].items() if k != "model"}
    if table_path:
        rec["table"] = table_path
    return rec


def final_line(full, table_path=None):
    """final_record as one line of JSON below FINAL_LINE_LIMIT.  Should a host with a long
    device or CPU name push it over, the optional tables go first (they are in the file)."""
    rec = final_record(full, table_path)
    for optional in (None, "step_ops", "baseline_rows", "baseline_rows_columns", "network", "network_bn_tail",
                     "network_tail"):
        rec.pop(optional, None)
        line = json.dumps(rec, separators=(",", ":"))
        if len(line) < FINAL_LINE_LIMIT:
            return line
    raise RuntimeError("bench.py: the final record is %d characters, the limit is %d" % (len(line), FINAL_LINE_LIMIT))


def write_table(full, path):
    """The whole measurement (every row, every note) as a JSON file; None when the
    directory cannot be written (the final line then names no table)."""
    try:
        os.makedirs(os.path.dirname(path), exist_ok=True)
        with open(path, "w") as f:
            json.dump(full, f, indent=1)
        return os.path.relpath(path, ROOT)
    except OSError:
        return None


def main():
    args = parse()
    if args.gpus != 1:
        raise SystemExit("bench.py: this build measures one GPU; the path shards by batch with no "
                         "exchange, so run one process per GPU (got --gpus %d)" % args.gpus)
    if args.launch_shapes:
        launch_shapes()
        return
    dev = Dev()
    if args.scaling:
        scaling(dev)
        return
    if args.sweep:
        sweep(dev)
        return
    if args.probe:
        probe(dev)
        return
    if args.probe_next:
        probe_next(dev)
        return
    ms_per_step, step_bytes, n, roofline, detail, host = headline(dev, args.steps, args.warmup, args.single_input)
    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    out = {
        "metric": "achieved HBM GB/s (% of MI355X peak) per op; speedup vs host-CPU Shadow",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "BASELINE configs[1]: fp32 [64,256,56,56] ~N(0,2) seed 201; relu, "
                               "sigmoid, exp, abs, sqrt(abs), tanh as single ops + fused per-channel "
                               "Scale+ReLU (7 launches per step); %s" % (
                                   "one resident input" if args.single_input else
                                   "two resident copies of the input take turns step by step"),
                   "elements": n, "bytes_per_step": step_bytes, "device": dev.info},
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
        "elements_per_s": round(7 * n / (ms_per_step * 1e-3), 1),
        "roofline": roofline, "step_ops": detail,
        "step_ops_note": "per-op times from an untimed pass of the same K steps with events around every "
                         "launch; roofline.avg_us from events around the dominant kernel inside the timed region",
    }
    cpu = None if args.no_cpu else Cpu(args.cpu_passes)
    if cpu is not None:
        out["cpu_baseline"] = cpu_headline(cpu, host, step_bytes)
        out["speedup_vs_cpu"] = round(value / out["cpu_baseline"]["value"], 1)
        for d in detail:
            c = out["cpu_baseline"]["ops"].get(d["op"])
            if c:
                d["cpu_us"] = c["best_us"]
                d["speedup_vs_cpu"] = round(c["best_us"] / d["us"], 1)
    host = None
    if not args.no_configs:
        out["configs"] = config_table(dev, args.operand_sets, cpu)
        out["configs_note"] = ("us: median of three batches of back-to-back launches rotating over operand sets; "
                               "ceiling_us: a plain copy / read / write of the same number of bytes timed the same "
                               "way (rows at the end); cpu_us: the oracle's C loop for the same operator on this "
                               "host, one thread, outputs allocated beforehand, best of %d" % args.cpu_passes)
        out["network"] = network_forward(dev)
        out["network_tail"] = network_tail(dev)
        out["network_bn_tail"] = network_tail(dev, batch_norm=True)
    table = write_table(out, args.table)
    for r in out.get("configs", []):
        print("%-8s %-62s %9.2f us  %.3f of 8 TB/s%s" % (r["cfg"], r["op"], r["us"], r["frac"],
              "  %.3f of ceiling" % r["frac_of_ceiling"] if "frac_of_ceiling" in r else ""), file=sys.stderr)
    sys.stderr.flush()
    print(final_line(out, table), flush=True)


if __name__ == "__main__":
    main()
