#!/usr/bin/env python3
"""Benchmark of the tensor-math hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--sections a,b,...] [--no-cpu]
    python bench.py --profile-plan FILE ...        (under rocprofv3: marks the segments of the run)
    python bench.py --summarize DIR [--out DIR2]   (turns rocprofv3 output into profiles/ summaries)
    python bench.py --summarize-counters RUN [--out DIR2]   (per-workload averages of any --pmc run)

The metric is achieved HBM bandwidth of ``binary-op!``, ``unary-reduce!`` and the
Adam step.  One step is one pass of those three workloads at their BASELINE
shapes over synthetic inputs that are resident in HBM before the timed region:

    configs[3]  fused Adam step over 2^28 float32 parameters (the dominant kernel)
    configs[2]  unary-reduce! :sum :max :magnitude-squared over the last axis of
                float32 [16384,4096] and over axis 0 through a transposed view, and
                the same six reductions of float64 [4096,4096]
    configs[0]  binary-op! :+ of float32 [1024,1024] with a broadcast [1024] row

``value`` is the algorithmic bytes of one step (each input element read once,
each output element written once) over the step's time.  ``roofline`` describes
the Adam kernel, timed with HIP events recorded on the launch stream around each
of its launches inside the timed region.  ``ops`` carries a roofline-shaped block
for every workload of the step (and the Adadelta step of configs[3]), each timed
on its own, back to back.  ``others`` holds BASELINE configs[1] and [4] and the
scaled form of configs[0]; ``patterns`` the access patterns off the three fast
kernel families; ``adjacent`` the neighbouring TensorMath methods.
``cpu_baseline`` times the CPU oracle (a C++ restatement of the cortex CPU
backend, OpenMP) on the same step.

``traffic`` figures are HBM bytes per call measured with rocprofv3 counters and
stored in ``profiles/traffic.json`` together with a hash of the kernel sources
they were measured on; when the sources have changed since, the run reports
``null`` and says so.
"""
from __future__ import annotations

import argparse
import collections
import csv
import ctypes as C
import glob
import hashlib
import json
import re
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

PEAK_HBM_GBS = 8000.0  # MI355X HBM3E, published
SECTIONS = ("headline", "others", "midsize", "small", "variants", "patterns", "adjacent")


def log(msg: str) -> None:
    print(msg, file=sys.stderr, flush=True)


# ----------------------------------------------------------------------------- sources hash / stored traffic

def csrc_hash() -> str:
    """SHA-256 over the kernel sources and the C header, in name order."""
    h = hashlib.sha256()
    files = sorted(p for p in (ROOT / "cortex_amd" / "csrc").iterdir() if p.suffix in (".hip", ".h", ".cpp"))
    for p in files + [ROOT / "include" / "cortex_hip.h"]:
        h.update(p.name.encode())
        h.update(p.read_bytes())
    return h.hexdigest()


def load_traffic():
    """Stored rocprofv3 traffic per workload key, or ({}, reason) when it does not describe these sources."""
    tfile = ROOT / "profiles" / "traffic.json"
    if not tfile.exists():
        return {}, "profiles/traffic.json is missing"
    try:
        stored = json.loads(tfile.read_text())
    except (ValueError, OSError) as err:
        return {}, f"profiles/traffic.json unreadable: {err}"
    if stored.get("csrc_sha256") != csrc_hash():
        return {}, ("kernel sources changed since profiles/traffic.json was measured "
                    f"({str(stored.get('csrc_sha256'))[:8]} -> {csrc_hash()[:8]}): traffic not reported")
    return stored.get("ops", {}), None


# ----------------------------------------------------------------------------- timing helpers

class Timer:
    """HIP-event timing on one stream."""

    def __init__(self, capi, stream):
        self.capi, self.stream = capi, stream

    def mark(self):
        e = C.c_void_p()
        self.capi.call("ct_event_record_timed", C.byref(e), self.stream.handle)
        return e

    def elapsed_ms(self, e0, e1) -> float:
        self.capi.call("ct_event_sync", e1)
        ms = C.c_float()
        self.capi.call("ct_event_elapsed_ms", e0, e1, C.byref(ms))
        return float(ms.value)

    def free(self, *events) -> None:
        for e in events:
            self.capi.call("ct_event_destroy", e)


def dims(shape, strides=None):
    if strides is None:
        strides, m = [], 1
        for s in reversed(shape):
            strides.insert(0, m)
            m *= s
    return {"shape": list(shape), "strides": list(strides)}


def gbs(nbytes: float, ms: float) -> float:
    return nbytes / (ms * 1e-3) / 1e9


class Op:
    """One timed call of the library: `fn()` issues it on the bench stream."""

    def __init__(self, key, label, nbytes, fn, iters=20, config=None):
        self.key, self.label, self.nbytes, self.fn, self.iters, self.config = key, label, nbytes, fn, iters, config
        self.kernel = ""


class Bench:
    def __init__(self, plan_path=None):
        from cortex_amd import capi, driver as drv

        self.capi, self.drv = capi, drv
        self.driver = drv.HipDriver()
        self.device = self.driver.default_device()
        self.device.make_current()
        self.stream = self.device.create_stream()
        self.timer = Timer(capi, self.stream)
        self.traffic, self.traffic_note = load_traffic()
        self.plan = [] if plan_path else None
        self.plan_path = plan_path
        self.marker_buf = self.device.allocate_device_buffer(256, "byte") if plan_path else None
        # Buffers stay allocated until the end: on this board a large buffer allocated after frees can land
        # less favourably and cost several percent of bandwidth, which would make figures depend on the order.
        self.keep = []

    # -- profile plan: under rocprofv3 every segment of the run starts with a marker launch (a one-byte
    # fill) so that the dispatches of the trace can be attributed to workloads by order alone
    def segment(self, key, label, calls, nbytes):
        if self.plan is None:
            return
        self.stream.memset(self.marker_buf, 0, 1, 1)
        self.plan.append({"key": key, "label": label, "calls": calls, "algorithmic_bytes": nbytes})

    def save_plan(self):
        if self.plan is not None:
            Path(self.plan_path).write_text(json.dumps({"csrc_sha256": csrc_hash(), "segments": self.plan}, indent=1))

    def upload(self, array: np.ndarray):
        flat = np.ascontiguousarray(array).reshape(-1)
        dt = self.drv.DATATYPE_OF_NUMPY[flat.dtype]
        buf = self.device.allocate_device_buffer(flat.size, dt)
        self.capi.call("ct_memcpy_async", buf.ptr, flat.ctypes.data, flat.nbytes, self.capi.COPY_H2D, self.stream.handle)
        self.stream.sync()
        return buf

    def alloc(self, n, dt):
        return self.device.allocate_device_buffer(n, dt)

    def time_op(self, op: Op, warm: int = 2) -> dict:
        """Average duration of `op` over op.iters back-to-back calls, as a roofline-shaped block."""
        # the marker precedes the warm-up calls, which therefore count among the segment's dispatches
        self.segment(op.key, op.label, op.iters + warm, op.nbytes)
        for _ in range(warm):
            op.fn()
        self.stream.sync()
        op.kernel = self.capi.last_kernel()
        t0 = time.perf_counter()
        e0 = self.timer.mark()
        for _ in range(op.iters):
            op.fn()
        e1 = self.timer.mark()
        host_ms = (time.perf_counter() - t0) * 1e3 / op.iters  # submission only: nothing has been waited for yet
        ms = self.timer.elapsed_ms(e0, e1) / op.iters
        self.timer.free(e0, e1)
        return self.block(op, ms, host_us=host_ms * 1e3)

    def block(self, op: Op, ms: float, **more) -> dict:
        return roofline_block(op, ms, self.traffic.get(op.key), **more)


def roofline_block(op: Op, ms: float, stored: dict | None, **more) -> dict:
    """A roofline-shaped record of one workload: `ms` per call, `stored` its entry of profiles/traffic.json or None."""
    rate = gbs(op.nbytes, ms)
    b = {"key": op.key, "bound": "hbm", "achieved": round(rate, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
         "frac": round(rate / PEAK_HBM_GBS, 4), "traffic": stored["traffic"] if stored else None,
         "avg_call_us": round(ms * 1e3, 2), "algorithmic_bytes_per_call": op.nbytes, "kernel": op.kernel}
    if stored:
        b["kernel_us_rocprof"] = stored.get("kernel_us")
    for k, v in more.items():
        b[k] = round(v, 2) if isinstance(v, float) else v
    return b


def headline(steps: int, warmup: int, adam_n: int, step_bytes: int, ms_per_step: float, wall_ms_per_step: float) -> dict:
    """The fields of the result that the benchmark contract names, up to `config`."""
    value = gbs(step_bytes, ms_per_step)
    return collections.OrderedDict([
        ("metric", "achieved HBM GB/s (% of MI355X peak) for binary-op!, unary-reduce!, Adam step"),
        ("value", round(value, 1)),
        ("unit", "GB/s"),
        ("n_gpus", 1),
        ("steps", steps),
        ("warmup", warmup),
        ("ms_per_step", round(ms_per_step, 4)),
        ("higher_is_better", True),
        ("scaling", "weak"),
        ("vs_baseline", None),
        ("dtype", "f32"),
        ("data", "synthetic"),
        ("config", {
            "workload": f"configs[3] fused Adam step over {adam_n} float32 parameters + configs[2] unary-reduce! :sum :max "
                        ":magnitude-squared over the last axis and over axis 0 (transposed view) of float32 [16384,4096] and of "
                        "float64 [4096,4096] + configs[0] binary-op! :+ float32 [1024,1024] with a broadcast [1024] row; "
                        "numpy default_rng seeds 6, 4, 5, 0",
            "algorithmic_bytes_per_step": step_bytes,
            "frac_of_peak": round(value / PEAK_HBM_GBS, 4),
            "host_wall_ms_per_step": round(wall_ms_per_step, 4),
            "csrc_sha256": csrc_hash()[:16],
        }),
    ])


def adam_roofline(adam: Op, adam_ms: float, stored: dict | None, traffic_note: str | None) -> dict:
    """The `roofline` object: the Adam kernel, `adam_ms` the average of the event pairs around its launches."""
    roof = roofline_block(adam, adam_ms, stored)
    del roof["key"]
    roof["kernel"] = f"adam_kernel<float, 4, 1, true> ({adam.kernel})"
    roof["avg_launch_us"] = roof.pop("avg_call_us")
    roof["algorithmic_bytes_per_launch"] = roof.pop("algorithmic_bytes_per_call")
    roof["note"] = "4 read + 3 write streams; the bare mix without arithmetic reaches 77-78 % of peak here, a copy 84-89 %"
    stored_us = roof.get("kernel_us_rocprof")
    if stored_us and abs(roof["avg_launch_us"] - stored_us) > 0.025 * stored_us:
        roof["note"] += "; kernel_us_rocprof is from the other of the pool's two groups of boxes"
    if traffic_note:
        roof["traffic_note"] = traffic_note
    return roof


# ----------------------------------------------------------------------------- the step: configs[3], [2], [0]

def pow_betas(t=10):
    pb1 = pb2 = 1.0
    for _ in range(t):
        pb1 *= 0.9
        pb2 *= 0.999
    return pb1, pb2


class StepData:
    """Host arrays of the step's workloads (also used by the CPU baseline)."""

    def __init__(self, adam_n: int):
        log("generating inputs (numpy default_rng, seeds 0, 4, 5, 6) ...")
        g0 = np.random.default_rng(0)
        self.x0 = g0.uniform(-1, 1, 1024 * 1024).astype(np.float32)
        self.b0 = g0.uniform(-1, 1, 1024).astype(np.float32)
        self.red32 = np.random.default_rng(4).standard_normal(16384 * 4096, dtype=np.float32)
        self.red64 = np.random.default_rng(5).standard_normal(4096 * 4096)
        g6 = np.random.default_rng(6)
        self.adam_n = adam_n
        self.p = g6.uniform(-0.05, 0.05, adam_n).astype(np.float32)
        self.g = g6.standard_normal(adam_n, dtype=np.float32) * np.float32(1e-3)


REDUCE_OPS = ("sum", "max", "magnitude-squared")


def build_step(b: Bench, data: StepData):
    """The workloads of one step, in the order they run.  Returns (ops, adam_op, extra_ops)."""
    s = b.stream
    ops = []
    # configs[3]: Adam
    n = data.adam_n
    p, g = b.upload(data.p), b.upload(data.g)
    m, v = b.alloc(n, "float"), b.alloc(n, "float")
    s.memset(m, 0, 0.0, n)
    s.memset(v, 0, 1e-6, n)
    pb1, pb2 = pow_betas()
    adam = Op("c3_adam", f"configs[3] Adam step, {n} float32 parameters", 28 * n,
              lambda: s.adam_step(1e-3, 0.9, 0.999, 1e-8, pb1, pb2, 1.0, g, p, m, v, n), iters=10)
    ops.append(adam)
    # configs[2]: reductions
    r, c = 16384, 4096
    x32 = b.upload(data.red32)
    o_rows, o_cols = b.alloc(r, "float"), b.alloc(c, "float")
    for op in REDUCE_OPS:
        ops.append(Op(f"c2_{op}_rows_f32", f"configs[2] unary-reduce! :{op} last axis of float32 [{r},{c}]", 4 * r * c + 4 * r,
                      lambda op=op: s.unary_reduce(o_rows, dims([r, 1]), 1.0, x32, dims([r, c]), op)))
        ops.append(Op(f"c2_{op}_cols_f32", f"configs[2] unary-reduce! :{op} axis 0 of float32 [{r},{c}] (transposed view)",
                      4 * r * c + 4 * c,
                      lambda op=op: s.unary_reduce(o_cols, dims([c, 1]), 1.0, x32, dims([c, r], [1, c]), op)))
    q = 4096
    x64 = b.upload(data.red64)
    o64 = b.alloc(q, "double")
    for op in REDUCE_OPS:
        ops.append(Op(f"c2_{op}_rows_f64", f"configs[2] unary-reduce! :{op} last axis of float64 [{q},{q}]", 8 * q * q + 8 * q,
                      lambda op=op: s.unary_reduce(o64, dims([q, 1]), 1.0, x64, dims([q, q]), op)))
        ops.append(Op(f"c2_{op}_cols_f64", f"configs[2] unary-reduce! :{op} axis 0 of float64 [{q},{q}] (transposed view)",
                      8 * q * q + 8 * q,
                      lambda op=op: s.unary_reduce(o64, dims([q, 1]), 1.0, x64, dims([q, q], [1, q]), op)))
    # configs[0]: bias add at its stated shape (8 MiB: cache resident, launch bound)
    x0, b0 = b.upload(data.x0), b.upload(data.b0)
    d0 = b.alloc(1024 * 1024, "float")
    ops.append(Op("c0_bias_add", "configs[0] binary-op! :+ float32 [1024,1024] + [1024] row", 8392704,
                  lambda: s.binary_op(d0, dims([1024, 1024]), x0, dims([1024, 1024]), 1.0, b0, dims([1024]), 1.0,
                                      1024 * 1024, "+"), iters=200))
    # the Adadelta step of configs[3]: timed on its own, not part of the step (the metric names Adam)
    acc_g, acc_d = b.alloc(n, "float"), b.alloc(n, "float")
    s.memset(acc_g, 0, 0.0, n)
    s.memset(acc_d, 0, 0.0, n)
    adadelta = Op("c3_adadelta", f"configs[3] Adadelta step, {n} float32 parameters", 28 * n,
                  lambda: s.adadelta_step(0.05, 1e-6, acc_g, acc_d, 1.0, g, p, n), iters=10)
    return ops, adam, [adadelta]


# ----------------------------------------------------------------------------- others: configs[0] scaled, [1], [4]

def build_others(b: Bench):
    s = b.stream
    ops = []
    rng = np.random.default_rng(0)
    n = 16384
    x = b.upload(rng.standard_normal(n * n, dtype=np.float32))
    bias = b.upload(rng.uniform(-1, 1, n).astype(np.float32))
    d = b.alloc(n * n, "float")
    ops.append(Op("c0_bias_add_scaled", "configs[0] scaled: binary-op! :+ float32 [16384,16384] + [16384] row", 8 * n * n + 4 * n,
                  lambda: s.binary_op(d, dims([n, n]), x, dims([n, n]), 1.0, bias, dims([n]), 1.0, n * n, "+")))
    # configs[1]: transposed views of [8192,8192]
    e = 8192
    ee = e * e
    xs = [b.upload(np.random.default_rng(seed).standard_normal(ee).astype(np.float32)) for seed in (1, 2, 3)]
    cont, view = dims([e, e]), dims([e, e], [1, e])
    dest = d  # reuse (larger than needed)
    ops.append(Op("c1_exp_t", "configs[1] unary-op! :exp on a transposed float32 [8192,8192] view", 8 * ee,
                  lambda: s.unary_op(dest, cont, xs[0], view, 1.0, "exp", ee)))
    ops.append(Op("c1_tanh_t", "configs[1] unary-op! :tanh on a transposed float32 [8192,8192] view", 8 * ee,
                  lambda: s.unary_op(dest, cont, xs[0], view, 1.0, "tanh", ee)))
    ops.append(Op("c1_select_t", "configs[1] ternary-op! :select, three transposed float32 [8192,8192] views", 16 * ee,
                  lambda: s.ternary_op(dest, cont, xs[0], view, 1.0, xs[1], view, 1.0, xs[2], view, 1.0, ee, "select")))
    ops.append(Op("calibration_copy", "calibration: unary-op! :noop, contiguous float32 [8192,8192] (256 MiB in, 256 MiB out)", 8 * ee,
                  lambda: s.unary_op(dest, cont, xs[0], cont, 1.0, "noop", ee)))
    # configs[4]: mixed-dtype image normalise
    shp = [256, 3, 224, 224]
    ni = int(np.prod(shp))
    u8 = b.upload(np.random.default_rng(7).integers(0, 256, ni, dtype=np.uint8))
    f, f2 = b.alloc(ni, "float"), b.alloc(ni, "float")
    mean = b.upload((np.array([0.485, 0.456, 0.406]) * 255).astype(np.float32))
    std = b.upload((np.array([0.229, 0.224, 0.225]) * 255).astype(np.float32))
    ops.append(Op("c4_u8_f32", "configs[4] assign! uint8 -> float32 [256,3,224,224]", 5 * ni,
                  lambda: s.assign(f, dims(shp), u8, dims(shp), ni)))
    ops.append(Op("c4_sub_mean", "configs[4] binary-op! :- per-channel mean [3,1,1]", 8 * ni + 12,
                  lambda: s.binary_op(f2, dims(shp), f, dims(shp), 1.0, mean, dims([3, 1, 1]), -1.0, ni, "+")))
    ops.append(Op("c4_div_std", "configs[4] binary-op! :/ per-channel std [3,1,1]", 8 * ni + 12,
                  lambda: s.binary_op(f2, dims(shp), f, dims(shp), 1.0, std, dims([3, 1, 1]), 1.0, ni, "/")))
    nv = 1 << 26
    i32 = b.upload(np.random.default_rng(8).integers(-2 ** 31, 2 ** 31, nv, dtype=np.int64).astype(np.int32))
    f64 = b.alloc(nv, "double")
    ops.append(Op("c4_i32_f64", "configs[4] assign! int32 -> float64 [64M]", 12 * nv,
                  lambda: s.assign(f64, dims([nv]), i32, dims([nv]), nv)))
    return ops


# ----------------------------------------------------------------------------- the same methods at layer sizes

def build_midsize(b: Bench):
    """The methods of the step at the sizes of one layer of a network (a [4096,4096] float matrix, 64 MiB): the operands
    fit the 256 MiB last-level cache, the calls last 10-70 us, and launch ramps and second launches weigh more than at
    the benchmark's sizes."""
    s = b.stream
    side = 4096
    n = side * side
    rng = np.random.default_rng(11)
    x = b.upload(rng.standard_normal(n, dtype=np.float32))
    g = b.upload(rng.standard_normal(n, dtype=np.float32) * 1e-3)
    m, v, d = b.alloc(n, "float"), b.alloc(n, "float"), b.alloc(n, "float")
    bias = b.upload(rng.standard_normal(side, dtype=np.float32))
    out = b.alloc(side, "float")
    sq, tr = dims([side, side]), dims([side, side], [1, side])
    pb1, pb2 = pow_betas()
    return [
        Op("m_adam", "Adam step, 2^24 float32 parameters", 28 * n,
           lambda: s.adam_step(1e-3, 0.9, 0.999, 1e-8, pb1, pb2, 1.0, g, x, m, v, n)),
        Op("m_bias_add", "binary-op! :+ float32 [4096,4096] + [4096] row", 8 * n + 4 * side,
           lambda: s.binary_op(d, sq, x, sq, 1.0, bias, dims([side]), 1.0, n, "+")),
        Op("m_sum_rows", "unary-reduce! :sum last axis of float32 [4096,4096]", 4 * n + 4 * side,
           lambda: s.unary_reduce(out, dims([side, 1]), 1.0, x, sq, "sum")),
        Op("m_sum_cols", "unary-reduce! :sum axis 0 of float32 [4096,4096] (transposed view)", 4 * n + 4 * side,
           lambda: s.unary_reduce(out, dims([side, 1]), 1.0, x, tr, "sum")),
        Op("m_bias_gradient", "binary-op! :+ accumulate (bias gradient): float32 [4096] += rows of [4096,4096]", 4 * n + 8 * side,
           lambda: s.binary_accum(out, dims([side]), 1.0, x, sq, 1.0, n, "+", False, True)),
        Op("m_exp_t", "unary-op! :exp on a transposed float32 [4096,4096] view", 8 * n,
           lambda: s.unary_op(d, sq, x, tr, 1.0, "exp", n)),
        Op("m_select_t", "ternary-op! :select, three transposed float32 [4096,4096] views", 16 * n,
           lambda: s.ternary_op(d, sq, x, tr, 1.0, g, tr, 1.0, m, tr, 1.0, n, "select")),
        Op("m_softmax", "softmax! float32 [16384,1024]", 8 * n,
           lambda: s.softmax_eltwise(d, dims([16384, 1024]), x, dims([16384, 1024]))),
    ]


# ----------------------------------------------------------------------------- the reference's own sizes

def build_small(b: Bench):
    """The calls of one training step of the networks the reference trains itself (src/cortex/verify/nn/train.clj:185-187:
    batches of 128 images of 784 pixels, ten classes; a [64,32,7,7] activation for the spatial forms).  Everything here is
    bound by the launch: avg_call_us is what one call costs back to back, and c_caller holds the same calls from a
    compiled loop."""
    s = b.stream
    rng = np.random.default_rng(12)
    batch, pixels, classes = 128, 784, 10
    n = batch * pixels
    x = b.upload(rng.standard_normal(n, dtype=np.float32))
    g = b.upload(rng.standard_normal(n, dtype=np.float32) * 1e-3)
    d, m, v = b.alloc(n, "float"), b.alloc(n, "float"), b.alloc(n, "float")
    s.memset(m, 0, 0.0, n)
    s.memset(v, 0, 1e-6, n)
    row = b.upload(rng.standard_normal(pixels, dtype=np.float32))
    out = b.alloc(pixels, "float")
    s.memset(out, 0, 0.0, pixels)
    st = [b.upload(rng.uniform(0.5, 1.5, pixels).astype(np.float32)) for _ in range(8)]
    act, act_t = dims([batch, pixels]), dims([pixels, batch], [1, pixels])
    logits = dims([batch, classes])
    sb, sc, se = 64, 32, 49
    ns = sb * sc * se
    pb1, pb2 = pow_betas()
    it = 200
    return [
        Op("s_bias_add", f"binary-op! :+ float32 [{batch},{pixels}] + [{pixels}] row", 8 * n + 4 * pixels,
           lambda: s.binary_op(d, act, x, act, 1.0, row, dims([pixels]), 1.0, n, "+"), iters=it),
        Op("s_bias_gradient", f"binary-op! :+ accumulate (bias gradient): float32 [{pixels}] += rows of [{batch},{pixels}]",
           4 * n + 8 * pixels, lambda: s.binary_accum(out, dims([pixels]), 1.0, x, act, 1.0, n, "+", False, True), iters=it),
        Op("s_bias_gradient_classes", f"binary-op! :+ accumulate: float32 [{classes}] += rows of [{batch},{classes}]",
           4 * batch * classes + 8 * classes,
           lambda: s.binary_accum(out, dims([classes]), 1.0, x, logits, 1.0, batch * classes, "+", False, True), iters=it),
        Op("s_sum_over_batch", f"unary-reduce! :sum axis 0 of float32 [{batch},{pixels}] (transposed view)", 4 * n + 4 * pixels,
           lambda: s.unary_reduce(out, dims([pixels, 1]), 1.0, x, act_t, "sum"), iters=it),
        Op("s_sum_rows", f"unary-reduce! :sum last axis of float32 [{batch},{pixels}]", 4 * n + 4 * batch,
           lambda: s.unary_reduce(out, dims([batch, 1]), 1.0, x, act, "sum"), iters=it),
        Op("s_softmax", f"softmax! float32 [{batch},{classes}]", 8 * batch * classes,
           lambda: s.softmax_eltwise(d, logits, x, logits), iters=it),
        Op("s_bn_update_eltwise", f"batch-normalize-update-and-apply! eltwise float32 [{batch},{pixels}]", 8 * n,
           lambda: s.batch_normalize_update_and_apply_eltwise(d, x, st[0], st[1], st[4], st[5], 0.9, st[2], st[3], 1e-3,
                                                              batch, pixels), iters=it),
        Op("s_bn_gradients_eltwise", f"batch-normalize-gradients! eltwise float32 [{batch},{pixels}]", 12 * n,
           lambda: s.batch_normalize_gradients_eltwise(d, st[6], st[7], g, d, x, st[0], st[1], st[2], st[3], 1e-3, batch,
                                                       pixels), iters=it),
        Op("s_bn_update_spatial", f"batch-normalize-update-and-apply! spatial float32 [{sb},{sc},7,7]", 8 * ns,
           lambda: s.batch_normalize_update_and_apply_spatial(d, x, st[0], st[1], st[4], st[5], 0.9, st[2], st[3], 1e-3,
                                                              sb, sc, se), iters=it),
        Op("s_bn_gradients_spatial", f"batch-normalize-gradients! spatial float32 [{sb},{sc},7,7]", 12 * ns,
           lambda: s.batch_normalize_gradients_spatial(d, st[6], st[7], g, d, x, st[0], st[1], st[2], st[3], 1e-3, sb, sc,
                                                       se), iters=it),
        Op("s_adam", f"Adam step, {n} float32 parameters (the weights of a [{pixels},{batch}] layer)", 28 * n,
           lambda: s.adam_step(1e-3, 0.9, 0.999, 1e-8, pb1, pb2, 1.0, g, x, m, v, n), iters=it),
    ]


# ----------------------------------------------------------------------------- the constant and accumulate forms

def build_variants(b: Bench):
    """The TensorMath methods of the path that no BASELINE config names: assign-constant!, the accumulate (in place)
    forms and the forms that take constants, each over 2^26 contiguous float32 (256 MiB per stream)."""
    s = b.stream
    n = 1 << 26
    rng = np.random.default_rng(10)
    x = b.upload(rng.standard_normal(n, dtype=np.float32))
    y = b.upload(rng.standard_normal(n, dtype=np.float32))
    d = b.alloc(n, "float")
    flat = dims([n])
    ops = [
        Op("v_assign_constant", "assign-constant! float32 [2^26] (a write stream)", 4 * n,
           lambda: s.assign_constant(d, flat, 1.5, n)),
        Op("v_unary_accum", "unary-accum! :logistic float32 [2^26] (in place)", 8 * n,
           lambda: s.unary_accum(d, flat, 1.0, "logistic", n)),
        Op("v_binary_op_constant", "binary-op-constant! :* float32 [2^26], x * 0.5 with alpha 2", 8 * n,
           lambda: s.binary_op_constant(d, flat, x, flat, 2.0, 0.5, n, "*", False)),
        Op("v_binary_accum_constant", "binary-accum-constant! :max float32 [2^26] (in place, relu)", 8 * n,
           lambda: s.binary_accum_constant(d, flat, 1.0, 0.0, n, "max", False)),
        Op("v_binary_accum_same_shape", "binary-accum! :+ float32 [2^26] += y (destination is the max shape: no ordering needed)", 12 * n,
           lambda: s.binary_accum(d, flat, 1.0, y, flat, 1.0, n, "+", False, False)),
        Op("v_ternary_constant", "ternary-op! :select float32 [2^26], x >= 0 ? y : 0 (one constant)", 12 * n,
           lambda: s.ternary_op_constant(d, flat, x, flat, 1.0, y, flat, 1.0, 0.0, n, "select", ["x", "z", "y"])),
        Op("v_ternary_constant_constant", "ternary-op! :select float32 [2^26], x >= 0 ? 1 : 0 (two constants)", 8 * n,
           lambda: s.ternary_op_constant_constant(d, flat, x, flat, 1.0, 0.0, 1.0, n, "select", ["x", "y", "z"])),
    ]
    return ops


# ----------------------------------------------------------------------------- patterns off the fast families

class _Tensor:
    """What the driver's dimension maps accept as an index tensor: an object with a `.buffer`."""

    def __init__(self, buffer):
        self.buffer = buffer


def build_patterns(b: Bench):
    """Access patterns that real cortex callers produce beside the contiguous / broadcast / transposed
    ones (the census of the tensor layer's callers): gather and scatter-add through an index tensor
    (center loss), strided vectors (ct/columns, select :all k), planar <-> interleaved images, and
    accumulation into a broadcast destination with an op other than :+."""
    s = b.stream
    ops = []
    rng = np.random.default_rng(21)
    # center loss (loss/center.clj:32, 75, 92): rows of [1000,512] centers selected by 4096 labels
    n_cls, width, batch = 1000, 512, 4096
    centers = b.upload(rng.standard_normal(n_cls * width, dtype=np.float32))
    labels = b.upload(rng.integers(0, n_cls, batch, dtype=np.int64).astype(np.int32))
    feats = b.upload(rng.standard_normal(batch * width, dtype=np.float32))
    gathered = b.alloc(batch * width, "float")
    idx_dims = {"shape": [_Tensor(labels), width], "strides": [width, 1]}
    ops.append(Op("p_gather_rows", f"assign! gather: float32 [{batch},{width}] <- centers [{n_cls},{width}] through {batch} labels",
                  8 * batch * width + 4 * batch,
                  lambda: s.assign(gathered, dims([batch, width]), centers, idx_dims, batch * width)))
    ops.append(Op("p_scatter_add_rows", f"binary-op! :+ scatter-add: centers [{n_cls},{width}] (indexed by {batch} labels) += float32 [{batch},{width}]",
                  4 * batch * width + 8 * min(batch, n_cls) * width + 4 * batch,
                  lambda: s.binary_accum(centers, idx_dims, 1.0, feats, dims([batch, width]), 1e-3, batch * width, "+", False, True),
                  iters=5))
    # large gather: 2^16 rows of 1024 floats out of 2^15
    rows_src, rows_out, w2 = 1 << 15, 1 << 16, 1024
    table = b.upload(rng.standard_normal(rows_src * w2, dtype=np.float32))
    picks = b.upload(rng.integers(0, rows_src, rows_out, dtype=np.int64).astype(np.int32))
    out2 = b.alloc(rows_out * w2, "float")
    big_idx = {"shape": [_Tensor(picks), w2], "strides": [w2, 1]}
    ops.append(Op("p_gather_rows_large", f"assign! gather: float32 [{rows_out},{w2}] <- table [{rows_src},{w2}] through an index tensor",
                  8 * rows_out * w2 + 4 * rows_out,
                  lambda: s.assign(out2, dims([rows_out, w2]), table, big_idx, rows_out * w2)))
    scat = b.upload(rng.standard_normal(rows_src * w2, dtype=np.float32))
    upd = b.upload(rng.standard_normal(rows_out * w2, dtype=np.float32))
    scat_idx = {"shape": [_Tensor(picks), w2], "strides": [w2, 1]}
    ops.append(Op("p_scatter_add_rows_large", f"binary-op! :+ scatter-add: table [{rows_src},{w2}] (indexed by {rows_out} entries) += float32 [{rows_out},{w2}]",
                  4 * rows_out * w2 + 8 * rows_src * w2 + 4 * rows_out,
                  lambda: s.binary_accum(scat, scat_idx, 1.0, upd, dims([rows_out, w2]), 1e-3, rows_out * w2, "+", False, True),
                  iters=10))
    # strided vector: one column of a [2^22, 16] matrix (ct/columns, select :all k)
    rows_v, pitch = 1 << 22, 16
    mat = b.upload(rng.standard_normal(rows_v * pitch, dtype=np.float32))
    colv = b.alloc(rows_v, "float")
    ops.append(Op("p_strided_vector", f"assign! strided vector: float32 [{rows_v}] <- column of [{rows_v},{pitch}] (stride {pitch}; "
                                      "every 64-byte line of the matrix is fetched for one float: the memory system moves 8.5x these bytes)",
                  8 * rows_v,  # the elements asked for; the lines they sit in are 16 times that
                  lambda: s.assign(colv, dims([rows_v]), mat, dims([rows_v], [pitch]), rows_v)))
    # blocks of a wider matrix copied out (ct/submatrix, tensor.clj:490-513): rows off the 16-byte grid
    sub_rows, sub_w, sub_pitch = 65536, 999, 1024
    wide = b.upload(rng.standard_normal(sub_rows * sub_pitch, dtype=np.float32))
    block = b.alloc(sub_rows * sub_w, "float")
    ops.append(Op("p_submatrix_copy", f"assign! float32 [{sub_rows},{sub_w}] <- block of a pitch-{sub_pitch} matrix", 8 * sub_rows * sub_w,
                  lambda: s.assign(block, dims([sub_rows, sub_w]), wide, dims([sub_rows, sub_w], [sub_pitch, 1]), sub_rows * sub_w)))
    ops.append(Op("p_submatrix_store", f"assign! block of a pitch-{sub_pitch} matrix <- float32 [{sub_rows},{sub_w}]", 8 * sub_rows * sub_w,
                  lambda: s.assign(wide, dims([sub_rows, sub_w], [sub_pitch, 1]), block, dims([sub_rows, sub_w]), sub_rows * sub_w)))
    short_rows, short_w, short_pitch = 1 << 22, 10, 16
    ops.append(Op("p_short_rows_of_pitch", f"assign! float32 [{short_rows},{short_w}] <- rows of {short_w} out of a pitch of {short_pitch} "
                                           "(the memory system moves whole 64-byte lines: 1.3x these bytes)", 8 * short_rows * short_w,
                  lambda: s.assign(block, dims([short_rows, short_w]), wide, dims([short_rows, short_w], [short_pitch, 1]),
                                   short_rows * short_w)))
    # planar <-> interleaved images (verify/tensor.clj:668-684, 785-805)
    nb, hh, ww, ch = 256, 224, 224, 3
    npx = nb * hh * ww * ch
    inter = b.upload(rng.standard_normal(npx, dtype=np.float32))
    planar = b.alloc(npx, "float")
    planar_dims = dims([nb, ch, hh, ww])
    inter_as_planar = dims([nb, ch, hh, ww], [hh * ww * ch, 1, ww * ch, ch])
    ops.append(Op("p_interleaved_to_planar", f"assign! planar [{nb},{ch},{hh},{ww}] <- interleaved [{nb},{hh},{ww},{ch}] float32",
                  8 * npx, lambda: s.assign(planar, planar_dims, inter, inter_as_planar, npx)))
    inter_dims = dims([nb, hh, ww, ch])
    planar_as_inter = dims([nb, hh, ww, ch], [ch * hh * ww, ww, 1, hh * ww])
    ops.append(Op("p_planar_to_interleaved", f"assign! interleaved [{nb},{hh},{ww},{ch}] <- planar [{nb},{ch},{hh},{ww}] float32",
                  8 * npx, lambda: s.assign(inter, inter_dims, planar, planar_as_inter, npx)))
    # accumulate into a broadcast destination with :max (owner kernel) and with :+ (staged sums)
    bb, kk = 16384, 4096
    y = b.upload(rng.standard_normal(bb * kk, dtype=np.float32))
    acc = b.alloc(kk, "float")
    s.memset(acc, 0, 0.0, kk)
    ops.append(Op("p_accum_max_rows", f"binary-op! :max accumulate: float32 [{kk}] <- max over rows of [{bb},{kk}]",
                  4 * bb * kk + 8 * kk,
                  lambda: s.binary_accum(acc, dims([kk]), 1.0, y, dims([bb, kk]), 1.0, bb * kk, "max", False, True), iters=10))
    ops.append(Op("p_accum_sum_rows", f"binary-op! :+ accumulate (bias gradient): float32 [{kk}] += rows of [{bb},{kk}]",
                  4 * bb * kk + 8 * kk,
                  lambda: s.binary_accum(acc, dims([kk]), 1.0, y, dims([bb, kk]), 1.0, bb * kk, "+", False, True)))
    # the same destination under operations with no staged form: every destination element is a serial chain of
    # 16384 steps, each rounded to float (streamed through LDS, one lane per chain)
    ones = b.upload((1.0 + 1e-3 * rng.standard_normal(bb * kk)).astype(np.float32))
    ops.append(Op("p_accum_mul_rows", f"binary-op! :* accumulate: float32 [{kk}] <- product over rows of [{bb},{kk}] (one float "
                                      "multiplication per step of a chain)",
                  4 * bb * kk + 8 * kk,
                  lambda: s.binary_accum(acc, dims([kk]), 1.0, ones, dims([bb, kk]), 1.0, bb * kk, "*", False, True), iters=10))
    ops.append(Op("p_accum_decay_rows", f"binary-op! :+ accumulate with dest_alpha 0.9: float32 [{kk}] <- rows of [{bb},{kk}] "
                                        "(a step is widen, multiply, add, round: four dependent instructions)",
                  4 * bb * kk + 8 * kk,
                  lambda: s.binary_accum(acc, dims([kk]), 0.9, y, dims([bb, kk]), 1.0, bb * kk, "+", False, True), iters=10))
    return ops


# ----------------------------------------------------------------------------- adjacent TensorMath methods

def build_adjacent(b: Bench):
    """activation-gradient!, softmax!, batch normalization, rand!, local response normalization, gemv!: HBM-bound like the hot path.
    Bytes are algorithmic (every operand read once, every result written once) although the
    batch-normalization forms that need batch statistics read their operands twice."""
    s = b.stream
    ops = []
    rng = np.random.default_rng(9)
    n = 1 << 27
    x = b.upload(rng.standard_normal(n, dtype=np.float32))
    g = b.upload(rng.standard_normal(n, dtype=np.float32))
    o = b.alloc(n, "float")
    ops.append(Op("a_actgrad_tanh", "activation-gradient! :tanh float32 [2^27]", 12 * n,
                  lambda: s.activation_gradient(o, dims([n]), g, dims([n]), x, dims([n]), "tanh", n)))
    for k in (16, 1024):
        rows = n // k
        ops.append(Op(f"a_softmax_{k}", f"softmax! float32 [{rows},{k}]", 8 * n,
                      lambda rows=rows, k=k: s.softmax_eltwise(o, dims([rows, k]), x, dims([rows, k]))))
    bq, cq, eq = 64, 21, 65536
    ops.append(Op("a_softmax_spatial", f"softmax! spatial float32 [{bq},{cq},{eq}]", 8 * bq * cq * eq,
                  lambda: s.softmax_spatial(o, dims([bq, cq, eq]), x, dims([bq, cq, eq]))))
    ops.append(Op("a_rand_gaussian", "rand! gaussian float32 [2^27]", 4 * n,
                  lambda: s.rand(o, dims([n]), {"type": "gaussian", "mean": 0.0, "variance": 1.0})))
    ops.append(Op("a_rand_flat", "rand! flat float32 [2^27]", 4 * n,
                  lambda: s.rand(o, dims([n]), {"type": "flat", "minimum": 0.0, "maximum": 1.0})))
    # the bernoulli dropout mask (compute/nn/layers.clj:170-195): the reference's chain of tensor calls (rand!, then
    # ternary-op! :select in place; assign! drops out when the network runs in float) against the one-launch form
    prob = 0.9
    def chain():
        s.rand(o, dims([n]), {"type": "flat", "minimum": float(np.float32(prob)) - 1.0, "maximum": float(np.float32(prob))})
        s.ternary_op_constant_constant(o, dims([n]), o, dims([n]), 1.0, 0.0, 1.0 / prob, n, "select", ["x", "y", "z"])
    ops.append(Op("a_dropout_chain", "dropout mask float32 [2^27]: rand! + ternary-op! :select (the reference's chain; moves 12 B/element)", 4 * n, chain))
    ops.append(Op("a_dropout_fused", "dropout mask float32 [2^27]: ct_dropout_bernoulli_mask (one launch, same stored values)", 4 * n,
                  lambda: s.dropout_bernoulli_mask(o, None, prob)))
    bb, cc, ee = 64, 256, 3136
    nn_ = bb * cc * ee
    st = [b.upload(rng.uniform(0.5, 1.5, cc).astype(np.float32)) for _ in range(8)]
    ops.append(Op("a_bn_apply", f"batch-normalize! spatial float32 [{bb},{cc},{ee}]", 8 * nn_,
                  lambda: s.batch_normalize_spatial(o, x, st[0], st[1], st[2], st[3], 1e-3, bb, cc, ee)))
    ops.append(Op("a_bn_update", f"batch-normalize-update-and-apply! spatial float32 [{bb},{cc},{ee}] (moves 12 B/element)", 8 * nn_,
                  lambda: s.batch_normalize_update_and_apply_spatial(o, x, st[0], st[1], st[4], st[5], 0.9, st[2], st[3],
                                                                     1e-3, bb, cc, ee)))
    ops.append(Op("a_bn_gradients", f"batch-normalize-gradients! spatial float32 [{bb},{cc},{ee}] (moves 20 B/element)", 12 * nn_,
                  lambda: s.batch_normalize_gradients_spatial(o, st[6], st[7], g, o, x, st[0], st[1], st[2], st[3], 1e-3,
                                                              bb, cc, ee)))
    # local response normalization across the channels (AlexNet's n 5, k 2, alpha 1e-4, beta 0.75: the reference's defaults)
    lrn = {"n": 5, "k": 2.0, "alpha": 1e-4, "beta": 0.75}
    hw = 56
    o2 = b.alloc(nn_, "float")
    ops.append(Op("a_lrn_forward", f"lrn-forward! float32 [{bb},{cc},{hw},{hw}] n 5", 8 * nn_,
                  lambda: s.lrn_forward(o, dims([bb, cc, hw, hw]), x, dims([bb, cc, hw, hw]), lrn)))
    ops.append(Op("a_lrn_backward", f"lrn-backward! float32 [{bb},{cc},{hw},{hw}] n 5", 16 * nn_,
                  lambda: s.lrn_backward(o2, dims([bb, cc, hw, hw]), o, dims([bb, cc, hw, hw]), x, dims([bb, cc, hw, hw]),
                                         g, dims([bb, cc, hw, hw]), lrn)))
    mm = 8192
    a_ = b.upload(rng.standard_normal(mm * mm, dtype=np.float32))
    xv = b.upload(rng.standard_normal(mm, dtype=np.float32))
    yv = b.alloc(mm, "float")
    for trans, label in ((False, "A x"), (True, "A^T x")):
        ops.append(Op(f"a_gemv_{'t' if trans else 'n'}", f"gemv! float32 [{mm},{mm}] {label}", 4 * mm * mm,
                      lambda trans=trans: s.gemv(yv, 1, trans, 1.0, a_, mm, mm, mm, xv, 1, 0.0)))
    return ops


# ----------------------------------------------------------------------------- CPU baseline

def cpu_baseline(data: StepData) -> dict:
    """Times the CPU oracle on full steps of the same workload (about ten seconds)."""
    from cortex_amd import capi
    from oracle import binding as ob

    p_ = lambda a: a.ctypes.data
    n = data.adam_n
    params, grads = data.p.copy(), data.g
    m = np.zeros(n, np.float32)
    v = np.full(n, 1e-6, np.float32)
    pb1, pb2 = pow_betas()
    r, c, q = 16384, 4096, 4096
    o32, o64 = np.zeros(r, np.float32), np.zeros(q, np.float64)
    d0 = np.zeros(1024 * 1024, np.float32)
    D = lambda shape, strides: C.byref(capi.make_dims(shape, strides))

    def one_step():
        ob.call("adam_step", capi.F32, 1e-3, 0.9, 0.999, 1e-8, pb1, pb2, 1.0, p_(grads), p_(params), p_(m), p_(v), n)
        for op in REDUCE_OPS:
            code = capi.REDUCE_OPS[op]
            ob.call("unary_reduce", p_(o32), D([r, 1], [1, 1]), 1.0, p_(data.red32), D([r, c], [c, 1]), code, capi.F32)
            ob.call("unary_reduce", p_(o32), D([c, 1], [1, 1]), 1.0, p_(data.red32), D([c, r], [1, c]), code, capi.F32)
        for op in REDUCE_OPS:
            code = capi.REDUCE_OPS[op]
            ob.call("unary_reduce", p_(o64), D([q, 1], [1, 1]), 1.0, p_(data.red64), D([q, q], [q, 1]), code, capi.F64)
            ob.call("unary_reduce", p_(o64), D([q, 1], [1, 1]), 1.0, p_(data.red64), D([q, q], [1, q]), code, capi.F64)
        ob.call("binary_op", p_(d0), D([1024, 1024], [1024, 1]), p_(data.x0), D([1024, 1024], [1024, 1]), 1.0, p_(data.b0),
                D([1024], [1]), 1.0, 1024 * 1024, capi.BINARY_OPS["+"], capi.F32)

    one_step()  # first touch of the output pages
    steps, t0 = 0, time.perf_counter()
    while steps < 2 or (time.perf_counter() - t0 < 10.0 and steps < 100):
        one_step()
        steps += 1
    dt = time.perf_counter() - t0
    step_bytes = 28 * n + 6 * (4 * r * c) + 3 * 4 * (r + c) + 6 * (8 * q * q + 8 * q) + 8392704
    return {"value": round(steps * step_bytes / dt / 1e9, 3), "unit": "GB/s", "cores": ob.num_threads(), "kind": "port",
            "sample": f"{steps} full steps (Adam over {n} float32 parameters, the twelve configs[2] reductions, the configs[0] "
                      f"bias add) in {dt:.2f} s; C++ restatement of the cortex CPU backend, OpenMP over the index space the "
                      "reference hands to parallel-for"}


# ----------------------------------------------------------------------------- rocprofv3 output -> profiles/

def c_caller_rates() -> dict | None:
    """Builds tests/c_abi/callrate.c against the library and runs it as a child process: what a call
    costs a compiled caller (no interpreter between the loop and the C ABI).  None when it cannot be built."""
    import subprocess
    import tempfile
    src = ROOT / "tests" / "c_abi" / "callrate.c"
    libdir = ROOT / "cortex_amd"
    with tempfile.TemporaryDirectory() as tmp:
        exe = Path(tmp) / "callrate"
        cmd = ["gcc", "-std=c99", "-O1", f"-I{ROOT / 'include'}", str(src), "-o", str(exe), f"-L{libdir}", "-lcortex_hip",
               "-lm", f"-Wl,-rpath,{libdir}"]
        try:
            if subprocess.run(cmd, capture_output=True, text=True, timeout=120).returncode != 0:
                return None
            res = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
            if res.returncode != 0:
                return None
            out = json.loads(res.stdout.strip().splitlines()[-1])
        except (OSError, ValueError, subprocess.SubprocessError):
            return None
    out["note"] = ("a C99 loop over the C ABI (tests/c_abi/callrate.c), run as a child process: host_us is the loop's own time per "
                   "call, sustained_us includes the final wait for the stream; the interpreter's share of ops[...].host_us is the "
                   "difference to these")
    return out


def short_kernel_name(n: str) -> str:
    n = re.sub(r"^void ", "", n.strip('"')).replace("(anonymous namespace)::", "").replace("cthip::", "")
    depth = 0
    for i, ch in enumerate(n):
        if ch == "<":
            depth += 1
        elif ch == ">":
            depth -= 1
        elif ch == "(" and depth == 0:
            return n[:i]
    return n


MARKER = re.compile(r"ConstantF<signed char>")


def _segments(rows, plan, value_of):
    """Splits the dispatches (in dispatch order) at the marker launches; returns, per plan segment,
    {kernel short name: [values]} in first-seen order."""
    out, cur = [], None
    for row in rows:
        name = short_kernel_name(row["Kernel_Name"])
        if MARKER.search(name):
            cur = collections.OrderedDict()
            out.append(cur)
            continue
        if cur is not None:
            cur.setdefault(name, []).append(value_of(row))
    if len(out) != len(plan):
        raise SystemExit(f"profile has {len(out)} marked segments, the plan lists {len(plan)}")
    return out


def _read_sorted(path, key):
    with open(path) as fh:
        rows = list(csv.DictReader(fh))
    rows.sort(key=lambda r_: int(r_[key]))
    return rows


def summarize(prof_dir: str, out_dir: str) -> None:
    """Reads DIR/{trace,fetch,write}/*.csv and DIR/{trace,fetch,write}_plan.json (written by three runs of
    this program under rocprofv3, see the header of the summary) and writes OUT/bench_trace_and_traffic.txt
    and OUT/traffic.json."""
    d, out = Path(prof_dir), Path(out_dir)
    out.mkdir(parents=True, exist_ok=True)
    plans = {k: json.loads((d / f"{k}_plan.json").read_text()) for k in ("trace", "fetch", "write")}
    shas = {p["csrc_sha256"] for p in plans.values()}
    if len(shas) != 1:
        raise SystemExit("the three profile runs were made on different sources")
    trace = _segments(_read_sorted(glob.glob(str(d / "trace" / "*kernel_trace.csv"))[0], "Start_Timestamp"),
                      plans["trace"]["segments"],
                      lambda r_: (int(r_["End_Timestamp"]) - int(r_["Start_Timestamp"])) / 1e3)
    pmc = {}
    for kind in ("fetch", "write"):
        pmc[kind] = _segments(_read_sorted(glob.glob(str(d / kind / "*counter_collection.csv"))[0], "Dispatch_Id"),
                              plans[kind]["segments"], lambda r_: float(r_["Counter_Value"]))

    def seg_index(plan, key):
        return [i for i, s_ in enumerate(plan["segments"]) if s_["key"] == key]

    cal_kib = 8192 * 8192 * 4 / 1024
    if seg_index(plans["fetch"], "calibration_copy") and seg_index(plans["write"], "calibration_copy"):
        cal_f = pmc["fetch"][seg_index(plans["fetch"], "calibration_copy")[0]]
        cal_w = pmc["write"][seg_index(plans["write"], "calibration_copy")[0]]
        f_raw = float(np.mean(next(iter(cal_f.values()))))
        w_raw = float(np.mean(next(iter(cal_w.values()))))
    else:  # a run without the section that holds the calibration copy: the factors it measured before
        f_raw, w_raw = cal_kib / 2.0, cal_kib
    f_fac, w_fac = cal_kib / f_raw, cal_kib / w_raw

    lines = []
    traffic = {}
    for i, seg in enumerate(plans["trace"]["segments"]):
        key, calls, alg = seg["key"], seg["calls"], seg["algorithmic_bytes"]
        if key.startswith("_"):
            continue
        kernels = trace[i]
        fi, wi = seg_index(plans["fetch"], key), seg_index(plans["write"], key)
        fseg = pmc["fetch"][fi[0]] if fi else {}
        wseg = pmc["write"][wi[0]] if wi else {}
        fcalls = plans["fetch"]["segments"][fi[0]]["calls"] if fi else 1
        wcalls = plans["write"]["segments"][wi[0]]["calls"] if wi else 1
        per_call_us, per_call_bytes = 0.0, 0.0
        rows = []
        call_sums = np.zeros(calls)     # kernel time of each call, when every kernel runs a whole number of times per call
        for name, durs in kernels.items():
            per = len(durs) / calls
            fk = float(np.sum(fseg.get(name, [0.0]))) / fcalls
            wk = float(np.sum(wseg.get(name, [0.0]))) / wcalls
            per_call_us += float(np.sum(durs)) / calls
            per_call_bytes += (fk * f_fac + wk * w_fac) * 1024
            if call_sums is not None and len(durs) % calls == 0:
                call_sums = call_sums + np.asarray(durs).reshape(calls, -1).sum(axis=1)
            else:
                call_sums = None
            rows.append("      %-70s %5.2f/call %9.2f %9.2f %9.2f %9.2f %12.1f %12.1f" % (
                name[:70], per, float(np.mean(durs)), float(np.median(durs)), float(np.min(durs)), float(np.max(durs)), fk, wk))
        if key == "step":
            lines.append("%s\n    %d steps; kernels of the timed region (avg / median / best / max us per dispatch; FETCH / WRITE KiB per step):" % (seg["label"], calls))
            lines.extend(rows)
            continue
        rate = alg / per_call_us / 1e3 if per_call_us > 0 else 0.0
        spread = ""
        if call_sums is not None and calls > 0:
            med, best = float(np.median(call_sums)), float(np.min(call_sums))
            spread = " (median %.2f us = %.1f %%, best %.2f us = %.1f %%)" % (med, alg / med / 8e4, best, alg / best / 8e4)
        lines.append("%s\n    key %s: %d calls, kernel time %.2f us per call = %.0f GB/s = %.1f %% of 8 TB/s%s; HBM traffic %.0f bytes per call "
                     "= %.4f x the %d algorithmic bytes" % (seg["label"], key, calls, per_call_us, rate, rate / 80, spread,
                                                            per_call_bytes, per_call_bytes / alg, alg))
        lines.extend(rows)
        traffic[key] = {"traffic": int(round(per_call_bytes)), "kernel_us": round(per_call_us, 2),
                        "kernels": [name[:100] for name in kernels], "algorithmic_bytes": alg}
        if call_sums is not None and calls > 0:
            traffic[key]["kernel_us_median"] = round(float(np.median(call_sums)), 2)
            traffic[key]["kernel_us_best"] = round(float(np.min(call_sums)), 2)

    sha = shas.pop()
    head = f"""rocprofv3 summary of bench.py on one MI355X (gfx950): every workload of the step, the other BASELINE configs, the
access patterns off the fast kernel families and the adjacent TensorMath methods.  Kernel sources sha256 {sha[:16]}.

Commands (from the repository root, one rocprofv3 run each; P = gpurun_out/prof):
  cd /tmp && export TMPDIR=/tmp && cd <repo>
  rocprofv3 --kernel-trace --stats --output-format csv -d P/trace -o bench -- python3 bench.py --steps 20 --no-cpu --profile-plan P/trace_plan.json
  rocprofv3 --pmc FETCH_SIZE --output-format csv -d P/fetch -o bench -- python3 bench.py --steps 3 --warmup 1 --no-cpu --profile-plan P/fetch_plan.json
  rocprofv3 --pmc WRITE_SIZE --output-format csv -d P/write -o bench -- python3 bench.py --steps 3 --warmup 1 --no-cpu --profile-plan P/write_plan.json
  python3 bench.py --summarize P --out profiles

With --profile-plan every timed segment of the run starts with a one-byte fill, and the dispatches between two such markers
belong to one workload: durations and counters are attributed by dispatch order, not by kernel name.
Per kernel: launches per call, then avg / median / best / max duration in microseconds (kernel trace), then FETCH_SIZE and
WRITE_SIZE in KiB per call.  Per workload: the average kernel time of a call, and the median and the best call.  HBM traffic = FETCH x {f_fac:.4f} + WRITE x {w_fac:.4f}: the factors make the calibration copy (exactly
{cal_kib:.0f} KiB each way) read {cal_kib:.0f}; FETCH_SIZE reported {f_raw:.1f} KiB for it (it counts half the bytes on this part),
WRITE_SIZE {w_raw:.1f} KiB.  GB/s = algorithmic bytes / summed kernel time of one call; bench.py's own HIP-event figures
(avg_call_us) also contain the gaps between dispatches.

"""
    (out / "bench_trace_and_traffic.txt").write_text(head + "\n".join(lines) + "\n")
    (out / "traffic.json").write_text(json.dumps({
        "csrc_sha256": sha, "fetch_factor": round(f_fac, 6), "write_factor": round(w_fac, 6),
        "source": "profiles/bench_trace_and_traffic.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by the calibration copy)",
        "ops": traffic}, indent=1) + "\n")
    print((out / "bench_trace_and_traffic.txt").read_text())


def summarize_counters(run_dir: str, out_file: str) -> None:
    """Averages every counter of one `rocprofv3 --pmc ...` run of this program per workload and kernel:
    reads RUN/plan.json (written by --profile-plan) and RUN/*counter_collection.csv, writes a text table."""
    d = Path(run_dir)
    plan = json.loads((d / "plan.json").read_text())["segments"]
    rows = _read_sorted(glob.glob(str(d / "*counter_collection.csv"))[0], "Dispatch_Id")
    dispatches = collections.OrderedDict()
    for r_ in rows:
        rec = dispatches.setdefault(int(r_["Dispatch_Id"]), {"Kernel_Name": r_["Kernel_Name"], "c": {}})
        rec["c"][r_["Counter_Name"]] = float(r_["Counter_Value"])
    per_counter = {}
    names = sorted({c for rec in dispatches.values() for c in rec["c"]})
    for c in names:
        segs = _segments(dispatches.values(), plan, lambda rec, c=c: rec["c"].get(c, 0.0))
        per_counter[c] = segs
    lines = ["per dispatch averages; columns: " + "  ".join(names), ""]
    for i, seg in enumerate(plan):
        if seg["key"].startswith("_") or seg["key"] == "step":
            continue
        kernels = per_counter[names[0]][i]
        for kname in kernels:
            vals = ["%.4g" % float(np.mean(per_counter[c][i].get(kname, [0.0]))) for c in names]
            lines.append("%-22s %-60s %s" % (seg["key"], kname[:60], "  ".join(vals)))
    Path(out_file).write_text("\n".join(lines) + "\n")
    print("\n".join(lines))


# ----------------------------------------------------------------------------- main

# ----------------------------------------------------------------------------- the one line on stdout

FINAL_LINE_LIMIT = 4096  # characters; what reads the line keeps only the end of this program's output

# (section, key of the workload inside it) per BASELINE config, in the order the configs are listed
CONFIG_FRACS = (
    ("c0_bias_add_1024", "ops", "c0_bias_add"), ("c0_bias_add_16384", "others", "c0_bias_add_scaled"),
    ("c1_exp_t", "others", "c1_exp_t"), ("c1_tanh_t", "others", "c1_tanh_t"), ("c1_select_t", "others", "c1_select_t"),
    ("c2_sum_rows_f32", "ops", "c2_sum_rows_f32"), ("c2_sum_cols_f32", "ops", "c2_sum_cols_f32"),
    ("c2_max_rows_f32", "ops", "c2_max_rows_f32"), ("c2_max_cols_f32", "ops", "c2_max_cols_f32"),
    ("c2_magsq_rows_f32", "ops", "c2_magnitude-squared_rows_f32"), ("c2_magsq_cols_f32", "ops", "c2_magnitude-squared_cols_f32"),
    ("c2_sum_rows_f64", "ops", "c2_sum_rows_f64"), ("c2_sum_cols_f64", "ops", "c2_sum_cols_f64"),
    ("c2_max_rows_f64", "ops", "c2_max_rows_f64"), ("c2_max_cols_f64", "ops", "c2_max_cols_f64"),
    ("c2_magsq_rows_f64", "ops", "c2_magnitude-squared_rows_f64"), ("c2_magsq_cols_f64", "ops", "c2_magnitude-squared_cols_f64"),
    ("c3_adam", "ops", "c3_adam"), ("c3_adadelta", "ops", "c3_adadelta"),
    ("c4_u8_f32", "others", "c4_u8_f32"), ("c4_sub_mean", "others", "c4_sub_mean"), ("c4_div_std", "others", "c4_div_std"),
    ("c4_i32_f64", "others", "c4_i32_f64"),
)


def final_line(result: dict) -> dict:
    """The object printed as the last line of stdout: the headline fields, `roofline`, `cpu_baseline` and one fraction
    of the HBM peak per BASELINE config (each workload timed on its own, back to back).  Everything else the run
    measured stays in the detail file.  Raises if the line would outgrow FINAL_LINE_LIMIT."""
    head = ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline",
            "dtype", "data", "config", "roofline")
    out = collections.OrderedDict((k, result[k]) for k in head)
    if result.get("cpu_baseline") is not None:
        out["cpu_baseline"] = result["cpu_baseline"]
    fracs = collections.OrderedDict()
    for name, section, key in CONFIG_FRACS:
        block = next((blk for blk in result.get(section, {}).values() if blk.get("key") == key), None)
        if block is not None:
            fracs[name] = block["frac"]
    out["frac_of_peak_by_config"] = fracs
    size = len(json.dumps(out))
    if size >= FINAL_LINE_LIMIT:
        raise RuntimeError(f"the final line has {size} characters; the limit is {FINAL_LINE_LIMIT}")
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--sections", default=",".join(SECTIONS), help="comma-separated subset of " + ",".join(SECTIONS))
    ap.add_argument("--no-extras", action="store_true", help="only the headline step")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--adam-n", type=int, default=1 << 28, help="Adam parameter count (2^28 is the benchmark)")
    ap.add_argument("--profile-plan", default=None, help="write the segment plan here and mark segments (for rocprofv3 runs)")
    ap.add_argument("--summarize", default=None, help="directory holding trace/ fetch/ write/ rocprofv3 output")
    ap.add_argument("--summarize-counters", default=None,
                    help="directory of one rocprofv3 --pmc run (plan.json + *counter_collection.csv): per-workload averages")
    ap.add_argument("--out", default=str(ROOT / "profiles"))
    ap.add_argument("--detail", default=str(ROOT / "gpurun_out" / "bench_detail.json"),
                    help="file that receives every section in full (the last stdout line carries the headline only)")
    args = ap.parse_args()
    if args.summarize:
        summarize(args.summarize, args.out)
        return 0
    if args.summarize_counters:
        summarize_counters(args.summarize_counters, str(Path(args.out) / "counters.txt"))
        return 0
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path has no cross-GPU exchange); "
              f"--gpus {args.gpus} is not supported", file=sys.stderr)
        return 2
    sections = ["headline"] if args.no_extras else [s_ for s_ in args.sections.split(",") if s_]

    b = Bench(args.profile_plan)
    data = StepData(args.adam_n)
    step_ops, adam, extra = build_step(b, data)
    step_bytes = sum(op.nbytes for op in step_ops)

    adam_events = []

    def step(record: bool) -> None:
        for op in step_ops:
            if record and op is adam:
                e0 = b.timer.mark()
                op.fn()
                adam_events.append((e0, b.timer.mark()))
            else:
                op.fn()

    for _ in range(args.warmup):
        step(False)
    b.stream.sync()
    b.segment("step", "the timed region: Adam, twelve reductions, bias add per step", args.steps, step_bytes)
    t_host0 = time.perf_counter()
    e_start = b.timer.mark()
    for _ in range(args.steps):
        step(True)
    e_stop = b.timer.mark()
    total_ms = b.timer.elapsed_ms(e_start, e_stop)
    b.stream.sync()
    wall_ms = (time.perf_counter() - t_host0) * 1e3
    adam_ms = float(np.mean([b.timer.elapsed_ms(a_, b_) for a_, b_ in adam_events]))
    for a_, b_ in adam_events:
        b.timer.free(a_, b_)
    b.timer.free(e_start, e_stop)

    ms_per_step = total_ms / args.steps
    value = gbs(step_bytes, ms_per_step)

    log("timing every workload of the step on its own ...")
    ops_out = collections.OrderedDict()
    for op in step_ops + extra:
        ops_out[op.label] = b.time_op(op)
    adam.kernel = ops_out[adam.label]["kernel"]
    roof = adam_roofline(adam, adam_ms, b.traffic.get(adam.key), b.traffic_note)
    c0 = ops_out[step_ops[-1].label]
    c0["note"] = ("8 MiB, cache resident: avg_call_us is the GPU timeline per call with launches back to back, host_us the "
                  "time this program needs to submit one call (Python + ctypes + launch); when the two agree the loop is "
                  "bound by the host, and kernel_us_rocprof is what the kernel itself takes")

    result = headline(args.steps, args.warmup, args.adam_n, step_bytes, ms_per_step, wall_ms / args.steps)
    result["roofline"] = roof
    result["ops"] = ops_out
    builders = {"others": build_others, "midsize": build_midsize, "small": build_small, "variants": build_variants,
                "patterns": build_patterns, "adjacent": build_adjacent}
    for name in ("others", "midsize", "small", "variants", "patterns", "adjacent"):
        if name not in sections:
            continue
        log(f"timing section '{name}' ...")
        sect = collections.OrderedDict()
        b.segment("_setup_" + name, "fills that prepare the section's buffers", 1, 1)
        section_ops = builders[name](b)
        b.keep.append(section_ops)
        for op in section_ops:
            sect[op.label] = b.time_op(op)
        result[name] = sect
    b.save_plan()
    if not args.profile_plan and not args.no_extras:
        log("timing a compiled caller of the C ABI ...")
        result["c_caller"] = c_caller_rates()
    if not args.no_cpu:
        log("timing the CPU oracle on the step ...")
        result["cpu_baseline"] = cpu_baseline(data)
    b.stream.release()
    detail = Path(args.detail)
    try:
        detail.parent.mkdir(parents=True, exist_ok=True)
        detail.write_text(json.dumps(result, indent=1))
        log(f"every section in full: {detail}")
    except OSError as err:
        log(f"could not write {detail}: {err}")
    print(json.dumps(final_line(result)))
    return 0


if __name__ == "__main__":
    sys.exit(main())
