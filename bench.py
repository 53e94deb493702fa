#!/usr/bin/env python3
"""Benchmark of the tensor-math hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras] [--no-cpu]

One step is one pass of BASELINE.json configs[1] over its synthetic input:
``unary-op! :exp``, ``unary-op! :tanh`` and ``ternary-op! :select`` on
transposed views (strides [1, 8192]) of float32 [8192, 8192] tensors, output
contiguous.  Inputs are resident in HBM before the timed region.  The line
printed at the end follows the driver's contract; ``value`` is algorithmic
bytes per second (each input element read once, each output element written
once) over the K timed steps.

``roofline`` describes the dominant kernel of the step (the LDS-tiled kernel
running ``:select``, three transposed inputs), timed with HIP events recorded on
the launch stream around every one of its launches inside the timed region.
``cpu_baseline`` times the CPU oracle (a C++ restatement of the cortex CPU
backend, OpenMP) on the same step.  ``others`` reports the remaining BASELINE
configs and ``adjacent`` the neighbouring TensorMath methods, each timed the
same way, as additional information.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

PEAK_HBM_GBS = 8000.0  # MI355X HBM3E, published


def log(msg: str) -> None:
    print(msg, file=sys.stderr, flush=True)


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


def upload(driver_mod, device, stream, array: np.ndarray):
    """Copies a numpy array into a fresh device buffer."""
    flat = np.ascontiguousarray(array).reshape(-1)
    dt = driver_mod.DATATYPE_OF_NUMPY[flat.dtype]
    buf = device.allocate_device_buffer(flat.size, dt)
    from cortex_amd import capi

    capi.call("ct_memcpy_async", buf.ptr, flat.ctypes.data, flat.nbytes, capi.COPY_H2D, stream.handle)
    stream.sync()
    return buf


def dims(shape, strides=None):
    if strides is None:
        strides, m = [], 1
        for s in reversed(shape):
            strides.insert(0, m)
            m *= s
    return {"shape": list(shape), "strides": list(strides)}


def time_launches(timer, stream, fn, iters: int, warm: int = 2):
    """Average duration in ms of `fn` (one or more launches) over `iters` runs."""
    for _ in range(warm):
        fn()
    stream.sync()
    e0 = timer.mark()
    for _ in range(iters):
        fn()
    e1 = timer.mark()
    ms = timer.elapsed_ms(e0, e1) / iters
    timer.free(e0, e1)
    return ms


def gbs(nbytes: float, ms: float) -> float:
    return nbytes / (ms * 1e-3) / 1e9


def run_extras(drv, device, stream, timer, capi) -> dict:
    """BASELINE configs 0, 2, 3, 4 (additional information, not the headline).

    Buffers are not released between configs: on this board a large buffer
    allocated after frees can land less favourably and cost several percent of
    bandwidth, which would make the figures depend on the order of the configs."""
    out = {}
    rng = np.random.default_rng(0)

    def entry(nbytes, ms):
        return {"us": round(ms * 1e3, 2), "GB/s": round(gbs(nbytes, ms), 1), "frac": round(gbs(nbytes, ms) / PEAK_HBM_GBS, 4),
                "kernel": capi.last_kernel()}

    # configs[0]: bias add [1024,1024] + [1024] (8 MiB: cache resident, launch bound)
    x = upload(drv, device, stream, rng.uniform(-1, 1, 1024 * 1024).astype(np.float32))
    b = upload(drv, device, stream, rng.uniform(-1, 1, 1024).astype(np.float32))
    d = device.allocate_device_buffer(1024 * 1024, "float")
    ms = time_launches(timer, stream, lambda: stream.binary_op(d, dims([1024, 1024]), x, dims([1024, 1024]), 1.0, b,
                                                               dims([1024]), 1.0, 1024 * 1024, "+"), 200)
    out["config0 binary-op! :+ [1024,1024]+[1024]"] = entry(8392704, ms)
    # the same op at a size that exercises HBM
    n = 16384
    x = upload(drv, device, stream, rng.standard_normal(n * n, dtype=np.float32))
    b = upload(drv, device, stream, rng.uniform(-1, 1, n).astype(np.float32))
    d = device.allocate_device_buffer(n * n, "float")
    ms = time_launches(timer, stream, lambda: stream.binary_op(d, dims([n, n]), x, dims([n, n]), 1.0, b, dims([n]), 1.0,
                                                               n * n, "+"), 20)
    out["config0 scaled binary-op! :+ [16384,16384]+[16384]"] = entry(8 * n * n + 4 * n, ms)

    # configs[2]: unary-reduce!
    r, c = 16384, 4096
    x = upload(drv, device, stream, np.random.default_rng(4).standard_normal(r * c, dtype=np.float32))
    o_rows = device.allocate_device_buffer(r, "float")
    o_cols = device.allocate_device_buffer(c, "float")
    for op in ("sum", "max", "magnitude-squared"):
        ms = time_launches(timer, stream, lambda: stream.unary_reduce(o_rows, dims([r, 1]), 1.0, x, dims([r, c]), op), 20)
        out[f"config2 unary-reduce! :{op} last axis f32 [16384,4096]"] = entry(4 * r * c + 4 * r, ms)
        ms = time_launches(timer, stream, lambda: stream.unary_reduce(o_cols, dims([c, 1]), 1.0, x, dims([c, r], [1, c]), op), 20)
        out[f"config2 unary-reduce! :{op} axis 0 (transposed view) f32"] = entry(4 * r * c + 4 * c, ms)
    r = c = 4096
    x = upload(drv, device, stream, np.random.default_rng(5).standard_normal(r * c))
    o = device.allocate_device_buffer(r, "double")
    for op in ("sum", "max", "magnitude-squared"):
        ms = time_launches(timer, stream, lambda: stream.unary_reduce(o, dims([r, 1]), 1.0, x, dims([r, c]), op), 20)
        out[f"config2 unary-reduce! :{op} last axis f64 [4096,4096]"] = entry(8 * r * c + 8 * r, ms)
        ms = time_launches(timer, stream, lambda: stream.unary_reduce(o, dims([c, 1]), 1.0, x, dims([c, r], [1, c]), op), 20)
        out[f"config2 unary-reduce! :{op} axis 0 (transposed view) f64"] = entry(8 * r * c + 8 * r, ms)

    # configs[3]: Adam and Adadelta over 2^28 float parameters
    n = 1 << 28
    g6 = np.random.default_rng(6)
    p = upload(drv, device, stream, g6.uniform(-0.05, 0.05, n).astype(np.float32))
    g = upload(drv, device, stream, g6.standard_normal(n, dtype=np.float32) * np.float32(1e-3))
    m = device.allocate_device_buffer(n, "float")
    v = device.allocate_device_buffer(n, "float")
    stream.memset(m, 0, 0.0, n)
    stream.memset(v, 0, 1e-6, n)
    pb1 = pb2 = 1.0
    for _ in range(10):
        pb1 *= 0.9
        pb2 *= 0.999
    ms = time_launches(timer, stream, lambda: stream.adam_step(1e-3, 0.9, 0.999, 1e-8, pb1, pb2, 1.0, g, p, m, v, n), 10)
    out["config3 Adam step 2^28 f32"] = entry(28 * n, ms)
    stream.memset(m, 0, 0.0, n)
    stream.memset(v, 0, 0.0, n)
    ms = time_launches(timer, stream, lambda: stream.adadelta_step(0.05, 1e-6, m, v, 1.0, g, p, n), 10)
    out["config3 Adadelta step 2^28 f32"] = entry(28 * n, ms)

    # configs[4]: mixed-dtype image normalise
    shp = [256, 3, 224, 224]
    n = int(np.prod(shp))
    u8 = upload(drv, device, stream, np.random.default_rng(7).integers(0, 256, n, dtype=np.uint8))
    f = device.allocate_device_buffer(n, "float")
    f2 = device.allocate_device_buffer(n, "float")
    mean = upload(drv, device, stream, (np.array([0.485, 0.456, 0.406]) * 255).astype(np.float32))
    std = upload(drv, device, stream, (np.array([0.229, 0.224, 0.225]) * 255).astype(np.float32))
    ms = time_launches(timer, stream, lambda: stream.assign(f, dims(shp), u8, dims(shp), n), 20)
    out["config4 assign! u8->f32 [256,3,224,224]"] = entry(5 * n, ms)
    ms = time_launches(timer, stream, lambda: stream.binary_op(f2, dims(shp), f, dims(shp), 1.0, mean, dims([3, 1, 1]),
                                                               -1.0, n, "+"), 20)
    out["config4 binary-op! :- per-channel mean"] = entry(8 * n + 12, ms)
    ms = time_launches(timer, stream, lambda: stream.binary_op(f2, dims(shp), f, dims(shp), 1.0, std, dims([3, 1, 1]),
                                                               1.0, n, "/"), 20)
    out["config4 binary-op! :/ per-channel std"] = entry(8 * n + 12, ms)
    n = 1 << 26
    i32 = upload(drv, device, stream, np.random.default_rng(8).integers(-2 ** 31, 2 ** 31, n, dtype=np.int64).astype(np.int32))
    f64 = device.allocate_device_buffer(n, "double")
    ms = time_launches(timer, stream, lambda: stream.assign(f64, dims([n]), i32, dims([n]), n), 20)
    out["config4 assign! i32->f64 [64M]"] = entry(12 * n, ms)
    return out


def run_adjacent(drv, device, stream, timer, capi) -> dict:
    """The adjacent TensorMath methods built on the same machinery (activation-gradient!,
    softmax!, batch normalization, rand!, gemv!, gemm!), timed like the BASELINE configs.  Bytes
    are algorithmic: every operand read once, every result written once, although the
    batch-normalization forms that need batch statistics read their operands twice."""
    out = {}
    rng = np.random.default_rng(9)

    def entry(nbytes, ms, **more):
        e = {"us": round(ms * 1e3, 2), "GB/s": round(gbs(nbytes, ms), 1), "frac": round(gbs(nbytes, ms) / PEAK_HBM_GBS, 4),
             "kernel": capi.last_kernel()}
        e.update(more)
        return e

    n = 1 << 27
    x = upload(drv, device, stream, rng.standard_normal(n, dtype=np.float32))
    g = upload(drv, device, stream, rng.standard_normal(n, dtype=np.float32))
    o = device.allocate_device_buffer(n, "float")
    ms = time_launches(timer, stream, lambda: stream.activation_gradient(o, dims([n]), g, dims([n]), x, dims([n]), "tanh", n), 20)
    out["activation-gradient! :tanh f32 [2^27]"] = entry(12 * n, ms)
    for k in (16, 1024):
        rows = n // k
        ms = time_launches(timer, stream, lambda: stream.softmax_eltwise(o, dims([rows, k]), x, dims([rows, k])), 20)
        out[f"softmax! f32 [{rows},{k}]"] = entry(8 * n, ms)
    b, c, e = 64, 21, 65536
    ms = time_launches(timer, stream, lambda: stream.softmax_spatial(o, dims([b, c, e]), x, dims([b, c, e])), 20)
    out[f"softmax! spatial f32 [{b},{c},{e}]"] = entry(8 * b * c * e, ms)
    ms = time_launches(timer, stream, lambda: stream.rand(o, dims([n]), {"type": "gaussian", "mean": 0.0, "variance": 1.0}), 20)
    out["rand! gaussian f32 [2^27]"] = entry(4 * n, ms)
    ms = time_launches(timer, stream, lambda: stream.rand(o, dims([n]), {"type": "flat", "minimum": 0.0, "maximum": 1.0}), 20)
    out["rand! flat f32 [2^27]"] = entry(4 * n, ms)

    b, c, e = 64, 256, 3136
    nn_ = b * c * e
    st = [upload(drv, device, stream, rng.uniform(0.5, 1.5, c).astype(np.float32)) for _ in range(8)]
    ms = time_launches(timer, stream, lambda: stream.batch_normalize_spatial(o, x, st[0], st[1], st[2], st[3], 1e-3, b, c, e), 20)
    out[f"batch-normalize! spatial f32 [{b},{c},{e}]"] = entry(8 * nn_, ms)
    ms = time_launches(timer, stream, lambda: stream.batch_normalize_update_and_apply_spatial(
        o, x, st[0], st[1], st[4], st[5], 0.9, st[2], st[3], 1e-3, b, c, e), 20)
    out[f"batch-normalize-update-and-apply! spatial f32 [{b},{c},{e}]"] = entry(8 * nn_, ms, hbm_bytes_moved=12 * nn_)
    ms = time_launches(timer, stream, lambda: stream.batch_normalize_gradients_spatial(
        o, st[6], st[7], g, o, x, st[0], st[1], st[2], st[3], 1e-3, b, c, e), 20)
    out[f"batch-normalize-gradients! spatial f32 [{b},{c},{e}]"] = entry(12 * nn_, ms, hbm_bytes_moved=20 * nn_)

    # pooling: algorithmic bytes = input + output forward; gradient read and written, output gradient
    # (and, for max, input and output) backward
    pb, pc, ph = 32, 64, 256
    po = ph // 2
    in_dims, out_dims = dims([pb, pc, ph, ph]), dims([pb, pc, po, po])
    n_out = pb * pc * po * po
    ig = device.allocate_device_buffer(n, "float")
    stream.memset(ig, 0, 0.0, n)
    for kernel, pad, pool_op in ((2, 0, "max"), (3, 1, "max"), (3, 1, "avg")):
        desc = {"kernel-width": kernel, "kernel-height": kernel, "pad-x": pad, "pad-y": pad, "stride-x": 2,
                "stride-y": 2, "pool-op": pool_op}
        label = f"f32 [{pb},{pc},{ph},{ph}] {kernel}x{kernel} stride 2 :{pool_op}"
        ms = time_launches(timer, stream, lambda: stream.pooling_forward(o, out_dims, 0.0, x, in_dims, desc), 20)
        out[f"pooling-forward! {label}"] = entry(4 * (n + n_out), ms)
        ms = time_launches(timer, stream, lambda: stream.pooling_backward(ig, in_dims, 0.0, x, in_dims, o, out_dims, g,
                                                                         out_dims, desc), 20)
        out[f"pooling-backward! {label}"] = entry(4 * (2 * n + n_out) + (4 * (n + n_out) if pool_op == "max" else 0), ms)

    # convolution as the CPU backend decomposes it (unroll, gemm!, roll back): priced like gemm!
    cb, cc, ck, chw = 64, 64, 64, 56
    conv_desc = {"in-channels": cc, "out-channels": ck, "kernel-width": 3, "kernel-height": 3, "pad-x": 1, "pad-y": 1,
                 "stride-x": 1, "stride-y": 1}
    c_in, c_out = dims([cb, cc, chw, chw]), dims([cb, ck, chw, chw])
    n_cols, n_rows = cc * 9, chw * chw
    w_ = upload(drv, device, stream, (rng.standard_normal(ck * n_cols, dtype=np.float32) / 24))
    work = device.allocate_device_buffer(cb * n_rows * n_cols, "float")
    wgrad = device.allocate_device_buffer(ck * n_cols, "float")
    w_dims = dims([ck, n_cols])
    conv_flops = 2.0 * cb * ck * n_rows * n_cols
    conv_calls = (
        ("convolution-forward!", lambda: stream.convolution_forward(o, c_out, 0.0, x, c_in, w_, w_dims, work,
                                                                    cb * n_rows * n_cols, conv_desc, None)),
        ("convolution-backward-weights!", lambda: stream.convolution_backward_weights(
            wgrad, w_dims, 0.0, g, c_out, x, c_in, work, cb * n_rows * n_cols, conv_desc, None)),
        ("convolution-backward-data!", lambda: stream.convolution_backward_data(
            ig, c_in, 0.0, g, c_out, w_, w_dims, work, cb * n_rows * n_cols, conv_desc, None)),
    )
    for name, call in conv_calls:
        ms = time_launches(timer, stream, call, 5, warm=2)
        tflops = conv_flops / (ms * 1e-3) / 1e12
        out[f"{name} f32 [{cb},{cc}->{ck},{chw},{chw}] 3x3 pad 1"] = {
            "us": round(ms * 1e3, 1), "TFLOP/s": round(tflops, 1), "frac_of_fp32_matrix_peak": round(tflops / 157.3, 4),
            "workspace_bytes": 4 * cb * n_rows * n_cols, "kernel": capi.last_kernel()}

    # gemm! is the one MFMA-bound method (rocBLAS); priced against the dense fp32 matrix peak
    m = 8192
    a_ = upload(drv, device, stream, rng.standard_normal(m * m, dtype=np.float32))
    b_ = upload(drv, device, stream, rng.standard_normal(m * m, dtype=np.float32))
    c_ = device.allocate_device_buffer(m * m, "float")
    # gemv! reads the matrix once: HBM-bound like the rest
    xv = upload(drv, device, stream, rng.standard_normal(m, dtype=np.float32))
    yv = device.allocate_device_buffer(m, "float")
    for trans, label in ((False, "A x"), (True, "A^T x")):
        ms = time_launches(timer, stream, lambda: stream.gemv(yv, 1, trans, 1.0, a_, m, m, m, xv, 1, 0.0), 20)
        out[f"gemv! f32 [{m},{m}] {label}"] = entry(4 * m * m, ms)
    ms = time_launches(timer, stream, lambda: stream.gemm(c_, m, False, False, 1.0, a_, m, m, m, b_, m, m, 0.0), 5, warm=2)
    tflops = 2.0 * m ** 3 / (ms * 1e-3) / 1e12
    out[f"gemm! f32 [{m},{m}]x[{m},{m}] (rocBLAS)"] = {"us": round(ms * 1e3, 1), "TFLOP/s": round(tflops, 1),
                                                     "frac_of_fp32_matrix_peak": round(tflops / 157.3, 4),
                                                     "kernel": capi.last_kernel()}
    return out


def cpu_baseline(hosts, n: int) -> dict:
    """Times the CPU oracle on one full step of the workload."""
    from cortex_amd import capi
    from oracle import binding as ob

    shape, tr = [n, n], [1, n]
    dest = np.zeros(n * n, np.float32)
    cont = capi.make_dims(shape, [n, 1])
    view = capi.make_dims(shape, tr)
    p = lambda a: a.ctypes.data
    def one_step():
        ob.call("unary_op", p(dest), C.byref(cont), p(hosts[0]), C.byref(view), 1.0, capi.UNARY_OPS["exp"], capi.F32, n * n)
        ob.call("unary_op", p(dest), C.byref(cont), p(hosts[0]), C.byref(view), 1.0, capi.UNARY_OPS["tanh"], capi.F32, n * n)
        ob.call("ternary_op", p(dest), C.byref(cont), p(hosts[0]), C.byref(view), 1.0, p(hosts[1]), C.byref(view), 1.0,
                p(hosts[2]), C.byref(view), 1.0, n * n, 0, capi.F32)

    one_step()  # first touch of the destination pages
    steps, t0 = 0, time.perf_counter()
    while steps < 3 or (time.perf_counter() - t0 < 10.0 and steps < 200):
        one_step()
        steps += 1
    dt = time.perf_counter() - t0
    step_bytes = 8 * 4 * n * n
    return {"value": round(steps * step_bytes / dt / 1e9, 3), "unit": "GB/s", "cores": ob.num_threads(), "kind": "port",
            "sample": f"{steps} full steps (exp, tanh, select on transposed float32 [{n},{n}]) in {dt:.2f} s, "
                      "C++ restatement of the cortex CPU backend with OpenMP"}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-extras", action="store_true", help="skip the other BASELINE configs")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--size", type=int, default=8192, help="edge of the square tensors (8192 is the benchmark)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path has no cross-GPU exchange); "
              f"--gpus {args.gpus} is not supported", file=sys.stderr)
        return 2

    from cortex_amd import capi, driver as drv

    driver = drv.HipDriver()
    device = driver.default_device()
    device.make_current()
    stream = device.create_stream()
    timer = Timer(capi, stream)
    n = args.size

    log("generating inputs (numpy default_rng, seeds 1-3) ...")
    hosts = [np.random.default_rng(seed).standard_normal(n * n).astype(np.float32) for seed in (1, 2, 3)]
    xs = [upload(drv, device, stream, h) for h in hosts]
    dest = device.allocate_device_buffer(n * n, "float")
    cont, view = dims([n, n]), dims([n, n], [1, n])
    nn = n * n

    sel_events = []

    def step(record: bool) -> None:
        stream.unary_op(dest, cont, xs[0], view, 1.0, "exp", nn)
        stream.unary_op(dest, cont, xs[0], view, 1.0, "tanh", nn)
        e0 = timer.mark() if record else None
        stream.ternary_op(dest, cont, xs[0], view, 1.0, xs[1], view, 1.0, xs[2], view, 1.0, nn, "select")
        if record:
            sel_events.append((e0, timer.mark()))

    for _ in range(args.warmup):
        step(False)
    stream.sync()
    dominant_kernel = capi.last_kernel()
    t_host0 = time.perf_counter()
    e_start = timer.mark()
    for _ in range(args.steps):
        step(True)
    e_stop = timer.mark()
    total_ms = timer.elapsed_ms(e_start, e_stop)
    stream.sync()
    wall_ms = (time.perf_counter() - t_host0) * 1e3
    sel_ms = [timer.elapsed_ms(a, b) for a, b in sel_events]
    for a, b in sel_events:
        timer.free(a, b)
    timer.free(e_start, e_stop)

    step_bytes = 2 * 4 * nn + 2 * 4 * nn + 4 * 4 * nn  # exp + tanh + select
    ms_per_step = total_ms / args.steps
    value = gbs(step_bytes, ms_per_step)
    sel_avg = float(np.mean(sel_ms))
    achieved = gbs(4 * 4 * nn, sel_avg)

    traffic = None
    tfile = ROOT / "profiles" / "traffic.json"
    if tfile.exists():
        try:
            traffic = json.loads(tfile.read_text()).get("ew_tile_kernel_select_f32_8192")
        except (ValueError, OSError):
            traffic = None

    # per-op times of the other two kernels of the step
    ms_exp = time_launches(timer, stream, lambda: stream.unary_op(dest, cont, xs[0], view, 1.0, "exp", nn), 20)
    ms_tanh = time_launches(timer, stream, lambda: stream.unary_op(dest, cont, xs[0], view, 1.0, "tanh", nn), 20)
    # a plain contiguous copy of the same size: the reference point for the hardware counters
    ms_copy = time_launches(timer, stream, lambda: stream.unary_op(dest, cont, xs[0], cont, 1.0, "noop", nn), 20)

    result = {
        "metric": "achieved HBM GB/s (% of MI355X peak) for binary-op!, unary-reduce!, Adam step",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "configs[1]: unary-op! :exp, unary-op! :tanh and ternary-op! :select on transposed views "
                        f"(strides [1,{n}]) of float32 [{n},{n}], inputs N(0,1) seeds 1-3, output contiguous",
            "algorithmic_bytes_per_step": step_bytes,
            "frac_of_peak": round(value / PEAK_HBM_GBS, 4),
            "host_wall_ms_per_step": round(wall_ms / args.steps, 4),
        },
        "roofline": {
            "bound": "hbm",
            "kernel": f"ew_tile_kernel<SelectF<float>> ({dominant_kernel})",
            "achieved": round(achieved, 1),
            "peak": PEAK_HBM_GBS,
            "unit": "GB/s",
            "frac": round(achieved / PEAK_HBM_GBS, 4),
            "traffic": traffic,
            "avg_launch_us": round(sel_avg * 1e3, 2),
            "algorithmic_bytes_per_launch": 4 * 4 * nn,
        },
        "kernels": {
            "unary-op! :exp (transposed)": {"us": round(ms_exp * 1e3, 2), "GB/s": round(gbs(8 * nn, ms_exp), 1)},
            "unary-op! :tanh (transposed)": {"us": round(ms_tanh * 1e3, 2), "GB/s": round(gbs(8 * nn, ms_tanh), 1)},
            "unary-op! :noop (contiguous copy, calibration)": {"us": round(ms_copy * 1e3, 2), "GB/s": round(gbs(8 * nn, ms_copy), 1)},
            "ternary-op! :select (3 transposed)": {"us": round(sel_avg * 1e3, 2), "GB/s": round(achieved, 1)},
        },
    }
    if not args.no_extras:
        log("timing the other BASELINE configs ...")
        result["others"] = run_extras(drv, device, stream, timer, capi)
        log("timing the adjacent TensorMath methods ...")
        result["adjacent"] = run_adjacent(drv, device, stream, timer, capi)
    if not args.no_cpu:
        log("timing the CPU oracle on one step ...")
        result["cpu_baseline"] = cpu_baseline(hosts, n)
    stream.release()
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
