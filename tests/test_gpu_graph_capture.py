"""The library's calls recorded into a HIP graph and replayed.

A caller whose step is a fixed sequence of small calls (the reference's own networks: batches of 128 x 784)
can record the sequence once with hipStreamBeginCapture on the stream it hands to the library and replay it
with one launch per step.  That needs every recorded call to do nothing but launch kernels on that stream:
no allocation, no wait, no memset node (scratch reserved ahead, debug-sync mode off).  The test records a bias
add, a bias gradient, a column reduction cut into row segments (two launches through the stream's scratch),
the same through the entry point that allocates nothing, a softmax, a one-launch batch-normalization update
and an Adam step, replays the graph three times with new inputs and eager work on the stream in between, and
compares every replay, bit for bit, with the same calls made eagerly on the same inputs.
"""
import ctypes as C

import numpy as np
import pytest

from cortex_amd import capi

pytestmark = pytest.mark.gpu

HIP_STREAM_CAPTURE_MODE_THREAD_LOCAL = 1


def hip_runtime():
    rt = C.CDLL("libamdhip64.so")
    for name, argtypes in (("hipStreamBeginCapture", [C.c_void_p, C.c_int]),
                           ("hipStreamEndCapture", [C.c_void_p, C.POINTER(C.c_void_p)]),
                           ("hipGraphInstantiate", [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]),
                           ("hipGraphLaunch", [C.c_void_p, C.c_void_p]),
                           ("hipGraphExecDestroy", [C.c_void_p]),
                           ("hipGraphDestroy", [C.c_void_p]),
                           ("hipGraphGetNodes", [C.c_void_p, C.c_void_p, C.POINTER(C.c_size_t)])):
        fn = getattr(rt, name)
        fn.argtypes = argtypes
        fn.restype = C.c_int
    return rt


class Dev:
    def __init__(self, host: np.ndarray):
        self.host = np.ascontiguousarray(host).reshape(-1)
        p = C.c_void_p()
        capi.call("ct_malloc", C.byref(p), max(1, self.host.nbytes))
        self.ptr = p.value
        self.upload(self.host, None)

    def upload(self, host: np.ndarray, stream):
        host = np.ascontiguousarray(host).reshape(-1)
        assert host.nbytes == self.host.nbytes
        capi.call("ct_memcpy_async", self.ptr, host.ctypes.data, host.nbytes, capi.COPY_H2D, stream)
        capi.call("ct_stream_sync", stream)

    def download(self, stream) -> np.ndarray:
        out = np.empty_like(self.host)
        capi.call("ct_stream_sync", stream)
        capi.call("ct_memcpy_async", out.ctypes.data, self.ptr, out.nbytes, capi.COPY_D2H, stream)
        capi.call("ct_stream_sync", stream)
        return out

    def free(self):
        capi.call("ct_free", self.ptr)


def dims(shape, strides=None):
    if strides is None:
        strides, m = [], 1
        for s in reversed(shape):
            strides.insert(0, m)
            m *= s
    return capi.make_dims(shape, strides)


def test_a_recorded_step_replays_to_the_eager_results():
    rt = hip_runtime()
    capi.call("ct_set_device", 0)
    capi.call("ct_set_debug_sync", 0)
    stream = C.c_void_p()
    capi.call("ct_stream_create", C.byref(stream))
    capi.call("ct_stream_reserve_scratch", stream, 4 << 20, 4 << 20)
    batch, pixels, classes = 128, 784, 10
    rows, cols = 4096, 2048            # a column reduction above the size one launch over narrow strips takes
    rng = np.random.default_rng(41)
    f32 = np.float32
    act = Dev(rng.standard_normal(batch * pixels).astype(f32))
    bias = Dev(rng.standard_normal(pixels).astype(f32))
    logits = Dev(rng.standard_normal(batch * classes).astype(f32))
    big = Dev(rng.standard_normal(rows * cols).astype(f32))
    stats = [Dev(rng.uniform(0.5, 1.5, pixels).astype(f32)) for _ in range(6)]
    params, grads = Dev(rng.standard_normal(pixels * 16).astype(f32)), Dev(rng.standard_normal(pixels * 16).astype(f32))
    m, v = Dev(np.zeros(pixels * 16, f32)), Dev(np.full(pixels * 16, 1e-6, f32))
    # every output twice: one set for the eager calls, one for the graph's
    outs = {side: {"added": Dev(np.zeros(batch * pixels, f32)), "grad": Dev(np.zeros(pixels, f32)),
                   "colsum": Dev(np.zeros(cols, f32)), "colmax": Dev(np.zeros(cols, f32)),
                   "soft": Dev(np.zeros(batch * classes, f32)), "norm": Dev(np.zeros(batch * pixels, f32))}
            for side in ("eager", "graph")}
    state = {side: {"params": Dev(params.host), "m": Dev(m.host), "v": Dev(v.host),
                    "bmean": Dev(np.zeros(pixels, f32)), "bvar": Dev(np.zeros(pixels, f32)),
                    "rmean": Dev(stats[2].host), "rvar": Dev(stats[3].host)} for side in ("eager", "graph")}
    d_act, d_row, d_grad = dims([batch, pixels]), dims([pixels]), dims([batch, pixels], [0, 1])
    d_logits = dims([batch, classes])
    d_cols_view, d_cols_out = dims([cols, rows], [1, cols]), dims([cols, 1])
    ref = C.byref

    def step(side):
        o, st = outs[side], state[side]
        capi.call("ct_binary_op", stream, o["added"].ptr, ref(d_act), act.ptr, ref(d_act), 1.0, bias.ptr, ref(d_row), 1.0,
                  batch * pixels, capi.BINARY_OPS["+"], capi.F32)
        capi.call("ct_binary_accum", stream, o["grad"].ptr, ref(d_grad), 1.0, o["added"].ptr, ref(d_act), 1.0, batch * pixels,
                  capi.BINARY_OPS["+"], 0, 1, capi.F32)
        capi.call("ct_unary_reduce", stream, o["colsum"].ptr, ref(d_cols_out), 1.0, big.ptr, ref(d_cols_view),
                  capi.REDUCE_OPS["sum"], capi.F32)
        capi.call("ct_unary_reduce_noalloc", stream, o["colmax"].ptr, ref(d_cols_out), 1.0, big.ptr, ref(d_cols_view),
                  capi.REDUCE_OPS["max"], capi.F32)
        capi.call("ct_softmax_eltwise", stream, o["soft"].ptr, ref(d_logits), logits.ptr, ref(d_logits), capi.F32)
        capi.call("ct_batch_normalize_update_and_apply_eltwise", stream, o["norm"].ptr, act.ptr, st["bmean"].ptr, st["bvar"].ptr,
                  st["rmean"].ptr, st["rvar"].ptr, 0.9, stats[4].ptr, stats[5].ptr, 1e-3, batch, pixels, capi.F32)
        capi.call("ct_adam_step", stream, capi.F32, 1e-3, 0.9, 0.999, 1e-8, 0.9, 0.999, 1.0, grads.ptr, st["params"].ptr,
                  st["m"].ptr, st["v"].ptr, pixels * 16)

    everything = []
    try:
        step("graph")          # once eagerly: kernels are loaded and scratch is in place before anything is recorded
        for name in ("params", "m", "v", "rmean", "rvar"):
            state["graph"][name].upload(state["eager"][name].host, stream)
        capi.call("ct_memset", stream, outs["graph"]["grad"].ptr, capi.F32, 0.0, pixels)
        capi.call("ct_stream_sync", stream)
        assert rt.hipStreamBeginCapture(stream, HIP_STREAM_CAPTURE_MODE_THREAD_LOCAL) == 0
        try:
            step("graph")
        finally:
            graph = C.c_void_p()
            ended = rt.hipStreamEndCapture(stream, C.byref(graph))
        assert ended == 0 and graph.value, f"the capture did not end cleanly (hipError {ended})"
        n_nodes = C.c_size_t(0)
        assert rt.hipGraphGetNodes(graph, None, C.byref(n_nodes)) == 0
        assert n_nodes.value >= 9, n_nodes.value      # seven calls, two of them two launches
        graph_exec = C.c_void_p()
        assert rt.hipGraphInstantiate(C.byref(graph_exec), graph, None, None, 0) == 0
        for replay in range(3):
            # new inputs, written by eager work on the same stream between the replays
            act.upload(rng.standard_normal(batch * pixels).astype(f32), stream)
            big.upload(rng.standard_normal(rows * cols).astype(f32), stream)
            logits.upload(rng.standard_normal(batch * classes).astype(f32), stream)
            grads.upload(rng.standard_normal(pixels * 16).astype(f32), stream)
            step("eager")
            capi.call("ct_stream_sync", stream)
            assert rt.hipGraphLaunch(graph_exec, stream) == 0
            capi.call("ct_stream_sync", stream)
            for name in outs["eager"]:
                a, b = outs["eager"][name].download(stream), outs["graph"][name].download(stream)
                assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), (replay, name)
            for name in state["eager"]:
                a, b = state["eager"][name].download(stream), state["graph"][name].download(stream)
                assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), (replay, name)
        assert np.any(outs["graph"]["colsum"].download(stream) != 0)
        assert rt.hipGraphExecDestroy(graph_exec) == 0
        assert rt.hipGraphDestroy(graph) == 0
    finally:
        capi.call("ct_stream_sync", stream)
        for group in (outs["eager"], outs["graph"], state["eager"], state["graph"]):
            everything.extend(group.values())
        everything.extend([act, bias, logits, big, params, grads, m, v] + stats)
        for t in everything:
            t.free()
        capi.call("ct_stream_destroy", stream)
        capi.call("ct_set_debug_sync", 1)
