"""Test harness: runs one tensor-math call on the CPU oracle and/or on the HIP
library through their C entry points, on identical inputs.

The oracle (``oracle/libcortex_cpu_oracle.so``) and the library
(``cortex_amd/libcortex_hip.so``) take the same argument lists; the library
takes a leading stream.  A :class:`Buf` owns one flat allocation on each side,
a :class:`View` is a ``{:shape :strides}`` window into it (with an element
offset, as the reference's sub-buffers).
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path
from typing import List, Optional, Sequence

import numpy as np

from cortex_amd import capi
from oracle import binding as oracle_binding

ROOT = Path(__file__).resolve().parent.parent

NP_DTYPES = {capi.I8: np.int8, capi.I16: np.int16, capi.I32: np.int32, capi.I64: np.int64,
             capi.F32: np.float32, capi.F64: np.float64, capi.U8: np.uint8}
CODE_OF = {np.dtype(v): k for k, v in NP_DTYPES.items()}
ALL_DTYPES = [capi.I8, capi.I16, capi.I32, capi.I64, capi.F32, capi.F64, capi.U8]
REFERENCE_DTYPES = ALL_DTYPES[:6]

_P, _D, _I, _L = C.c_void_p, C.c_double, C.c_int, C.c_int64
_DP = C.POINTER(capi.CtDims)


def oracle_lib() -> C.CDLL:
    return oracle_binding.lib()


OracleError = oracle_binding.OracleError


class Buf:
    """One flat buffer: a host array for the oracle and, when a GPU is in play,
    a device allocation holding the same initial bytes."""

    def __init__(self, data: np.ndarray, gpu: bool):
        self.init = np.ascontiguousarray(data).reshape(-1).copy()
        self.host = self.init.copy()          # mutated by the oracle
        self.dtype = CODE_OF[self.init.dtype]
        self.nbytes = self.init.nbytes
        self.dev = None
        if gpu:
            p = _P()
            capi.call("ct_malloc", C.byref(p), max(self.nbytes, 1))
            self.dev = p.value
            self.upload(self.init)

    def upload(self, data: np.ndarray) -> None:
        data = np.ascontiguousarray(data).reshape(-1)
        assert data.nbytes == self.nbytes
        capi.call("ct_memcpy_async", self.dev, data.ctypes.data, data.nbytes, capi.COPY_H2D, None)
        capi.call("ct_stream_sync", None)

    def download(self) -> np.ndarray:
        out = np.empty_like(self.init)
        capi.call("ct_stream_sync", None)
        capi.call("ct_memcpy_async", out.ctypes.data, self.dev, out.nbytes, capi.COPY_D2H, None)
        capi.call("ct_stream_sync", None)
        return out

    def reset(self) -> None:
        self.host[...] = self.init
        if self.dev is not None:
            self.upload(self.init)

    def free(self) -> None:
        if self.dev is not None:
            capi.call("ct_free", self.dev)
            self.dev = None


def row_major(shape: Sequence[int]) -> List[int]:
    strides, m = [], 1
    for s in reversed(shape):
        strides.append(m)
        m *= s
    return list(reversed(strides))


class View:
    """{:shape :strides} over a Buf, starting ``offset`` elements in.
    ``index[d]`` may be a Buf of int32 making dimension d indirect."""

    def __init__(self, buf: Buf, shape, strides=None, offset: int = 0, index=None):
        self.buf = buf
        self.shape = [int(s) for s in shape]
        self.strides = [int(s) for s in (strides if strides is not None else row_major(shape))]
        self.offset = int(offset)
        self.index = list(index) if index is not None else [None] * len(self.shape)

    @property
    def ecount(self) -> int:
        return int(np.prod(self.shape))

    def transpose(self, order) -> "View":
        return View(self.buf, [self.shape[i] for i in order], [self.strides[i] for i in order], self.offset,
                    [self.index[i] for i in order])

    def gather_host(self, data: Optional[np.ndarray] = None) -> np.ndarray:
        """The view's logical contents (row-major) read from ``data`` (default: the oracle's host copy)."""
        data = self.buf.host if data is None else data
        idx = np.zeros(self.shape, dtype=np.int64) + self.offset
        for d, (n, st) in enumerate(zip(self.shape, self.strides)):
            coord = np.arange(n, dtype=np.int64)
            if self.index[d] is not None:
                coord = self.index[d].init.astype(np.int64)
            shp = [1] * len(self.shape)
            shp[d] = n
            idx = idx + coord.reshape(shp) * st
        return data[idx.reshape(-1)].reshape(self.shape)


class Side:
    """One implementation (oracle or HIP) seen through the common call shape."""

    def __init__(self, gpu: bool):
        self.gpu = gpu
        self.stream = None

    def ptr(self, v: View) -> int:
        itemsize = v.buf.init.itemsize
        base = v.buf.dev if self.gpu else v.buf.host.ctypes.data
        return base + v.offset * itemsize

    def dims(self, v: View) -> capi.CtDims:
        index = []
        for ib in v.index:
            if ib is None:
                index.append(None)
            else:
                index.append(ib.dev if self.gpu else ib.host.ctypes.data)
        return capi.make_dims(v.shape, v.strides, index)

    def call(self, name: str, *args) -> None:
        if self.gpu:
            capi.call("ct_" + name, self.stream, *args)
            capi.call("ct_stream_sync", self.stream)
        else:
            oracle_binding.call(name, *args)


def _pd(side: Side, v: View):
    return side.ptr(v), C.byref(side.dims(v))


# ---- one wrapper per TensorMath method; `side` picks the implementation

def assign_constant(side, dest: View, value, n=None):
    p, d = _pd(side, dest)
    side.call("assign_constant", p, d, dest.buf.dtype, float(value), dest.ecount if n is None else n)


def assign(side, dest: View, src: View, n=None):
    n = max(dest.ecount, src.ecount) if n is None else n
    side.call("assign", *_pd(side, dest), dest.buf.dtype, *_pd(side, src), src.buf.dtype, n)


def unary_accum(side, dest: View, alpha, op, n=None):
    side.call("unary_accum", *_pd(side, dest), float(alpha), capi.UNARY_OPS[op], dest.buf.dtype,
              dest.ecount if n is None else n)


def unary_op(side, dest: View, x: View, alpha, op, n=None):
    n = max(dest.ecount, x.ecount) if n is None else n
    side.call("unary_op", *_pd(side, dest), *_pd(side, x), float(alpha), capi.UNARY_OPS[op], dest.buf.dtype, n)


def binary_accum_constant(side, dest: View, dest_alpha, scalar, op, reverse=False, n=None):
    side.call("binary_accum_constant", *_pd(side, dest), float(dest_alpha), float(scalar),
              dest.ecount if n is None else n, capi.BINARY_OPS[op], int(reverse), dest.buf.dtype)


def binary_op_constant(side, dest: View, x: View, x_alpha, scalar, op, reverse=False, n=None):
    n = max(dest.ecount, x.ecount) if n is None else n
    side.call("binary_op_constant", *_pd(side, dest), *_pd(side, x), float(x_alpha), float(scalar), n,
              capi.BINARY_OPS[op], int(reverse), dest.buf.dtype)


def binary_accum(side, dest: View, dest_alpha, y: View, y_alpha, op, reverse=False, requires_cas=True, n=None):
    n = max(dest.ecount, y.ecount) if n is None else n
    side.call("binary_accum", *_pd(side, dest), float(dest_alpha), *_pd(side, y), float(y_alpha), n,
              capi.BINARY_OPS[op], int(reverse), int(requires_cas), dest.buf.dtype)


def binary_op(side, dest: View, x: View, x_alpha, y: View, y_alpha, op, n=None):
    n = max(dest.ecount, x.ecount, y.ecount) if n is None else n
    side.call("binary_op", *_pd(side, dest), *_pd(side, x), float(x_alpha), *_pd(side, y), float(y_alpha), n,
              capi.BINARY_OPS[op], dest.buf.dtype)


def ternary_op(side, dest: View, x: View, xa, y: View, ya, z: View, za, n=None):
    n = max(dest.ecount, x.ecount, y.ecount, z.ecount) if n is None else n
    side.call("ternary_op", *_pd(side, dest), *_pd(side, x), float(xa), *_pd(side, y), float(ya), *_pd(side, z),
              float(za), n, 0, dest.buf.dtype)


def ternary_op_constant(side, dest: View, a: View, aa, b: View, ba, constant, arg_idx, n=None):
    n = max(dest.ecount, a.ecount, b.ecount) if n is None else n
    side.call("ternary_op_constant", *_pd(side, dest), *_pd(side, a), float(aa), *_pd(side, b), float(ba),
              float(constant), n, 0, capi.arg_idx(arg_idx), dest.buf.dtype)


def ternary_op_constant_constant(side, dest: View, a: View, aa, c1, c2, arg_idx, n=None):
    n = max(dest.ecount, a.ecount) if n is None else n
    side.call("ternary_op_constant_constant", *_pd(side, dest), *_pd(side, a), float(aa), float(c1), float(c2), n,
              0, capi.arg_idx(arg_idx), dest.buf.dtype)


def unary_reduce(side, out: View, alpha, inp: View, op):
    side.call("unary_reduce", *_pd(side, out), float(alpha), *_pd(side, inp), capi.REDUCE_OPS[op], out.buf.dtype)


def activation_gradient(side, ig: View, og: View, out: View, op, n):
    side.call("activation_gradient", *_pd(side, ig), *_pd(side, og), *_pd(side, out), capi.ACTIVATION_OPS[op], n,
              ig.buf.dtype)


def softmax(side, out: View, inp: View, spatial=False):
    side.call("softmax_spatial" if spatial else "softmax_eltwise", *_pd(side, out), *_pd(side, inp), out.buf.dtype)


def conv_desc(in_channels, out_channels, kw, kh, px, py, sx, sy):
    return {"in-channels": in_channels, "out-channels": out_channels, "kernel-width": kw, "kernel-height": kh,
            "pad-x": px, "pad-y": py, "stride-x": sx, "stride-y": sy}


def convolution(side, which, dest: View, alpha, a: View, b: View, workspace: View, desc, batch, in_h, in_w, out_h,
                out_w):
    """which: "forward" (dest output, a input, b weights), "backward_weights" (dest weight gradient, a output
    gradient, b input), "backward_data" (dest input gradient, a output gradient, b weights)."""
    d = capi.make_conv_desc(desc)
    side.call("convolution_" + which, side.ptr(dest), float(alpha), side.ptr(a), side.ptr(b), side.ptr(workspace),
              int(np.prod(workspace.shape)), C.byref(d), batch, in_h, in_w, out_h, out_w, dest.buf.dtype)


def pool_desc(kw, kh, px, py, sx, sy, op):
    return {"kernel-width": kw, "kernel-height": kh, "pad-x": px, "pad-y": py, "stride-x": sx, "stride-y": sy,
            "pool-op": op}


def pooling_forward(side, out: View, inp: View, desc, batch, channels, in_h, in_w, out_h, out_w):
    d = capi.make_pool_desc(desc)
    side.call("pooling_forward", side.ptr(out), 0.0, side.ptr(inp), C.byref(d), batch, channels, in_h, in_w, out_h,
              out_w, out.buf.dtype)


def pooling_backward(side, ig: View, inp: View, out: View, og: View, desc, batch, channels, in_h, in_w, out_h, out_w):
    d = capi.make_pool_desc(desc)
    side.call("pooling_backward", side.ptr(ig), 0.0, side.ptr(inp), side.ptr(out), side.ptr(og), C.byref(d), batch,
              channels, in_h, in_w, out_h, out_w, ig.buf.dtype)


def lrn_forward(side, out: View, inp: View, n, k, alpha, beta):
    side.call("lrn_forward", *_pd(side, out), *_pd(side, inp), int(n), float(k), float(alpha), float(beta), out.buf.dtype)


def lrn_backward(side, ig: View, out: View, inp: View, og: View, n, k, alpha, beta):
    side.call("lrn_backward", *_pd(side, ig), *_pd(side, out), *_pd(side, inp), *_pd(side, og), int(n), float(k),
              float(alpha), float(beta), out.buf.dtype)


def batch_normalize(side, out: View, inp: View, means: View, variances: View, scale: View, bias: View, epsilon,
                    batch, channels, elements=None):
    """elements=None selects the eltwise form ([batch, channels] with one statistic per element)."""
    ptrs = [side.ptr(v) for v in (out, inp, means, variances, scale, bias)]
    if elements is None:
        side.call("batch_normalize_eltwise", *ptrs, float(epsilon), batch, channels, out.buf.dtype)
    else:
        side.call("batch_normalize_spatial", *ptrs, float(epsilon), batch, channels, elements, out.buf.dtype)


def batch_normalize_update_and_apply(side, out: View, inp: View, batch_means: View, batch_variances: View,
                                     running_means: View, running_variances: View, average_factor, scale: View,
                                     bias: View, epsilon, batch, channels, elements=None):
    head = [side.ptr(v) for v in (out, inp, batch_means, batch_variances, running_means, running_variances)]
    tail = [side.ptr(scale), side.ptr(bias), float(epsilon), batch, channels]
    if elements is None:
        side.call("batch_normalize_update_and_apply_eltwise", *head, float(average_factor), *tail, out.buf.dtype)
    else:
        side.call("batch_normalize_update_and_apply_spatial", *head, float(average_factor), *tail, elements,
                  out.buf.dtype)


def batch_normalize_gradients(side, input_gradient: View, scale_gradient: View, bias_gradient: View,
                              output_gradient: View, output: View, inp: View, batch_means: View,
                              batch_variances: View, scale: View, bias: View, epsilon, batch, channels,
                              elements=None):
    ptrs = [side.ptr(v) for v in (input_gradient, scale_gradient, bias_gradient, output_gradient, output, inp,
                                  batch_means, batch_variances, scale, bias)]
    if elements is None:
        side.call("batch_normalize_gradients_eltwise", *ptrs, float(epsilon), batch, channels,
                  input_gradient.buf.dtype)
    else:
        side.call("batch_normalize_gradients_spatial", *ptrs, float(epsilon), batch, channels, elements,
                  input_gradient.buf.dtype)


def gemm(side, c: View, c_colstride, trans_a, trans_b, alpha, a: View, a_rows, a_cols, a_colstride, b: View, b_cols,
         b_colstride, beta):
    side.call("gemm", side.ptr(c), c_colstride, int(trans_a), int(trans_b), float(alpha), side.ptr(a), a_rows, a_cols,
              a_colstride, side.ptr(b), b_cols, b_colstride, float(beta), c.buf.dtype)


def gemv(side, c: View, inc_c, trans_a, alpha, a: View, a_rows, a_cols, a_colstride, x: View, inc_x, beta):
    side.call("gemv", side.ptr(c), inc_c, int(trans_a), float(alpha), side.ptr(a), a_rows, a_cols, a_colstride,
              side.ptr(x), inc_x, float(beta), c.buf.dtype)


def rand(side, dest: View, n, distribution, a, b, seed, offset):
    """distribution: "gaussian" (a = mean, b = variance) or "flat" (a = minimum, b = maximum)."""
    side.call("rand", side.ptr(dest), n, dest.buf.dtype, capi.DISTRIBUTIONS[distribution], float(a), float(b),
              int(seed), int(offset))


def adam_step(side, alpha, beta1, beta2, eps, pb1, pb2, ga, grad: View, params: View, m: View, v: View, n):
    args = (grad.buf.dtype, float(alpha), float(beta1), float(beta2), float(eps), float(pb1), float(pb2), float(ga),
            side.ptr(grad), side.ptr(params), side.ptr(m), side.ptr(v), n)
    side.call("adam_step", *args)


def adadelta_step(side, decay, eps, gacc: View, dacc: View, ga, grad: View, params: View, n):
    args = (grad.buf.dtype, float(decay), float(eps), side.ptr(gacc), side.ptr(dacc), float(ga), side.ptr(grad),
            side.ptr(params), n)
    side.call("adadelta_step", *args)


def memset(side, buf_view: View, value, n):
    if side.gpu:
        capi.call("ct_memset", side.stream, side.ptr(buf_view), buf_view.buf.dtype, float(value), n)
        capi.call("ct_stream_sync", side.stream)
    else:
        oracle_lib().co_memset(side.ptr(buf_view), buf_view.buf.dtype, float(value), n)


ORACLE = Side(gpu=False)


def gpu_side() -> Side:
    return Side(gpu=True)


class Pair:
    """Runs every call on both sides and compares buffers afterwards."""

    def __init__(self):
        self.hip = gpu_side()
        self.bufs: List[Buf] = []

    def buf(self, data: np.ndarray) -> Buf:
        b = Buf(np.asarray(data), gpu=True)
        self.bufs.append(b)
        return b

    def run(self, fn, *args, **kwargs) -> str:
        fn(ORACLE, *args, **kwargs)
        fn(self.hip, *args, **kwargs)
        return capi.last_kernel()

    def close(self) -> None:
        for b in self.bufs:
            b.free()
        self.bufs.clear()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()
        return False


def ulp_diff_f32(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """Distance in units in the last place between two float32 arrays (NaN == NaN)."""
    a = np.asarray(a, dtype=np.float32)
    b = np.asarray(b, dtype=np.float32)
    ai = a.view(np.int32).astype(np.int64)
    bi = b.view(np.int32).astype(np.int64)
    ai = np.where(ai < 0, -(ai & 0x7FFFFFFF), ai)
    bi = np.where(bi < 0, -(bi & 0x7FFFFFFF), bi)
    d = np.abs(ai - bi)
    both_nan = np.isnan(a) & np.isnan(b)
    return np.where(both_nan, 0, d)


def assert_bit_exact(got: np.ndarray, want: np.ndarray, what: str = "") -> None:
    got = np.asarray(got)
    want = np.asarray(want)
    assert got.dtype == want.dtype and got.shape == want.shape, (what, got.dtype, want.dtype, got.shape, want.shape)
    if got.dtype.kind == "f":
        same = (got.view(f"u{got.itemsize}") == want.view(f"u{want.itemsize}")) | (np.isnan(got) & np.isnan(want))
    else:
        same = got == want
    if not np.all(same):
        bad = np.flatnonzero(~same.reshape(-1))
        i = int(bad[0])
        raise AssertionError(f"{what}: {bad.size} of {got.size} elements differ; first at {i}: "
                             f"got {got.reshape(-1)[i]!r}, want {want.reshape(-1)[i]!r}")
