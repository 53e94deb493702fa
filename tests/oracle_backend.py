"""A CPU driver over the oracle with the interface of ``cortex_amd.driver``
(TEST INFRASTRUCTURE).  It lets the backend-neutral tensor API and the
reference-style test bodies run against the oracle exactly as they run against
the HIP driver: "one test body, many backends"
(``/root/reference/test/clj/cortex/compute/cpu/tensor_test.clj``)."""
from __future__ import annotations

import ctypes as C

import numpy as np

from cortex_amd import capi
from cortex_amd.driver import NUMPY_OF, _arg_order_indexes
from oracle import binding as ob


class OracleBuffer:
    def __init__(self, device, array: np.ndarray, datatype: str):
        self.device = device
        self.array = array  # 1-D numpy view
        self.datatype = datatype

    @property
    def ptr(self) -> int:
        return self.array.ctypes.data

    def ecount(self) -> int:
        return int(self.array.size)

    def get_datatype(self) -> str:
        return self.datatype

    @property
    def nbytes(self) -> int:
        return int(self.array.nbytes)

    def sub_buffer(self, offset, length):
        if offset < 0 or length < 0 or offset + length > self.array.size:
            raise ValueError("Sub buffer out of range")
        return OracleBuffer(self.device, self.array[offset:offset + length], self.datatype)

    def alias(self, other) -> bool:
        return self.ptr == other.ptr

    def partially_alias(self, other) -> bool:
        a0, a1, b0, b1 = self.ptr, self.ptr + self.nbytes, other.ptr, other.ptr + other.nbytes
        return a0 != b0 and a0 < b1 and b0 < a1

    def release(self) -> None:
        pass


class OracleEvent:
    def wait_for_event(self) -> None:
        pass


def _dims(d: dict) -> capi.CtDims:
    shape, index = [], []
    for entry in d["shape"]:
        if hasattr(entry, "buffer"):
            shape.append(entry.buffer.ecount())
            index.append(entry.buffer.ptr)
        else:
            shape.append(int(entry))
            index.append(None)
    return capi.make_dims(shape, d["strides"], index)


class OracleStream:
    def __init__(self, device):
        self.device = device

    def get_device(self):
        return self.device

    def get_driver(self):
        return self.device.driver

    def copy_host_to_device(self, host, ho, dev, do, n):
        dev.array[do:do + n] = host.array[ho:ho + n]

    def copy_device_to_host(self, dev, do, host, ho, n):
        host.array[ho:ho + n] = dev.array[do:do + n]

    def copy_device_to_device(self, src, so, dst, do, n):
        dst.array[do:do + n] = src.array[so:so + n].copy()

    def memset(self, dev, offset, value, n):
        ob.call("memset", dev.ptr + offset * dev.array.itemsize, capi.DTYPE_CODES[dev.datatype], float(value), n)

    def create_event(self):
        return OracleEvent()

    def sync_event(self, event):
        pass

    def sync(self):
        pass

    def release(self):
        pass

    # TensorMath
    def assign_constant(self, buffer, dimensions, value, n):
        ob.call("assign_constant", buffer.ptr, C.byref(_dims(dimensions)), capi.DTYPE_CODES[buffer.datatype], float(value), int(n))

    def assign(self, dest, dd, src, sd, n):
        ob.call("assign", dest.ptr, C.byref(_dims(dd)), capi.DTYPE_CODES[dest.datatype], src.ptr, C.byref(_dims(sd)),
                capi.DTYPE_CODES[src.datatype], int(n))

    def unary_accum(self, dest, dd, alpha, op, n):
        ob.call("unary_accum", dest.ptr, C.byref(_dims(dd)), float(alpha), capi.UNARY_OPS[op], capi.DTYPE_CODES[dest.datatype], int(n))

    def unary_op(self, dest, dd, x, xd, alpha, op, n):
        ob.call("unary_op", dest.ptr, C.byref(_dims(dd)), x.ptr, C.byref(_dims(xd)), float(alpha), capi.UNARY_OPS[op],
                capi.DTYPE_CODES[dest.datatype], int(n))

    def binary_accum_constant(self, dest, dd, da, scalar, n, op, rev):
        ob.call("binary_accum_constant", dest.ptr, C.byref(_dims(dd)), float(da), float(scalar), int(n),
                capi.BINARY_OPS[op], int(bool(rev)), capi.DTYPE_CODES[dest.datatype])

    def binary_op_constant(self, dest, dd, x, xd, xa, scalar, n, op, rev):
        ob.call("binary_op_constant", dest.ptr, C.byref(_dims(dd)), x.ptr, C.byref(_dims(xd)), float(xa), float(scalar),
                int(n), capi.BINARY_OPS[op], int(bool(rev)), capi.DTYPE_CODES[dest.datatype])

    def binary_accum(self, dest, dd, da, y, yd, ya, n, op, rev, cas):
        ob.call("binary_accum", dest.ptr, C.byref(_dims(dd)), float(da), y.ptr, C.byref(_dims(yd)), float(ya), int(n),
                capi.BINARY_OPS[op], int(bool(rev)), int(bool(cas)), capi.DTYPE_CODES[dest.datatype])

    def binary_op(self, dest, dd, x, xd, xa, y, yd, ya, n, op):
        ob.call("binary_op", dest.ptr, C.byref(_dims(dd)), x.ptr, C.byref(_dims(xd)), float(xa), y.ptr,
                C.byref(_dims(yd)), float(ya), int(n), capi.BINARY_OPS[op], capi.DTYPE_CODES[dest.datatype])

    def ternary_op(self, dest, dd, x, xd, xa, y, yd, ya, z, zd, za, n, op):
        ob.call("ternary_op", dest.ptr, C.byref(_dims(dd)), x.ptr, C.byref(_dims(xd)), float(xa), y.ptr,
                C.byref(_dims(yd)), float(ya), z.ptr, C.byref(_dims(zd)), float(za), int(n), capi.TERNARY_OPS[op],
                capi.DTYPE_CODES[dest.datatype])

    def ternary_op_constant(self, dest, dd, a, ad, aa, b, bd, ba, constant, n, op, arg_order):
        ob.call("ternary_op_constant", dest.ptr, C.byref(_dims(dd)), a.ptr, C.byref(_dims(ad)), float(aa), b.ptr,
                C.byref(_dims(bd)), float(ba), float(constant), int(n), capi.TERNARY_OPS[op],
                _arg_order_indexes(arg_order), capi.DTYPE_CODES[dest.datatype])

    def ternary_op_constant_constant(self, dest, dd, a, ad, aa, c1, c2, n, op, arg_order):
        ob.call("ternary_op_constant_constant", dest.ptr, C.byref(_dims(dd)), a.ptr, C.byref(_dims(ad)), float(aa),
                float(c1), float(c2), int(n), capi.TERNARY_OPS[op], _arg_order_indexes(arg_order),
                capi.DTYPE_CODES[dest.datatype])

    def unary_reduce(self, out, od, alpha, inp, idims, op):
        ob.call("unary_reduce", out.ptr, C.byref(_dims(od)), float(alpha), inp.ptr, C.byref(_dims(idims)),
                capi.REDUCE_OPS[op], capi.DTYPE_CODES[out.datatype])

    def activation_gradient(self, ig, igd, og, ogd, out, od, op, n):
        ob.call("activation_gradient", ig.ptr, C.byref(_dims(igd)), og.ptr, C.byref(_dims(ogd)), out.ptr,
                C.byref(_dims(od)), capi.ACTIVATION_OPS[op], int(n), capi.DTYPE_CODES[ig.datatype])

    def softmax_eltwise(self, out, od, inp, idims):
        ob.call("softmax_eltwise", out.ptr, C.byref(_dims(od)), inp.ptr, C.byref(_dims(idims)),
                capi.DTYPE_CODES[out.datatype])

    def softmax_spatial(self, out, od, inp, idims):
        ob.call("softmax_spatial", out.ptr, C.byref(_dims(od)), inp.ptr, C.byref(_dims(idims)),
                capi.DTYPE_CODES[out.datatype])

    def batch_normalize_eltwise(self, out, inp, means, variances, scale, bias, eps, batch, elems):
        ob.call("batch_normalize_eltwise", out.ptr, inp.ptr, means.ptr, variances.ptr, scale.ptr, bias.ptr, float(eps),
                int(batch), int(elems), capi.DTYPE_CODES[out.datatype])

    def batch_normalize_spatial(self, out, inp, means, variances, scale, bias, eps, batch, chans, elems):
        ob.call("batch_normalize_spatial", out.ptr, inp.ptr, means.ptr, variances.ptr, scale.ptr, bias.ptr, float(eps),
                int(batch), int(chans), int(elems), capi.DTYPE_CODES[out.datatype])

    def batch_normalize_update_and_apply_eltwise(self, out, inp, bm, bv, rm, rv, af, scale, bias, eps, batch, elems):
        ob.call("batch_normalize_update_and_apply_eltwise", out.ptr, inp.ptr, bm.ptr, bv.ptr, rm.ptr, rv.ptr, float(af),
                scale.ptr, bias.ptr, float(eps), int(batch), int(elems), capi.DTYPE_CODES[out.datatype])

    def batch_normalize_update_and_apply_spatial(self, out, inp, bm, bv, rm, rv, af, scale, bias, eps, batch, chans,
                                                 elems):
        ob.call("batch_normalize_update_and_apply_spatial", out.ptr, inp.ptr, bm.ptr, bv.ptr, rm.ptr, rv.ptr, float(af),
                scale.ptr, bias.ptr, float(eps), int(batch), int(chans), int(elems), capi.DTYPE_CODES[out.datatype])

    def batch_normalize_gradients_eltwise(self, ig, sg, bg, og, out, inp, bm, bv, scale, bias, eps, batch, elems):
        ob.call("batch_normalize_gradients_eltwise", ig.ptr, sg.ptr, bg.ptr, og.ptr, out.ptr, inp.ptr, bm.ptr, bv.ptr,
                scale.ptr, bias.ptr, float(eps), int(batch), int(elems), capi.DTYPE_CODES[ig.datatype])

    def batch_normalize_gradients_spatial(self, ig, sg, bg, og, out, inp, bm, bv, scale, bias, eps, batch, chans,
                                          elems):
        ob.call("batch_normalize_gradients_spatial", ig.ptr, sg.ptr, bg.ptr, og.ptr, out.ptr, inp.ptr, bm.ptr, bv.ptr,
                scale.ptr, bias.ptr, float(eps), int(batch), int(chans), int(elems), capi.DTYPE_CODES[ig.datatype])

    def convolution_descriptor(self, *args):
        return None

    def choose_convolution_algorithms(self, desc, input_width, input_height, output_width, output_height, batch_size,
                                      max_ideal_workspace_size, use_defaults):
        n_cols = int(desc["kernel-width"]) * int(desc["kernel-height"]) * int(desc["in-channels"])
        return {"workspace-size": n_cols * int(output_width) * int(output_height) * int(batch_size)}

    def _conv(self, name, dest, alpha, a, b, workspace, workspace_ecount, desc, in_shape, out_shape):
        batch, _, in_h, in_w = (int(v) for v in in_shape)
        out_h, out_w = (int(v) for v in out_shape[2:])
        ob.call(name, dest.ptr, float(alpha), a.ptr, b.ptr, workspace.ptr, int(workspace_ecount),
                C.byref(capi.make_conv_desc(desc)), int(out_shape[0]), in_h, in_w, out_h, out_w,
                capi.DTYPE_CODES[dest.datatype])

    def convolution_forward(self, out, od, out_alpha, inp, idims, weights, wd, workspace, ecount, desc, algorithms):
        self._conv("convolution_forward", out, out_alpha, inp, weights, workspace, ecount, desc, idims["shape"],
                   od["shape"])

    def convolution_backward_weights(self, wg, wgd, wg_alpha, og, ogd, inp, idims, workspace, ecount, desc, algorithms):
        self._conv("convolution_backward_weights", wg, wg_alpha, og, inp, workspace, ecount, desc, idims["shape"],
                   ogd["shape"])

    def convolution_backward_data(self, ig, igd, ig_alpha, og, ogd, weights, wd, workspace, ecount, desc, algorithms):
        self._conv("convolution_backward_data", ig, ig_alpha, og, weights, workspace, ecount, desc, igd["shape"],
                   ogd["shape"])

    def pooling_forward(self, out, od, out_alpha, inp, idims, desc):
        batch, channels, in_h, in_w = (int(v) for v in idims["shape"])
        out_h, out_w = (int(v) for v in od["shape"][2:])
        ob.call("pooling_forward", out.ptr, float(out_alpha), inp.ptr, C.byref(capi.make_pool_desc(desc)), batch,
                channels, in_h, in_w, out_h, out_w, capi.DTYPE_CODES[out.datatype])

    def pooling_backward(self, ig, igd, ig_alpha, inp, idims, out, od, og, ogd, desc):
        batch, channels, in_h, in_w = (int(v) for v in idims["shape"])
        out_h, out_w = (int(v) for v in od["shape"][2:])
        ob.call("pooling_backward", ig.ptr, float(ig_alpha), inp.ptr, out.ptr, og.ptr,
                C.byref(capi.make_pool_desc(desc)), batch, channels, in_h, in_w, out_h, out_w,
                capi.DTYPE_CODES[out.datatype])

    def lrn_forward(self, out, od, inp, idims, desc):
        ob.call("lrn_forward", out.ptr, C.byref(_dims(od)), inp.ptr, C.byref(_dims(idims)), int(desc["n"]),
                float(desc["k"]), float(desc["alpha"]), float(desc["beta"]), capi.DTYPE_CODES[out.datatype])

    def lrn_backward(self, ig, igd, out, od, inp, idims, og, ogd, desc):
        ob.call("lrn_backward", ig.ptr, C.byref(_dims(igd)), out.ptr, C.byref(_dims(od)), inp.ptr, C.byref(_dims(idims)),
                og.ptr, C.byref(_dims(ogd)), int(desc["n"]), float(desc["k"]), float(desc["alpha"]), float(desc["beta"]),
                capi.DTYPE_CODES[out.datatype])

    def gemm(self, c, ldc, ta, tb, alpha, a, a_rows, a_cols, lda, b, b_cols, ldb, beta):
        ob.call("gemm", c.ptr, int(ldc), int(bool(ta)), int(bool(tb)), float(alpha), a.ptr, int(a_rows), int(a_cols),
                int(lda), b.ptr, int(b_cols), int(ldb), float(beta), capi.DTYPE_CODES[c.datatype])

    def gemv(self, c, inc_c, ta, alpha, a, a_rows, a_cols, lda, x, inc_x, beta):
        ob.call("gemv", c.ptr, int(inc_c), int(bool(ta)), float(alpha), a.ptr, int(a_rows), int(a_cols), int(lda),
                x.ptr, int(inc_x), float(beta), capi.DTYPE_CODES[c.datatype])

    def seed_random(self, seed):
        self._rand_seed, self._rand_calls = int(seed) & 0xFFFFFFFFFFFFFFFF, 0

    def rand(self, dest, dest_dims, distribution):
        if getattr(self, "_rand_seed", None) is None:
            self.seed_random(0x5EED)
        kind = distribution["type"]
        a, b = ((distribution["mean"], distribution["variance"]) if kind == "gaussian"
                else (distribution["minimum"], distribution["maximum"]))
        n = int(np.prod([int(v) for v in dest_dims["shape"]]))
        ob.call("rand", dest.ptr, n, capi.DTYPE_CODES[dest.datatype], capi.DISTRIBUTIONS[kind], float(a), float(b),
                self._rand_seed, self._rand_calls)
        self._rand_calls += 1

    def adam_step(self, alpha, beta1, beta2, eps, pb1, pb2, ga, gradient, parameters, m, v, n):
        ob.call("adam_step", capi.DTYPE_CODES[gradient.datatype], float(alpha), float(beta1), float(beta2), float(eps),
                float(pb1), float(pb2), float(ga), gradient.ptr, parameters.ptr, m.ptr, v.ptr, int(n))

    def adadelta_step(self, decay, eps, gacc, dacc, ga, gradient, parameters, n):
        ob.call("adadelta_step", capi.DTYPE_CODES[gradient.datatype], float(decay), float(eps), gacc.ptr, dacc.ptr,
                float(ga), gradient.ptr, parameters.ptr, int(n))


class OracleDevice:
    def __init__(self, driver):
        self.driver = driver

    def get_driver(self):
        return self.driver

    def make_current(self):
        pass

    def create_stream(self):
        return OracleStream(self)

    def allocate_device_buffer(self, n, datatype):
        return OracleBuffer(self, np.zeros(max(int(n), 0), dtype=NUMPY_OF[datatype]), datatype)


class OracleDriver:
    type = "cpu-oracle"

    def __init__(self):
        self._device = OracleDevice(self)

    def get_devices(self):
        return [self._device]

    def default_device(self):
        return self._device

    def allocate_host_buffer(self, n, datatype, usage_type="one-time"):
        return OracleBuffer(self._device, np.zeros(int(n), dtype=NUMPY_OF[datatype]), datatype)
