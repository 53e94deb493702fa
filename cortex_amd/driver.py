"""The ``:hip`` compute driver: a Python mirror of the reference's driver
protocols for the tensor-math path, on top of the C ABI.

It provides what ``cortex.compute.driver`` asks of a backend
(``src/cortex/compute/driver.clj:46-221``) with the same names and argument
meaning:

* :class:`HipDriver`   -- ``PDriver``: ``get_devices``, ``allocate_host_buffer``
* :class:`HipDevice`   -- ``PDevice``: ``memory_info``, ``create_stream``,
  ``allocate_device_buffer``
* :class:`HipStream`   -- ``PStream``: ``copy_host_to_device``,
  ``copy_device_to_host``, ``copy_device_to_device``, ``memset``,
  ``create_event``, ``sync_event``; and the twelve ``TensorMath`` methods of
  ``src/cortex/tensor/math.clj:14-104`` (template:
  ``src/cortex/compute/cuda/tensor_math.clj:289-631``)
* :class:`DeviceBuffer` -- ``PBuffer``: ``sub_buffer``, ``alias``,
  ``partially_alias`` (``src/cortex/compute/cuda/driver.clj:465-510``)
* :class:`Event`       -- ``PEvent``: ``wait_for_event``

Dimensions are the reference's ``{:shape :strides}`` maps as Python dicts
``{"shape": [...], "strides": [...]}``; a shape entry may be an int32
:class:`DeviceBuffer`-backed tensor (anything with ``.buffer``) for an
indirectly addressed dimension.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional, Sequence

import numpy as np

from . import capi

DATATYPES = ("byte", "short", "int", "long", "float", "double", "ubyte")
NUMPY_OF = {"byte": np.int8, "short": np.int16, "int": np.int32, "long": np.int64, "float": np.float32,
            "double": np.float64, "ubyte": np.uint8}
DATATYPE_OF_NUMPY = {np.dtype(v): k for k, v in NUMPY_OF.items()}


def dtype_size(datatype: str) -> int:
    return capi.DTYPE_SIZES[capi.DTYPE_CODES[datatype]]


class DeviceBuffer:
    """A typed range of device memory.  The owner frees it on ``release``;
    sub-buffers share the owner's memory and own nothing
    (``src/cortex/compute/cuda/driver.clj:502-506``)."""

    def __init__(self, device: "HipDevice", ptr: int, ecount: int, datatype: str, owner: Optional["DeviceBuffer"] = None):
        self.device = device
        self.ptr = ptr
        self._ecount = int(ecount)
        self.datatype = datatype
        self._owner = owner
        self._released = False

    def ecount(self) -> int:
        return self._ecount

    def get_datatype(self) -> str:
        return self.datatype

    @property
    def nbytes(self) -> int:
        return self._ecount * dtype_size(self.datatype)

    def sub_buffer(self, offset: int, length: int) -> "DeviceBuffer":
        """``drv/sub-buffer`` (``src/cortex/compute/driver.clj:206-214``)."""
        offset, length = int(offset), int(length)
        if offset < 0 or length < 0 or offset + length > self._ecount:
            raise ValueError(f"Sub buffer out of range: offset {offset} length {length} of {self._ecount}")
        return DeviceBuffer(self.device, self.ptr + offset * dtype_size(self.datatype), length, self.datatype,
                            owner=self._owner or self)

    def alias(self, other: "DeviceBuffer") -> bool:
        """Same start address (``cuda/driver.clj:465-472``)."""
        return self.ptr == other.ptr

    def partially_alias(self, other: "DeviceBuffer") -> bool:
        """Overlapping byte ranges that do not start at the same address
        (``cuda/driver.clj:473-486``)."""
        a0, a1 = self.ptr, self.ptr + self.nbytes
        b0, b1 = other.ptr, other.ptr + other.nbytes
        if a0 == b0:
            return False
        return a0 < b1 and b0 < a1

    def release(self) -> None:
        if self._owner is None and not self._released and self.ptr:
            capi.call("ct_free", self.ptr)
            self._released = True


class HostBuffer:
    """Pinned host memory exposed as a numpy array (``allocate-host-buffer``)."""

    def __init__(self, ecount: int, datatype: str):
        self.datatype = datatype
        self._ecount = int(ecount)
        p = C.c_void_p()
        nbytes = max(1, self._ecount * dtype_size(datatype))
        capi.call("ct_host_alloc", C.byref(p), nbytes)
        self.ptr = p.value
        raw = (C.c_char * nbytes).from_address(self.ptr)
        self.array = np.frombuffer(raw, dtype=NUMPY_OF[datatype], count=self._ecount)
        self._released = False

    def ecount(self) -> int:
        return self._ecount

    def get_datatype(self) -> str:
        return self.datatype

    def release(self) -> None:
        if not self._released:
            self.array = None
            capi.call("ct_host_free", self.ptr)
            self._released = True


class Event:
    def __init__(self, handle: int):
        self.handle = handle

    def wait_for_event(self) -> None:
        """``PEvent wait-for-event``: blocks the host."""
        capi.call("ct_event_sync", self.handle)

    def release(self) -> None:
        if self.handle:
            capi.call("ct_event_destroy", self.handle)
            self.handle = None


# ct_dims structs of directly addressed dimensions, by (shape, strides): building one costs 2 us of interpreter
# time, three of them most of what a small call costs from Python.  The library reads a struct during the call
# only and never writes it, so one struct serves every call with those dimensions, from any thread.
_DIMS_CACHE: dict = {}
_DIMS_CACHE_LIMIT = 4096


def _dims_struct(dims: dict) -> capi.CtDims:
    shape_in, strides_in = dims["shape"], dims["strides"]
    direct = True
    for entry in shape_in:
        if type(entry) is not int:
            direct = False
            break
    if direct:
        key = (tuple(shape_in), tuple(strides_in))
        try:
            hit = _DIMS_CACHE.get(key)
        except TypeError:       # a stride that does not hash: take the long way
            hit, key = None, None
        if hit is not None:
            return hit
        made = capi.make_dims(shape_in, strides_in, None)
        if key is not None:
            if len(_DIMS_CACHE) >= _DIMS_CACHE_LIMIT:
                _DIMS_CACHE.clear()
            _DIMS_CACHE[key] = made
        return made
    shape, index = [], []
    for entry in dims["shape"]:
        if isinstance(entry, (int, np.integer)):
            shape.append(int(entry))
            index.append(None)
        else:  # an index tensor: int32, dense (cpu/tensor_math.clj:68-80)
            buf = entry.buffer
            if buf.get_datatype() != "int":
                raise TypeError("Index buffers must be integer tensors")
            shape.append(int(buf.ecount()))
            index.append(buf.ptr)
    return capi.make_dims(shape, dims["strides"], index)


def _arg_order_indexes(arg_order: Sequence[str]):
    """``arg-order->indexes`` (``cpu/tensor_math.clj:500-504``)."""
    pos = {name: i for i, name in enumerate(arg_order)}
    return capi.arg_idx([pos["x"], pos["y"], pos["z"]])


class HipStream:
    """A HIP stream.  Calls are ordered on the stream and asynchronous to the
    host; observe completion through ``create_event().wait_for_event()`` or
    ``sync``."""

    def __init__(self, device: "HipDevice", handle: Optional[int]):
        self.device = device
        self.handle = handle

    def get_device(self) -> "HipDevice":
        return self.device

    def get_driver(self) -> "HipDriver":
        return self.device.driver

    # -- PStream ----------------------------------------------------------
    def copy_host_to_device(self, host: HostBuffer, host_offset: int, dev: DeviceBuffer, dev_offset: int, n: int) -> None:
        self._check_copy(host, host_offset, dev, dev_offset, n)
        es = dtype_size(dev.datatype)
        capi.call("ct_memcpy_async", dev.ptr + dev_offset * es, host.ptr + host_offset * es, n * es, capi.COPY_H2D,
                  self.handle)

    def copy_device_to_host(self, dev: DeviceBuffer, dev_offset: int, host: HostBuffer, host_offset: int, n: int) -> None:
        self._check_copy(host, host_offset, dev, dev_offset, n)
        es = dtype_size(dev.datatype)
        capi.call("ct_memcpy_async", host.ptr + host_offset * es, dev.ptr + dev_offset * es, n * es, capi.COPY_D2H,
                  self.handle)

    def copy_device_to_device(self, src: DeviceBuffer, src_offset: int, dst: DeviceBuffer, dst_offset: int, n: int) -> None:
        self._check_copy(src, src_offset, dst, dst_offset, n)
        es = dtype_size(dst.datatype)
        capi.call("ct_memcpy_async", dst.ptr + dst_offset * es, src.ptr + src_offset * es, n * es, capi.COPY_D2D,
                  self.handle)

    @staticmethod
    def _check_copy(a, a_offset, b, b_offset, n) -> None:
        # cuda/driver.clj:901-919: datatypes must match and both ranges must fit
        if a.get_datatype() != b.get_datatype():
            raise TypeError(f"Copy datatypes differ: {a.get_datatype()} vs {b.get_datatype()}")
        if a_offset < 0 or b_offset < 0 or n < 0 or a_offset + n > a.ecount() or b_offset + n > b.ecount():
            raise ValueError("Copy out of range")

    def memset(self, dev: DeviceBuffer, offset: int, value, n: int) -> None:
        if offset < 0 or n < 0 or offset + n > dev.ecount():
            raise ValueError("memset out of range")
        capi.call("ct_memset", self.handle, dev.ptr + offset * dtype_size(dev.datatype),
                  capi.DTYPE_CODES[dev.datatype], float(value), n)

    def create_event(self) -> Event:
        h = C.c_void_p()
        capi.call("ct_event_record", C.byref(h), self.handle)
        return Event(h.value)

    def sync_event(self, event: Event) -> None:
        """Makes this stream wait for ``event`` (``PStream sync-event``)."""
        capi.call("ct_stream_wait_event", self.handle, event.handle)

    def sync(self) -> None:
        """``drv/sync-stream`` (``compute/driver.clj:217-221``)."""
        capi.call("ct_stream_sync", self.handle)

    def release(self) -> None:
        if self.handle:
            capi.call("ct_stream_destroy", self.handle)
            self.handle = None

    # -- TensorMath (src/cortex/tensor/math.clj:14-104) ---------------------
    def assign_constant(self, buffer, dimensions, value, n_elems) -> None:
        capi.call("ct_assign_constant", self.handle, buffer.ptr, C.byref(_dims_struct(dimensions)),
                  capi.DTYPE_CODES[buffer.datatype], float(value), int(n_elems))

    def assign(self, dest, dest_dims, src, src_dims, n_elems) -> None:
        capi.call("ct_assign", self.handle, dest.ptr, C.byref(_dims_struct(dest_dims)), capi.DTYPE_CODES[dest.datatype],
                  src.ptr, C.byref(_dims_struct(src_dims)), capi.DTYPE_CODES[src.datatype], int(n_elems))

    def unary_accum(self, dest, dest_dims, alpha, op, n_elems) -> None:
        capi.call("ct_unary_accum", self.handle, dest.ptr, C.byref(_dims_struct(dest_dims)), float(alpha),
                  capi.UNARY_OPS[op], capi.DTYPE_CODES[dest.datatype], int(n_elems))

    def unary_op(self, dest, dest_dims, x, x_dims, alpha, op, n_elems) -> None:
        capi.call("ct_unary_op", self.handle, dest.ptr, C.byref(_dims_struct(dest_dims)), x.ptr,
                  C.byref(_dims_struct(x_dims)), float(alpha), capi.UNARY_OPS[op], capi.DTYPE_CODES[dest.datatype],
                  int(n_elems))

    def binary_accum_constant(self, dest, dest_dims, dest_alpha, scalar, n_elems, operation, reverse_operands) -> None:
        capi.call("ct_binary_accum_constant", self.handle, dest.ptr, C.byref(_dims_struct(dest_dims)), float(dest_alpha),
                  float(scalar), int(n_elems), capi.BINARY_OPS[operation], int(bool(reverse_operands)),
                  capi.DTYPE_CODES[dest.datatype])

    def binary_op_constant(self, dest, dest_dims, x, x_dims, x_alpha, scalar, n_elems, operation, reverse_operands) -> None:
        capi.call("ct_binary_op_constant", self.handle, dest.ptr, C.byref(_dims_struct(dest_dims)), x.ptr,
                  C.byref(_dims_struct(x_dims)), float(x_alpha), float(scalar), int(n_elems),
                  capi.BINARY_OPS[operation], int(bool(reverse_operands)), capi.DTYPE_CODES[dest.datatype])

    def binary_accum(self, dest, dest_dims, dest_alpha, y, y_dims, y_alpha, n_elems, operation, reverse_operands,
                     dest_requires_cas) -> None:
        capi.call("ct_binary_accum", self.handle, dest.ptr, C.byref(_dims_struct(dest_dims)), float(dest_alpha), y.ptr,
                  C.byref(_dims_struct(y_dims)), float(y_alpha), int(n_elems), capi.BINARY_OPS[operation],
                  int(bool(reverse_operands)), int(bool(dest_requires_cas)), capi.DTYPE_CODES[dest.datatype])

    def binary_op(self, dest, dest_dims, x, x_dims, x_alpha, y, y_dims, y_alpha, n_elems, operation) -> None:
        capi.call("ct_binary_op", self.handle, dest.ptr, C.byref(_dims_struct(dest_dims)), x.ptr,
                  C.byref(_dims_struct(x_dims)), float(x_alpha), y.ptr, C.byref(_dims_struct(y_dims)), float(y_alpha),
                  int(n_elems), capi.BINARY_OPS[operation], capi.DTYPE_CODES[dest.datatype])

    def ternary_op(self, dest, dest_dims, x, x_dims, x_alpha, y, y_dims, y_alpha, z, z_dims, z_alpha, n_elems,
                   operation) -> None:
        capi.call("ct_ternary_op", self.handle, dest.ptr, C.byref(_dims_struct(dest_dims)), x.ptr,
                  C.byref(_dims_struct(x_dims)), float(x_alpha), y.ptr, C.byref(_dims_struct(y_dims)), float(y_alpha),
                  z.ptr, C.byref(_dims_struct(z_dims)), float(z_alpha), int(n_elems), capi.TERNARY_OPS[operation],
                  capi.DTYPE_CODES[dest.datatype])

    def ternary_op_constant(self, dest, dest_dims, a, a_dims, a_alpha, b, b_dims, b_alpha, constant, n_elems, operation,
                            arg_order) -> None:
        capi.call("ct_ternary_op_constant", self.handle, dest.ptr, C.byref(_dims_struct(dest_dims)), a.ptr,
                  C.byref(_dims_struct(a_dims)), float(a_alpha), b.ptr, C.byref(_dims_struct(b_dims)), float(b_alpha),
                  float(constant), int(n_elems), capi.TERNARY_OPS[operation], _arg_order_indexes(arg_order),
                  capi.DTYPE_CODES[dest.datatype])

    def ternary_op_constant_constant(self, dest, dest_dims, a, a_dims, a_alpha, const_1, const_2, n_elems, operation,
                                     arg_order) -> None:
        capi.call("ct_ternary_op_constant_constant", self.handle, dest.ptr, C.byref(_dims_struct(dest_dims)), a.ptr,
                  C.byref(_dims_struct(a_dims)), float(a_alpha), float(const_1), float(const_2), int(n_elems),
                  capi.TERNARY_OPS[operation], _arg_order_indexes(arg_order), capi.DTYPE_CODES[dest.datatype])

    def unary_reduce(self, output, output_dims, input_alpha, input, input_dims, op) -> None:
        capi.call("ct_unary_reduce", self.handle, output.ptr, C.byref(_dims_struct(output_dims)), float(input_alpha),
                  input.ptr, C.byref(_dims_struct(input_dims)), capi.REDUCE_OPS[op], capi.DTYPE_CODES[output.datatype])

    # -- neural-network tensor ops (tensor/math.clj:176-189) ------------------
    def activation_gradient(self, input_gradient, input_grad_dims, output_gradient, output_grad_dims, output,
                            output_dims, op, element_count) -> None:
        capi.call("ct_activation_gradient", self.handle, input_gradient.ptr, C.byref(_dims_struct(input_grad_dims)),
                  output_gradient.ptr, C.byref(_dims_struct(output_grad_dims)), output.ptr,
                  C.byref(_dims_struct(output_dims)), capi.ACTIVATION_OPS[op], int(element_count),
                  capi.DTYPE_CODES[input_gradient.datatype])

    def softmax_eltwise(self, output, output_dims, input, input_dims) -> None:
        capi.call("ct_softmax_eltwise", self.handle, output.ptr, C.byref(_dims_struct(output_dims)), input.ptr,
                  C.byref(_dims_struct(input_dims)), capi.DTYPE_CODES[output.datatype])

    def softmax_spatial(self, output, output_dims, input, input_dims) -> None:
        capi.call("ct_softmax_spatial", self.handle, output.ptr, C.byref(_dims_struct(output_dims)), input.ptr,
                  C.byref(_dims_struct(input_dims)), capi.DTYPE_CODES[output.datatype])

    # -- convolution (tensor/math.clj:185-220); buffers are packed, the workspace is the caller's --
    def convolution_descriptor(self, datatype, out_channels, in_channels, kern_width, kern_height, pad_x, pad_y,
                               stride_x, stride_y):
        return None   # no native object, as on the CPU backend (cpu/tensor_math.clj:1665-1668)

    def choose_convolution_algorithms(self, conv_descriptor, input_width, input_height, output_width, output_height,
                                      batch_size, max_ideal_workspace_size, use_defaults):
        """Workspace for the unrolled input (cpu/tensor_math.clj:1670-1680)."""
        n_cols = int(conv_descriptor["kernel-width"]) * int(conv_descriptor["kernel-height"]) * \
            int(conv_descriptor["in-channels"])
        return {"workspace-size": n_cols * int(output_width) * int(output_height) * int(batch_size)}

    def _conv(self, name, dest, alpha, a, b, workspace, workspace_ecount, conv_descriptor, in_shape, out_shape):
        batch, _, in_h, in_w = (int(v) for v in in_shape)
        out_h, out_w = (int(v) for v in out_shape[2:])
        desc = capi.make_conv_desc(conv_descriptor)
        capi.call(name, self.handle, dest.ptr, float(alpha), a.ptr, b.ptr, workspace.ptr, int(workspace_ecount),
                  C.byref(desc), int(out_shape[0]), in_h, in_w, out_h, out_w, capi.DTYPE_CODES[dest.datatype])

    def convolution_forward(self, output, output_dims, output_alpha, input, input_dims, weights, weight_dims,
                            workspace, workspace_ecount, conv_descriptor, algorithms) -> None:
        self._conv("ct_convolution_forward", output, output_alpha, input, weights, workspace, workspace_ecount,
                   conv_descriptor, input_dims["shape"], output_dims["shape"])

    def convolution_backward_weights(self, weight_gradient, weight_gradient_dims, weight_gradient_alpha,
                                     output_gradient, output_gradient_dims, input, input_dims, workspace,
                                     workspace_ecount, conv_descriptor, algorithms) -> None:
        self._conv("ct_convolution_backward_weights", weight_gradient, weight_gradient_alpha, output_gradient, input,
                   workspace, workspace_ecount, conv_descriptor, input_dims["shape"], output_gradient_dims["shape"])

    def convolution_backward_data(self, input_gradient, input_gradient_dims, input_gradient_alpha, output_gradient,
                                  output_gradient_dims, weights, weights_dims, workspace, workspace_ecount,
                                  conv_descriptor, algorithms) -> None:
        self._conv("ct_convolution_backward_data", input_gradient, input_gradient_alpha, output_gradient, weights,
                   workspace, workspace_ecount, conv_descriptor, input_gradient_dims["shape"],
                   output_gradient_dims["shape"])

    # -- pooling (tensor/math.clj:221-236); buffers are packed [batch channels height width] --
    def pooling_forward(self, output, output_dims, output_alpha, input, input_dims, pool_descriptor) -> None:
        batch, channels, in_h, in_w = (int(v) for v in input_dims["shape"])
        out_h, out_w = (int(v) for v in output_dims["shape"][2:])
        desc = capi.make_pool_desc(pool_descriptor)
        capi.call("ct_pooling_forward", self.handle, output.ptr, float(output_alpha), input.ptr, C.byref(desc), batch,
                  channels, in_h, in_w, out_h, out_w, capi.DTYPE_CODES[output.datatype])

    def pooling_backward(self, input_grad, input_grad_dims, input_grad_alpha, input, input_dims, output, output_dims,
                         output_grad, output_grad_dims, pool_descriptor) -> None:
        batch, channels, in_h, in_w = (int(v) for v in input_dims["shape"])
        out_h, out_w = (int(v) for v in output_dims["shape"][2:])
        desc = capi.make_pool_desc(pool_descriptor)
        capi.call("ct_pooling_backward", self.handle, input_grad.ptr, float(input_grad_alpha), input.ptr, output.ptr,
                  output_grad.ptr, C.byref(desc), batch, channels, in_h, in_w, out_h, out_w,
                  capi.DTYPE_CODES[output.datatype])

    # -- local response normalization (tensor/math.clj:240-252); the descriptor is a plain map --
    def lrn_forward(self, output, output_dims, input, input_dims, lrn_descriptor) -> None:
        d = lrn_descriptor
        capi.call("ct_lrn_forward", self.handle, output.ptr, C.byref(_dims_struct(output_dims)), input.ptr,
                  C.byref(_dims_struct(input_dims)), int(d["n"]), float(d["k"]), float(d["alpha"]), float(d["beta"]),
                  capi.DTYPE_CODES[output.datatype])

    def lrn_backward(self, input_grad, input_grad_dims, output, output_dims, input, input_dims, output_grad,
                     output_grad_dims, lrn_descriptor) -> None:
        d = lrn_descriptor
        capi.call("ct_lrn_backward", self.handle, input_grad.ptr, C.byref(_dims_struct(input_grad_dims)), output.ptr,
                  C.byref(_dims_struct(output_dims)), input.ptr, C.byref(_dims_struct(input_dims)), output_grad.ptr,
                  C.byref(_dims_struct(output_grad_dims)), int(d["n"]), float(d["k"]), float(d["alpha"]),
                  float(d["beta"]), capi.DTYPE_CODES[output.datatype])

    # -- gemm!, gemv! (tensor/math.clj:106-123) ---------------------------------
    def gemm(self, c, c_colstride, trans_a, trans_b, alpha, a, a_row_count, a_col_count, a_colstride, b, b_col_count,
             b_colstride, beta) -> None:
        capi.call("ct_gemm", self.handle, c.ptr, int(c_colstride), int(bool(trans_a)), int(bool(trans_b)), float(alpha),
                  a.ptr, int(a_row_count), int(a_col_count), int(a_colstride), b.ptr, int(b_col_count),
                  int(b_colstride), float(beta), capi.DTYPE_CODES[c.datatype])

    def gemv(self, c, inc_c, trans_a, alpha, a, a_row_count, a_col_count, a_colstride, x, inc_x, beta) -> None:
        capi.call("ct_gemv", self.handle, c.ptr, int(inc_c), int(bool(trans_a)), float(alpha), a.ptr, int(a_row_count),
                  int(a_col_count), int(a_colstride), x.ptr, int(inc_x), float(beta), capi.DTYPE_CODES[c.datatype])

    # -- batch normalization (tensor/math.clj:124-174); every buffer is packed --
    def batch_normalize_eltwise(self, output, input, means, variances, scale, bias, epsilon, batch_count,
                                element_count) -> None:
        capi.call("ct_batch_normalize_eltwise", self.handle, output.ptr, input.ptr, means.ptr, variances.ptr,
                  scale.ptr, bias.ptr, float(epsilon), int(batch_count), int(element_count),
                  capi.DTYPE_CODES[output.datatype])

    def batch_normalize_spatial(self, output, input, means, variances, scale, bias, epsilon, batch_count,
                                channel_count, element_count) -> None:
        capi.call("ct_batch_normalize_spatial", self.handle, output.ptr, input.ptr, means.ptr, variances.ptr,
                  scale.ptr, bias.ptr, float(epsilon), int(batch_count), int(channel_count), int(element_count),
                  capi.DTYPE_CODES[output.datatype])

    def batch_normalize_update_and_apply_eltwise(self, output, input, batch_means, batch_variances, running_means,
                                                 running_variances, average_factor, scale, bias, epsilon,
                                                 batch_count, element_count) -> None:
        capi.call("ct_batch_normalize_update_and_apply_eltwise", self.handle, output.ptr, input.ptr, batch_means.ptr,
                  batch_variances.ptr, running_means.ptr, running_variances.ptr, float(average_factor), scale.ptr,
                  bias.ptr, float(epsilon), int(batch_count), int(element_count), capi.DTYPE_CODES[output.datatype])

    def batch_normalize_update_and_apply_spatial(self, output, input, batch_means, batch_variances, running_means,
                                                 running_variances, average_factor, scale, bias, epsilon,
                                                 batch_count, channel_count, element_count) -> None:
        capi.call("ct_batch_normalize_update_and_apply_spatial", self.handle, output.ptr, input.ptr, batch_means.ptr,
                  batch_variances.ptr, running_means.ptr, running_variances.ptr, float(average_factor), scale.ptr,
                  bias.ptr, float(epsilon), int(batch_count), int(channel_count), int(element_count),
                  capi.DTYPE_CODES[output.datatype])

    def batch_normalize_gradients_eltwise(self, input_gradient, scale_gradient, bias_gradient, output_gradient,
                                          output, input, batch_means, batch_variances, scale, bias, epsilon,
                                          batch_count, element_count) -> None:
        capi.call("ct_batch_normalize_gradients_eltwise", self.handle, input_gradient.ptr, scale_gradient.ptr,
                  bias_gradient.ptr, output_gradient.ptr, output.ptr, input.ptr, batch_means.ptr, batch_variances.ptr,
                  scale.ptr, bias.ptr, float(epsilon), int(batch_count), int(element_count),
                  capi.DTYPE_CODES[input_gradient.datatype])

    def batch_normalize_gradients_spatial(self, input_gradient, scale_gradient, bias_gradient, output_gradient,
                                          output, input, batch_means, batch_variances, scale, bias, epsilon,
                                          batch_count, channel_count, element_count) -> None:
        capi.call("ct_batch_normalize_gradients_spatial", self.handle, input_gradient.ptr, scale_gradient.ptr,
                  bias_gradient.ptr, output_gradient.ptr, output.ptr, input.ptr, batch_means.ptr, batch_variances.ptr,
                  scale.ptr, bias.ptr, float(epsilon), int(batch_count), int(channel_count), int(element_count),
                  capi.DTYPE_CODES[input_gradient.datatype])

    # -- rand! (tensor/math.clj:237) ------------------------------------------
    def seed_random(self, seed: int) -> None:
        """Restarts this stream's generator.  The reference's generators are
        seeded by their libraries (SecureRandom, cuRAND); an unseeded stream
        draws its seed from the operating system."""
        self._rand_seed = int(seed) & 0xFFFFFFFFFFFFFFFF
        self._rand_calls = 0

    def rand(self, dest, dest_dims, distribution) -> None:
        if getattr(self, "_rand_seed", None) is None:
            self.seed_random(int.from_bytes(os.urandom(8), "little"))
        kind = distribution["type"]
        if kind == "gaussian":
            a, b = distribution["mean"], distribution["variance"]
        elif kind == "flat":
            a, b = distribution["minimum"], distribution["maximum"]
        else:
            raise ValueError(f"Unrecognized distribution: {distribution}")
        n = int(np.prod([int(v) for v in dest_dims["shape"]], dtype=np.int64))
        capi.call("ct_rand", self.handle, dest.ptr, n, capi.DTYPE_CODES[dest.datatype], capi.DISTRIBUTIONS[kind],
                  float(a), float(b), self._rand_seed, self._rand_calls)
        self._rand_calls += 1

    def dropout_bernoulli_mask(self, mult_buffer, rand_buffer, probability) -> None:
        """The three tensor calls of ``dropout-prepare-forward!`` (``compute/nn/layers.clj:170-195``: ``rand!``,
        ``assign!``, ``ternary-op! :select``) as one launch with the same stored values.  ``rand_buffer`` may be
        None (or ``mult_buffer`` itself) when the draws need not be kept.  Advances the stream's generator state
        as one ``rand!`` call does."""
        if getattr(self, "_rand_seed", None) is None:
            self.seed_random(int.from_bytes(os.urandom(8), "little"))
        seed, offset = self._rand_seed, self._rand_calls
        self._rand_calls += 1
        capi.call("ct_dropout_bernoulli_mask", self.handle, mult_buffer.ptr, capi.DTYPE_CODES[mult_buffer.datatype],
                  None if rand_buffer is None else rand_buffer.ptr, int(mult_buffer.ecount()), float(probability),
                  seed, offset)

    # -- optimizers ---------------------------------------------------------
    def adam_step(self, alpha, beta1, beta2, epsilon, pow_beta1_t, pow_beta2_t, gradient_alpha, gradient, parameters,
                  m, v, n) -> None:
        capi.call("ct_adam_step", self.handle, capi.DTYPE_CODES[gradient.datatype], float(alpha), float(beta1),
                  float(beta2), float(epsilon), float(pow_beta1_t), float(pow_beta2_t), float(gradient_alpha),
                  gradient.ptr, parameters.ptr, m.ptr, v.ptr, int(n))

    def adadelta_step(self, decay, epsilon, grad_accum, dx_accum, gradient_alpha, gradient, parameters, n) -> None:
        capi.call("ct_adadelta_step", self.handle, capi.DTYPE_CODES[gradient.datatype], float(decay), float(epsilon),
                  grad_accum.ptr, dx_accum.ptr, float(gradient_alpha), gradient.ptr, parameters.ptr, int(n))


class HipDevice:
    def __init__(self, driver: "HipDriver", index: int):
        self.driver = driver
        self.index = index

    def get_driver(self) -> "HipDriver":
        return self.driver

    def make_current(self) -> None:
        capi.call("ct_set_device", self.index)

    def memory_info(self) -> dict:
        self.make_current()
        free, total = C.c_size_t(), C.c_size_t()
        capi.call("ct_memory_info", C.byref(free), C.byref(total))
        return {"free": free.value, "total": total.value}

    def create_stream(self) -> HipStream:
        self.make_current()
        h = C.c_void_p()
        capi.call("ct_stream_create", C.byref(h))
        return HipStream(self, h.value)

    def default_stream(self) -> HipStream:
        return HipStream(self, None)

    def allocate_device_buffer(self, elem_count: int, elem_type: str) -> DeviceBuffer:
        if elem_type not in capi.DTYPE_CODES:
            raise TypeError(f"Unknown datatype {elem_type!r}")
        self.make_current()
        p = C.c_void_p()
        capi.call("ct_malloc", C.byref(p), max(1, int(elem_count) * dtype_size(elem_type)))
        return DeviceBuffer(self, p.value, elem_count, elem_type)


class HipDriver:
    """``PDriver`` for the HIP backend."""

    type = "hip"

    def __init__(self):
        n = C.c_int(0)
        capi.call("ct_device_count", C.byref(n))
        self._devices = [HipDevice(self, i) for i in range(n.value)]

    def get_devices(self):
        return list(self._devices)

    def default_device(self) -> HipDevice:
        if not self._devices:
            raise RuntimeError("No HIP device is visible")
        return self._devices[0]

    def allocate_host_buffer(self, elem_count: int, elem_type: str, usage_type: str = "one-time") -> HostBuffer:
        if usage_type not in ("one-time", "reusable"):
            raise ValueError("Usage type is not in expected set")
        return HostBuffer(elem_count, elem_type)
