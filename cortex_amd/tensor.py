"""Backend-neutral tensor API: a Python mirror of the front half of
``src/cortex/tensor.clj`` (lines 1-884) for the tensor-math path.

It does what the reference's tensor layer does before it reaches a backend:
validation, alias detection, scalar folding, the ``:-`` to ``:+`` rewrite, the
``x * const`` strength reduction, the choice between the plain / accumulate /
constant variants, and the ``arg-order`` bookkeeping of ``ternary-op!``.  The
backend is whatever *stream* is bound (:func:`tensor_context`); it must
implement the ``TensorMath`` methods (``src/cortex/tensor/math.clj:14-104``)
and the ``PStream`` copies.  :class:`cortex_amd.driver.HipStream` is the HIP
backend; the tests bind a CPU-oracle stream to the very same functions.

Names follow the reference with ``!`` dropped and ``-`` turned into ``_``.
"""
from __future__ import annotations

import contextlib
import contextvars
import itertools
import math
from typing import Sequence

import numpy as np

from . import dimensions as dims

_stream = contextvars.ContextVar("cortex_stream", default=None)
_datatype = contextvars.ContextVar("cortex_datatype", default="double")

UNARY_OPERATIONS = ["floor", "ceil", "round", "-", "tanh", "logistic", "exp", "sqrt", "noop"]  # tensor.clj:607-609
BINARY_OPERATIONS = ["+", "-", "*", "/", "max", "min", "bit-and", "bit-xor", "eq", ">", ">=", "<", "<="]  # :764-765
UNARY_REDUCTION_OPERATIONS = ["max", "min", "sum", "mean", "magnitude-squared", "magnitude"]  # :857-858

NUMPY_OF = {"byte": np.int8, "short": np.int16, "int": np.int32, "long": np.int64, "float": np.float32,
            "double": np.float64, "ubyte": np.uint8}


class TensorError(ValueError):
    """Stands in for the ``ex-info`` of ``when-not-error``."""


@contextlib.contextmanager
def tensor_context(stream, datatype: str = "double"):
    """Binds ``*stream*`` and ``*datatype*`` (``tensor.clj:89-111``;
    ``src/cortex/verify/tensor.clj:11-17``)."""
    t1 = _stream.set(stream)
    t2 = _datatype.set(datatype)
    try:
        yield stream
    finally:
        _stream.reset(t1)
        _datatype.reset(t2)


def check_stream():
    s = _stream.get()
    if s is None:
        raise TensorError("Tensor stream is nil")
    return s


def current_datatype() -> str:
    return _datatype.get()


class Tensor:
    """``(defrecord Tensor [device dimensions buffer])`` (``tensor.clj:174-195``)."""

    def __init__(self, device, dimensions, buffer):
        self.device = device
        self.dimensions = dimensions
        self.buffer = buffer

    def get_datatype(self) -> str:
        return self.buffer.get_datatype()

    def ecount(self) -> int:
        return dims.ecount(self.dimensions)

    def shape(self):
        return dims.shape(self.dimensions)

    def _with(self, dimensions=None, buffer=None) -> "Tensor":
        return Tensor(self.device, dimensions if dimensions is not None else self.dimensions,
                      buffer if buffer is not None else self.buffer)


def is_tensor(x) -> bool:
    return isinstance(x, Tensor)


def _is_number(x) -> bool:
    return isinstance(x, (int, float, np.integer, np.floating)) and not isinstance(x, bool)


def ecount(t) -> int:
    return t.ecount()


def shape(t):
    return t.shape()


def get_datatype(t) -> str:
    return t.get_datatype()


def dense(t: Tensor) -> bool:
    return dims.dense(t.dimensions)


def _dtype_cast(value, datatype: str):
    """``drv/dtype-cast`` (``src/cortex/compute/driver.clj:17-43``) for scalars
    folded on the host."""
    if datatype in ("float", "double"):
        return float(np.float32(value)) if datatype == "float" else float(value)
    return int(value)


# ---------------------------------------------------------------- construction

def to_tensor(data, datatype: str = None) -> Tensor:
    """``->tensor`` (``tensor.clj:415-435``): uploads nested data."""
    datatype = datatype or current_datatype()
    stream = check_stream()
    arr = np.asarray(data)
    flat = arr.astype(NUMPY_OF[datatype]).reshape(-1)
    device = stream.get_device()
    driver = device.get_driver()
    host = driver.allocate_host_buffer(flat.size, datatype)
    dev = device.allocate_device_buffer(flat.size, datatype)
    host.array[...] = flat
    stream.copy_host_to_device(host, 0, dev, 0, flat.size)
    stream.sync()
    host.release()
    return Tensor(device, dims.dimensions(list(arr.shape)), dev)


def new_tensor(shape_: Sequence[int], datatype: str = None, init_value=0) -> Tensor:
    """``new-tensor`` (``tensor.clj:438-450``)."""
    datatype = datatype or current_datatype()
    stream = check_stream()
    n = int(np.prod(shape_)) if len(shape_) else 1
    device = stream.get_device()
    dev = device.allocate_device_buffer(n, datatype)
    if init_value is not None:
        stream.memset(dev, 0, 0, n)
    return Tensor(device, dims.dimensions(list(shape_)), dev)


def as_dense(t: Tensor):
    return t if dense(t) and dims.access_increasing(t.dimensions) else None


def make_dense(t: Tensor) -> Tensor:
    d = as_dense(t)
    if d is not None:
        return d
    out = new_tensor(shape(t), datatype=t.get_datatype(), init_value=None)
    assign(out, t)
    return out


def to_array_of_type(t: Tensor, datatype: str) -> np.ndarray:
    """``copy-to-java-type`` (``tensor.clj:375-395``)."""
    d = make_dense(t)
    n = d.ecount()
    stream = check_stream()
    host = stream.get_driver().allocate_host_buffer(n, d.get_datatype())
    stream.copy_device_to_host(d.buffer, 0, host, 0, n)
    stream.create_event().wait_for_event()
    out = np.array(host.array, dtype=NUMPY_OF[datatype])
    host.release()
    return out


def to_double_array(t: Tensor) -> np.ndarray:
    return to_array_of_type(t, "double")


# ---------------------------------------------------------------- views

def in_place_reshape(t: Tensor, shape_) -> Tensor:
    return t._with(dimensions=dims.in_place_reshape(t.dimensions, list(shape_)))


def as_vector(t: Tensor):
    """``PVectorView as-vector`` (``tensor.clj:1647-1650``)."""
    if dense(t):
        return t._with(dimensions=dims.dimensions([t.ecount()]))
    return None


def to_vector(t: Tensor) -> Tensor:
    d = make_dense(t)
    return d._with(dimensions=dims.dimensions([d.ecount()]))


def as_2d_matrix(t: Tensor) -> Tensor:
    return in_place_reshape(t, dims.to_2d_shape(t.dimensions))


def as_batch_matrix(t: Tensor) -> Tensor:
    return in_place_reshape(t, dims.to_batch_shape(t.dimensions))


def transpose(t: Tensor, reorder_vec) -> Tensor:
    """``transpose`` (``tensor.clj:453-459``): a view; no data moves."""
    return t._with(dimensions=dims.transpose(t.dimensions, list(reorder_vec)))


def select(t: Tensor, *args) -> Tensor:
    """``select`` (``tensor.clj:462-477``)."""
    res = dims.select(t.dimensions, *args)
    off = int(res["elem-offset"])
    buf = t.buffer.sub_buffer(off, t.buffer.ecount() - off)
    return t._with(dimensions=res["dimensions"], buffer=buf)


def subvector(t: Tensor, offset: int, length: int = None) -> Tensor:
    if offset < 0:
        raise TensorError("Offset must be >= 0")
    v = as_vector(t)
    stop = offset + length if length is not None else v.ecount()
    return select(v, list(range(offset, stop)))


def submatrix(t: Tensor, row_start, row_length, col_start, col_length) -> Tensor:
    """``submatrix`` (``tensor.clj:490-513``)."""
    t2 = as_2d_matrix(t)
    n_rows, n_cols = t2.shape()
    d = t2.dimensions
    rev_shape, rev_strides = list(reversed(d["shape"])), list(reversed(d["strides"]))
    addr = dims.elem_idx_to_addr(rev_shape, rev_strides, rev_shape, row_start * n_cols + col_start)
    buf = t2.buffer.sub_buffer(addr, t2.buffer.ecount() - addr)
    return t2._with(dimensions={"shape": [row_length, col_length], "strides": list(d["strides"])}, buffer=buf)


def rows(t: Tensor):
    n_rows, n_cols = dims.to_2d_shape(t.dimensions)
    return [select(t, r, list(range(n_cols))) for r in range(n_rows)]


def columns(t: Tensor):
    n_rows, n_cols = dims.to_2d_shape(t.dimensions)
    return [select(t, list(range(n_rows)), c) for c in range(n_cols)]


# ---------------------------------------------------------------- checks

def _ensure_datatypes(datatype, *args) -> None:
    if not all(a.get_datatype() == datatype for a in args):
        raise TensorError(f"Not all arguments match required datatype {datatype}: {[a.get_datatype() for a in args]}")


def _ensure_same_device(*args) -> None:
    if not all(a.device is args[0].device for a in args[1:]):
        raise TensorError("Tensor arguments are not all on same device")


def _check_partial_alias(*args) -> None:
    for a, b in itertools.combinations([t.buffer for t in args], 2):
        if a.partially_alias(b):
            raise TensorError("Partially overlapping arguments detected.")


def _ensure_broadcast_rules(*args) -> None:
    """``ensure-broadcast-rules`` (``tensor.clj:592-604``): every operand
    dimension must divide the max dimension."""
    info = dims.dimension_seq_to_max_shape(*[a.dimensions for a in args])
    max_shape = info["max-shape"]
    for d in info["dimensions"]:
        for mx, s in zip(max_shape, dims.shape(d)):
            if mx % s != 0:
                raise TensorError("Shapes are not broadcast-compatible (dimension counts must be commensurate) "
                                  f"{[dims.shape(x) for x in info['dimensions']]} vs {max_shape}")


# ---------------------------------------------------------------- assign!

def _memcpy_semantics(dest: Tensor, src: Tensor) -> bool:
    return (dest.ecount() == src.ecount() and dense(dest) and dense(src)
            and dims.access_increasing(dest.dimensions) and dims.access_increasing(src.dimensions)
            and dest.get_datatype() == src.get_datatype())


def assign(dest: Tensor, src) -> Tensor:
    """``assign!`` / ``typed-assign!`` (``tensor.clj:535-589``)."""
    stream = check_stream()
    if _is_number(src):
        if dense(dest):
            stream.memset(dest.buffer, 0, src, dest.ecount())
        else:
            stream.assign_constant(dest.buffer, dest.dimensions, src, dest.ecount())
        return dest
    de, se = dest.ecount(), src.ecount()
    if not de >= se:
        raise TensorError("destination element count must be >= src element count")
    if se != 0 and de % se != 0:
        raise TensorError("Src element count must evenly divide dest ecount.")
    _ensure_same_device(dest, src)
    _check_partial_alias(dest, src)
    if _memcpy_semantics(dest, src):
        stream.copy_device_to_device(src.buffer, 0, dest.buffer, 0, se)
    else:
        stream.assign(dest.buffer, dest.dimensions, src.buffer, src.dimensions, max(se, de))
    return dest


# ---------------------------------------------------------------- unary-op!

def _perform_unary_op(value: float, op: str) -> float:
    """``perform-unary-op`` (``tensor.clj:612-624``)."""
    if op == "ceil":
        return math.ceil(value)
    if op == "round":
        return math.floor(value + 0.5)
    if op == "floor":
        return math.floor(value)
    if op == "-":
        return -value
    if op == "tanh":
        return math.tanh(value)
    if op == "logistic":
        return 1.0 / (1.0 + math.exp(-value))
    if op == "exp":
        return math.exp(value)
    if op == "sqrt":
        return math.sqrt(value)
    if op == "noop":
        return value
    raise TensorError(f"Unknown unary operation {op}")


def unary_op(dest: Tensor, alpha, x, op: str) -> Tensor:
    """``unary-op!`` (``tensor.clj:627-651``): dest = op(alpha * x)."""
    if op not in UNARY_OPERATIONS:
        raise TensorError(f"Unknown unary operation {op}")
    if _is_number(x):
        dt = dest.get_datatype()
        return assign(dest, _perform_unary_op(float(_dtype_cast(alpha, dt)) * float(_dtype_cast(x, dt)), op))
    stream = check_stream()
    if dest.buffer.alias(x.buffer):
        stream.unary_accum(dest.buffer, dest.dimensions, alpha, op, dest.ecount())
    else:
        _ensure_datatypes(dest.get_datatype(), x)
        _ensure_same_device(dest, x)
        _ensure_broadcast_rules(dest, x)
        _check_partial_alias(dest, x)
        stream.unary_op(dest.buffer, dest.dimensions, x.buffer, x.dimensions, alpha, op, max(dest.ecount(), x.ecount()))
    return dest


# ---------------------------------------------------------------- binary-op!

def _binary_op_constant(dest, alpha, x, beta, y, op, reverse_operands) -> Tensor:
    """``binary-op-constant!`` (``tensor.clj:676-703``)."""
    _ensure_broadcast_rules(dest, x)
    _ensure_datatypes(dest.get_datatype(), x)
    y = float(beta) * float(y)
    stream = check_stream()
    if op == "*":  # strength reduction
        return unary_op(dest, float(alpha) * y, x, "noop")
    if dest.buffer.alias(x.buffer):
        stream.binary_accum_constant(dest.buffer, dest.dimensions, alpha, y, dest.ecount(), op, reverse_operands)
    else:
        _check_partial_alias(dest, x)
        stream.binary_op_constant(dest.buffer, dest.dimensions, x.buffer, x.dimensions, alpha, y,
                                  max(x.ecount(), dest.ecount()), op, reverse_operands)
    return dest


def _typed_binary_op(dest, alpha, x, beta, y, op) -> Tensor:
    xn, yn = _is_number(x), _is_number(y)
    if xn and yn:  # tensor.clj:662-673
        a, b = float(alpha) * float(x), float(beta) * float(y)
        table = {"+": lambda: a + b, "-": lambda: a - b, "*": lambda: a * b, "/": lambda: a / b,
                 "max": lambda: max(a, b), "min": lambda: min(a, b)}
        return assign(dest, table[op]())
    if yn:
        return _binary_op_constant(dest, alpha, x, beta, y, op, False)
    if xn:
        return _binary_op_constant(dest, beta, y, alpha, x, op, True)
    # [:tensor :tensor] (tensor.clj:716-761)
    stream = check_stream()
    info = dims.dimension_seq_to_max_shape(dest.dimensions, x.dimensions, y.dimensions)
    max_shape = info["max-shape"]
    dest_dims, x_dims, y_dims = info["dimensions"]
    x_alias = dest.buffer.alias(x.buffer)
    arg_alias = x_alias or dest.buffer.alias(y.buffer)
    # the comparison is against the raw shape vector, index tensors included
    dest_is_max_shape = list(dest_dims["shape"]) == list(max_shape) and dims.direct(dest_dims)
    if not dest_is_max_shape and not arg_alias:
        raise TensorError("If destination is a broadcast target then it must be one of the operands")
    if arg_alias:
        if x_alias:
            a, b, other, rev = alpha, beta, y, False
        else:
            a, b, other, rev = beta, alpha, x, True
        _ensure_broadcast_rules(dest, other)
        _ensure_datatypes(dest.get_datatype(), other)
        stream.binary_accum(dest.buffer, dest.dimensions, a, other.buffer, other.dimensions, b,
                            max(dest.ecount(), other.ecount()), op, rev, not dest_is_max_shape)
    else:
        _ensure_broadcast_rules(dest, x, y)
        _ensure_datatypes(x.get_datatype(), y, dest)
        stream.binary_op(dest.buffer, dest_dims, x.buffer, x_dims, alpha, y.buffer, y_dims, beta,
                         max(dest.ecount(), x.ecount(), y.ecount()), op)
    return dest


def binary_op(dest: Tensor, alpha, x, beta, y, op: str) -> Tensor:
    """``binary-op!`` (``tensor.clj:768-779``): dest = alpha*x op beta*y."""
    if op not in BINARY_OPERATIONS:
        raise TensorError(f"Unknown binary operation {op}")
    if op == "-":
        return _typed_binary_op(dest, alpha, x, -float(beta), y, "+")
    return _typed_binary_op(dest, alpha, x, beta, y, op)


# ---------------------------------------------------------------- ternary-op!

def ternary_op(dest: Tensor, alpha, x, beta, y, gamma, z, op: str = "select") -> Tensor:
    """``ternary-op!`` (``tensor.clj:808-854``).  select: ``(x >= 0) ? z : y``
    (``cpu/tensor_math.clj:464-466``)."""
    if op != "select":
        raise TensorError(f"Unknown ternary operation {op}")
    args = [(x, alpha, "x"), (y, beta, "y"), (z, gamma, "z")]
    tensors = [(v, a, n) for v, a, n in args if is_tensor(v)]
    consts = [(v, a, n) for v, a, n in args if not is_tensor(v)]
    if not tensors:
        value = float(gamma) * float(z) if float(alpha) * float(x) >= 0.0 else float(beta) * float(y)
        return assign(dest, value)
    max_ecount = max(t.ecount() for t, _, _ in tensors)
    constants = [float(v) * float(a) for v, a, _ in consts]
    arg_order = [n for _, _, n in tensors] + [n for _, _, n in consts]
    tens_only = [t for t, _, _ in tensors]
    _ensure_datatypes(dest.get_datatype(), *tens_only)
    _ensure_same_device(dest, *tens_only)
    for t in tens_only:
        _ensure_broadcast_rules(dest, t)
    stream = check_stream()
    if len(tensors) == 3:
        stream.ternary_op(dest.buffer, dest.dimensions, x.buffer, x.dimensions, alpha, y.buffer, y.dimensions, beta,
                          z.buffer, z.dimensions, gamma, max_ecount, op)
    elif len(tensors) == 2:
        (a, am, _), (b, bm, _) = tensors
        stream.ternary_op_constant(dest.buffer, dest.dimensions, a.buffer, a.dimensions, am, b.buffer, b.dimensions, bm,
                                   constants[0], max_ecount, op, arg_order)
    else:
        (a, am, _), = tensors
        stream.ternary_op_constant_constant(dest.buffer, dest.dimensions, a.buffer, a.dimensions, am, constants[0],
                                            constants[1], max_ecount, op, arg_order)
    return dest


# ---------------------------------------------------------------- unary-reduce!

def unary_reduce(output: Tensor, alpha, input: Tensor, op: str) -> Tensor:
    """``unary-reduce!`` (``tensor.clj:861-884``): reduces the last axis of the
    input view into an output whose last dimension is 1."""
    if op not in UNARY_REDUCTION_OPERATIONS:
        raise TensorError(f"Unknown reduction operation {op}")
    out_shape, in_shape = output.shape(), input.shape()
    if out_shape[:-1] != in_shape[:-1]:
        raise TensorError(f"Output leading dimensions must match input leading dimensions {out_shape} {in_shape}")
    if out_shape[-1] != 1:
        raise TensorError(f"Last dimension of output must be 1 {out_shape}")
    _ensure_same_device(output, input)
    _ensure_datatypes(output.get_datatype(), input)
    check_stream().unary_reduce(output.buffer, output.dimensions, alpha, input.buffer, input.dimensions, op)
    return output


# ---------------------------------------------------------------- activation-gradient!, softmax!

def _external_library_check(method_name: str, *tensors) -> None:
    """``external-library-check!`` (``tensor.clj:895-917``)."""
    _ensure_datatypes(tensors[0].get_datatype(), *tensors[1:])
    _ensure_same_device(*tensors)
    if tensors[0].get_datatype() not in ("float", "double"):
        raise TensorError(f"{method_name} is only defined for float and double tensors")
    if not all(dims.access_increasing(t.dimensions) for t in tensors):
        raise TensorError("External libraries (blas (gemm gemv) and cudnn require dimensions access to be increasing")


def activation_gradient(input_gradient: Tensor, output_gradient: Tensor, output: Tensor, op: str) -> Tensor:
    """``activation-gradient!`` (``tensor.clj:1256-1284``)."""
    _external_library_check("activation-gradient!", input_gradient, output, output_gradient)
    if op not in ("logistic", "tanh", "relu"):
        raise TensorError("Only :logistic :tanh and :relu are supported")
    n = ecount(output)
    if n != ecount(input_gradient) or n != ecount(output_gradient):
        raise TensorError("All element ecounts must match")
    check_stream().activation_gradient(input_gradient.buffer, input_gradient.dimensions, output_gradient.buffer,
                                       output_gradient.dimensions, output.buffer, output.dimensions, op, n)
    return input_gradient


def softmax(output: Tensor, input: Tensor) -> Tensor:
    """``softmax!`` (``tensor.clj:1286-1312``): three dimensions mean
    [batch channels elements] and a softmax across the channels; anything else
    is squashed to [batch, n] and normalised along n."""
    _external_library_check("softmax!", output, input)
    if output.shape() != input.shape():
        raise TensorError(f"Input, output shapes do not match {input.shape()} {output.shape()}")
    stream = check_stream()
    if len(input.shape()) == 3:
        stream.softmax_spatial(output.buffer, output.dimensions, input.buffer, input.dimensions)
    else:
        i, o = as_batch_matrix(input), as_batch_matrix(output)
        stream.softmax_eltwise(o.buffer, o.dimensions, i.buffer, i.dimensions)
    return output


# ---------------------------------------------------------------- convolution

def convolution_descriptor(datatype, out_channels, in_channels, kern_width, kern_height, pad_x, pad_y, stride_x,
                           stride_y):
    """``convolution-descriptor`` (``tensor.clj:1320-1348``)."""
    args = {"out-channels": out_channels, "in-channels": in_channels, "kern-width": kern_width,
            "kern-height": kern_height, "pad-x": pad_x, "pad-y": pad_y, "stride-x": stride_x, "stride-y": stride_y}
    missing = [k for k, v in args.items() if v is None]
    if missing:
        raise TensorError(f"Arguments were nil: {missing}")
    return {"datatype": datatype, "out-channels": out_channels, "in-channels": in_channels,
            "kernel-width": kern_width, "kernel-height": kern_height, "pad-x": pad_x, "pad-y": pad_y,
            "stride-x": stride_x, "stride-y": stride_y,
            "descriptor": check_stream().convolution_descriptor(datatype, out_channels, in_channels, kern_width,
                                                                kern_height, pad_x, pad_y, stride_x, stride_y)}


def choose_convolution_algorithms(descriptor, input_width, input_height, batch_size, max_ideal_workspace_size,
                                  use_defaults=False):
    """``choose-convolution-algorithms`` (``tensor.clj:1385-1401``)."""
    out = get_convolution_output_dimensions(descriptor, input_width, input_height)
    return check_stream().choose_convolution_algorithms(descriptor, input_width, input_height, out["output-width"],
                                                        out["output-height"], batch_size, max_ideal_workspace_size,
                                                        use_defaults)


def _ensure_conv_weight_dims_match(input: Tensor, weights: Tensor, descriptor) -> None:
    """``ensure-conv-weight-dims-match`` (``tensor.clj:1403-1423``)."""
    out_size, in_size = as_2d_matrix(weights).shape()
    if not dense(weights):
        raise TensorError("Convolution weights must be dense tensors")
    expected = int(descriptor["kernel-width"]) * int(descriptor["kernel-height"]) * int(descriptor["in-channels"])
    if int(in_size) != expected:
        raise TensorError(f"Weight column length does not equal kernel-width * kernel-height * in-channels: "
                          f"{in_size} {expected}")
    if int(out_size) != int(descriptor["out-channels"]):
        raise TensorError(f"Weight row count does not match out-channels: {out_size} {descriptor['out-channels']}")


def convolution_forward(output: Tensor, output_alpha, input: Tensor, weights: Tensor, workspace: Tensor,
                        conv_descriptor, algorithms) -> Tensor:
    """``convolution-forward!`` (``tensor.clj:1454-1467``)."""
    _external_library_check("convolution-forward!", output, input, weights)
    _ensure_conv_io(conv_descriptor, [input], [output])
    check_stream().convolution_forward(output.buffer, output.dimensions, output_alpha, input.buffer, input.dimensions,
                                       weights.buffer, weights.dimensions, workspace.buffer, ecount(workspace),
                                       conv_descriptor, algorithms)
    return output


def convolution_backward_weights(weight_gradient: Tensor, weight_gradient_alpha, output_gradient: Tensor,
                                 input: Tensor, workspace: Tensor, conv_descriptor, algorithms) -> Tensor:
    """``convolution-backward-weights!`` (``tensor.clj:1470-1481``)."""
    _external_library_check("convolution-backward-weights!", weight_gradient, output_gradient, input)
    check_stream().convolution_backward_weights(weight_gradient.buffer, weight_gradient.dimensions,
                                                weight_gradient_alpha, output_gradient.buffer,
                                                output_gradient.dimensions, input.buffer, input.dimensions,
                                                workspace.buffer, ecount(workspace), conv_descriptor, algorithms)
    return weight_gradient


def convolution_backward_data(input_gradient: Tensor, input_gradient_alpha, output_gradient: Tensor, weights: Tensor,
                              workspace: Tensor, conv_descriptor, algorithms) -> Tensor:
    """``convolution-backward-data!`` (``tensor.clj:1484-1496``)."""
    _external_library_check("convolution-backward-data!", input_gradient, output_gradient, weights)
    _ensure_conv_io(conv_descriptor, [input_gradient], [output_gradient])
    check_stream().convolution_backward_data(input_gradient.buffer, input_gradient.dimensions, input_gradient_alpha,
                                             output_gradient.buffer, output_gradient.dimensions, weights.buffer,
                                             weights.dimensions, workspace.buffer, ecount(workspace),
                                             conv_descriptor, algorithms)
    return input_gradient


# ---------------------------------------------------------------- pooling

POOL_OPERATIONS = ("max", "avg", "avg-exc-pad")


def _padded_strided_dimension(input_dim, pad, kernel_size, stride, dimension_op) -> int:
    """``get-padded-strided-dimension`` (``tensor.clj:1351-1365``)."""
    partial = (float(input_dim) + 2.0 * float(pad) - float(kernel_size)) / float(stride)
    if dimension_op == "floor":
        partial = math.floor(partial)
    elif dimension_op == "ceil":
        partial = math.ceil(partial)
    else:
        raise TensorError(f"No matching clause: {dimension_op}")
    return int(partial + 1)


def get_convolution_output_dimensions(descriptor, input_width, input_height):
    """``get-convolution-output-dimensions`` (``tensor.clj:1368-1382``)."""
    op = descriptor.get("dimension-op") or "floor"
    return {"output-width": _padded_strided_dimension(input_width, descriptor["pad-x"], descriptor["kernel-width"],
                                                      descriptor["stride-x"], op),
            "output-height": _padded_strided_dimension(input_height, descriptor["pad-y"],
                                                       descriptor["kernel-height"], descriptor["stride-y"], op)}


def pooling_descriptor(datatype, channels, kern_width, kern_height, pad_x, pad_y, stride_x, stride_y, *,
                       dimension_op="ceil", pool_op="max"):
    """``pooling-descriptor`` (``tensor.clj:1499-1524``); the library keeps no
    descriptor object of its own, as the CPU backend keeps none
    (``cpu/tensor_math.clj:1794-1798``)."""
    retval = {"in-channels": channels, "out-channels": channels, "datatype": datatype, "kernel-width": kern_width,
              "kernel-height": kern_height, "pad-x": pad_x, "pad-y": pad_y, "stride-x": stride_x,
              "stride-y": stride_y, "pool-op": pool_op, "dimension-op": dimension_op}
    missing = [k for k, v in retval.items() if v is None]
    if missing:
        raise TensorError(f"Nil values detected in map: {missing}")
    if pool_op not in POOL_OPERATIONS:
        raise TensorError(f"Max pooling layers have three possible pool operations: {POOL_OPERATIONS}, got {pool_op}")
    check_stream()
    return retval


def _ensure_conv_io(descriptor, input_args, output_args) -> None:
    """``ensure-conv-io`` (``tensor.clj:1425-1451``).  As there, the output is
    expected as [batch channels output-width output-height] and only the first
    tensor of each list is compared."""
    batch_size, _, in_height, in_width = input_args[0].shape()
    out = get_convolution_output_dimensions(descriptor, in_height, in_width)
    expected_input = [batch_size, int(descriptor["in-channels"]), in_height, in_width]
    expected_output = [batch_size, int(descriptor["out-channels"]), out["output-width"], out["output-height"]]
    if not all(dense(t) for t in list(input_args) + list(output_args)):
        raise TensorError("Convolution arguments must be dense tensors")
    if list(input_args[0].shape()) != expected_input:
        raise TensorError(f"Input dimensions do not match expected dimensions {expected_input} "
                          f"{list(input_args[0].shape())}")
    if list(output_args[0].shape()) != expected_output:
        raise TensorError(f"Output dimensions do not match expected dimensions {expected_output} "
                          f"{list(output_args[0].shape())}")


def pooling_forward(output: Tensor, output_alpha, input: Tensor, pool_descriptor) -> Tensor:
    """``pooling-forward!`` (``tensor.clj:1527-1538``)."""
    _external_library_check("pooling-forward!", output, input)
    _ensure_conv_io(pool_descriptor, [input], [output])
    check_stream().pooling_forward(output.buffer, output.dimensions, output_alpha, input.buffer, input.dimensions,
                                   pool_descriptor)
    return output


def pooling_backward(input_gradient: Tensor, input_grad_alpha, input: Tensor, output: Tensor,
                     output_gradient: Tensor, pool_descriptor) -> Tensor:
    """``pooling-backward!`` (``tensor.clj:1541-1551``)."""
    _external_library_check("pooling-backward!", input_gradient, input, output, output_gradient)
    _ensure_conv_io(pool_descriptor, [input_gradient, input], [output, output_gradient])
    check_stream().pooling_backward(input_gradient.buffer, input_gradient.dimensions, input_grad_alpha, input.buffer,
                                    input.dimensions, output.buffer, output.dimensions, output_gradient.buffer,
                                    output_gradient.dimensions, pool_descriptor)
    return input_gradient


# ---------------------------------------------------------------- local response normalization

def lrn_descriptor(*, n=5, k=2, alpha=1e-4, beta=0.75) -> dict:
    """``lrn-descriptor`` (``tensor.clj:1554-1560``): the window and the three
    constants, with the reference's defaults.  The library keeps no native
    object for it."""
    return {"n": int(n), "k": float(k), "alpha": float(alpha), "beta": float(beta)}


def _lrn_shapes(*named) -> None:
    first = named[0][1].shape()
    if any(t.shape() != first for _, t in named[1:]):
        raise TensorError("Input and output shapes must match " + str({name: t.shape() for name, t in named}))
    if len(first) < 3:
        raise TensorError(f"tensor must be of at least rank 3: {first}")


def lrn_forward(output: Tensor, input: Tensor, lrn_desc: dict) -> Tensor:
    """``lrn-forward!`` (``tensor.clj:1563-1583``): every value divided by
    ``(k + alpha / n * sum of squares over the n neighbouring channels) ** beta``."""
    _lrn_shapes(("input-shape", input), ("output-shape", output))
    _external_library_check("lrn-forward", output, input)
    check_stream().lrn_forward(output.buffer, output.dimensions, input.buffer, input.dimensions, lrn_desc)
    return output


def lrn_backward(input_gradient: Tensor, output: Tensor, input: Tensor, output_gradient: Tensor, lrn_desc: dict) -> Tensor:
    """``lrn-backward!`` (``tensor.clj:1586-1616``)."""
    _lrn_shapes(("input-shape", input), ("output-shape", output), ("in-grad-shape", input_gradient),
                ("out-grad-shape", output_gradient))
    _external_library_check("lrn-forward", output, input, input_gradient, output_gradient)
    check_stream().lrn_backward(input_gradient.buffer, input_gradient.dimensions, output.buffer, output.dimensions,
                                input.buffer, input.dimensions, output_gradient.buffer, output_gradient.dimensions, lrn_desc)
    return input_gradient


# ---------------------------------------------------------------- gemm!, gemv!

def _column_stride(t: Tensor) -> int:
    """``dimensions->column-stride`` (``tensor.clj:198-204``)."""
    strides, shp = t.dimensions["strides"], t.dimensions["shape"]
    return int(strides[-2]) if len(strides) > 1 else int(shp[0]) if shp else 1


def _2d_shape(t: Tensor):
    return dims.to_2d_shape(t.dimensions)


def gemm(C: Tensor, trans_a, trans_b, alpha, A: Tensor, B: Tensor, beta) -> Tensor:
    """``gemm!`` (``tensor.clj:920-951``): C = alpha * (trans-a? A) * (trans-b? B) + beta * C."""
    _external_library_check("gemm!", C, A, B)
    a_shape = _2d_shape(A)[::-1] if trans_a else _2d_shape(A)
    b_shape = _2d_shape(B)[::-1] if trans_b else _2d_shape(B)
    c_shape = _2d_shape(C)
    if a_shape[1] != b_shape[0]:
        raise TensorError(f"A {a_shape} col count doesn't match B {b_shape} row count")
    if a_shape[0] != c_shape[0]:
        raise TensorError(f"C {c_shape} rows count doesn't match A {a_shape} row count")
    if b_shape[1] != c_shape[1]:
        raise TensorError(f"C {c_shape} col count doesn't match B {b_shape} col count")
    check_stream().gemm(C.buffer, _column_stride(C), trans_a, trans_b, alpha, A.buffer, a_shape[0], a_shape[1],
                        _column_stride(A), B.buffer, b_shape[1], _column_stride(B), beta)
    return C


def _blas_vector_increment(t: Tensor) -> int:
    """``blas-vector-increment`` (``tensor.clj:966-972``)."""
    if dense(t):
        return 1
    strides = t.dimensions["strides"]
    return int(strides[-1]) if strides else 1


def gemv(c: Tensor, trans_a, alpha, A: Tensor, x: Tensor, beta) -> Tensor:
    """``gemv!`` (``tensor.clj:975-989``): c = alpha * (trans-a? A) * x + beta * c."""
    _external_library_check("gemv!", c, A, x)
    for t in (x, c):
        if not (dense(t) or _num_columns(t) == 1):
            raise TensorError("Argument is not vector-indexable")
    a_rows, a_cols = _2d_shape(A)
    check_stream().gemv(c.buffer, _blas_vector_increment(c), trans_a, alpha, A.buffer, a_rows, a_cols,
                        _column_stride(A), x.buffer, _blas_vector_increment(x), beta)
    return c


# ---------------------------------------------------------------- rand!

def gaussian_distribution(mean=0, variance=1) -> dict:
    """``gaussian-distribution`` (``tensor.clj:989-996``)."""
    return {"type": "gaussian", "mean": float(mean), "variance": float(variance)}


def flat_distribution(minimum=0, maximum=1) -> dict:
    """``flat-distribution`` (``tensor.clj:999-1013``): [minimum, maximum)."""
    if not float(minimum) < float(maximum):
        raise TensorError("Minimum must be less than maximum")
    return {"type": "flat", "minimum": float(minimum), "maximum": float(maximum)}


def rand(dest: Tensor, distribution: dict) -> Tensor:
    """``rand!`` (``tensor.clj:1026-1044``): float tensors with simple dense buffers only."""
    if dest.get_datatype() != "float":
        raise TensorError("Can only generate rands into floating point buffers")
    if not (dense(dest) and dims.access_increasing(dest.dimensions)):
        raise TensorError("Rand generation must have simple dense buffers")
    if distribution.get("type") not in ("gaussian", "flat"):
        raise TensorError("Invalid distibution type")
    check_stream().rand(dest.buffer, dest.dimensions, distribution)
    return dest


# ---------------------------------------------------------------- batch normalization

def _num_columns(t: Tensor) -> int:
    """``dimensions->num-columns`` (``tensor.clj:207-209``): the second shape entry, 1 if there is none."""
    shp = t.shape()
    return int(shp[1]) if len(shp) > 1 else 1


def as_row_vector(t: Tensor) -> Tensor:
    """``as-row-vector`` (``tensor.clj:307-314``)."""
    if not (_num_columns(t) == 1 or dense(t)):
        raise TensorError("Row vectors must either be dense or have num-columns = 1")
    return t._with(dimensions=dims.dimensions([t.ecount()]))


def _batch_normalize_setup(io_args, mvbs_args, epsilon):
    """``batch-normalize-setup`` (``tensor.clj:1040-1099``).  Returns
    (kind, row-vector statistics tensors, input shape).  The backends take
    packed buffers (``tensor/math.clj:124-137``); the reference does not check
    that, this mirror does."""
    all_args = list(io_args) + list(mvbs_args)
    inp = io_args[0]
    input_shape = list(inp.shape())
    if len(input_shape) == 1:
        input_shape = [1, input_shape[0]]
    _external_library_check("batch-normalize", *all_args)
    if not float(epsilon) > 1e-5:
        raise TensorError("Epsilon cannot be smaller than 1e-5 (cudnn limitation")
    for t in mvbs_args:
        if not (dense(t) or _num_columns(t) == 1):
            raise TensorError("Argument is not vector-indexable")
    vectors = [as_row_vector(t) for t in mvbs_args]
    if len(input_shape) < 2:
        raise TensorError("Input shape needs at least 2 dimensions")
    if len({tuple(t.shape()) for t in io_args}) != 1:
        raise TensorError("Tensor input and output shapes do not match")
    if len({tuple(t.shape()) for t in vectors}) != 1:
        raise TensorError("means, variances, scale, bias must have same shape")
    if not all(dense(t) for t in all_args):
        raise TensorError("batch-normalize: all tensors must be packed")
    n_stats = vectors[0].shape()[0]
    if len(input_shape) == 2:
        if input_shape[1] != n_stats:
            raise TensorError("Means, variances, scale, bias must match input element count.")
        return "eltwise", vectors, input_shape
    if input_shape[-2] != n_stats:
        raise TensorError("means, variances, scale bias size must match input channel count")
    return "spatial", vectors, input_shape


def _bn_counts(input_shape):
    batch_count = int(np.prod(input_shape[:-2], dtype=np.int64))
    return batch_count, int(input_shape[-2]), int(input_shape[-1])


def batch_normalize(output: Tensor, input: Tensor, means: Tensor, variances: Tensor, scale: Tensor, bias: Tensor,
                    epsilon) -> Tensor:
    """``batch-normalize!`` (``tensor.clj:1102-1147``):
    output = (input - mean) / sqrt(variance + epsilon) * scale + bias, per
    trailing element for two dimensions, per channel (second to last dimension)
    for more."""
    kind, (means, variances, scale, bias), input_shape = _batch_normalize_setup(
        [output, input], [means, variances, scale, bias], epsilon)
    stream = check_stream()
    if kind == "eltwise":
        stream.batch_normalize_eltwise(output.buffer, input.buffer, means.buffer, variances.buffer, scale.buffer,
                                       bias.buffer, epsilon, input_shape[0], input_shape[1])
    else:
        stream.batch_normalize_spatial(output.buffer, input.buffer, means.buffer, variances.buffer, scale.buffer,
                                       bias.buffer, epsilon, *_bn_counts(input_shape))
    return output


def batch_normalize_update_and_apply(output: Tensor, input: Tensor, batch_means: Tensor, batch_variances: Tensor,
                                     running_means: Tensor, running_variances: Tensor, ave_factor, scale: Tensor,
                                     bias: Tensor, epsilon):
    """``batch-normalize-update-and-apply!`` (``tensor.clj:1149-1202``)."""
    kind, vecs, input_shape = _batch_normalize_setup(
        [output, input], [batch_means, batch_variances, running_means, running_variances, scale, bias], epsilon)
    batch_means, batch_variances, running_means, running_variances, scale, bias = vecs
    stream = check_stream()
    bufs = (output.buffer, input.buffer, batch_means.buffer, batch_variances.buffer, running_means.buffer,
            running_variances.buffer, ave_factor, scale.buffer, bias.buffer, epsilon)
    if kind == "eltwise":
        stream.batch_normalize_update_and_apply_eltwise(*bufs, input_shape[0], input_shape[1])
    else:
        stream.batch_normalize_update_and_apply_spatial(*bufs, *_bn_counts(input_shape))
    return [output, batch_means, batch_variances, running_means, running_variances]


def batch_normalize_gradients(input_gradient: Tensor, scale_gradient: Tensor, bias_gradient: Tensor,
                              output_gradient: Tensor, output: Tensor, input: Tensor, batch_means: Tensor,
                              batch_variances: Tensor, scale: Tensor, bias: Tensor, epsilon):
    """``batch-normalize-gradients!`` (``tensor.clj:1205-1253``)."""
    kind, vecs, input_shape = _batch_normalize_setup(
        [output, input, output_gradient, input_gradient],
        [batch_means, batch_variances, scale, bias, scale_gradient, bias_gradient], epsilon)
    batch_means, batch_variances, scale, bias, scale_gradient, bias_gradient = vecs
    stream = check_stream()
    bufs = (input_gradient.buffer, scale_gradient.buffer, bias_gradient.buffer, output_gradient.buffer, output.buffer,
            input.buffer, batch_means.buffer, batch_variances.buffer, scale.buffer, bias.buffer, epsilon)
    if kind == "eltwise":
        stream.batch_normalize_gradients_eltwise(*bufs, input_shape[0], input_shape[1])
    else:
        stream.batch_normalize_gradients_spatial(*bufs, *_bn_counts(input_shape))
    return [input_gradient, scale_gradient, bias_gradient]


# ---------------------------------------------------------------- composites

def normalize(dest: Tensor, mag_vec: Tensor, radius_length, epsilon=1e-6) -> Tensor:
    """``normalize!`` (``tensor.clj:1618-1626``)."""
    unary_reduce(mag_vec, 1.0, dest, "magnitude")
    binary_op(mag_vec, 1.0, mag_vec, 1.0, 1e-6, "+")
    return binary_op(dest, 1.0, dest, 1.0 / float(radius_length), mag_vec, "/")


def constrain_inside_hypersphere(dest: Tensor, mag_vec: Tensor, radius_length) -> Tensor:
    """``constrain-inside-hypersphere!`` (``tensor.clj:1629-1644``)."""
    unary_reduce(mag_vec, 1.0, dest, "magnitude")
    binary_op(mag_vec, 1.0, mag_vec, 1.0, radius_length, "-")
    ternary_op(mag_vec, 1.0, mag_vec, 0.0, 0.0, 1.0, mag_vec, "select")
    binary_op(mag_vec, 1.0, mag_vec, 1.0, radius_length, "+")
    return binary_op(dest, 1.0, dest, 1.0 / float(radius_length), mag_vec, "/")
