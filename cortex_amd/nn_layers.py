"""Backend-neutral layers, loss gradients and regularisers that are written
purely against the tensor API: a Python mirror of
``src/cortex/compute/nn/layers.clj``, ``src/cortex/compute/nn/activations.clj``,
``src/cortex/compute/nn/backend.clj:98-139`` and the compute halves of
``src/cortex/loss/{mse,softmax,regularization}.clj``.

Every function here is a fixed sequence of ``assign!``, ``unary-op!``,
``binary-op!``, ``ternary-op!``, ``gemm!``, ``rand!``, ``softmax!``,
``activation-gradient!`` and ``batch-normalize-*!`` calls on the stream bound
by ``tensor_context``; nothing is computed on the host, so the same code runs
on any driver that implements the tensor-math calls.

A layer is described by a dict as in ``src/cortex/nn/layers.clj`` (``{"type":
"dropout", "distribution": "bernoulli", "probability": 0.8}``).  Where the
reference asks its graph for sizes, the description carries them itself:
``"input-size"`` (elements per batch item) and ``"input-dimension"``
(``{"channels", "height", "width"}``).  Buffers are passed as the reference
passes them: lists of ``{"buffer": Tensor, "gradient": Tensor}`` whose tensors
have the batch as their first dimension, and dicts of such entries for
parameters.
"""
from __future__ import annotations

import numpy as np

from . import operations as tops
from . import tensor as ct


def first_buffer(buffer_vec):
    return buffer_vec[0]["buffer"]


def first_gradient(buffer_vec):
    return buffer_vec[0]["gradient"]


def _simple_batch_tensor(t: ct.Tensor) -> ct.Tensor:
    """[batch, everything else]; a vector becomes one row (``layers.clj:41-47``)."""
    out = ct.as_batch_matrix(t)
    if len(out.shape()) < 2:
        return ct.in_place_reshape(out, [1, out.shape()[0]])
    return out


def _batch_tensor(t: ct.Tensor, batch_count: int, input_dimension: dict, spatial: bool) -> ct.Tensor:
    """[batch, channels, height*width] for spatial layers, else the simple batch
    matrix; shares the storage (``layers.clj:50-64``)."""
    if spatial:
        return ct.in_place_reshape(
            t, [batch_count, input_dimension["channels"], input_dimension["height"] * input_dimension["width"]])
    return _simple_batch_tensor(t)


def _batch_size(t: ct.Tensor) -> int:
    return t.shape()[0] if len(t.shape()) > 1 else 1


def _vector(t: ct.Tensor) -> ct.Tensor:
    """``math/->vector-ct``: the whole dense buffer as one vector."""
    v = ct.as_vector(t)
    if v is None:
        raise ct.TensorError("buffer must be dense")
    return v


def _input_size(node: dict) -> int:
    if "input-size" in node:
        return int(node["input-size"])
    d = node["input-dimension"]
    return int(d["channels"]) * int(d["height"]) * int(d["width"])


# ------------------------------------------------------------------ linear

def biased_multiply(input, weights, bias, output):
    """``biased-multiply!`` (``backend.clj:98-112``): every output row starts as
    the bias, then ``output += input * weights^T``."""
    input = ct.as_batch_matrix(input)
    output = ct.as_batch_matrix(output)
    ct.assign(output, bias)
    return ct.gemm(output, False, True, 1.0, input, weights, 1.0)


def biased_multiply_backward(input, weights, bias, output, input_gradient, weight_gradient, bias_gradient,
                             output_gradient):
    """``biased-multiply-backward!`` (``backend.clj:115-139``).  The bias and
    weight gradients accumulate; the input gradient is overwritten."""
    if bias_gradient is not None:
        ct.binary_op(bias_gradient, 1.0, output_gradient, 1.0, bias_gradient, "+")
    if input_gradient is not None:
        ct.gemm(ct.as_batch_matrix(input_gradient), False, False, 1.0, ct.as_batch_matrix(output_gradient), weights,
                0.0)
    if weight_gradient is not None:
        ct.gemm(weight_gradient, True, False, 1.0, ct.as_batch_matrix(output_gradient), ct.as_batch_matrix(input),
                1.0)


class Linear:
    """``Linear`` (``layers.clj:67-87``)."""

    def forward(self, parameter_buffers, input_buffers, output_buffers):
        biased_multiply(first_buffer(input_buffers), parameter_buffers["weights"]["buffer"],
                        parameter_buffers["bias"]["buffer"], first_buffer(output_buffers))

    def backward(self, parameter_buffers, output_buffers, input_buffers):
        biased_multiply_backward(first_buffer(input_buffers), parameter_buffers["weights"]["buffer"],
                                 parameter_buffers["bias"]["buffer"], first_buffer(output_buffers),
                                 first_gradient(input_buffers), parameter_buffers["weights"].get("gradient"),
                                 parameter_buffers["bias"].get("gradient"), first_gradient(output_buffers))


# ------------------------------------------------------------------ activations

SELU_ALPHA = 1.6732632423543772848170429916717   # activations.clj:23
SELU_LAMBDA = 1.0507009873554804934193349852946  # activations.clj:24


def logistic(input, output):
    return tops.logistic(output, input)


def tanh(input, output):
    return tops.tanh(output, input)


def relu(input, output):
    return tops.max_(output, input, 0)


def swish(input, output):
    """sigmoid(x)*x (``activations.clj:17-21``)."""
    return tops.mul(tops.logistic(output, input), input)


def selu(input, output):
    """lambda*x for x > 0, lambda*(alpha*exp(x) - alpha) otherwise
    (``activations.clj:26-37``)."""
    test = tops.gt(tops.new_tensor(input), input, 0)
    then = tops.mul(tops.new_tensor(input), input, SELU_LAMBDA)
    else_ = tops.mul(tops.sub(tops.mul(tops.exp(tops.new_tensor(input), input), SELU_ALPHA), SELU_ALPHA), SELU_LAMBDA)
    return tops.where(output, test, then, else_)


def default_gradient(input_gradient, output_gradient, output, act_type):
    """tanh, logistic and relu (``activations.clj:41-53``)."""
    return ct.activation_gradient(input_gradient, output_gradient, output, act_type)


def swish_gradient(input_gradient, output_gradient, output):
    """``(fx + sigm*(1 - fx)) * output-gradient`` with ``fx = sigm(v)*v`` taken,
    as in the reference, at the layer's output (``activations.clj:55-67``)."""
    fx = tops.mul(tops.logistic(tops.new_tensor(output), output), output)
    sigm = tops.logistic(tops.new_tensor(output), output)
    tops.sub(input_gradient, 1.0, fx)
    tops.mul(input_gradient, sigm)
    tops.add(input_gradient, fx)
    return tops.mul(input_gradient, output_gradient)


def selu_gradient(input_gradient, output_gradient, output):
    """lambda for v > 0, lambda*alpha*exp(v) otherwise, at the layer's output
    (``activations.clj:69-81``)."""
    test = tops.gt(tops.new_tensor(output), output, 0)
    then = tops.add(tops.new_tensor(output), SELU_LAMBDA)
    else_ = tops.mul(tops.mul(tops.exp(tops.new_tensor(output), output), SELU_ALPHA), SELU_LAMBDA)
    return tops.mul(tops.where(input_gradient, test, then, else_), output_gradient)


_FORWARD = {"logistic": logistic, "tanh": tanh, "relu": relu, "swish": swish, "selu": selu}
_GRADIENT = {"swish": swish_gradient, "selu": selu_gradient}


class ActivationLayer:
    """``ActivationLayer`` (``layers.clj:95-121``)."""

    def __init__(self, act_type: str, layer: dict = None):
        if act_type not in _FORWARD:
            raise ValueError(f"Unknown activation {act_type}")
        self.act_type, self.layer = act_type, layer

    def forward(self, parameter_buffers, input_buffers, output_buffers):
        output = _simple_batch_tensor(first_buffer(output_buffers))
        input = _simple_batch_tensor(first_buffer(input_buffers))
        _FORWARD[self.act_type](input, output)

    def backward(self, parameter_buffers, output_buffers, input_buffers):
        output = _simple_batch_tensor(first_buffer(output_buffers))
        input_gradient = _simple_batch_tensor(first_gradient(input_buffers))
        output_gradient = _simple_batch_tensor(first_gradient(output_buffers))
        if self.act_type in _GRADIENT:
            _GRADIENT[self.act_type](input_gradient, output_gradient, output)
        else:
            default_gradient(input_gradient, output_gradient, output, self.act_type)


# ------------------------------------------------------------------ softmax

class SoftmaxLayer:
    """``SoftmaxLayer`` (``layers.clj:147-173``).  The gradient is passed
    through: the softmax loss already differentiates through the softmax."""

    def __init__(self, layer: dict):
        self.layer = layer

    def _tensor(self, t: ct.Tensor) -> ct.Tensor:
        channels = int(self.layer.get("output-channels", 1))
        if channels > 1:
            return ct.in_place_reshape(t, [t.ecount() // channels, channels])
        dimension = self.layer.get("input-dimension", {"channels": 1})
        spatial = dimension.get("channels", 1) != 1
        return _batch_tensor(t, _batch_size(t), dimension, spatial)

    def forward(self, parameter_buffers, input_buffers, output_buffers):
        ct.softmax(self._tensor(first_buffer(output_buffers)), self._tensor(first_buffer(input_buffers)))

    def backward(self, parameter_buffers, output_buffers, input_buffers):
        ct.assign(self._tensor(first_gradient(input_buffers)), self._tensor(first_gradient(output_buffers)))


# ------------------------------------------------------------------ dropout

class Dropout:
    """``Dropout`` (``layers.clj:176-232``).  ``prepare_forward`` draws the
    multipliers once; forward and backward multiply by them, so a gradient
    check can call forward many times against one draw."""

    def __init__(self, layer: dict, batch_size: int, datatype: str = None):
        n_items = _input_size(layer)
        self.layer, self.batch_size = layer, batch_size
        self.mult_buffer = ct.new_tensor([batch_size, n_items], datatype=datatype)
        # the generator fills float buffers only
        self.rand_buffer = (self.mult_buffer if self.mult_buffer.get_datatype() == "float"
                            else ct.new_tensor([batch_size, n_items], datatype="float"))

    def prepare_forward(self, parameter_buffers=None, input_buffers=None, output_buffers=None):
        kind = self.layer["distribution"]
        if kind not in ("bernoulli", "gaussian"):
            raise ValueError(f"Unknown dropout distribution {kind}")
        if kind == "bernoulli":
            maximum = float(np.float32(self.layer["probability"]))
            distribution = ct.flat_distribution(minimum=maximum - 1.0, maximum=maximum)
        else:
            distribution = ct.gaussian_distribution(mean=1, variance=self.layer["variance"])
        ct.rand(self.rand_buffer, distribution)
        if self.mult_buffer is not self.rand_buffer:
            ct.assign(self.mult_buffer, self.rand_buffer)
        if kind == "bernoulli":
            # survivors are scaled so the expected signal keeps its magnitude
            ct.ternary_op(self.mult_buffer, 1.0, self.mult_buffer, 0.0, 0.0, 1.0,
                          1.0 / float(self.layer["probability"]), "select")

    def forward(self, parameter_buffers, input_buffers, output_buffers):
        input = _simple_batch_tensor(first_buffer(input_buffers))
        output = _simple_batch_tensor(first_buffer(output_buffers))
        ct.binary_op(output, 1.0, input, 1.0, self.mult_buffer, "*")

    def backward(self, parameter_buffers, output_buffers, input_buffers):
        input_gradient = _simple_batch_tensor(first_gradient(input_buffers))
        output_gradient = _simple_batch_tensor(first_gradient(output_buffers))
        ct.binary_op(input_gradient, 1.0, output_gradient, 1.0, self.mult_buffer, "*")


# ------------------------------------------------------------------ batch normalization

class BatchNormalization:
    """``BatchNormalization`` (``layers.clj:235-314``).  The first training
    batch sets the running statistics (average factor 1); later batches blend
    with the layer's ``average-factor``."""

    def __init__(self, layer: dict, datatype: str = None):
        self.layer = layer
        n = self._param_size()
        self.batch_means = ct.new_tensor([n], datatype=datatype)
        self.batch_variances = ct.new_tensor([n], datatype=datatype)
        self.local_average_factor = 1.0

    def _spatial(self) -> bool:
        return self.layer.get("mode", "elementwise") == "spatial"

    def _param_size(self) -> int:
        return int(self.layer["input-dimension"]["channels"]) if self._spatial() else _input_size(self.layer)

    def _tensor(self, t, input_buffers):
        return _batch_tensor(t, _batch_size(first_buffer(input_buffers)), self.layer.get("input-dimension"),
                             self._spatial())

    def forward(self, parameter_buffers, input_buffers, output_buffers):
        p = parameter_buffers
        ct.batch_normalize_update_and_apply(
            self._tensor(first_buffer(output_buffers), input_buffers),
            self._tensor(first_buffer(input_buffers), input_buffers),
            self.batch_means, self.batch_variances, p["means"]["buffer"], p["variances"]["buffer"],
            self.local_average_factor, p["scale"]["buffer"], p["bias"]["buffer"], self.layer["epsilon"])
        self.local_average_factor = self.layer["average-factor"]

    def backward(self, parameter_buffers, output_buffers, input_buffers):
        p = parameter_buffers
        ct.batch_normalize_gradients(
            self._tensor(first_gradient(input_buffers), input_buffers), p["scale"]["gradient"],
            p["bias"]["gradient"], self._tensor(first_gradient(output_buffers), input_buffers),
            self._tensor(first_buffer(output_buffers), input_buffers),
            self._tensor(first_buffer(input_buffers), input_buffers), self.batch_means, self.batch_variances,
            p["scale"]["buffer"], p["bias"]["buffer"], self.layer["epsilon"])

    def infer(self, parameter_buffers, input_buffers, output_buffers):
        p = parameter_buffers
        ct.batch_normalize(
            self._tensor(first_buffer(output_buffers), input_buffers),
            self._tensor(first_buffer(input_buffers), input_buffers), p["means"]["buffer"],
            p["variances"]["buffer"], p["scale"]["buffer"], p["bias"]["buffer"], self.layer["epsilon"])


# ------------------------------------------------------------------ prelu

def convolutional(kernel_dim: int, pad: int, stride: int, num_kernels: int, input_dimension: dict) -> dict:
    """The description of a convolutional layer as ``layers/convolutional``
    (``src/cortex/nn/layers.clj:394-408``) writes it and ``build-convolutional-type-node``
    (``:449-465``) completes it; the dimension operation is always ``:floor``
    (``:467-475``).  Weights are [num-kernels, kernel-width * kernel-height * channels]
    (``:410-413``), the bias [num-kernels]."""
    if stride < 1:
        raise ValueError("Convolutional layers must have stride >= 1")
    if kernel_dim < 1:
        raise ValueError("Convolutional layers must have kernel dimensions >= 1")
    node = {"type": "convolutional", "kernel-width": kernel_dim, "kernel-height": kernel_dim, "pad-x": pad,
            "pad-y": pad, "stride-x": stride, "stride-y": stride, "num-kernels": num_kernels, "dimension-op": "floor"}
    out = ct.get_convolution_output_dimensions(node, input_dimension["width"], input_dimension["height"])
    node["input-dimension"] = dict(input_dimension)
    node["output-dimension"] = {"channels": num_kernels, "height": out["output-height"], "width": out["output-width"]}
    return node


class ConvolutionLayer:
    """``ConvolutionLayer`` (``layers.clj:306-368``): the workspace for the
    unrolled input lives with the layer and carries the unrolled input from the
    forward pass to the weight gradient."""

    def __init__(self, layer: dict, batch_size: int, datatype: str = None):
        self.layer = layer
        datatype = datatype or ct.current_datatype()
        dimension = layer["input-dimension"]
        self.conv_desc = ct.convolution_descriptor(datatype, layer["num-kernels"], dimension["channels"],
                                                   layer["kernel-width"], layer["kernel-height"], layer["pad-x"],
                                                   layer["pad-y"], layer["stride-x"], layer["stride-y"])
        self.algorithms = ct.choose_convolution_algorithms(self.conv_desc, dimension["width"], dimension["height"],
                                                           batch_size, 100000)
        self.workspace = ct.new_tensor([self.algorithms["workspace-size"]], datatype)

    def forward(self, parameter_buffers, input_buffers, output_buffers):
        batch_size = _batch_size(first_buffer(input_buffers))
        output = _conv_tensor(self.layer["output-dimension"], batch_size, first_buffer(output_buffers))
        input = _conv_tensor(self.layer["input-dimension"], batch_size, first_buffer(input_buffers))
        weights = parameter_buffers["weights"]["buffer"]
        # set the bias up so that it broadcasts over the output
        bias = ct.in_place_reshape(parameter_buffers["bias"]["buffer"], [self.conv_desc["out-channels"], 1, 1])
        ct.convolution_forward(output, 0.0, input, weights, self.workspace, self.conv_desc, self.algorithms)
        ct.binary_op(output, 1.0, output, 1.0, bias, "+")

    def backward(self, parameter_buffers, output_buffers, input_buffers):
        batch_size = _batch_size(first_buffer(input_buffers))
        output_gradient = _conv_tensor(self.layer["output-dimension"], batch_size, first_gradient(output_buffers))
        input = _conv_tensor(self.layer["input-dimension"], batch_size, first_buffer(input_buffers))
        input_gradient = _conv_tensor(self.layer["input-dimension"], batch_size, first_gradient(input_buffers))
        weights = parameter_buffers["weights"]["buffer"]
        weight_gradient = parameter_buffers["weights"]["gradient"]
        out_chan = output_gradient.shape()[1]
        bias_gradient = ct.in_place_reshape(parameter_buffers["bias"]["gradient"], [out_chan, 1, 1])
        ct.binary_op(bias_gradient, 1.0, output_gradient, 1.0, bias_gradient, "+")
        ct.convolution_backward_weights(weight_gradient, 0.0, output_gradient, input, self.workspace, self.conv_desc,
                                        self.algorithms)
        ct.convolution_backward_data(input_gradient, 0.0, output_gradient, weights, self.workspace, self.conv_desc,
                                     self.algorithms)


def max_pooling(kernel_dim: int, pad: int, stride: int, input_dimension: dict, **args) -> dict:
    """The description of a pooling layer as ``layers/max-pooling``
    (``src/cortex/nn/layers.clj:492-511``) writes it and
    ``build-convolutional-type-node`` (``:449-465``) completes it: square kernel,
    padding and stride, ``:dimension-op :ceil`` and ``:pool-op :max`` unless
    given, output dimensions from the padded-strided formula (``:421-446``)."""
    if stride < 1:
        raise ValueError("Convolutional layers must have stride >= 1")
    if kernel_dim < 1:
        raise ValueError("Convolutional layers must have kernel dimensions >= 1")
    node = {"type": "max-pooling", "kernel-width": kernel_dim, "kernel-height": kernel_dim, "pad-x": pad,
            "pad-y": pad, "stride-x": stride, "stride-y": stride, "num-kernels": 0, "dimension-op": "ceil"}
    node.update({k.replace("_", "-"): v for k, v in args.items()})
    node.setdefault("pool-op", "max")
    if node["pool-op"] not in ct.POOL_OPERATIONS:
        raise ValueError(f"Max pooling layers have three possible pool operations: {ct.POOL_OPERATIONS}")
    out = ct.get_convolution_output_dimensions(node, input_dimension["width"], input_dimension["height"])
    node["input-dimension"] = dict(input_dimension)
    node["output-dimension"] = {"channels": input_dimension["channels"], "height": out["output-height"],
                                "width": out["output-width"]}
    return node


def _conv_tensor(dimension: dict, batch_size: int, t: ct.Tensor) -> ct.Tensor:
    """``->conv-tensor`` (``layers.clj:297-303``)."""
    return ct.in_place_reshape(t, [batch_size, dimension["channels"], dimension["height"], dimension["width"]])


class PoolingLayer:
    """``PoolingLayer`` (``layers.clj:390-428``)."""

    def __init__(self, layer: dict, batch_size: int, datatype: str = None):
        self.layer, self.batch_size = layer, batch_size
        self.pool_desc = ct.pooling_descriptor(datatype or ct.current_datatype(), layer["input-dimension"]["channels"],
                                               layer["kernel-width"], layer["kernel-height"], layer["pad-x"],
                                               layer["pad-y"], layer["stride-x"], layer["stride-y"],
                                               dimension_op=layer.get("dimension-op"),
                                               pool_op=layer.get("pool-op") or "max")

    def forward(self, parameter_buffers, input_buffers, output_buffers):
        output = _conv_tensor(self.layer["output-dimension"], self.batch_size, first_buffer(output_buffers))
        input = _conv_tensor(self.layer["input-dimension"], self.batch_size, first_buffer(input_buffers))
        ct.pooling_forward(output, 0.0, input, self.pool_desc)

    def backward(self, parameter_buffers, output_buffers, input_buffers):
        output = _conv_tensor(self.layer["output-dimension"], self.batch_size, first_buffer(output_buffers))
        output_gradient = _conv_tensor(self.layer["output-dimension"], self.batch_size,
                                       first_gradient(output_buffers))
        input = _conv_tensor(self.layer["input-dimension"], self.batch_size, first_buffer(input_buffers))
        input_gradient = _conv_tensor(self.layer["input-dimension"], self.batch_size, first_gradient(input_buffers))
        ct.pooling_backward(input_gradient, 0.0, input, output, output_gradient, self.pool_desc)


def local_response_normalization(input_dimension: dict, *, k=2, n=5, alpha=1e-4, beta=0.75, **args) -> dict:
    """The description ``layers/local-response-normalization``
    (``src/cortex/nn/layers.clj:586-594``) writes, with its defaults; the output
    has the input's dimensions."""
    node = {"type": "local-response-normalization", "k": k, "n": n, "alpha": alpha, "beta": beta}
    node.update({key.replace("_", "-"): v for key, v in args.items()})
    node["input-dimension"] = dict(input_dimension)
    node["output-dimension"] = dict(input_dimension)
    return node


class LocalResponseNormalization:
    """``LocalResponseNormalization`` (``layers.clj:363-388``)."""

    def __init__(self, layer: dict, batch_size: int):
        self.layer, self.batch_size = layer, batch_size
        self.lrn_desc = ct.lrn_descriptor(n=layer["n"], k=layer["k"], alpha=layer["alpha"], beta=layer["beta"])

    def forward(self, parameter_buffers, input_buffers, output_buffers):
        output = _conv_tensor(self.layer["output-dimension"], self.batch_size, first_buffer(output_buffers))
        input = _conv_tensor(self.layer["input-dimension"], self.batch_size, first_buffer(input_buffers))
        ct.lrn_forward(output, input, self.lrn_desc)

    def backward(self, parameter_buffers, output_buffers, input_buffers):
        output = _conv_tensor(self.layer["output-dimension"], self.batch_size, first_buffer(output_buffers))
        input = _conv_tensor(self.layer["input-dimension"], self.batch_size, first_buffer(input_buffers))
        output_gradient = _conv_tensor(self.layer["output-dimension"], self.batch_size, first_gradient(output_buffers))
        input_gradient = _conv_tensor(self.layer["output-dimension"], self.batch_size, first_gradient(input_buffers))
        ct.lrn_backward(input_gradient, output, input, output_gradient, self.lrn_desc)


def prelu_size(layer: dict) -> int:
    """One slope per channel, or per element when there is one channel
    (``src/cortex/nn/layers.clj:241-246``)."""
    d = layer["input-dimension"]
    if int(d["channels"]) == 1:
        return int(d["channels"]) * int(d["height"]) * int(d["width"])
    return int(d["channels"])


class Prelu:
    """``Prelu`` (``layers.clj:465-522``): ``scale = x >= 0 ? 1 : neg-scale``,
    ``output = x * scale``."""

    def __init__(self, layer: dict, batch_size: int, datatype: str = None):
        self.layer = layer
        self.scale_buffer = ct.new_tensor([batch_size, _input_size(layer)], datatype=datatype)

    def _views(self, input_buffers):
        n_channels = prelu_size(self.layer)
        spatial = n_channels != 1
        batch = _batch_size(first_buffer(input_buffers))

        def batch_tensor(t):
            return _batch_tensor(t, batch, self.layer["input-dimension"], spatial)

        def parameter(t):
            # [channels, 1] broadcasts over [batch, channels, pixels]
            return ct.in_place_reshape(t, [n_channels, 1]) if spatial else t
        return batch_tensor, parameter

    def forward(self, parameter_buffers, input_buffers, output_buffers):
        batch_tensor, parameter = self._views(input_buffers)
        input = batch_tensor(first_buffer(input_buffers))
        output = batch_tensor(first_buffer(output_buffers))
        neg_scale = parameter(parameter_buffers["neg-scale"]["buffer"])
        scale_buffer = batch_tensor(self.scale_buffer)
        ct.ternary_op(scale_buffer, 1.0, input, 1.0, neg_scale, 1.0, 1.0, "select")
        ct.binary_op(output, 1.0, input, 1.0, scale_buffer, "*")

    def backward(self, parameter_buffers, output_buffers, input_buffers):
        batch_tensor, parameter = self._views(input_buffers)
        input_gradient = batch_tensor(first_gradient(input_buffers))
        input = batch_tensor(first_buffer(input_buffers))
        output_gradient = batch_tensor(first_gradient(output_buffers))
        neg_scale_gradient = parameter(parameter_buffers["neg-scale"]["gradient"])
        scale_buffer = batch_tensor(self.scale_buffer)
        # the input gradient doubles as the temporary; it is overwritten below
        ct.binary_op(input_gradient, 1.0, output_gradient, 1, input, "*")
        ct.binary_op(neg_scale_gradient, 1.0, neg_scale_gradient, 1.0, input_gradient, "+")
        ct.binary_op(input_gradient, 1.0, output_gradient, 1.0, scale_buffer, "*")


# ------------------------------------------------------------------ concatenate / split / join

def _do_concat(input_buffers, output_buffers, buffer_key: str) -> int:
    """Copies column blocks into (``"buffer"``) or out of (``"gradient"``) the
    output (``layers.clj:535-560``)."""
    output = _simple_batch_tensor(output_buffers[0][buffer_key])
    num_batches, num_output = output.shape()
    offset = 0
    for entry in input_buffers:
        input_buffer = _simple_batch_tensor(entry[buffer_key])
        _, in_num_cols = input_buffer.shape()
        target_output = ct.submatrix(output, 0, num_batches, offset, in_num_cols)
        if buffer_key == "buffer":
            ct.assign(target_output, input_buffer)
        else:
            ct.assign(input_buffer, target_output)
        offset += in_num_cols
    return offset


class Concatenate:
    """``Concatenate`` (``layers.clj:563-568``)."""

    def forward(self, parameter_buffers, input_buffers, output_buffers):
        return _do_concat(input_buffers, output_buffers, "buffer")

    def backward(self, parameter_buffers, output_buffers, input_buffers):
        return _do_concat(input_buffers, output_buffers, "gradient")


class Split:
    """``Split`` (``layers.clj:575-595``): every output is a copy of the input;
    the input gradient is the sum of the output gradients."""

    def forward(self, parameter_buffers, input_buffers, output_buffers):
        input_tensor = _simple_batch_tensor(first_buffer(input_buffers))
        for entry in output_buffers:
            ct.assign(_simple_batch_tensor(entry["buffer"]), input_tensor)

    def backward(self, parameter_buffers, output_buffers, input_buffers):
        input_gradient = _simple_batch_tensor(first_gradient(input_buffers))
        ct.assign(input_gradient, 0)
        for entry in output_buffers:
            ct.binary_op(input_gradient, 1.0, input_gradient, 1.0, _simple_batch_tensor(entry["gradient"]), "+")


class Join:
    """``Join`` (``layers.clj:603-660``): sums inputs of possibly different
    widths into the widest, or multiplies their common leading columns."""

    def __init__(self, layer: dict = None):
        self.layer = layer or {}

    def forward(self, parameter_buffers, input_buffers, output_buffers):
        output = _simple_batch_tensor(first_buffer(output_buffers))
        inputs = [_simple_batch_tensor(e["buffer"]) for e in input_buffers]
        operation = self.layer.get("operation", "+")
        min_num_columns = min(t.shape()[1] for t in inputs)
        ct.assign(output, 0)
        for idx, input in enumerate(inputs):
            num_rows, num_columns = input.shape()
            if operation != "+":
                num_columns = min_num_columns
            out = ct.submatrix(output, 0, num_rows, 0, num_columns)
            inp = ct.submatrix(input, 0, num_rows, 0, num_columns)
            if operation == "+":
                ct.binary_op(out, 1.0, out, 1.0, inp, "+")
            elif operation == "*":
                if idx == 0:
                    ct.assign(out, inp)
                else:
                    ct.binary_op(out, 1.0, out, 1.0, inp, "*")
            else:
                raise ValueError(f"Unknown join operation {operation}")

    def backward(self, parameter_buffers, output_buffers, input_buffers):
        output_gradient = _simple_batch_tensor(first_gradient(output_buffers))
        input_gradients = [_simple_batch_tensor(e["gradient"]) for e in input_buffers]
        inputs = [_simple_batch_tensor(e["buffer"]) for e in input_buffers]
        operation = self.layer.get("operation", "+")
        min_num_columns = min(t.shape()[1] for t in inputs)
        for idx, input_gradient in enumerate(input_gradients):
            num_rows, num_columns = input_gradient.shape()
            if operation != "+":
                num_columns = min_num_columns
            og = ct.submatrix(output_gradient, 0, num_rows, 0, num_columns)
            ig = ct.submatrix(input_gradient, 0, num_rows, 0, num_columns)
            ct.assign(ig, og)
            if operation == "*":
                for other_idx in range(len(inputs)):
                    if other_idx != idx:
                        other = ct.submatrix(inputs[other_idx], 0, num_rows, 0, num_columns)
                        ct.binary_op(ig, 1, ig, 1, other, "*")


# ------------------------------------------------------------------ create

def create(node: dict, batch_size: int, datatype: str = None):
    """``create`` (``layers.clj:35-39`` and its methods): the compute layer of a
    layer description."""
    kind = node["type"]
    if kind == "linear":
        return Linear()
    if kind in _FORWARD:
        return ActivationLayer(kind, node)
    if kind == "softmax":
        return SoftmaxLayer(node)
    if kind == "dropout":
        return Dropout(node, batch_size, datatype)
    if kind == "batch-normalization":
        return BatchNormalization(node, datatype)
    if kind == "prelu":
        return Prelu(node, batch_size, datatype)
    if kind == "max-pooling":
        return PoolingLayer(node, batch_size, datatype)
    if kind == "convolutional":
        return ConvolutionLayer(node, batch_size, datatype)
    if kind == "local-response-normalization":
        return LocalResponseNormalization(node, batch_size)
    if kind == "concatenate":
        return Concatenate()
    if kind == "split":
        return Split()
    if kind == "join":
        return Join(node)
    raise ValueError(f"No tensor-math implementation for layer type {kind}")


# ------------------------------------------------------------------ loss gradients

def mse_loss_gradient(buffer_map: dict):
    """``MSELoss compute-loss-gradient`` (``loss/mse.clj:12-21``):
    ``gradient = (2/output-size) * (v - target)``."""
    v = ct.as_batch_matrix(buffer_map["output"]["buffer"])
    gradient = ct.as_batch_matrix(buffer_map["output"]["gradient"])
    target = ct.as_batch_matrix(buffer_map["labels"]["buffer"])
    _, output_size = v.shape()
    alpha = 2.0 / float(output_size)
    return ct.binary_op(gradient, alpha, v, alpha, target, "-")


def softmax_loss_gradient(buffer_map: dict):
    """``SoftmaxLoss compute-loss-gradient`` (``loss/softmax.clj:13-29``):
    ``gradient = v - target``."""
    v = ct.as_batch_matrix(buffer_map["output"]["buffer"])
    gradient = ct.as_batch_matrix(buffer_map["output"]["gradient"])
    target = ct.as_batch_matrix(buffer_map["labels"]["buffer"])
    return ct.binary_op(gradient, 1.0, v, 1.0, target, "-")


class L1RegularizationLoss:
    """``L1RegularizationLoss`` (``loss/regularization.clj:16-46``):
    ``gradient += sign(param)`` with ``sign(0) = 1``."""

    def __init__(self, term_size: int, datatype: str = None):
        self.l1_buffer = ct.new_tensor([term_size], datatype=datatype)

    def compute_loss_gradient(self, buffer_map: dict):
        param_buf = _vector(buffer_map["output"]["buffer"])
        gradient = _vector(buffer_map["output"]["gradient"])
        ct.ternary_op(self.l1_buffer, 1.0, param_buf, 1.0, -1, 1.0, 1, "select")
        return ct.binary_op(gradient, 1.0, gradient, 1.0, self.l1_buffer, "+")


class L2RegularizationLoss:
    """``L2RegularizationLoss`` (``loss/regularization.clj:49-56``):
    ``gradient += param``."""

    def compute_loss_gradient(self, buffer_map: dict):
        target = _vector(buffer_map["output"]["buffer"])
        gradient = _vector(buffer_map["output"]["gradient"])
        return ct.binary_op(gradient, 1.0, target, 1.0, gradient, "+")
