"""Gradient optimizers of the tensor-math path: a Python mirror of
``src/cortex/optimize.clj:5-24``, ``src/cortex/optimize/adam.clj:116-200``,
``src/cortex/optimize/adadelta.clj:19-132`` and ``src/cortex/optimize/sgd.clj``.

An optimizer object implements ``PGradientOptimizer``: ``batch_update`` is
called once per batch, ``compute_parameters`` once per parameter buffer with
the running ``offset`` of that buffer inside the flat optimizer state
(``src/cortex/nn/compute_binding.clj:817-854``).  The Adam and Adadelta steps
are one fused kernel each on the backend's stream; SGD is, as in the reference,
four calls of the tensor API.
"""
from __future__ import annotations

import dataclasses


def adam(**kwargs) -> dict:
    """Default Adam description (``adam.clj:191-200``)."""
    out = {"type": "adam", "alpha": 0.001, "beta1": 0.9, "beta2": 0.999, "epsilon": 1e-8}
    out.update(kwargs)
    return out


def adadelta(**kwargs) -> dict:
    """Default Adadelta description (``adadelta.clj:124-132``)."""
    out = {"type": "adadelta", "decay": 0.05, "epsilon": 1e-6}
    out.update(kwargs)
    return out


def sgd(**kwargs) -> dict:
    """Default SGD description (``sgd.clj:74-80``)."""
    out = {"type": "sgd", "learning-rate": 0.001, "momentum": 0.9}
    out.update(kwargs)
    return out


@dataclasses.dataclass
class Backend:
    """What the optimizers need of a compute backend: its stream and datatype
    (``src/cortex/compute/cuda/backend.clj:33-72``)."""
    stream: object
    datatype: str = "float"
    type: str = "hip"


def _buffer(x):
    return x.buffer if hasattr(x, "buffer") else x


def _ensure_datatype(datatype, *buffers) -> None:
    actual = [b.get_datatype() for b in buffers]
    if any(a != datatype for a in actual):
        raise TypeError(f"Buffer datatype mismatch: expected {datatype}, got {actual}")


@dataclasses.dataclass
class Adam:
    backend: Backend
    optimizer: dict
    pow_beta1_t: float = 1.0
    pow_beta2_t: float = 1.0

    def batch_update(self, optimizer_parameters=None) -> "Adam":
        """``batch-update`` (``adam.clj:149-153``): beta^t by repeated multiplication."""
        return dataclasses.replace(self, pow_beta1_t=self.pow_beta1_t * float(self.optimizer["beta1"]),
                                   pow_beta2_t=self.pow_beta2_t * float(self.optimizer["beta2"]))

    def compute_parameters(self, state: dict, gradient_alpha, offset: int, gradient, parameters) -> None:
        """``compute-parameters!`` (``adam.clj:154-158`` -> ``adam-optimise-step!`` :116-134)."""
        g, p, m, v = _buffer(gradient), _buffer(parameters), _buffer(state["m"]), _buffer(state["v"])
        _ensure_datatype(self.backend.datatype, g, p, m, v)
        n = g.ecount()
        o = self.optimizer
        self.backend.stream.adam_step(o["alpha"], o["beta1"], o["beta2"], o["epsilon"], self.pow_beta1_t,
                                      self.pow_beta2_t, gradient_alpha, g, p,
                                      m.sub_buffer(offset, m.ecount() - offset),
                                      v.sub_buffer(offset, v.ecount() - offset), n)


@dataclasses.dataclass
class Adadelta:
    backend: Backend
    optimizer: dict

    def batch_update(self, optimizer_parameters=None) -> "Adadelta":
        return self

    def compute_parameters(self, state: dict, gradient_alpha, offset: int, gradient, parameters) -> None:
        """``compute-parameters!`` (``adadelta.clj:19-26``)."""
        g, p = _buffer(gradient), _buffer(parameters)
        ga, da = _buffer(state["grad-accum"]), _buffer(state["dx-accum"])
        _ensure_datatype(self.backend.datatype, g, p, ga, da)
        o = self.optimizer
        self.backend.stream.adadelta_step(o["decay"], o["epsilon"], ga.sub_buffer(offset, ga.ecount() - offset),
                                          da.sub_buffer(offset, da.ecount() - offset), gradient_alpha, g, p, g.ecount())


@dataclasses.dataclass
class SGD:
    backend: Backend
    optimizer: dict
    _temp: object = None   # the allocator's reusable :sgd-temp tensor (sgd.clj:27)

    def batch_update(self, optimizer_parameters=None) -> "SGD":
        return self

    def compute_parameters(self, state: dict, gradient_alpha, offset: int, gradient, parameters) -> None:
        """``tensor-sgd`` (``sgd.clj:16-40``): momentum with the look-ahead correction,
            dxm = momentum * v;  v = dxm + learning-rate * gradient-alpha * g;
            dx = dxm - (1 + momentum) * v;  p = p + dx
        as one ``unary-op!`` and three ``binary-op!`` calls."""
        from . import tensor as ct
        from . import dimensions as dims

        g, p, mv = _buffer(gradient), _buffer(parameters), _buffer(state["momentum-vals"])
        _ensure_datatype(self.backend.datatype, g, p, mv)
        n = g.ecount()
        device = self.backend.stream.get_device()
        vec = lambda buf, count: ct.Tensor(device, dims.dimensions([count]), buf)
        momentum = float(self.optimizer["momentum"])
        with ct.tensor_context(self.backend.stream, self.backend.datatype):
            grad, params = vec(g, n), vec(p, p.ecount())
            momentum_vals = vec(mv.sub_buffer(offset, n), n)
            if self._temp is None or self._temp.ecount() < n:
                self._temp = ct.new_tensor([n], init_value=None)
            temp = vec(self._temp.buffer.sub_buffer(0, n), n)
            dxm = ct.unary_op(temp, momentum, momentum_vals, "noop")
            ct.binary_op(momentum_vals, 1.0, dxm, float(self.optimizer["learning-rate"]) * float(gradient_alpha), grad, "+")
            dx = ct.binary_op(temp, 1.0, dxm, 1 + momentum, momentum_vals, "-")
            ct.binary_op(params, 1.0, params, 1.0, dx, "+")


def create_optimizer(backend: Backend, optimizer: dict):
    """``create-optimizer`` multimethod on ``[(:type backend) (:type optimizer)]``
    (``optimize.clj:19-24``)."""
    if backend.datatype not in ("float", "double"):
        raise TypeError("optimizers support float and double only")
    kind = optimizer["type"]
    if kind == "adam":
        return Adam(backend, optimizer)
    if kind == "adadelta":
        return Adadelta(backend, optimizer)
    if kind == "sgd":
        return SGD(backend, optimizer)
    raise KeyError(f"No optimizer {kind!r} for backend {backend.type!r}")
