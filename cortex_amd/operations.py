"""Tensor operations with short names: a Python mirror of
``src/cortex/tensor/operations.clj``.  Every function mutates and returns its
first argument; with two arguments the output is also the first operand
(``operations.clj:8-127``).  The names that shadow Python built-ins carry a
trailing underscore.
"""
from __future__ import annotations

from . import tensor as ct


def _binary(op):
    def apply(output, x1, x2=None):
        if x2 is None:
            output, x1, x2 = output, output, x1
        return ct.binary_op(output, 1.0, x1, 1.0, x2, op)
    apply.__doc__ = f"output = x1 {op} x2; with two arguments output = output {op} x1."
    return apply


def _unary(op):
    def apply(output, input=None):
        return ct.unary_op(output, 1.0, output if input is None else input, op)
    apply.__doc__ = f"output = {op}(input); with one argument in place."
    return apply


max_ = _binary("max")          # operations.clj:8-13
min_ = _binary("min")          # operations.clj:15-20
ceil = _unary("ceil")          # operations.clj:22-27
floor = _unary("floor")        # operations.clj:29-34
logistic = _unary("logistic")  # operations.clj:36-41
tanh = _unary("tanh")          # operations.clj:43-48
exp = _unary("exp")            # operations.clj:50-55
mul = _binary("*")             # operations.clj:57-62
sub = _binary("-")             # operations.clj:64-69
add = _binary("+")             # operations.clj:71-76
gt = _binary(">")              # operations.clj:78-83
ge = _binary(">=")             # operations.clj:85-90
lt = _binary("<")              # operations.clj:92-97
le = _binary("<=")             # operations.clj:99-104
bit_xor = _binary("bit-xor")   # operations.clj:106-111
bit_and = _binary("bit-and")   # operations.clj:113-118


def new_tensor(output: ct.Tensor) -> ct.Tensor:
    """A zeroed tensor of the shape and datatype of ``output``
    (``operations.clj:120-123``)."""
    return ct.new_tensor(output.shape(), datatype=output.get_datatype())


def where(output, test, then, else_):
    """``output = then*test + else*(test xor 1)`` for a test tensor of ones and
    zeros; ``then`` and ``else_`` are overwritten with their masked values
    (``operations.clj:125-137``)."""
    compl = bit_xor(new_tensor(test), test, 1)
    x1 = mul(then, test)
    x2 = mul(else_, compl)
    return add(output, x1, x2)
