"""ctypes binding of ``libcortex_hip.so`` (see ``include/cortex_hip.h``).

This is the lowest Python layer: one Python callable per C entry point, a
``ct_dims`` structure, and error translation.  A failing call raises
:class:`CortexHipError` carrying ``ct_last_error()``, as the reference turns
every failed native call into an exception
(``src/cortex/compute/cuda/driver.clj:40-49``).

The library must have been built (``python -m cortex_amd.build``); there is no
fallback implementation: if the shared object is missing, importing this module
raises.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path
from typing import Optional, Sequence

MAX_DIMS = 8

# Datatype codes (include/cortex_hip.h: ct_dtype).  The first six are the
# reference's datatypes in its order (src/cortex/compute/cuda/driver.clj:354-367).
I8, I16, I32, I64, F32, F64, U8 = range(7)
DTYPE_CODES = {"byte": I8, "short": I16, "int": I32, "long": I64, "float": F32, "double": F64, "ubyte": U8}
DTYPE_SIZES = {I8: 1, I16: 2, I32: 4, I64: 8, F32: 4, F64: 8, U8: 1}

# Operation codes (resources/operations.h:27-45, 88-102; tensor_unary_reduce.cu:9-20).
UNARY_OPS = {"floor": 0, "ceil": 1, "round": 2, "-": 3, "tanh": 4, "logistic": 5, "exp": 6, "sqrt": 7, "noop": 8}
BINARY_OPS = {"+": 0, "-": 1, "*": 2, "/": 3, "min": 4, "max": 5, "bit-and": 6, "bit-xor": 7, "eq": 8,
              ">": 9, ">=": 10, "<": 11, "<=": 12}
TERNARY_OPS = {"select": 0}
ACTIVATION_OPS = {"logistic": 0, "tanh": 1, "relu": 2}
DISTRIBUTIONS = {"gaussian": 0, "flat": 1}
POOL_OPS = {"max": 0, "avg": 1, "avg-exc-pad": 2}
REDUCE_OPS = {"max": 0, "min": 1, "sum": 2, "mean": 3, "magnitude": 4, "magnitude-squared": 5}

COPY_H2D, COPY_D2H, COPY_D2D = 0, 1, 2


class CtDims(C.Structure):
    """``ct_dims``: shape and strides in elements, slowest dimension first."""

    _fields_ = [
        ("ndim", C.c_int32),
        ("shape", C.c_int64 * MAX_DIMS),
        ("strides", C.c_int64 * MAX_DIMS),
        ("index", C.c_void_p * MAX_DIMS),
    ]


class CtPoolDesc(C.Structure):
    """``ct_pool_desc``: the geometry of a pooling descriptor."""

    _fields_ = [
        ("kernel_width", C.c_int32), ("kernel_height", C.c_int32),
        ("pad_x", C.c_int32), ("pad_y", C.c_int32),
        ("stride_x", C.c_int32), ("stride_y", C.c_int32),
        ("pool_op", C.c_int32),
    ]


class CtConvDesc(C.Structure):
    """``ct_conv_desc``: the geometry of a convolution descriptor."""

    _fields_ = [
        ("in_channels", C.c_int32), ("out_channels", C.c_int32),
        ("kernel_width", C.c_int32), ("kernel_height", C.c_int32),
        ("pad_x", C.c_int32), ("pad_y", C.c_int32),
        ("stride_x", C.c_int32), ("stride_y", C.c_int32),
    ]


def make_conv_desc(descriptor) -> CtConvDesc:
    """Builds a ``ct_conv_desc`` from a convolution descriptor map."""
    return CtConvDesc(int(descriptor["in-channels"]), int(descriptor["out-channels"]), int(descriptor["kernel-width"]),
                      int(descriptor["kernel-height"]), int(descriptor["pad-x"]), int(descriptor["pad-y"]),
                      int(descriptor["stride-x"]), int(descriptor["stride-y"]))


def make_pool_desc(descriptor) -> CtPoolDesc:
    """Builds a ``ct_pool_desc`` from a pooling descriptor map."""
    return CtPoolDesc(int(descriptor["kernel-width"]), int(descriptor["kernel-height"]), int(descriptor["pad-x"]),
                      int(descriptor["pad-y"]), int(descriptor["stride-x"]), int(descriptor["stride-y"]),
                      POOL_OPS[descriptor["pool-op"]])


def make_dims(shape: Sequence[int], strides: Sequence[int], index: Optional[Sequence[Optional[int]]] = None) -> CtDims:
    """Builds a ``ct_dims``.  ``index[d]`` is a device address of an int32
    index array for an indirectly addressed dimension, or None."""
    if len(shape) != len(strides):
        raise ValueError("shape and strides differ in length")
    if not 1 <= len(shape) <= MAX_DIMS:
        raise ValueError(f"rank {len(shape)} outside 1..{MAX_DIMS}")
    d = CtDims()
    d.ndim = len(shape)
    for i, (s, st) in enumerate(zip(shape, strides)):
        d.shape[i] = int(s)
        d.strides[i] = int(st)
        d.index[i] = None if index is None or index[i] is None else int(index[i])
    return d


class CortexHipError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"[ct_status {status}] {message}")
        self.status = status
        self.message = message


LIB_PATH = Path(__file__).resolve().parent / "libcortex_hip.so"

_P, _D, _I, _L = C.c_void_p, C.c_double, C.c_int, C.c_int64
_DP = C.POINTER(CtDims)

# name -> argument types, exactly the prototypes of include/cortex_hip.h
PROTOTYPES = {
    "ct_set_debug_sync": [_I],
    "ct_device_count": [C.POINTER(C.c_int)],
    "ct_set_device": [_I],
    "ct_get_device": [C.POINTER(C.c_int)],
    "ct_memory_info": [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)],
    "ct_malloc": [C.POINTER(_P), C.c_size_t],
    "ct_free": [_P],
    "ct_host_alloc": [C.POINTER(_P), C.c_size_t],
    "ct_host_free": [_P],
    "ct_stream_create": [C.POINTER(_P)],
    "ct_stream_destroy": [_P],
    "ct_stream_reserve_scratch": [_P, C.c_size_t, C.c_size_t],
    "ct_check_index_range": [_P, _P, _L, _L],
    "ct_stream_sync": [_P],
    "ct_event_record": [C.POINTER(_P), _P],
    "ct_event_record_timed": [C.POINTER(_P), _P],
    "ct_stream_wait_event": [_P, _P],
    "ct_event_sync": [_P],
    "ct_event_destroy": [_P],
    "ct_event_elapsed_ms": [_P, _P, C.POINTER(C.c_float)],
    "ct_memcpy_async": [_P, _P, C.c_size_t, _I, _P],
    "ct_memset": [_P, _P, _I, _D, _L],
    "ct_assign_constant": [_P, _P, _DP, _I, _D, _L],
    "ct_assign": [_P, _P, _DP, _I, _P, _DP, _I, _L],
    "ct_unary_accum": [_P, _P, _DP, _D, _I, _I, _L],
    "ct_unary_op": [_P, _P, _DP, _P, _DP, _D, _I, _I, _L],
    "ct_binary_accum_constant": [_P, _P, _DP, _D, _D, _L, _I, _I, _I],
    "ct_binary_op_constant": [_P, _P, _DP, _P, _DP, _D, _D, _L, _I, _I, _I],
    "ct_binary_accum": [_P, _P, _DP, _D, _P, _DP, _D, _L, _I, _I, _I, _I],
    "ct_binary_op": [_P, _P, _DP, _P, _DP, _D, _P, _DP, _D, _L, _I, _I],
    "ct_ternary_op": [_P, _P, _DP, _P, _DP, _D, _P, _DP, _D, _P, _DP, _D, _L, _I, _I],
    "ct_ternary_op_constant": [_P, _P, _DP, _P, _DP, _D, _P, _DP, _D, _D, _L, _I, C.POINTER(C.c_int8), _I],
    "ct_ternary_op_constant_constant": [_P, _P, _DP, _P, _DP, _D, _D, _D, _L, _I, C.POINTER(C.c_int8), _I],
    "ct_unary_reduce": [_P, _P, _DP, _D, _P, _DP, _I, _I],
    "ct_unary_reduce_noalloc": [_P, _P, _DP, _D, _P, _DP, _I, _I],
    "ct_activation_gradient": [_P, _P, _DP, _P, _DP, _P, _DP, _I, _L, _I],
    "ct_softmax_eltwise": [_P, _P, _DP, _P, _DP, _I],
    "ct_softmax_spatial": [_P, _P, _DP, _P, _DP, _I],
    "ct_batch_normalize_eltwise": [_P, _P, _P, _P, _P, _P, _P, _D, _L, _L, _I],
    "ct_batch_normalize_spatial": [_P, _P, _P, _P, _P, _P, _P, _D, _L, _L, _L, _I],
    "ct_batch_normalize_update_and_apply_eltwise": [_P, _P, _P, _P, _P, _P, _P, _D, _P, _P, _D, _L, _L, _I],
    "ct_batch_normalize_update_and_apply_spatial": [_P, _P, _P, _P, _P, _P, _P, _D, _P, _P, _D, _L, _L, _L, _I],
    "ct_batch_normalize_gradients_eltwise": [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _D, _L, _L, _I],
    "ct_batch_normalize_gradients_spatial": [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _D, _L, _L, _L, _I],
    "ct_convolution_forward": [_P, _P, _D, _P, _P, _P, _L, C.POINTER(CtConvDesc), _L, _L, _L, _L, _L, _I],
    "ct_convolution_backward_weights": [_P, _P, _D, _P, _P, _P, _L, C.POINTER(CtConvDesc), _L, _L, _L, _L, _L, _I],
    "ct_convolution_backward_data": [_P, _P, _D, _P, _P, _P, _L, C.POINTER(CtConvDesc), _L, _L, _L, _L, _L, _I],
    "ct_pooling_forward": [_P, _P, _D, _P, C.POINTER(CtPoolDesc), _L, _L, _L, _L, _L, _L, _I],
    "ct_pooling_backward": [_P, _P, _D, _P, _P, _P, C.POINTER(CtPoolDesc), _L, _L, _L, _L, _L, _L, _I],
    "ct_lrn_forward": [_P, _P, _DP, _P, _DP, _I, _D, _D, _D, _I],
    "ct_lrn_backward": [_P, _P, _DP, _P, _DP, _P, _DP, _P, _DP, _I, _D, _D, _D, _I],
    "ct_gemm": [_P, _P, _L, _I, _I, _D, _P, _L, _L, _L, _P, _L, _L, _D, _I],
    "ct_gemv": [_P, _P, _L, _I, _D, _P, _L, _L, _L, _P, _L, _D, _I],
    "ct_rand": [_P, _P, _L, _I, _I, _D, _D, C.c_uint64, C.c_uint64],
    "ct_dropout_bernoulli_mask": [_P, _P, _I, _P, _L, _D, C.c_uint64, C.c_uint64],
    "ct_adam_step": [_P, _I, _D, _D, _D, _D, _D, _D, _D, _P, _P, _P, _P, _L],
    "ct_adadelta_step": [_P, _I, _D, _D, _P, _P, _D, _P, _P, _L],
}
STRING_FUNCTIONS = ("ct_last_error", "ct_last_kernel")


def load_library(path: Optional[Path] = None) -> C.CDLL:
    path = Path(path) if path else LIB_PATH
    if not path.exists():
        raise ImportError(
            f"{path} is missing: build it with `python -m cortex_amd.build` (hipcc, gfx950). "
            "There is no CPU fallback for the HIP backend."
        )
    lib = C.CDLL(str(path))
    for name, argtypes in PROTOTYPES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = C.c_int
    for name in STRING_FUNCTIONS:
        fn = getattr(lib, name)
        fn.argtypes = []
        fn.restype = C.c_char_p
    return lib


_lib: Optional[C.CDLL] = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        _lib = load_library()
    return _lib


def check(status: int) -> None:
    if status != 0:
        raise CortexHipError(status, lib().ct_last_error().decode("utf-8", "replace"))


def call(name: str, *args) -> None:
    """Calls entry point ``name`` and raises on a non-zero status."""
    check(getattr(lib(), name)(*args))


def last_kernel() -> str:
    return lib().ct_last_kernel().decode()


def arg_idx(values: Sequence[int]):
    return (C.c_int8 * 3)(*values)
