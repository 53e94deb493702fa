"""ct_unary_reduce_noalloc: the reduction entry point that allocates nothing.

Its partial accumulators live in a fixed array in device memory, shared by all
calls on a device and holding whatever the previous call left there.  Every
case below therefore runs two calls in a row through the C ABI, the second on
a smaller input, and compares each output with ct_unary_reduce's on the same
input: both run the same kernels with the same plan, so the bar is bit-exact
for every datatype.  The oracle is checked as well (max / min and integers
bit-exact, float sums to 2e-6 of the sum of magnitudes, 1e-12 for doubles).
"""
import ctypes as C

import numpy as np
import pytest

import harness as H
from cortex_amd import capi

pytestmark = pytest.mark.gpu


def _reduce(entry, side, out: H.View, alpha, inp: H.View, op):
    capi.call(entry, side.stream, side.ptr(out), C.byref(side.dims(out)), float(alpha), side.ptr(inp),
              C.byref(side.dims(inp)), capi.REDUCE_OPS[op], out.buf.dtype)
    capi.call("ct_stream_sync", side.stream)


def _check(pair, data: np.ndarray, shape, strides, op, alpha=1.0):
    """Reduces the last axis of the view (shape, strides) of `data` through both entry points."""
    n_out = int(np.prod(shape[:-1]))
    src = pair.buf(data)
    want = pair.buf(np.zeros(n_out, data.dtype))
    got = pair.buf(np.full(n_out, 77, data.dtype))
    view = H.View(src, shape, strides)
    out_shape = list(shape[:-1]) + [1]
    H.unary_reduce(H.ORACLE, H.View(want, out_shape), alpha, view, op)
    _reduce("ct_unary_reduce", pair.hip, H.View(want, out_shape), alpha, view, op)
    kernel = capi.last_kernel()
    _reduce("ct_unary_reduce_noalloc", pair.hip, H.View(got, out_shape), alpha, view, op)
    assert capi.last_kernel() == kernel
    what = f"{op} {data.dtype} view {shape} strides {strides} ({kernel})"
    H.assert_bit_exact(got.download(), want.download(), "noalloc vs ct_unary_reduce: " + what)
    oracle = want.host
    if data.dtype.kind != "f" or op in ("max", "min"):
        H.assert_bit_exact(got.download(), oracle, "noalloc vs oracle: " + what)
    else:
        k = shape[-1]
        scale = np.abs(view.gather_host(src.init).astype(np.float64) * alpha)
        scale = (scale ** 2 if op.startswith("magnitude") else scale).reshape(n_out, k).sum(axis=1)
        if op == "magnitude":
            scale = np.sqrt(scale)
        if op == "mean":
            scale = scale / k
        tol = 2e-6 if data.dtype == np.float32 else 1e-12
        err = np.abs(got.download().astype(np.float64) - oracle.astype(np.float64))
        assert np.all(err <= tol * np.maximum(scale, 1e-30)), what
    return kernel


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32, np.int8])
@pytest.mark.parametrize("op", ["sum", "max", "magnitude-squared", "mean"])
def test_column_reduction_twice_second_smaller(pair_factory, dtype, op):
    rng = np.random.default_rng(11)
    with pair_factory() as pair:
        # both calls are cut into row segments whose partials go through the fixed array (inputs above the 4 MiB
        # that a single launch over narrow strips takes); the second is smaller and meets the first one's leftovers
        for rows, cols in ((4096, 2048), (3072, 1536)):
            if np.dtype(dtype).kind == "f":
                data = rng.standard_normal(rows * cols).astype(dtype)
            else:
                info = np.iinfo(dtype)
                data = rng.integers(info.min, info.max, rows * cols, dtype=np.int64).astype(dtype)
            kernel = _check(pair, data, [cols, rows], [1, cols], op)
            assert kernel.startswith("reduce_col"), kernel


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_split_rows_twice_second_smaller(pair_factory, dtype):
    """A few very long rows: each row is cut into chunks whose partials go through the fixed array."""
    rng = np.random.default_rng(12)
    with pair_factory() as pair:
        for rows, cols in ((3, 1 << 20), (2, 1 << 18)):
            data = rng.standard_normal(rows * cols).astype(dtype)
            for op in ("sum", "min", "magnitude"):
                _check(pair, data, [rows, cols], [cols, 1], op, alpha=1.0 if op == "min" else 0.5)


def test_unsplit_shapes_and_ragged_views(pair_factory):
    """Shapes that need no partial accumulators run unchanged."""
    rng = np.random.default_rng(13)
    with pair_factory() as pair:
        data = rng.standard_normal(4096 * 96).astype(np.float32)
        _check(pair, data, [4096, 96], [96, 1], "sum")
        _check(pair, data, [96, 4096], [1, 96], "max")
        _check(pair, data, [7, 13, 5], [65, 5, 1], "mean")
        _check(pair, data[:1], [1, 1], [1, 1], "sum")


def test_rejects_what_the_fixed_array_cannot_hold(pair_factory):
    """1024 byte-wide columns of 132200 rows under a multiplier of 127: the sums can leave 32 bits, so they run on
    long accumulators, and the 512 row segments need 4 MiB of them: refused, nothing launched.  With a
    multiplier of 1 the same reduction runs on int accumulators, 2 MiB, and fits."""
    rows, cols = 132200, 1024
    with pair_factory() as pair:
        data = np.random.default_rng(14).integers(-128, 128, rows * cols, dtype=np.int64).astype(np.int8)
        src = pair.buf(data)
        out = pair.buf(np.full(cols, 5, np.int8))
        view = H.View(src, [cols, rows], [1, cols])
        with pytest.raises(capi.CortexHipError) as err:
            _reduce("ct_unary_reduce_noalloc", pair.hip, H.View(out, [cols, 1]), 127.0, view, "sum")
        assert err.value.status == 1 and "fixed scratch holds 2097152" in err.value.message
        assert np.all(out.download() == 5)
        _reduce("ct_unary_reduce", pair.hip, H.View(out, [cols, 1]), 127.0, view, "sum")  # the allocating form takes it
        sums = data.reshape(rows, cols).astype(np.int64).sum(axis=0)
        assert np.array_equal(out.download(), (sums * 127).astype(np.int8))
        _reduce("ct_unary_reduce_noalloc", pair.hip, H.View(out, [cols, 1]), 1.0, view, "sum")  # int accumulators: fits
        assert np.array_equal(out.download(), sums.astype(np.int8))


def test_float_extreme_under_a_multiplier_on_a_large_input(pair_factory):
    """Float :max / :min with a multiplier other than 1 on 32 MiB and more run the multiplier-free kernel and a
    small multiplying launch: two launches through the fixed array, second call smaller (below 32 MiB it is the
    widening form, one kernel family)."""
    rng = np.random.default_rng(15)
    with pair_factory() as pair:
        for rows, cols in ((8192, 1024), (4096, 512)):
            data = rng.standard_normal(rows * cols).astype(np.float32)
            for op, alpha in (("max", 0.5), ("min", -3.0)):
                kernel = _check(pair, data, [cols, rows], [1, cols], op, alpha=alpha)
                if rows == 8192:  # the last launch is the multiplying one, an elementwise kernel
                    assert not kernel.startswith("reduce"), kernel
                else:
                    assert kernel.startswith("reduce_col"), kernel


def test_allocates_nothing_on_a_fresh_stream(pair_factory):
    """The property the entry point exists for: on a stream whose scratch has never been grown, a split column
    reduction and a split row reduction through it leave the device's free memory where it was."""
    rows, cols = 16384, 1024
    free0, free1, free2, total = C.c_size_t(0), C.c_size_t(0), C.c_size_t(0), C.c_size_t(0)
    with pair_factory() as pair:
        data = np.random.default_rng(16).standard_normal(rows * cols).astype(np.float32)
        src = pair.buf(data)
        out = pair.buf(np.zeros(cols, np.float32))
        few = pair.buf(np.zeros(4, np.float32))
        fresh = C.c_void_p()
        capi.call("ct_stream_create", C.byref(fresh))
        try:
            side = H.Side(gpu=True)
            side.stream = fresh
            col_view, row_view = H.View(src, [cols, rows], [1, cols]), H.View(src, [4, rows * cols // 4])
            capi.call("ct_stream_sync", fresh)
            capi.call("ct_memory_info", C.byref(free0), C.byref(total))
            for op in ("sum", "max"):
                _reduce("ct_unary_reduce_noalloc", side, H.View(out, [cols, 1]), 1.0, col_view, op)
                assert capi.last_kernel().startswith("reduce_col"), capi.last_kernel()
                _reduce("ct_unary_reduce_noalloc", side, H.View(few, [4, 1]), 1.0, row_view, op)
            capi.call("ct_memory_info", C.byref(free1), C.byref(total))
            assert free1.value == free0.value, (free0.value, free1.value)
            want = data.reshape(rows, cols).max(axis=0)
            assert np.array_equal(out.download(), want)
            # the probe does see allocations (a 64 MiB one: the runtime may serve a block as small as a stream's
            # first scratch, 1 MiB, from a chunk it already holds, depending on what was freed before)
            block = C.c_void_p()
            capi.call("ct_malloc", C.byref(block), 64 << 20)
            capi.call("ct_memory_info", C.byref(free2), C.byref(total))
            capi.call("ct_free", block)
            assert free2.value < free1.value, "ct_memory_info did not register a 64 MiB allocation"
        finally:
            capi.call("ct_stream_destroy", fresh)
