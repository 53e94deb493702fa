"""The fused bernoulli dropout mask against the reference's three-call chain (rand!, assign!,
ternary-op! :select; src/cortex/compute/nn/layers.clj:170-195), and the integer division by zero
that the reference's CPU backend throws on (src/cortex/compute/cpu/tensor_math.clj:278-304)."""
import ctypes as C

import numpy as np
import pytest

import harness as H
from cortex_amd import capi
from harness import View

pytestmark = pytest.mark.gpu


@pytest.fixture()
def P(pair_factory):
    with pair_factory() as pair:
        yield pair


def fused(pair, mult: View, rand, n, probability, seed, offset):
    side = pair.hip
    capi.call("ct_dropout_bernoulli_mask", side.stream, side.ptr(mult), mult.buf.dtype,
              side.ptr(rand) if rand is not None else None, n, float(probability), seed, offset)
    capi.call("ct_stream_sync", side.stream)


@pytest.mark.parametrize("n,offset_elems", [(1, 0), (5, 0), (4096, 0), (1000003, 0), (777, 1), (4099, 3)])
@pytest.mark.parametrize("probability", [0.5, 0.9, 0.3])
def test_dropout_mask_equals_the_three_call_chain(P, n, offset_elems, probability):
    seed, offset = 1234567, 42
    maximum = float(np.float32(probability))
    minimum = maximum - 1.0
    for code in (capi.F32, capi.F64):
        np_t = H.NP_DTYPES[code]
        total = n + offset_elems + 4
        # the chain, on the oracle and on the device: rand! -> assign! -> select
        rand_chain = P.buf(np.zeros(total, np.float32))
        mult_chain = rand_chain if code == capi.F32 else P.buf(np.zeros(total, np_t))
        rv, mv = View(rand_chain, [n], offset=offset_elems), View(mult_chain, [n], offset=offset_elems)
        P.run(H.rand, rv, n, "flat", minimum, maximum, seed, offset)
        if mult_chain is not rand_chain:
            P.run(H.assign, mv, rv)
        P.run(H.ternary_op_constant_constant, mv, mv, 1.0, 0.0 * 0.0, 1.0 * (1.0 / probability), [0, 1, 2])
        H.assert_bit_exact(mult_chain.download(), mult_chain.host, "three-call chain, device against oracle")
        # the fused call, with and without a separate buffer for the draws
        mult_f = P.buf(np.zeros(total, np_t))
        rand_f = P.buf(np.zeros(total, np.float32)) if code == capi.F64 else None
        fused(P, View(mult_f, [n], offset=offset_elems), View(rand_f, [n], offset=offset_elems) if rand_f else None, n,
              probability, seed, offset)
        assert capi.last_kernel() == "dropout_mask"
        H.assert_bit_exact(mult_f.download(), mult_chain.host, f"fused mask {np_t.__name__} n={n} p={probability}")
        if rand_f is not None:
            H.assert_bit_exact(rand_f.download(), rand_chain.host, "draws kept by the fused call")
        kept = mult_chain.host[offset_elems:offset_elems + n]
        assert set(np.unique(kept)) <= {np_t(0), np_t(1.0 / probability)}
        if n >= 4096:
            assert abs(np.count_nonzero(kept) / n - probability) < 0.05


def test_dropout_mask_rejects_bad_arguments(P):
    buf = P.buf(np.zeros(16, np.int32))
    with pytest.raises(capi.CortexHipError, match="float or double"):
        fused(P, View(buf, [16]), None, 16, 0.5, 1, 0)


@pytest.mark.parametrize("code", [capi.I32, capi.I8, capi.I64])
def test_integer_division_by_zero_is_reported_in_debug_sync_mode(P, code):
    np_t = H.NP_DTYPES[code]
    x = P.buf(np.arange(1, 65).astype(np_t))
    y = P.buf(np.where(np.arange(64) % 7 == 3, 0, 2).astype(np_t))
    d = P.buf(np.full(64, 9, np_t))
    with pytest.raises(H.OracleError, match="Divide by zero"):
        H.binary_op(H.ORACLE, View(d, [64]), View(x, [64]), 1.0, View(y, [64]), 1.0, "/")
    with pytest.raises(capi.CortexHipError) as err:
        H.binary_op(P.hip, View(d, [64]), View(x, [64]), 1.0, View(y, [64]), 1.0, "/")
    assert err.value.status == 1 and "Divide by zero" in err.value.message
    got = d.download()
    want = np.where(y.init == 0, 0, x.init // 2).astype(np_t)
    assert np.array_equal(got, want)          # the other elements are computed; the offending ones hold 0
    # the flag was cleared: a clean division passes, and so does an unrelated call
    y2 = P.buf(np.full(64, 3, np_t))
    H.binary_op(P.hip, View(d, [64]), View(x, [64]), 1.0, View(y2, [64]), 1.0, "/")
    assert np.array_equal(d.download(), (x.init // 3).astype(np_t))
    # constant and accumulate forms
    with pytest.raises(capi.CortexHipError, match="Divide by zero"):
        H.binary_op_constant(P.hip, View(d, [64]), View(x, [64]), 1.0, 0.0, "/")
    with pytest.raises(capi.CortexHipError, match="Divide by zero"):
        H.binary_accum(P.hip, View(d, [8]), 1.0, View(y, [8, 8]), 1.0, "/", requires_cas=True)
    # with debug-sync off the same call succeeds (0 where the division by zero happened)
    capi.call("ct_set_debug_sync", 0)
    try:
        H.binary_op(P.hip, View(d, [64]), View(x, [64]), 1.0, View(y, [64]), 1.0, "/")
        assert np.array_equal(d.download(), want)
    finally:
        capi.call("ct_set_debug_sync", 1)
    # what that call left in the device's error word does not surface at a later, clean division
    H.binary_op(P.hip, View(d, [64]), View(x, [64]), 1.0, View(y2, [64]), 1.0, "/")
    assert np.array_equal(d.download(), (x.init // 3).astype(np_t))


def test_reserved_scratch_serves_later_calls(P):
    """After a reservation a split reduction and a scatter-add give the results they give without one."""
    capi.call("ct_stream_reserve_scratch", P.hip.stream, 16 << 20, 8 << 20)
    capi.call("ct_stream_reserve_scratch", P.hip.stream, 0, 0)
    rng = np.random.default_rng(21)
    rows, cols = 4096, 512
    data = P.buf(rng.standard_normal(rows * cols).astype(np.float32))
    out = P.buf(np.zeros(cols, np.float32))
    P.run(H.unary_reduce, View(out, [cols, 1]), 1.0, View(data, [cols, rows], [1, cols]), "max")
    assert capi.last_kernel().startswith("reduce_col")
    H.assert_bit_exact(out.download(), out.host, "column max after a reservation")
    table = P.buf(rng.integers(-50, 50, 64 * 32).astype(np.float32))
    updates = P.buf(rng.integers(-50, 50, 4096 * 32).astype(np.float32))
    index = P.buf(rng.integers(0, 64, 4096).astype(np.int32))
    P.run(H.binary_accum, View(table, [4096, 32], [32, 1], index=[index, None]), 1.0, View(updates, [4096, 32]), 1.0, "+")
    assert capi.last_kernel().startswith("accum_grouped")
    H.assert_bit_exact(table.download(), table.host, "scatter-add after a reservation")


def test_index_range_check_names_the_first_bad_entry(P):
    """ct_check_index_range accepts entries in [0, limit) and reports the first one outside without using it."""
    rng = np.random.default_rng(22)
    for n in (1, 77, 5000, 300001):
        good = rng.integers(0, 1000, n).astype(np.int32)
        buf = P.buf(good)
        capi.call("ct_check_index_range", P.hip.stream, P.hip.ptr(View(buf, [n])), n, 1000)
        for bad_value, where in ((1000, n // 2), (-1, n - 1), (2**31 - 1, 0)):
            bad = good.copy()
            bad[where] = bad_value
            if where + 3 < n:
                bad[where + 3] = -7  # a later offender must not be the one reported
            bbuf = P.buf(bad)
            with pytest.raises(capi.CortexHipError) as err:
                capi.call("ct_check_index_range", P.hip.stream, P.hip.ptr(View(bbuf, [n])), n, 1000)
            assert err.value.status == 1
            assert f"entry {where} of the index tensor is {bad_value}, outside [0, 1000)" in err.value.message
    capi.call("ct_check_index_range", P.hip.stream, None, 0, 10)
