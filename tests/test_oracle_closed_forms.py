"""Pins the CPU oracle where the reference holds no stored vector: closed forms
(IEEE-754, Java primitive conversion rules), brute force on tiny shapes, and
hand-computed optimizer steps the reference keeps in its examples.  CPU only.
"""
import itertools
import math

import numpy as np
import pytest

import harness as H
from cortex_amd import capi
from harness import ORACLE, Buf, View

NP = H.NP_DTYPES


def hbuf(a):
    return Buf(np.asarray(a), gpu=False)


# ------------------------------------------------------------------ Java conversion rules (JLS 5.1.3), restated independently

INT_BITS = {capi.I8: 8, capi.I16: 16, capi.I32: 32, capi.I64: 64, capi.U8: 8}


def java_narrow_int(v: int, code: int) -> int:
    bits = INT_BITS[code]
    v &= (1 << bits) - 1
    if code != capi.U8 and v >= 1 << (bits - 1):
        v -= 1 << bits
    return v


def java_fp_to_int(v: float, code: int) -> int:
    if math.isnan(v):
        wide = 0
    elif code == capi.I64:
        wide = max(-(1 << 63), min((1 << 63) - 1, int(v))) if math.isfinite(v) else ((1 << 63) - 1 if v > 0 else -(1 << 63))
        return wide
    else:  # through int (saturating), then truncated
        wide = max(-(1 << 31), min((1 << 31) - 1, int(v))) if math.isfinite(v) else ((1 << 31) - 1 if v > 0 else -(1 << 31))
    return java_narrow_int(wide, code)


def java_convert(value, src_code: int, dst_code: int):
    if dst_code in (capi.F32, capi.F64):
        return NP[dst_code](value)  # numpy rounds to nearest even from ints and from double
    if src_code in (capi.F32, capi.F64):
        return java_fp_to_int(float(value), dst_code)
    return java_narrow_int(int(value), dst_code)


EDGE_VALUES = {
    capi.F64: [0.0, -0.0, 1.5, -1.5, 300.7, -300.7, 127.9, 128.0, -129.2, 65535.6, 2147483647.0, 2147483648.0,
               -2147483649.0, 4294967296.0 + 44.9, 1e19, -1e19, 9.3e18, float("inf"), float("-inf"), float("nan"),
               2.0 ** 53 + 2, 16777217.0],
    capi.I64: [0, 1, -1, 127, 128, -129, 255, 256, 32767, 32768, 65536 + 5, 2 ** 31 - 1, 2 ** 31, -2 ** 31 - 1,
               2 ** 53 + 1, 2 ** 63 - 1, -2 ** 63, 16777217, 2 ** 24 + 3],
}
EDGE_VALUES[capi.F32] = [np.float32(v) for v in EDGE_VALUES[capi.F64][:-2]] + [np.float32(16777216.0)]
EDGE_VALUES[capi.I32] = [v for v in EDGE_VALUES[capi.I64] if -2 ** 31 <= v < 2 ** 31]
EDGE_VALUES[capi.I16] = [v for v in EDGE_VALUES[capi.I64] if -2 ** 15 <= v < 2 ** 15]
EDGE_VALUES[capi.I8] = [v for v in EDGE_VALUES[capi.I64] if -2 ** 7 <= v < 2 ** 7]
EDGE_VALUES[capi.U8] = [0, 1, 127, 128, 200, 255]


@pytest.mark.parametrize("src", H.ALL_DTYPES)
@pytest.mark.parametrize("dst", H.ALL_DTYPES)
def test_assign_conversion_edge_values(src, dst):
    vals = np.array(EDGE_VALUES[src], dtype=NP[src])
    s, d = hbuf(vals), hbuf(np.zeros(vals.size, NP[dst]))
    H.assign(ORACLE, View(d, [vals.size]), View(s, [vals.size]))
    with np.errstate(all="ignore"):
        want = np.array([java_convert(v, src, dst) for v in vals], dtype=NP[dst])
    H.assert_bit_exact(d.host, want, f"assign {src}->{dst}")


def test_assign_exhaustive_int16_and_bytes():
    all16 = np.arange(-32768, 32768, dtype=np.int16)
    s = hbuf(all16)
    for dst in (capi.I8, capi.U8, capi.I32, capi.F32):
        d = hbuf(np.zeros(all16.size, NP[dst]))
        H.assign(ORACLE, View(d, [all16.size]), View(s, [all16.size]))
        want = all16.astype(np.int64)
        want = (want & 0xFF).astype(np.uint8).view(np.int8 if dst == capi.I8 else np.uint8) if dst in (capi.I8, capi.U8) \
            else want.astype(NP[dst])
        H.assert_bit_exact(d.host, want.astype(NP[dst]), f"int16->{dst}")
    u8 = np.arange(256, dtype=np.uint8)
    d = hbuf(np.zeros(256, np.float32))
    H.assign(ORACLE, View(d, [256]), View(hbuf(u8), [256]))
    H.assert_bit_exact(d.host, u8.astype(np.float32), "u8->f32 is exact")
    # the reference's own marshal example in the narrowing direction: 300.7 -> (byte)(int)300.7 = 44
    d = hbuf(np.zeros(1, np.int8))
    H.assign(ORACLE, View(d, [1]), View(hbuf(np.array([300.7], np.float32)), [1]))
    assert int(d.host[0]) == 44


# ------------------------------------------------------------------ address functions: every fast path against the general formula

def general_address(shape, strides, max_shape, e):
    """elem-idx->addr (dimensions.clj:226-252) written out: dims reversed, index
    = running quotient mod the operand's dim, quotient by the max dim."""
    rank = len(max_shape)
    pad = rank - len(shape)
    mi = max(range(len(shape)), key=lambda i: (strides[i], -i))
    shp = [1] * pad + list(shape)
    st = [strides[mi] * shape[mi]] * pad + list(strides)
    off, arg = 0, e
    for i in reversed(range(rank)):
        off += st[i] * (arg % shp[i])
        arg //= max_shape[i]
    return off


def oracle_address(all_dims, which, e):
    import ctypes as C
    from oracle import binding as ob

    structs = [capi.make_dims(s, st) for s, st in all_dims]
    arr = (C.POINTER(capi.CtDims) * len(structs))(*[C.pointer(s) for s in structs])
    addr, mode = C.c_int64(), C.c_int()
    rc = ob.lib().co_elem_address(arr, len(structs), which, e, C.byref(addr), C.byref(mode))
    assert rc == 0
    return addr.value, mode.value


def test_fast_address_paths_equal_the_general_formula():
    """All shapes of rank <= 3 with dims in {1,2,3,4} as the max-shape, every
    operand shape whose dims divide it (dense row-major and transposed)."""
    seen_modes = set()
    for rank in (1, 2, 3):
        for max_shape in itertools.product([1, 2, 3, 4], repeat=rank):
            full = (list(max_shape), H.row_major(max_shape))
            n = int(np.prod(max_shape))
            for op_rank in range(1, rank + 1):
                tail = max_shape[rank - op_rank:]
                for shp in itertools.product(*[[d for d in (1, 2, 3, 4) if m % d == 0] for m in tail]):
                    for perm in itertools.permutations(range(op_rank)):
                        base = H.row_major([shp[i] for i in perm])
                        strides = [0] * op_rank
                        for pos, i in enumerate(perm):
                            strides[i] = base[pos]
                        for e in range(n):
                            got, mode = oracle_address([full, (list(shp), strides)], 1, e)
                            seen_modes.add(mode)
                            assert got == general_address(list(shp), strides, list(max_shape), e), \
                                (max_shape, shp, strides, e, mode)
    assert seen_modes == {0, 1, 2, 3}  # identity, broadcast, repeat and general were all exercised


# ------------------------------------------------------------------ arithmetic closed forms

def f32_special():
    vals = [0.0, -0.0, 1.0, -1.0, 0.1, -0.1, 3.4e38, -3.4e38, 1e-45, -1e-45, 1.17549435e-38, 16777216.0, 16777217.0,
            float("inf"), float("-inf"), float("nan"), 0.5, 1.5, 2.5, -0.5, -1.5, 0.49999997, 123456.789, -7.25]
    return np.array(vals, dtype=np.float32)


def pairs(v):
    a, b = np.meshgrid(v, v)
    return a.reshape(-1).copy(), b.reshape(-1).copy()


@pytest.mark.parametrize("op", ["+", "*", "/", "max", "min", "eq", ">", ">=", "<", "<=", "bit-and", "bit-xor"])
def test_binary_float_closed_form(op):
    """One operation in double, one rounding to float."""
    x, y = pairs(f32_special())
    n = x.size
    bx, by, bd = hbuf(x), hbuf(y), hbuf(np.zeros(n, np.float32))
    H.binary_op(ORACLE, View(bd, [n]), View(bx, [n]), 1.0, View(by, [n]), 1.0, op)
    xd, yd = x.astype(np.float64), y.astype(np.float64)
    with np.errstate(all="ignore"):
        if op == "+":
            want = (xd + yd).astype(np.float32)
        elif op == "*":
            want = (xd * yd).astype(np.float32)
        elif op == "/":
            want = (xd / yd).astype(np.float32)
        elif op == "max":   # (if (> x y) x y): NaN in either place yields y
            want = np.where(xd > yd, x, y)
        elif op == "min":   # (if (> x y) y x)
            want = np.where(xd > yd, y, x)
        elif op in ("bit-and", "bit-xor"):
            to_int = lambda a: np.array([java_fp_to_int(float(t), capi.I32) for t in a], dtype=np.int64)
            r = to_int(xd) & to_int(yd) if op == "bit-and" else to_int(xd) ^ to_int(yd)
            want = r.astype(np.float32)
        else:
            fn = {"eq": np.equal, ">": np.greater, ">=": np.greater_equal, "<": np.less, "<=": np.less_equal}[op]
            want = fn(xd, yd).astype(np.float32)
    H.assert_bit_exact(bd.host, want.astype(np.float32), op)


def test_binary_alpha_is_applied_in_double_before_the_op():
    x = np.array([0.1, 1e30, 3.0, -7.5], np.float32)
    y = np.array([0.2, 1e30, 1e-3, 2.25], np.float32)
    bd = hbuf(np.zeros(4, np.float32))
    H.binary_op(ORACLE, View(bd, [4]), View(hbuf(x), [4]), 2.5, View(hbuf(y), [4]), -0.3, "+")
    a, b = np.float64(np.float32(2.5)), np.float64(np.float32(-0.3))
    want = (x.astype(np.float64) * a + y.astype(np.float64) * b).astype(np.float32)
    H.assert_bit_exact(bd.host, want, "alpha in double")


@pytest.mark.parametrize("code", [capi.I8, capi.I16, capi.I32, capi.I64, capi.U8])
def test_binary_integer_wraps_and_truncates(code):
    info = np.iinfo(NP[code])
    v = np.array([info.min, info.min + 1, -3 if info.min < 0 else 3, 0, 1, 2, 7, info.max - 1, info.max], dtype=NP[code])
    x, y = pairs(v)
    n = x.size
    for op in ("+", "*", "/", "max", "min", "bit-and", "eq", "<"):
        yy = np.where(y == 0, 1, y).astype(NP[code]) if op == "/" else y
        bd = hbuf(np.zeros(n, NP[code]))
        H.binary_op(ORACLE, View(bd, [n]), View(hbuf(x), [n]), 1.0, View(hbuf(yy), [n]), 1.0, op)
        want = []
        for a, b in zip(x.tolist(), yy.tolist()):
            if op == "+":
                r = a + b
            elif op == "*":
                r = a * b
            elif op == "/":
                q = abs(a) // abs(b) * (1 if (a >= 0) == (b >= 0) else -1)  # toward zero
                exact = q * b == a
                if exact or code == capi.I64:
                    r = q
                else:                      # Ratio.intValue saturates at the int range
                    r = max(-2 ** 31, min(2 ** 31 - 1, q))
            elif op == "max":
                r = a if a > b else b
            elif op == "min":
                r = b if a > b else a
            elif op == "bit-and":
                r = java_narrow_int(a, capi.I32) & java_narrow_int(b, capi.I32)
            elif op == "eq":
                r = int(a == b)
            else:
                r = int(a < b)
            want.append(java_narrow_int(r, code))
        H.assert_bit_exact(bd.host, np.array(want, dtype=NP[code]), f"{op} {code}")


def test_integer_division_by_zero_is_an_error():
    bd = hbuf(np.zeros(2, np.int32))
    with pytest.raises(H.OracleError, match="Divide by zero"):
        H.binary_op(ORACLE, View(bd, [2]), View(hbuf(np.array([1, 2], np.int32)), [2]), 1.0,
                    View(hbuf(np.array([1, 0], np.int32)), [2]), 1.0, "/")


def java_round(v: float) -> int:
    if math.isnan(v):
        return 0
    if math.isinf(v):
        return (1 << 63) - 1 if v > 0 else -(1 << 63)
    r = math.floor(v)
    if v - r >= 0.5:
        r += 1
    return max(-(1 << 63), min((1 << 63) - 1, int(r)))


@pytest.mark.parametrize("op", H.capi.UNARY_OPS.keys())
def test_unary_float_closed_form(op):
    x = f32_special()
    n = x.size
    for alpha in (1.0, -2.5):
        bd = hbuf(np.zeros(n, np.float32))
        H.unary_op(ORACLE, View(bd, [n]), View(hbuf(x), [n]), alpha, op)
        v = x.astype(np.float64) * np.float64(np.float32(alpha))
        with np.errstate(all="ignore"):
            if op == "round":
                want = np.array([java_round(float(t)) for t in v], dtype=np.float64).astype(np.float32)
            else:
                fn = {"floor": np.floor, "ceil": np.ceil, "-": np.negative, "tanh": np.tanh, "exp": np.exp,
                      "sqrt": np.sqrt, "noop": lambda t: t, "logistic": lambda t: 1.0 / (1.0 + np.exp(-t))}[op]
                want = fn(v).astype(np.float32)
        if op in ("tanh", "exp", "logistic"):
            # libm's double results are below one double ulp from correctly rounded, so after the
            # rounding to float they can differ from numpy's by at most one float ulp, and rarely
            assert H.ulp_diff_f32(bd.host, want).max() <= 1
        else:
            H.assert_bit_exact(bd.host, want, f"{op} alpha={alpha}")


def test_unary_integer_routes():
    # floor/ceil/noop go through double and saturate; round and negate stay in long and wrap
    x = np.array([2 ** 30, -2 ** 30, 7, -7], np.int32)
    for op, want in (("noop", [2 ** 31 - 1, -2 ** 31, 28, -28]),      # (int)(double)(x*4)
                     ("round", [0, 0, 28, -28]),                      # (int)(long)2^32 wraps
                     ("-", [0, 0, -28, 28]),
                     ("sqrt", [65536, 0, 5, 0]),                      # sqrt(2^32); NaN -> 0
                     ("logistic", [1, 0, 0, 0])):                     # 1/(1+exp(-28)) < 1 truncates to 0
        bd = hbuf(np.zeros(4, np.int32))
        H.unary_op(ORACLE, View(bd, [4]), View(hbuf(x), [4]), 4.0, op)
        assert bd.host.tolist() == want, (op, bd.host.tolist())
    # alpha is cast to the tensor datatype first: (int 2.5) = 2
    bd = hbuf(np.zeros(2, np.int32))
    H.unary_op(ORACLE, View(bd, [2]), View(hbuf(np.array([3, -3], np.int32)), [2]), 2.5, "noop")
    assert bd.host.tolist() == [6, -6]


def test_select_semantics():
    x = np.array([1.0, -1.0, 0.0, -0.0, float("nan"), 1e-30, -1e-30], np.float32)
    y = np.full(7, 10.0, np.float32)
    z = np.full(7, 20.0, np.float32)
    bd = hbuf(np.zeros(7, np.float32))
    H.ternary_op(ORACLE, View(bd, [7]), View(hbuf(x), [7]), 1.0, View(hbuf(y), [7]), 1.0, View(hbuf(z), [7]), 1.0)
    # (>= x 0) ? z : y; -0.0 >= 0 is true, NaN >= 0 is false
    assert bd.host.tolist() == [20.0, 10.0, 20.0, 20.0, 10.0, 20.0, 10.0]
    # with a constant every argument is cast to float BEFORE the comparison:
    # -1e-30 * 1e-30 underflows to -0.0f, and -0.0 >= 0 holds
    H.ternary_op_constant(ORACLE, View(bd, [7]), View(hbuf(x), [7]), 1e-30, View(hbuf(y), [7]), 1.0, 20.0, [0, 1, 2])
    assert bd.host.tolist() == [20.0, 10.0, 20.0, 20.0, 10.0, 20.0, 20.0]
    # three tensors compare the unrounded double product
    H.ternary_op(ORACLE, View(bd, [7]), View(hbuf(x), [7]), 1e-30, View(hbuf(y), [7]), 1.0, View(hbuf(z), [7]), 1.0)
    assert bd.host.tolist() == [20.0, 10.0, 20.0, 20.0, 10.0, 20.0, 10.0]


# ------------------------------------------------------------------ reductions

@pytest.mark.parametrize("code", [capi.F32, capi.F64])
def test_reduce_is_sequential_double(code):
    rng = np.random.default_rng(3)
    x = (rng.standard_normal((7, 1000)) * 1e3).astype(NP[code])
    for alpha in (1.0, 0.37):
        a = np.float64(NP[code](alpha))
        for op in capi.REDUCE_OPS:
            out = hbuf(np.zeros(7, NP[code]))
            H.unary_reduce(ORACLE, View(out, [7, 1]), alpha, View(hbuf(x), [7, 1000]), op)
            want = []
            for row in x.astype(np.float64):
                v = row * a
                if op in ("sum", "mean"):
                    acc = float(np.cumsum(v)[-1])  # numpy cumsum is the same left-to-right sum
                    want.append(acc / 1000 if op == "mean" else acc)
                elif op in ("magnitude", "magnitude-squared"):
                    acc = float(np.cumsum(v * v)[-1])
                    want.append(math.sqrt(acc) if op == "magnitude" else acc)
                else:
                    want.append(float(v.max() if op == "max" else v.min()))
            H.assert_bit_exact(out.host, np.array(want, dtype=np.float64).astype(NP[code]), f"{op} {alpha}")


def test_reduce_nan_and_signed_zero():
    x = np.array([[1.0, float("nan"), 3.0], [-0.0, 0.0, -0.0], [0.0, -0.0, -0.0]], np.float32)
    out = hbuf(np.zeros(3, np.float32))
    H.unary_reduce(ORACLE, View(out, [3, 1]), 1.0, View(hbuf(x), [3, 3]), "max")
    assert math.isnan(out.host[0]) and not np.signbit(out.host[1]) and not np.signbit(out.host[2])
    H.unary_reduce(ORACLE, View(out, [3, 1]), 1.0, View(hbuf(x), [3, 3]), "min")
    assert math.isnan(out.host[0]) and np.signbit(out.host[1]) and np.signbit(out.host[2])


def test_reduce_integer_mean_truncates_toward_zero():
    x = np.array([[1, 2, 4], [-1, -2, -4], [100, 27, 0]], np.int32)
    out = hbuf(np.zeros(3, np.int32))
    H.unary_reduce(ORACLE, View(out, [3, 1]), 1.0, View(hbuf(x), [3, 3]), "mean")
    assert out.host.tolist() == [2, -2, 42]
    H.unary_reduce(ORACLE, View(out, [3, 1]), 1.0, View(hbuf(x), [3, 3]), "magnitude")
    assert out.host.tolist() == [4, 4, 103]


def test_reduce_through_a_transposed_view():
    x = np.arange(12, dtype=np.float64).reshape(3, 4)
    out = hbuf(np.zeros(4))
    H.unary_reduce(ORACLE, View(out, [4, 1]), 1.0, View(hbuf(x), [3, 4]).transpose([1, 0]), "sum")
    assert out.host.tolist() == x.sum(axis=0).tolist()


# ------------------------------------------------------------------ accumulate: serial order

def test_binary_accum_applies_updates_in_increasing_order():
    # dest [3] <- y [4,3], op :*, dest_alpha 2: d = ((d*2*y0)*2*y1)...; the order matters once rounding bites
    y = (np.arange(12, dtype=np.float32) + 1.1).reshape(4, 3)
    d0 = np.array([1.0, 2.0, 3.0], np.float32)
    dest = hbuf(d0)
    H.binary_accum(ORACLE, View(dest, [3]), 2.0, View(hbuf(y), [4, 3]), 1.0, "*", requires_cas=True)
    want = d0.copy()
    for r in range(4):
        want = (want.astype(np.float64) * 2.0 * y[r].astype(np.float64)).astype(np.float32)
    H.assert_bit_exact(dest.host, want, "serial accumulate")
    # reversed operands: dest = y - dest
    dest = hbuf(d0)
    H.binary_accum(ORACLE, View(dest, [3]), 1.0, View(hbuf(y), [4, 3]), 1.0, "-", reverse=True, requires_cas=True)
    want = d0.copy()
    for r in range(4):
        want = (y[r].astype(np.float64) - want.astype(np.float64)).astype(np.float32)
    H.assert_bit_exact(dest.host, want, "reversed accumulate")


# ------------------------------------------------------------------ optimizers

def test_adam_hand_computed_step():
    """examples/optimise/test/cortex/optimise/optimisers_test.clj:71-87: step size 5, decays
    0.75 / 0.3, conditioning 0.2, third step."""
    p, g = hbuf(np.array([1.0, 2.0, -5.0])), hbuf(np.array([5.0, 3.0, 7.0]))
    m, v = hbuf(np.array([5.0, 2.0, -3.0])), hbuf(np.array([-1.0, -3.0, -8.0]))
    V = lambda b: View(b, [3])
    H.adam_step(ORACLE, 5, 0.75, 0.3, 0.2, 0.75 ** 3, 0.3 ** 3, 1.0, V(g), V(p), V(m), V(v), 3)
    assert np.allclose(p.host, [-8.81811015, -5.613809809, -4.270259223], atol=1e-8, rtol=0)
    assert np.allclose(m.host, [5.0, 2.25, -0.5], atol=1e-12, rtol=0)
    assert np.allclose(v.host, [17.2, 5.4, 31.9], atol=1e-12, rtol=0)


def test_adam_float_runs_in_double_and_rounds_once():
    rng = np.random.default_rng(5)
    n = 257
    p0 = rng.uniform(-0.05, 0.05, n).astype(np.float32)
    g0 = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    m0 = (rng.standard_normal(n) * 1e-4).astype(np.float32)
    v0 = (rng.random(n) * 1e-6).astype(np.float32)
    p, g, m, v = hbuf(p0), hbuf(g0), hbuf(m0), hbuf(v0)
    V = lambda b: View(b, [n])
    pb1, pb2 = 0.9 ** 7, 0.999 ** 7
    H.adam_step(ORACLE, 1e-3, 0.9, 0.999, 1e-8, pb1, pb2, 0.5, V(g), V(p), V(m), V(v), n)
    f = lambda t: np.float64(np.float32(t))
    gv = f(0.5) * g0.astype(np.float64)
    lm = f(0.9) * m0.astype(np.float64) + (1.0 - f(0.9)) * gv
    lv = f(0.999) * v0.astype(np.float64) + ((1.0 - f(0.999)) * gv) * gv
    dx = f(1e-3) * (lm / ((1.0 - f(pb1)) * (np.sqrt(lv / (1.0 - f(pb2))) + f(1e-8))))
    H.assert_bit_exact(m.host, lm.astype(np.float32), "m")
    H.assert_bit_exact(v.host, lv.astype(np.float32), "v")
    H.assert_bit_exact(p.host, (p0.astype(np.float64) - dx).astype(np.float32), "params")


def test_adadelta_hand_computed_step():
    """examples/optimise/test/cortex/optimise/optimisers_test.clj:57-69 (decay 0.5 is where the
    example's and the core's conventions coincide), conditioning 1."""
    p, g = hbuf(np.array([1.0, 2.0, 3.0])), hbuf(np.array([2.0, 4.0, 8.0]))
    ga, da = hbuf(np.array([6.0, 3.0, 9.0])), hbuf(np.array([7.0, 8.0, 7.0]))
    V = lambda b: View(b, [3])
    H.adadelta_step(ORACLE, 0.5, 1.0, V(ga), V(da), 1.0, V(g), V(p), 3)
    assert np.allclose(p.host, [-1.309401077, -1.703280399, -0.6950417228], atol=1e-8, rtol=0)
    assert np.allclose(ga.host, [5.0, 9.5, 36.5], atol=1e-12, rtol=0)
    assert np.allclose(da.host, [6.166666667, 10.85714286, 10.32666667], atol=1e-7, rtol=0)


def test_adadelta_float_follows_the_java_step():
    rng = np.random.default_rng(9)
    n = 130
    p0 = rng.uniform(-1, 1, n).astype(np.float32)
    g0 = rng.standard_normal(n).astype(np.float32)
    a0, d0 = rng.random(n).astype(np.float32), rng.random(n).astype(np.float32)
    p, g, ga, da = hbuf(p0), hbuf(g0), hbuf(a0), hbuf(d0)
    V = lambda b: View(b, [n])
    H.adadelta_step(ORACLE, 0.05, 1e-6, V(ga), V(da), 0.7, V(g), V(p), n)
    dec, eps = np.float64(np.float32(0.05)), np.float64(np.float32(1e-6))
    grad = (np.float32(0.7) * g0).astype(np.float64)            # float product, then widened
    acc = grad * grad * dec + a0.astype(np.float64) * (1.0 - dec)
    dx = (-1.0 * np.sqrt(d0.astype(np.float64) + eps) * grad) / np.sqrt(acc + eps)
    dacc = dx * dx * dec + d0.astype(np.float64) * (1.0 - dec)
    H.assert_bit_exact(ga.host, acc.astype(np.float32), "grad accum")
    H.assert_bit_exact(da.host, dacc.astype(np.float32), "dx accum")
    H.assert_bit_exact(p.host, p0 + dx.astype(np.float32), "params (float +=)")


# ------------------------------------------------------------------ activation-gradient!, softmax

@pytest.mark.parametrize("code", [capi.F32, capi.F64])
def test_activation_gradient_closed_form(code):
    rng = np.random.default_rng(21)
    n = 257
    out = rng.standard_normal(n).astype(NP[code])
    grad = rng.standard_normal(n).astype(NP[code])
    out[:4] = [0.0, -0.0, np.nan, 1.0]
    o64, g64 = out.astype(np.float64), grad.astype(np.float64)
    want = {"logistic": (o64 * (1.0 - o64)) * g64, "tanh": (1.0 - o64 * o64) * g64,
            "relu": np.where(o64 > 0.0, 1.0, 0.0) * g64}
    for op, w in want.items():
        ob, gb, ib = hbuf(out), hbuf(grad), hbuf(np.zeros(n, NP[code]))
        H.activation_gradient(ORACLE, View(ib, [n]), View(gb, [n]), View(ob, [n]), op, n)
        H.assert_bit_exact(ib.host, w.astype(NP[code]), op)   # one rounding of the double result


def test_activation_gradient_broadcasts_like_the_other_elementwise_ops():
    out, grad = hbuf(np.array([2.0, -1.0, 0.5], np.float32)), hbuf(np.arange(6, dtype=np.float32))
    ib = hbuf(np.zeros(6, np.float32))
    H.activation_gradient(ORACLE, View(ib, [2, 3]), View(grad, [2, 3]), View(out, [3]), "relu", 6)
    assert ib.host.tolist() == [0.0, 0.0, 2.0, 3.0, 0.0, 5.0]


@pytest.mark.parametrize("code", [capi.F32, capi.F64])
def test_softmax_closed_form_and_invariants(code):
    rng = np.random.default_rng(22)
    rows, k = 7, 13
    x = (rng.standard_normal((rows, k)) * 5).astype(NP[code])
    xb, ob = hbuf(x.ravel()), hbuf(np.zeros(rows * k, NP[code]))
    H.softmax(ORACLE, View(ob, [rows, k]), View(xb, [rows, k]))
    got = ob.host.reshape(rows, k).astype(np.float64)
    x64 = x.astype(np.float64)
    e = np.exp(x64 - x64.max(axis=1, keepdims=True))
    want = e / e.sum(axis=1, keepdims=True)
    tol = 1e-6 if code == capi.F32 else 1e-14
    assert np.allclose(got, want, rtol=tol, atol=0)
    assert np.allclose(got.sum(axis=1), 1.0, atol=k * tol)
    # a shifted input gives the same distribution; the largest entry of a row is exp(0)/sum
    sb, o2 = hbuf((x + NP[code](3.0)).ravel()), hbuf(np.zeros(rows * k, NP[code]))
    H.softmax(ORACLE, View(o2, [rows, k]), View(sb, [rows, k]))
    assert np.allclose(o2.host.astype(np.float64), ob.host.astype(np.float64), rtol=20 * tol)
    assert np.allclose(got.max(axis=1), 1.0 / e.sum(axis=1), rtol=tol)


def test_softmax_spatial_runs_across_channels_and_three_dims_batch():
    rng = np.random.default_rng(23)
    b, c, e = 2, 5, 6
    x = rng.standard_normal((b, c, e))
    xb, ob = hbuf(x.ravel()), hbuf(np.zeros(b * c * e))
    H.softmax(ORACLE, View(ob, [b, c, e]), View(xb, [b, c, e]), spatial=True)
    ex = np.exp(x - x.max(axis=1, keepdims=True))
    assert np.allclose(ob.host.reshape(b, c, e), ex / ex.sum(axis=1, keepdims=True), rtol=1e-14)
    # the eltwise form on three dimensions normalises the last axis of every [outer, row]
    H.softmax(ORACLE, View(ob, [b, c, e]), View(xb, [b, c, e]))
    ex = np.exp(x - x.max(axis=2, keepdims=True))
    assert np.allclose(ob.host.reshape(b, c, e), ex / ex.sum(axis=2, keepdims=True), rtol=1e-14)


def test_softmax_stores_float_exponentials_before_summing():
    # every stage rounds to the tensor type: e_i = float(exp(x_i - max)), s = float(sum of e_i), y_i = e_i / s in float
    x = np.array([0.1, 0.2, 0.3, 0.7, -1.5], np.float32)
    xb, ob = hbuf(x), hbuf(np.zeros(5, np.float32))
    H.softmax(ORACLE, View(ob, [1, 5]), View(xb, [1, 5]))
    e = np.exp(x.astype(np.float64) - np.float64(x.max())).astype(np.float32)
    s = np.float32(np.cumsum(e.astype(np.float64))[-1])
    H.assert_bit_exact(ob.host, e / s, "softmax staging")


# ------------------------------------------------------------------ batch normalization
# Pinned by the reference's stored vectors (tests/reference_suite.py) and, here, by what the
# mathematics fixes: numpy's mean / var for the statistics, the running-average rule, a
# normalized output, and a finite-difference derivative of the forward pass for the gradients.

def _bn_buffers(rng, b, c, e, f):
    n = b * c * e
    t = dict(x=(rng.standard_normal(n) * 2 + 3).astype(f), out=np.zeros(n, f), og=rng.standard_normal(n).astype(f),
             ig=np.zeros(n, f), means=np.zeros(c, f), variances=np.zeros(c, f), rmeans=rng.standard_normal(c).astype(f),
             rvars=rng.uniform(0.5, 2, c).astype(f), scale=rng.uniform(0.5, 1.5, c).astype(f),
             bias=rng.standard_normal(c).astype(f), sg=np.zeros(c, f), bg=np.zeros(c, f))
    bufs = {k: H.Buf(v, gpu=False) for k, v in t.items()}
    return bufs, {k: H.View(v, [v.init.size]) for k, v in bufs.items()}


@pytest.mark.parametrize("layout", [(6, 5, None), (4, 3, 7)], ids=["eltwise", "spatial"])
def test_batch_normalize_statistics_closed_form(layout):
    b, c, e = layout
    rng = np.random.default_rng(50)
    bufs, V = _bn_buffers(rng, b, c, e or 1, np.float64)
    rm0, rv0 = bufs["rmeans"].init.copy(), bufs["rvars"].init.copy()
    H.batch_normalize_update_and_apply(H.ORACLE, V["out"], V["x"], V["means"], V["variances"], V["rmeans"], V["rvars"],
                                       0.3, V["scale"], V["bias"], 1e-3, b, c, e)
    x = bufs["x"].init.reshape(b, c, e or 1)
    mean, var = x.mean(axis=(0, 2)), x.var(axis=(0, 2))
    np.testing.assert_allclose(bufs["means"].host, mean, rtol=1e-13)
    np.testing.assert_allclose(bufs["variances"].host, var, rtol=1e-12)
    np.testing.assert_allclose(bufs["rmeans"].host, rm0 * 0.7 + mean * 0.3, rtol=1e-12)
    np.testing.assert_allclose(bufs["rvars"].host, rv0 * 0.7 + x.var(axis=(0, 2), ddof=1) * 0.3, rtol=1e-12)
    want = (x - mean[None, :, None]) / np.sqrt(var + 1e-3)[None, :, None] * bufs["scale"].init[None, :, None] \
        + bufs["bias"].init[None, :, None]
    np.testing.assert_allclose(bufs["out"].host.reshape(x.shape), want, rtol=1e-11, atol=1e-12)


@pytest.mark.parametrize("layout", [(5, 4, None), (3, 2, 6)], ids=["eltwise", "spatial"])
def test_batch_normalize_gradients_against_finite_differences(layout):
    b, c, e = layout
    ee = e or 1
    rng = np.random.default_rng(51)
    bufs, V = _bn_buffers(rng, b, c, ee, np.float64)
    eps = 1e-3

    def forward(x, scale, bias):
        x = x.reshape(b, c, ee)
        mean, var = x.mean(axis=(0, 2), keepdims=True), x.var(axis=(0, 2), keepdims=True)
        return ((x - mean) / np.sqrt(var + eps) * scale[None, :, None] + bias[None, :, None]).reshape(-1)

    x0, og = bufs["x"].init.copy(), bufs["og"].init.copy()
    scale0, bias0 = bufs["scale"].init.copy(), bufs["bias"].init.copy()
    loss = lambda x, s, bb: float(np.dot(forward(x, s, bb), og))
    H.batch_normalize_update_and_apply(H.ORACLE, V["out"], V["x"], V["means"], V["variances"], V["rmeans"], V["rvars"],
                                       0.3, V["scale"], V["bias"], eps, b, c, e)
    H.batch_normalize_gradients(H.ORACLE, V["ig"], V["sg"], V["bg"], V["og"], V["out"], V["x"], V["means"],
                                V["variances"], V["scale"], V["bias"], eps, b, c, e)
    h = 1e-6
    num_ig = np.zeros_like(x0)
    for i in range(x0.size):
        xp, xm = x0.copy(), x0.copy()
        xp[i] += h
        xm[i] -= h
        num_ig[i] = (loss(xp, scale0, bias0) - loss(xm, scale0, bias0)) / (2 * h)
    np.testing.assert_allclose(bufs["ig"].host, num_ig, rtol=1e-5, atol=1e-7)
    for name, which in (("sg", 0), ("bg", 1)):
        num = np.zeros(c)
        for j in range(c):
            d = np.zeros(c)
            d[j] = h
            if which == 0:
                num[j] = (loss(x0, scale0 + d, bias0) - loss(x0, scale0 - d, bias0)) / (2 * h)
            else:
                num[j] = (loss(x0, scale0, bias0 + d) - loss(x0, scale0, bias0 - d)) / (2 * h)
        np.testing.assert_allclose(bufs[name].host, num, rtol=1e-6, atol=1e-8)


def test_batch_normalize_float_rounding_points():
    """Where the float form rounds: the inverse standard deviation is rounded to float before it
    is used (cpu/tensor_math.clj:772-773) and the store rounds once."""
    x = np.array([0.1, 0.7, 1.3, 2.9], np.float32)
    m, v, s, bb = np.float32(0.3), np.float32(0.77), np.float32(1.7), np.float32(-0.2)
    bufs = [H.Buf(a, gpu=False) for a in (np.zeros(4, np.float32), x, np.array([m]), np.array([v]), np.array([s]),
                                          np.array([bb]))]
    views = [H.View(bf, [bf.init.size]) for bf in bufs]
    H.batch_normalize(H.ORACLE, *views, 1e-2, 4, 1)
    inv = np.float32(np.sqrt(1.0 / (np.float64(v) + np.float64(np.float32(1e-2)))))
    want = ((x.astype(np.float64) - np.float64(m)) * np.float64(inv) * np.float64(s) + np.float64(bb)).astype(np.float32)
    H.assert_bit_exact(bufs[0].host, want, "batch-normalize float rounding")


# ------------------------------------------------------------------ rand!
# The generator is not the reference's (it draws from SecureRandom / cuRAND and fixes only the
# distribution).  Philox4x32-10 is pinned by the known-answer vectors published with Random123
# (kat_vectors: zero, all-ones and digits-of-pi inputs); the mapping to floats by its closed form
# and by the moments of the two distributions.

PHILOX_KAT = [
    ([0, 0, 0, 0], [0, 0], [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]),
    ([0xffffffff] * 4, [0xffffffff] * 2, [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]),
    ([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], [0xa4093822, 0x299f31d0],
     [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1]),
]


def _philox(counter, key):
    import ctypes as C
    c, k, o = (C.c_uint32 * 4)(*counter), (C.c_uint32 * 2)(*key), (C.c_uint32 * 4)()
    H.oracle_lib().co_philox4x32_10(c, k, o)
    return list(o)


@pytest.mark.parametrize("counter,key,want", PHILOX_KAT)
def test_philox_known_answers(counter, key, want):
    assert _philox(counter, key) == want


def test_rand_flat_is_the_philox_stream():
    n, seed, offset = 1003, 0x0123456789ABCDEF, 7
    buf = H.Buf(np.zeros(n, np.float32), gpu=False)
    H.rand(H.ORACLE, H.View(buf, [n]), n, "flat", -1.5, 2.5, seed, offset)
    key = [seed & 0xFFFFFFFF, seed >> 32]
    words = np.array([w for i in range((n + 3) // 4) for w in _philox([i, 0, offset, 0], key)][:n], dtype=np.uint64)
    u = (words >> np.uint64(8)).astype(np.float64) * 2.0 ** -24
    want = (np.float64(np.float32(-1.5)) + u * (np.float64(np.float32(2.5)) - np.float64(np.float32(-1.5)))).astype(np.float32)
    H.assert_bit_exact(buf.host, want, "flat rand")
    assert buf.host.min() >= -1.5 and buf.host.max() < 2.5
    # another offset or seed gives another stream; the same pair repeats
    again = H.Buf(np.zeros(n, np.float32), gpu=False)
    H.rand(H.ORACLE, H.View(again, [n]), n, "flat", -1.5, 2.5, seed, offset)
    assert np.array_equal(again.host, buf.host)
    H.rand(H.ORACLE, H.View(again, [n]), n, "flat", -1.5, 2.5, seed, offset + 1)
    assert not np.array_equal(again.host, buf.host)


def test_rand_moments():
    n = 1 << 20
    buf = H.Buf(np.zeros(n, np.float32), gpu=False)
    H.rand(H.ORACLE, H.View(buf, [n]), n, "gaussian", 3.0, 4.0, 11, 0)
    v = buf.host.astype(np.float64)
    assert abs(v.mean() - 3.0) < 0.01 and abs(v.var() - 4.0) < 0.03
    z = (v - 3.0) / 2.0
    assert abs(np.mean(z ** 3)) < 0.02 and abs(np.mean(z ** 4) - 3.0) < 0.05      # skewness, kurtosis
    assert abs(np.corrcoef(z[:-1], z[1:])[0, 1]) < 0.005                           # neighbours (cos / sin of one pair)
    from scipy import stats
    assert stats.kstest(z[:200000], "norm").pvalue > 1e-3
    H.rand(H.ORACLE, H.View(buf, [n]), n, "flat", 0.0, 1.0, 11, 1)
    u = buf.host.astype(np.float64)
    assert abs(u.mean() - 0.5) < 0.002 and abs(u.var() - 1 / 12) < 0.001
    counts = np.histogram(u, bins=64, range=(0, 1))[0]
    assert stats.chisquare(counts).pvalue > 1e-3


# ------------------------------------------------------------------ gemm!, gemv!
# The product is netlib BLAS in the reference (not under /root/reference); its definition
# C = alpha op(A) op(B) + beta C is checked against numpy's matmul in float64, with row pitches
# wider than the rows, all four transposition pairs, and beta = 0 over a NaN-filled C.

@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
def test_gemm_matches_numpy(ta, tb):
    rng = np.random.default_rng(60)
    M, K, N, lda, ldb, ldc = 5, 7, 4, 9, 8, 6
    a_rows, a_cols = (K, M) if ta else (M, K)
    b_rows, b_cols = (N, K) if tb else (K, N)
    a, b, c = rng.standard_normal((a_rows, lda)), rng.standard_normal((b_rows, ldb)), rng.standard_normal((M, ldc))
    A, B = a[:, :a_cols], b[:, :b_cols]
    want = c.copy()
    want[:, :N] = 1.5 * (A.T if ta else A) @ (B.T if tb else B) - 0.5 * c[:, :N]
    bufs = [H.Buf(v, gpu=False) for v in (c, a, b)]
    vc, va, vb = (H.View(bf, [bf.init.size]) for bf in bufs)
    H.gemm(H.ORACLE, vc, ldc, ta, tb, 1.5, va, M, K, lda, vb, N, ldb, -0.5)
    np.testing.assert_allclose(bufs[0].host.reshape(M, ldc), want, rtol=1e-13, atol=1e-13)
    bufs[0].host[...] = np.nan
    H.gemm(H.ORACLE, vc, ldc, ta, tb, 1.0, va, M, K, lda, vb, N, ldb, 0.0)
    got = bufs[0].host.reshape(M, ldc)
    np.testing.assert_allclose(got[:, :N], (A.T if ta else A) @ (B.T if tb else B), rtol=1e-13, atol=1e-13)
    assert np.all(np.isnan(got[:, N:]))          # the padding between rows is not touched


@pytest.mark.parametrize("ta", [False, True])
def test_gemv_matches_numpy(ta):
    rng = np.random.default_rng(61)
    rows, cols, lda, incx, incy = 6, 5, 8, 3, 2
    a = rng.standard_normal((rows, lda))
    n_in, n_out = (rows, cols) if ta else (cols, rows)
    x, y = rng.standard_normal(n_in * incx), rng.standard_normal(n_out * incy)
    A = a[:, :cols]
    want = y.copy()
    want[::incy] = 2.0 * ((A.T if ta else A) @ x[::incx]) + 0.25 * y[::incy]
    bufs = [H.Buf(v, gpu=False) for v in (y, a, x)]
    vy, va, vx = (H.View(bf, [bf.init.size]) for bf in bufs)
    H.gemv(H.ORACLE, vy, incy, ta, 2.0, va, rows, cols, lda, vx, incx, 0.25)
    np.testing.assert_allclose(bufs[0].host, want, rtol=1e-13, atol=1e-13)


# ------------------------------------------------------------------ pooling against a windowed numpy restatement

POOL_GEOMETRIES = [(7, 9, 3, 3, 1, 1, 2, 2, 4, 5), (8, 8, 2, 2, 0, 0, 2, 2, 4, 4), (6, 5, 3, 2, 1, 1, 1, 2, 4, 5),
                   (9, 9, 2, 2, 1, 1, 1, 1, 10, 10)]


def _windows(h, w, kw, kh, px, py, sx, sy, oh, ow):
    """Per output position: the list of (y, x, inside-the-input) taps within the padded input."""
    for oy in range(oh):
        for ox in range(ow):
            taps = []
            for ky in range(kh):
                for kx in range(kw):
                    y, x = oy * sy - py + ky, ox * sx - px + kx
                    if -py <= y < h + py and -px <= x < w + px:
                        taps.append((y, x, 0 <= y < h and 0 <= x < w))
            yield oy, ox, taps


@pytest.mark.parametrize("geometry", POOL_GEOMETRIES, ids=str)
def test_pooling_matches_windowed_numpy(geometry):
    h, w, kw, kh, px, py, sx, sy, oh, ow = geometry
    rng = np.random.default_rng(60)
    planes = 3
    x = rng.standard_normal((planes, h, w))
    og = rng.standard_normal((planes, oh, ow))
    for op in capi.POOL_OPS:
        want = np.zeros((planes, oh, ow))
        want_ig = np.zeros((planes, h, w))
        for p in range(planes):
            for oy, ox, taps in _windows(h, w, kw, kh, px, py, sx, sy, oh, ow):
                vals = [x[p, y, xx] if inside else 0.0 for y, xx, inside in taps]
                inside_taps = [(y, xx) for y, xx, inside in taps if inside]
                if op == "max":
                    want[p, oy, ox] = max(vals)
                    for y, xx in inside_taps:
                        if x[p, y, xx] == want[p, oy, ox]:
                            want_ig[p, y, xx] += og[p, oy, ox]
                else:
                    count = kw * kh if op == "avg" else len(inside_taps)
                    want[p, oy, ox] = sum(vals) / count
                    for y, xx in inside_taps:
                        want_ig[p, y, xx] += og[p, oy, ox] / count
        inp, out = hbuf(x.reshape(-1)), hbuf(np.zeros(planes * oh * ow))
        grad, ig = hbuf(og.reshape(-1)), hbuf(np.zeros(planes * h * w))
        desc = H.pool_desc(kw, kh, px, py, sx, sy, op)
        H.pooling_forward(ORACLE, View(out, [out.host.size]), View(inp, [inp.host.size]), desc, 1, planes, h, w, oh, ow)
        np.testing.assert_allclose(out.host.reshape(want.shape), want, rtol=1e-12, atol=1e-14, err_msg=op)
        H.pooling_backward(ORACLE, View(ig, [ig.host.size]), View(inp, [inp.host.size]), View(out, [out.host.size]),
                           View(grad, [grad.host.size]), desc, 1, planes, h, w, oh, ow)
        np.testing.assert_allclose(ig.host.reshape(want_ig.shape), want_ig, rtol=1e-12, atol=1e-14, err_msg=op)


def test_average_pooling_backward_is_the_adjoint_of_forward():
    """<forward(x), g> = <x, backward(g)> for the two averages, which are linear maps."""
    h, w, kw, kh, px, py, sx, sy, oh, ow = 11, 13, 3, 3, 1, 1, 2, 2, 6, 7
    rng = np.random.default_rng(61)
    x, g = rng.standard_normal(2 * h * w), rng.standard_normal(2 * oh * ow)
    for op in ("avg", "avg-exc-pad"):
        inp, out, grad, ig = hbuf(x), hbuf(np.zeros(2 * oh * ow)), hbuf(g), hbuf(np.zeros(2 * h * w))
        desc = H.pool_desc(kw, kh, px, py, sx, sy, op)
        H.pooling_forward(ORACLE, View(out, [out.host.size]), View(inp, [x.size]), desc, 2, 1, h, w, oh, ow)
        H.pooling_backward(ORACLE, View(ig, [x.size]), View(inp, [x.size]), View(out, [g.size]), View(grad, [g.size]),
                           desc, 2, 1, h, w, oh, ow)
        assert abs(np.dot(out.host, g) - np.dot(x, ig.host)) < 1e-10


# ------------------------------------------------------------------ convolution against scipy's correlation

@pytest.mark.parametrize("geometry", [(5, 6, 3, 3, 0, 0, 1, 1), (7, 7, 3, 3, 1, 1, 2, 2), (6, 9, 2, 3, 1, 0, 1, 2)], ids=str)
def test_convolution_matches_correlation(geometry):
    from scipy.signal import correlate2d
    h, w, kw, kh, px, py, sx, sy = geometry
    batch, cin, cout = 2, 3, 4
    oh, ow = (h + 2 * py - kh) // sy + 1, (w + 2 * px - kw) // sx + 1
    rng = np.random.default_rng(62)
    x = rng.standard_normal((batch, cin, h, w))
    wt = rng.standard_normal((cout, cin, kh, kw))
    g = rng.standard_normal((batch, cout, oh, ow))
    desc = H.conv_desc(cin, cout, kw, kh, px, py, sx, sy)
    n_rows, n_cols = oh * ow, cin * kh * kw
    inp, weights, grad = hbuf(x.reshape(-1)), hbuf(wt.reshape(-1)), hbuf(g.reshape(-1))
    out, work = hbuf(np.full(batch * cout * n_rows, 9.0)), hbuf(np.zeros(batch * n_rows * n_cols))
    wg, ig = hbuf(np.full(cout * n_cols, 9.0)), hbuf(np.full(x.size, 9.0))
    V = lambda b: View(b, [b.host.size])
    geom = (desc, batch, h, w, oh, ow)
    H.convolution(ORACLE, "forward", V(out), 0.0, V(inp), V(weights), V(work), *geom)
    padded = np.pad(x, ((0, 0), (0, 0), (py, py), (px, px)))
    want = np.zeros((batch, cout, oh, ow))
    for b in range(batch):
        for o in range(cout):
            full = sum(correlate2d(padded[b, c], wt[o, c], mode="valid") for c in range(cin))
            want[b, o] = full[::sy, ::sx][:oh, :ow]
    np.testing.assert_allclose(out.host.reshape(want.shape), want, rtol=1e-12, atol=1e-12)
    # the gradients as the adjoints of the forward map: <conv(x, W), g> is linear in x and in W
    H.convolution(ORACLE, "backward_weights", V(wg), 0.0, V(grad), V(inp), V(work), *geom)
    H.convolution(ORACLE, "backward_data", V(ig), 0.0, V(grad), V(weights), V(work), *geom)
    inner = np.dot(want.reshape(-1), g.reshape(-1))
    assert abs(np.dot(wg.host, wt.reshape(-1)) - inner) < 1e-9 * max(1.0, abs(inner))
    assert abs(np.dot(ig.host, x.reshape(-1)) - inner) < 1e-9 * max(1.0, abs(inner))
    # finite differences pin the gradients element by element, not just their projections
    eps = 1e-6
    for idx in (0, x.size // 2, x.size - 1):
        bumped = x.reshape(-1).copy(); bumped[idx] += eps
        o2, w2 = hbuf(np.zeros(out.host.size)), hbuf(np.zeros(work.host.size))
        H.convolution(ORACLE, "forward", V(o2), 0.0, V(hbuf(bumped)), V(weights), V(w2), *geom)
        assert abs(np.dot(o2.host - out.host, g.reshape(-1)) / eps - ig.host[idx]) < 1e-5


# ------------------------------------------------------------------ local response normalization
# The reference's stored vectors (tests/reference_suite.py lrn_operator) fix k = alpha = beta = 1 and
# n = 1, 2, 3 on three channels.  These pin the other parameters through what the mathematics fixes.

def _lrn(x, dy, n, k, alpha, beta):
    xb, gb = hbuf(x.reshape(-1)), hbuf(dy.reshape(-1))
    yb, db = hbuf(np.zeros(x.size)), hbuf(np.zeros(x.size))
    shape = list(x.shape)
    H.lrn_forward(ORACLE, View(yb, shape), View(xb, shape), n, k, alpha, beta)
    H.lrn_backward(ORACLE, View(db, shape), View(yb, shape), View(xb, shape), View(gb, shape), n, k, alpha, beta)
    return yb.host.reshape(x.shape), db.host.reshape(x.shape)


def test_lrn_window_of_one_is_elementwise():
    """n = 1: y = x (k + alpha x^2)^-beta and its derivative, element by element."""
    rng = np.random.default_rng(71)
    x, dy = rng.standard_normal((2, 5, 3, 4)) * 2, rng.standard_normal((2, 5, 3, 4))
    k, alpha, beta = 1.7, 0.3, 0.75
    y, dx = _lrn(x, dy, 1, k, alpha, beta)
    s = k + alpha * x * x
    np.testing.assert_allclose(y, x * s ** -beta, rtol=1e-14)
    np.testing.assert_allclose(dx, dy * (s ** -beta - 2 * alpha * beta * x * x * s ** (-beta - 1)), rtol=1e-12, atol=1e-15)


def test_lrn_window_wider_than_the_channels_sees_all_of_them():
    """With n >= 2 C - 1 every window, clipped to the channels, is all of them: one scale per pixel,
    k + alpha / n * (sum over all channels of x^2)."""
    rng = np.random.default_rng(72)
    x = rng.standard_normal((3, 4, 2, 5))
    for n in (7, 8, 16):
        y, _ = _lrn(x, np.ones_like(x), n, 2.0, 0.5, 0.6)
        s = 2.0 + 0.5 / n * (x * x).sum(axis=1, keepdims=True)
        np.testing.assert_allclose(y, x * s ** -0.6, rtol=1e-14)


def test_lrn_window_placement_by_impulse_response():
    """One non-zero channel c0: the scales that rise above k are exactly those of the channels whose
    window holds c0, c0 - ahead <= c <= c0 + behind with behind = (n - 1) // 2 (cuDNN's lookBehind) and
    ahead = n - 1 - behind."""
    channels, c0 = 12, 6
    for n in range(1, 9):
        x = np.full((1, channels, 1, 1), 1e-3)
        x[0, c0] = 10.0
        y, _ = _lrn(x, np.ones_like(x), n, 1.0, 1.0, 1.0)
        scale = (x / y).reshape(-1)            # s, since beta = 1
        behind = (n - 1) // 2
        ahead = n - 1 - behind
        raised = {c for c in range(channels) if scale[c] > 2.0}
        assert raised == set(range(c0 - ahead, c0 + behind + 1)), (n, raised)


@pytest.mark.parametrize("n", [1, 3, 5, 7, 15])
def test_lrn_backward_against_central_differences(n):
    """For an odd n the window is centred and the backward pass is the exact derivative of
    sum(dy * forward(x)): checked against central differences in double.  (For an even n the stored
    vectors of the reference fix the unmirrored window, which is not that derivative.)"""
    rng = np.random.default_rng(73 + n)
    shape = (2, 9, 2, 3)
    x, dy = rng.standard_normal(shape), rng.standard_normal(shape)
    k, alpha, beta = 1.3, 0.8, 0.75
    _, dx = _lrn(x, dy, n, k, alpha, beta)
    h = 1e-6
    numeric = np.zeros(shape)
    for idx in np.ndindex(*shape):
        hi, lo = x.copy(), x.copy()
        hi[idx] += h
        lo[idx] -= h
        numeric[idx] = ((dy * _lrn(hi, dy, n, k, alpha, beta)[0]).sum() - (dy * _lrn(lo, dy, n, k, alpha, beta)[0]).sum()) / (2 * h)
    np.testing.assert_allclose(dx, numeric, rtol=2e-6, atol=2e-8)


def test_lrn_rank_three_is_one_image_and_strides_are_honoured():
    rng = np.random.default_rng(74)
    x = rng.standard_normal((6, 3, 4))
    y3, _ = _lrn(x, np.ones_like(x), 3, 1.0, 1.0, 0.5)
    y4, _ = _lrn(x.reshape(1, 6, 3, 4), np.ones((1, 6, 3, 4)), 3, 1.0, 1.0, 0.5)
    assert np.array_equal(y3.reshape(-1), y4.reshape(-1))
    # the same tensor stored channels-last: [b, c, h, w] strides [h w c, 1, w c, c]
    b, c, hh, w = 2, 5, 3, 4
    x = rng.standard_normal((b, c, hh, w))
    want, _ = _lrn(x, np.ones_like(x), 3, 1.0, 1.0, 0.5)
    xb, yb = hbuf(np.ascontiguousarray(x.transpose(0, 2, 3, 1)).reshape(-1)), hbuf(np.zeros(x.size))
    strides = [hh * w * c, 1, w * c, c]
    H.lrn_forward(ORACLE, View(yb, [b, c, hh, w], strides), View(xb, [b, c, hh, w], strides), 3, 1.0, 1.0, 0.5)
    assert np.array_equal(yb.host.reshape(b, hh, w, c).transpose(0, 3, 1, 2), want)
