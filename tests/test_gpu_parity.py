"""Parity of the HIP library with the CPU oracle, call by call through the C
ABI, on identical seeded inputs.  Bar: bit-exact for integer work, for
assign / convert / select / indexing and for the non-transcendental float ops;
<= 2e-6 relative for exp / tanh / logistic and for reductions.  Needs a GPU.
"""
import re

import numpy as np
import pytest

import harness as H
from cortex_amd import capi
from harness import View

pytestmark = pytest.mark.gpu

NP = H.NP_DTYPES
FLOATS = (capi.F32, capi.F64)
TRANSCENDENTAL = ("exp", "tanh", "logistic")
REL_TOL = 2e-6          # float32 transcendentals and reductions
REL_TOL_F64 = 1e-12


@pytest.fixture()
def P(pair_factory):
    with pair_factory() as pair:
        yield pair


def values(rng, code, n, lo=-100, hi=100, nonzero=False):
    if code in FLOATS:
        v = rng.standard_normal(n) * 3.0
        if nonzero:
            v = np.where(np.abs(v) < 0.1, 0.5, v)
        return v.astype(NP[code])
    info = np.iinfo(NP[code])
    lo, hi = max(lo, info.min), min(hi, info.max)
    v = rng.integers(lo, hi + 1, n)
    if nonzero:
        v = np.where(v == 0, 3, v)
    return v.astype(NP[code])


def compare(buf, what, tol=None, denormal_ulps=0):
    """tol: relative bar per element.  denormal_ulps: results below the smallest normal number of
    the type may instead differ by that many units of the denormal grid, where one unit is a
    large relative step."""
    got, want = buf.download(), buf.host
    if tol is None:
        H.assert_bit_exact(got, want, what)
        return
    g, w = got.astype(np.float64), want.astype(np.float64)
    ok = (np.abs(g - w) <= tol * np.abs(w)) | (np.isnan(g) & np.isnan(w)) | (g == w)
    if denormal_ulps:
        info = np.finfo(want.dtype)
        ok |= (np.abs(w) < info.tiny) & (np.abs(g - w) <= denormal_ulps * float(info.smallest_subnormal))
    assert np.all(ok), f"{what}: max rel err {np.nanmax(np.abs(g - w) / np.abs(w))}"


# ------------------------------------------------------------------ access patterns
# Each pattern builds (dest view, input views) over fresh buffers; `kernel` is the
# family the planner must choose for it.

def pat_flat(P, rng, code, n_in):
    n = 1003
    return View(P.buf(np.zeros(n, NP[code])), [n]), [View(P.buf(values(rng, code, n)), [n]) for _ in range(n_in)], "vec"


def pat_flat_misaligned(P, rng, code, n_in):
    n = 517
    d = View(P.buf(np.zeros(n + 8, NP[code])), [n], offset=1)
    return d, [View(P.buf(values(rng, code, n + 8)), [n], offset=3) for _ in range(n_in)], "vec1"


def pat_row_bcast(P, rng, code, n_in):
    r, c = 37, 64
    ins = [View(P.buf(values(rng, code, r * c)), [r, c])] + [View(P.buf(values(rng, code, c)), [c]) for _ in range(n_in - 1)]
    return View(P.buf(np.zeros(r * c, NP[code])), [r, c]), ins, "vec"


def pat_row_bcast_odd(P, rng, code, n_in):
    r, c = 33, 51
    ins = [View(P.buf(values(rng, code, r * c)), [r, c])] + [View(P.buf(values(rng, code, c)), [c]) for _ in range(n_in - 1)]
    return View(P.buf(np.zeros(r * c, NP[code])), [r, c]), ins, "vec1"


def pat_col_bcast(P, rng, code, n_in):
    r, c = 37, 64
    ins = [View(P.buf(values(rng, code, r * c)), [r, c])] + [View(P.buf(values(rng, code, r)), [r, 1]) for _ in range(n_in - 1)]
    return View(P.buf(np.zeros(r * c, NP[code])), [r, c]), ins, "vec"


def pat_channel(P, rng, code, n_in):
    shp = [4, 3, 8, 8]
    n = int(np.prod(shp))
    ins = [View(P.buf(values(rng, code, n)), shp)] + [View(P.buf(values(rng, code, 3)), [3, 1, 1]) for _ in range(n_in - 1)]
    return View(P.buf(np.zeros(n, NP[code])), shp), ins, "vec"


def pat_pitched(P, rng, code, n_in):
    d = View(P.buf(np.zeros(5 * 16 + 8, NP[code])), [5, 7], [16, 1], offset=3)
    return d, [View(P.buf(values(rng, code, 5 * 12 + 4)), [5, 7], [12, 1], offset=2) for _ in range(n_in)], "vec1"


def pat_transposed(P, rng, code, n_in):
    a, b = 70, 130
    ins = [View(P.buf(values(rng, code, a * b)), [b, a]).transpose([1, 0]) for _ in range(n_in)]
    return View(P.buf(np.zeros(a * b, NP[code])), [a, b]), ins, "tile"


def pat_transposed_mixed(P, rng, code, n_in):
    # first input transposed, the others contiguous / row vector
    a, b = 96, 80
    ins = [View(P.buf(values(rng, code, a * b)), [b, a]).transpose([1, 0])]
    if n_in >= 2:
        ins.append(View(P.buf(values(rng, code, a * b)), [a, b]))
    if n_in >= 3:
        ins.append(View(P.buf(values(rng, code, b)), [b]))
    # streams along the destination's rows in the majority: the mirrored tile
    return View(P.buf(np.zeros(a * b, NP[code])), [a, b]), ins, "tile_wide_a" if n_in >= 2 else "tile"


def pat_permuted_3d(P, rng, code, n_in):
    # planar <- interleaved: dest [3,20,24] contiguous, inputs [20,24,3] viewed through transpose [2 0 1]
    ins = [View(P.buf(values(rng, code, 20 * 24 * 3)), [20, 24, 3]).transpose([2, 0, 1]) for _ in range(n_in)]
    return View(P.buf(np.zeros(3 * 20 * 24, NP[code])), [3, 20, 24]), ins, None


def pat_dest_transposed(P, rng, code, n_in):
    a, b = 40, 72
    d = View(P.buf(np.zeros(a * b, NP[code])), [b, a]).transpose([1, 0])
    return d, [View(P.buf(values(rng, code, a * b)), [a, b]) for _ in range(n_in)], "tile"


def pat_strided_vector(P, rng, code, n_in):
    d = View(P.buf(np.zeros(50, NP[code])), [9], [5], offset=2)
    return d, [View(P.buf(values(rng, code, 40)), [9], [4], offset=1) for _ in range(n_in)], "general"


def pat_commensurate(P, rng, code, n_in):
    # [8,6] <- [4,3]: dimensions divide but are neither 1 nor full
    ins = [View(P.buf(values(rng, code, 12)), [4, 3]) for _ in range(n_in)]
    return View(P.buf(np.zeros(48, NP[code])), [8, 6]), ins, "general"


def pat_gather(P, rng, code, n_in):
    idx = P.buf(np.array([1, 2, 1, 0, 2, 1], np.int32))
    ins = [View(P.buf(values(rng, code, 2 * 3 * 3)), [2, 3, 6], [9, 3, 1], index=[None, None, idx]) for _ in range(n_in)]
    return View(P.buf(np.zeros(36, NP[code])), [2, 3, 6]), ins, "general"


def pat_single(P, rng, code, n_in):
    return View(P.buf(np.zeros(1, NP[code])), [1]), [View(P.buf(values(rng, code, 1)), [1]) for _ in range(n_in)], None


PATTERNS = [pat_flat, pat_flat_misaligned, pat_row_bcast, pat_row_bcast_odd, pat_col_bcast, pat_channel, pat_pitched,
            pat_transposed, pat_transposed_mixed, pat_permuted_3d, pat_dest_transposed, pat_strided_vector,
            pat_commensurate, pat_gather, pat_single]


@pytest.mark.parametrize("pattern", PATTERNS, ids=lambda f: f.__name__[4:])
@pytest.mark.parametrize("code", H.ALL_DTYPES)
def test_binary_op_patterns(P, pattern, code):
    rng = np.random.default_rng(1)
    dest, (x, y), kernel = pattern(P, rng, code, 2)
    for op, xa, ya in (("+", 1.0, 1.0), ("+", 1.0, -1.0), ("*", 2.0, 0.5 if code in FLOATS else 3.0), ("max", 1.0, 1.0)):
        k = P.run(H.binary_op, dest, x, xa, y, ya, op)
        compare(dest.buf, f"{pattern.__name__} {op} ({k})")
        if kernel:
            assert k == kernel, (pattern.__name__, k)


@pytest.mark.parametrize("pattern", PATTERNS, ids=lambda f: f.__name__[4:])
@pytest.mark.parametrize("code", [capi.F32, capi.I16, capi.F64])
def test_ternary_and_unary_patterns(P, pattern, code):
    rng = np.random.default_rng(2)
    dest, (x, y, z), kernel = pattern(P, rng, code, 3)
    k = P.run(H.ternary_op, dest, x, 1.0, y, 1.0, z, 1.0)
    compare(dest.buf, f"select {pattern.__name__} ({k})")
    if kernel:
        assert k == kernel
    k = P.run(H.ternary_op, dest, x, -1.0, y, 2.0, z, 3.0)
    compare(dest.buf, f"select alphas {pattern.__name__} ({k})")
    k = P.run(H.unary_op, dest, x, 1.0, "noop")
    compare(dest.buf, f"noop {pattern.__name__} ({k})")
    k = P.run(H.unary_op, dest, y, 1.0, "exp")
    compare(dest.buf, f"exp {pattern.__name__} ({k})", tol=REL_TOL if code == capi.F32 else (REL_TOL_F64 if code == capi.F64 else None))


@pytest.mark.parametrize("pattern", [pat_flat, pat_transposed, pat_pitched, pat_gather, pat_commensurate, pat_channel],
                         ids=lambda f: f.__name__[4:])
@pytest.mark.parametrize("src", H.ALL_DTYPES)
@pytest.mark.parametrize("dst", H.ALL_DTYPES)
def test_assign_all_dtype_pairs(P, pattern, src, dst):
    rng = np.random.default_rng(3)
    dest, (x,), _ = pattern(P, rng, src, 1)
    # swap the destination buffer for one of the destination datatype
    dbuf = P.buf(np.zeros(dest.buf.init.size, NP[dst]))
    dest = View(dbuf, dest.shape, dest.strides, dest.offset)
    # spread the source values over the whole range of its type, specials included
    raw = x.buf.init.copy()
    if src in FLOATS:
        raw = (raw.astype(np.float64) * 1e4).astype(NP[src])
        raw[:8] = np.array([np.nan, np.inf, -np.inf, 3e9, -3e9, 1e19, -1e19, 300.7][:min(8, raw.size)], NP[src])[:raw.size]
    else:
        info = np.iinfo(NP[src])
        raw = rng.integers(info.min, info.max, raw.size, endpoint=True).astype(NP[src])
    x.buf.init[...] = raw
    x.buf.reset()
    k = P.run(H.assign, dest, x)
    compare(dbuf, f"assign {src}->{dst} {pattern.__name__} ({k})")


@pytest.mark.parametrize("code", H.ALL_DTYPES)
@pytest.mark.parametrize("op", list(capi.UNARY_OPS))
def test_unary_ops_all_dtypes(P, code, op):
    rng = np.random.default_rng(4)
    n = 777
    x = values(rng, code, n, lo=-60, hi=60)
    if code in FLOATS:
        x[:12] = np.array([0.0, -0.0, 0.5, 1.5, 2.5, -0.5, -1.5, 0.49999997, np.nan, np.inf, -np.inf, 88.0], NP[code])
    xb, db = P.buf(x), P.buf(np.zeros(n, NP[code]))
    tol = None
    if op in TRANSCENDENTAL:
        # integer tensors evaluate these in double too; a long result above 2^53 shows the
        # last-ulp difference between the device's and the host's exp
        tol = REL_TOL if code == capi.F32 else REL_TOL_F64
    for alpha in (1.0, -1.0, 0.37 if code in FLOATS else 2.0):
        k = P.run(H.unary_op, View(db, [n]), View(xb, [n]), alpha, op)
        compare(db, f"{op} alpha {alpha} ({k})", tol=tol)
    # in place (unary-accum!)
    k = P.run(H.unary_accum, View(xb, [n]), 1.0, op)
    compare(xb, f"accum {op} ({k})", tol=tol)


def test_reduce_view_with_chained_kept_axes_stays_on_the_column_kernel(P):
    """[channels, 7, 7, batch] with the batch axis slowest in memory: the three kept axes chain into one."""
    rng = np.random.default_rng(61)
    batch, channels = 64, 24
    x = P.buf((rng.random(batch * channels * 49) + 0.5).astype(np.float32))
    out = P.buf(np.zeros(channels * 49, np.float32))
    k = P.run(H.unary_reduce, View(out, [channels, 7, 7, 1]), 1.0,
              View(x, [channels, 7, 7, batch], [49, 7, 1, channels * 49]), "sum")
    assert k.startswith("reduce_col"), k
    compare(out, f"sum over the batch axis ({k})", tol=REL_TOL)


@pytest.mark.parametrize("code", H.ALL_DTYPES)
def test_reduce_short_ragged_rows(P, code):
    """Dense rows of ten (seven, thirty-one ...) elements, no whole number of vectors: staged through LDS,
    one lane per row, accumulated first element to last as the reference does."""
    rng = np.random.default_rng(62)
    vmax = 16 // NP[code]().itemsize
    for rows, k in ((5000, 10), (1024, 7), (3001, 31), (1500, 3), (2048, 9)):
        if k % vmax == 0 or k * NP[code]().itemsize > 128:
            continue
        x = P.buf(values(rng, code, rows * k, -50, 50))
        if code in FLOATS:
            x.init[5 * k + 1] = np.nan
            x.init[7 * k: 8 * k] = 0.0
            x.init[7 * k + 2] = -0.0
            x = P.buf(x.init)
        out = P.buf(np.zeros(rows, NP[code]))
        for op, alpha in (("sum", 1.0), ("max", 1.0), ("min", 1.0), ("mean", 1.0), ("magnitude", 0.5), ("magnitude-squared", 1.0)):
            kname = P.run(H.unary_reduce, View(out, [rows, 1]), alpha, View(x, [rows, k]), op)
            assert kname == "reduce_short_rows", (kname, rows, k)
            compare(out, f"{op} rows of {k} ({kname})", tol=None if (code not in FLOATS or op in ("max", "min")) else
                    (REL_TOL if code == capi.F32 else REL_TOL_F64))


@pytest.mark.parametrize("code", [capi.I8, capi.U8, capi.I16])
def test_narrow_integer_reductions_at_the_edge_of_32_bits(P, code):
    """Byte and short reductions run on int accumulators while the host can prove that the result stays inside
    32 bits, on long ones otherwise: extreme elements, the largest multipliers, and row lengths on both sides of
    the bound, against the oracle's long arithmetic."""
    dt = NP[code]
    info = np.iinfo(dt)
    rng = np.random.default_rng(63)
    big_alpha = float(info.max)
    # sum: count * |alpha| * max|x| crosses 2^31 between these two row lengths
    per = int(max(abs(info.min), info.max)) * int(info.max)
    edge = (1 << 31) // per
    for k in sorted({max(1, edge - 3), edge + 5, 4096}):
        rows = 3
        x = np.full(rows * k, info.min, dt)
        x[k:2 * k] = info.max
        x[2 * k:] = rng.integers(info.min, int(info.max) + 1, k).astype(dt)
        xb = P.buf(x)
        out = P.buf(np.zeros(rows, dt))
        for op in ("sum", "mean", "max", "min", "magnitude-squared", "magnitude"):
            for alpha in (big_alpha, 1.0, -1.0):
                kname = P.run(H.unary_reduce, View(out, [rows, 1]), alpha, View(xb, [rows, k]), op)
                compare(out, f"{op} alpha {alpha} rows of {k} ({kname})")
        # down the columns of the same data viewed [k, rows]^T is a strided reduce of three rows: skip; a real column case:
    cols, rows = 512, 700
    x = rng.integers(info.min, int(info.max) + 1, rows * cols).astype(dt)
    x[:cols] = info.min
    xb = P.buf(x)
    out = P.buf(np.zeros(cols, dt))
    for op in ("sum", "mean", "max", "min", "magnitude-squared", "magnitude"):
        for alpha in (big_alpha, 1.0):
            kname = P.run(H.unary_reduce, View(out, [cols, 1]), alpha, View(xb, [cols, rows], [1, cols]), op)
            assert kname.startswith("reduce_col"), kname
            compare(out, f"column {op} alpha {alpha} ({kname})")


def test_float_tanh_dense_sweep(P):
    """unary-op! :tanh on float tensors runs a single-precision form of its own: a dense sweep of its
    argument range (the polynomial below 0.4, the seam, the exponential form up to saturation, tiny and
    huge arguments, both signs) against the oracle's double tanh rounded to float, to the 2e-6 relative
    bar of a transcendental and to the 6e-7 the form is built for."""
    pos = np.concatenate([np.linspace(0.0, 0.45, 1 << 21), np.linspace(0.35, 12.0, 1 << 22), np.logspace(-44, -2, 1 << 18),
                          np.logspace(1, 38, 1 << 16),
                          np.array([0.4, np.nextafter(np.float32(0.4), np.float32(0)), 88.0, 1e38, np.inf, 0.0])])
    x = np.concatenate([pos, -pos]).astype(np.float32)
    n = x.size
    xb, db = P.buf(x), P.buf(np.zeros(n, np.float32))
    k = P.run(H.unary_op, View(db, [n]), View(xb, [n]), 1.0, "tanh")
    got, want = db.download().astype(np.float64), db.host.astype(np.float64)
    assert np.array_equal(np.signbit(got), np.signbit(want)), k
    exact = np.tanh(x.astype(np.float64))
    scale = np.maximum(np.abs(exact), np.finfo(np.float32).tiny)  # denormal results: one denormal step is allowed
    rel = np.abs(got - exact) / scale
    worst = int(np.argmax(rel))
    assert rel[worst] <= 6e-7, (float(x[worst]), got[worst], exact[worst], float(rel[worst]))
    assert np.all(np.abs(got - want) <= REL_TOL * np.maximum(np.abs(want), np.finfo(np.float32).tiny))
    nan = P.buf(np.array([np.nan, -np.nan], np.float32))
    P.run(H.unary_op, View(nan, [2]), View(nan, [2]), 1.0, "tanh")
    assert np.all(np.isnan(nan.download()))


@pytest.mark.parametrize("code", [capi.I32, capi.I64])
def test_integer_division_edges(P, code):
    """Integer :/ truncates toward zero and wraps like the JVM's long division followed by the narrowing
    cast: the most negative value over -1 and over 1, operands on both sides of the 32-bit range (longs
    whose operands fit 32 bits divide in 32 bits), inexact quotients of either sign, multipliers that push
    int operands past 32 bits."""
    info = np.iinfo(NP[code])
    edge = [info.min, info.min + 1, info.max, info.max - 1, -(1 << 31), -(1 << 31) - 1, -(1 << 31) + 1, (1 << 31) - 1, 1 << 31,
            (1 << 31) + 1, -7, 7, -1, 1, 100, -100, 3, -3, (1 << 40) + 5, -(1 << 40) - 5]
    edge = [v for v in edge if info.min <= v <= info.max]
    divisors = [-1, 1, 2, -2, 3, -3, 7, -7, 1 << 16, -(1 << 16), (1 << 31) - 1, -(1 << 31), info.max, info.min]
    divisors = [v for v in divisors if info.min <= v <= info.max]
    xs = np.array([a for a in edge for _ in divisors], dtype=NP[code])
    ys = np.array([d for _ in edge for d in divisors], dtype=NP[code])
    n = xs.size
    xb, yb = P.buf(xs), P.buf(ys)
    for xa, ya in ((1.0, 1.0), (-1.0, 1.0), (3.0, 1.0), (65536.0, -3.0)):
        out = P.buf(np.zeros(n, NP[code]))
        P.run(H.binary_op, View(out, [n]), View(xb, [n]), xa, View(yb, [n]), ya, "/")
        H.assert_bit_exact(out.download(), out.host, f"integer / with alphas {xa}, {ya}")


def test_double_tanh_dense_sweep(P):
    """unary-op! :tanh on double tensors is 1 - 2 / (exp(2|x|) + 1) from 0.05 on and an odd polynomial
    below: a dense sweep of both pieces, the seam, tiny and huge arguments and both signs against the
    oracle's library tanh, to 1e-14 of the result (the transcendental bar for doubles is 1e-12)."""
    pos = np.concatenate([np.linspace(0.0, 0.07, 1 << 20), np.linspace(0.04, 25.0, 1 << 21), np.logspace(-300, -2, 1 << 16),
                          np.logspace(1.3, 300, 1 << 14),
                          np.array([0.05, np.nextafter(0.05, 0.0), np.nextafter(0.05, 1.0), 19.0, 19.06, 19.07, 20.0, 354.0,
                                    355.0, 710.0, np.inf, 0.0])])
    x = np.concatenate([pos, -pos])
    n = x.size
    xb, db = P.buf(x), P.buf(np.zeros(n, np.float64))
    P.run(H.unary_op, View(db, [n]), View(xb, [n]), 1.0, "tanh")
    got, want = db.download(), db.host
    assert np.array_equal(np.signbit(got), np.signbit(want))
    rel = np.abs(got - want) / np.maximum(np.abs(want), np.finfo(np.float64).tiny)
    worst = int(np.argmax(rel))
    assert rel[worst] <= 1e-14, (float(x[worst]), got[worst], want[worst], float(rel[worst]))
    nan = P.buf(np.array([np.nan, -np.nan]))
    P.run(H.unary_op, View(nan, [2]), View(nan, [2]), 1.0, "tanh")
    assert np.all(np.isnan(nan.download()))


@pytest.mark.parametrize("code", [capi.I8, capi.I16, capi.I32, capi.I64])
def test_integer_tanh_truncates_like_the_reference(P, code):
    """On integer tensors tanh(x * alpha) is truncated to the tensor's type: 0 until the double result
    is exactly +-1, which happens between |x * alpha| = 19 and 20.  Every value from -128 to 127 under
    multipliers 1, -1 and 3, bit for bit."""
    x = np.arange(-128, 128).astype(NP[code])
    for alpha in (1.0, -1.0, 3.0):
        xb, db = P.buf(x), P.buf(np.zeros(x.size, NP[code]))
        P.run(H.unary_op, View(db, [x.size]), View(xb, [x.size]), alpha, "tanh")
        H.assert_bit_exact(db.download(), db.host, f"integer tanh alpha {alpha}")
        assert set(np.unique(db.host).tolist()) <= {-1, 0, 1}


@pytest.mark.parametrize("code", H.ALL_DTYPES)
@pytest.mark.parametrize("op", list(capi.BINARY_OPS))
def test_binary_ops_all_dtypes(P, code, op):
    rng = np.random.default_rng(5)
    n = 640
    # every form below divides by x or by y somewhere, so both stay away from zero for :/
    x = values(rng, code, n, nonzero=(op == "/"))
    y = values(rng, code, n, nonzero=(op == "/"))
    if code in FLOATS:
        sp = np.array([0.0, -0.0, np.nan, np.inf, -np.inf, 1.0, -1.0, 1e30], NP[code])
        x[:8], y[:8] = sp, sp[::-1]
        x[8:16], y[8:16] = sp, sp
    xb, yb, db = P.buf(x), P.buf(y), P.buf(np.zeros(n, NP[code]))
    V = lambda b: View(b, [n])
    for xa, ya in ((1.0, 1.0), (1.0, -1.0), (2.0, 3.0)):
        k = P.run(H.binary_op, V(db), V(xb), xa, V(yb), ya, op)
        compare(db, f"binary {op} {xa},{ya} ({k})")
    scalar = 3.0
    for rev in (False, True):
        k = P.run(H.binary_op_constant, V(db), V(xb), 2.0, scalar, op, reverse=rev)
        compare(db, f"binary-constant {op} rev={rev} ({k})")
    # accumulate forms (dest is an operand)
    acc = P.buf(y)
    for rev in (False, True):
        k = P.run(H.binary_accum, V(acc), 1.0, V(xb), 1.0, op, reverse=rev, requires_cas=False)
        compare(acc, f"binary-accum {op} rev={rev} ({k})")
        acc.reset()
        k = P.run(H.binary_accum_constant, V(acc), 1.0, scalar, op, reverse=rev)
        compare(acc, f"binary-accum-constant {op} rev={rev} ({k})")
        acc.reset()


@pytest.mark.parametrize("code", H.ALL_DTYPES)
def test_ternary_constant_variants(P, code):
    rng = np.random.default_rng(6)
    n = 300
    a, b = P.buf(values(rng, code, n, -5, 5)), P.buf(values(rng, code, n, -5, 5))
    d = P.buf(np.zeros(n, NP[code]))
    V = lambda t: View(t, [n])
    import itertools
    for arg_idx in itertools.permutations([0, 1, 2]):
        k = P.run(H.ternary_op_constant, V(d), V(a), 1.0, V(b), 2.0, -1.5, list(arg_idx))
        compare(d, f"ternary-constant {arg_idx} ({k})")
        k = P.run(H.ternary_op_constant_constant, V(d), V(a), -1.0, 2.5, -3.0, list(arg_idx))
        compare(d, f"ternary-constant-constant {arg_idx} ({k})")


def test_select_compares_unrounded_products_and_casts_constants_first(P):
    x = np.array([1.0, -1.0, 0.0, -0.0, np.nan, 1e-30, -1e-30], np.float32)
    xb, yb, zb = P.buf(x), P.buf(np.full(7, 10.0, np.float32)), P.buf(np.full(7, 20.0, np.float32))
    d = P.buf(np.zeros(7, np.float32))
    V = lambda t: View(t, [7])
    P.run(H.ternary_op, V(d), V(xb), 1e-30, V(yb), 1.0, V(zb), 1.0)
    compare(d, "three tensors")
    assert d.host.tolist() == [20.0, 10.0, 20.0, 20.0, 10.0, 20.0, 10.0]
    P.run(H.ternary_op_constant, V(d), V(xb), 1e-30, V(yb), 1.0, 20.0, [0, 1, 2])
    compare(d, "two tensors and a constant")
    assert d.host.tolist() == [20.0, 10.0, 20.0, 20.0, 10.0, 20.0, 20.0]


@pytest.mark.parametrize("code", H.ALL_DTYPES)
def test_assign_constant_and_memset(P, code):
    n = 1000
    d = P.buf(np.zeros(n + 5, NP[code]))
    for value in (0.0, 7.0, -3.9, 300.7):
        P.run(H.memset, View(d, [n], offset=5), value, n)
        compare(d, f"memset {value}")
    s = P.buf(np.zeros(64, NP[code]))
    # a column of a [8,8] matrix (non dense): assign-constant!
    k = P.run(H.assign_constant, View(s, [8], [8], offset=3), 5.0)
    compare(s, f"assign-constant column ({k})")
    k = P.run(H.assign_constant, View(s, [4, 3], [8, 1], offset=9), -2.0)
    compare(s, f"assign-constant submatrix ({k})")


# ------------------------------------------------------------------ accumulate into a broadcast / indexed destination

@pytest.mark.parametrize("code", [capi.F32, capi.F64, capi.I32, capi.I64, capi.I8])
def test_binary_accum_broadcast_destination_is_serial_exact(P, code):
    rng = np.random.default_rng(7)
    for dshape, yshape in (([5, 1, 1], [3, 5, 4, 4]), ([7], [6, 7]), ([6, 1], [6, 9]), ([1], [50])):
        ny = int(np.prod(yshape))
        y = P.buf(values(rng, code, ny, -9, 9, nonzero=True))
        d = P.buf(values(rng, code, int(np.prod(dshape)), -9, 9))
        for op, da, ya, rev in (("+", 1.0, 1.0, False), ("+", 1.0, 2.0, True), ("-", 1.0, 1.0, True), ("max", 1.0, 1.0, False),
                                ("*", 1.0, 1.0, False) if code in FLOATS else ("bit-xor", 1.0, 1.0, False)):
            k = P.run(H.binary_accum, View(d, dshape), da, View(y, yshape), ya, op, reverse=rev, requires_cas=True)
            compare(d, f"accum {op} {dshape}<-{yshape} ({k})")
            assert k == "accum_owner", k
            d.reset()


def test_binary_accum_large_sum_uses_double_accumulation(P):
    # bias gradient: dest [C,1,1] += y [N,C,H,W]; the reference tolerates 1e-4 here
    rng = np.random.default_rng(8)
    n, c, hw = 16, 6, 32 * 32
    y = P.buf(rng.random(n * c * hw).astype(np.float32))
    d = P.buf(np.zeros(c, np.float32))
    k = P.run(H.binary_accum, View(d, [c, 1, 1]), 1.0, View(y, [n, c, 32, 32]), 1.0, "+", requires_cas=True)
    assert k == "accum_staged_sum"
    exact = y.init.astype(np.float64).reshape(n, c, hw).sum(axis=(0, 2))
    got = d.download().astype(np.float64)
    assert np.all(np.abs(got - exact) <= 1e-6 * exact)              # ours: sums formed in double
    assert np.all(np.abs(d.host - exact) <= 1e-4 * exact)           # the serial float sum drifts


# (dest shape, dest strides, y shape, y strides): every layout takes the staged-sum route
STAGED_LAYOUTS = [
    ([96], None, [400, 96], None),                       # sum the rows into a vector
    ([300, 1], None, [300, 130], None),                  # sum each row
    ([6, 1, 1], None, [8, 6, 24, 24], None),             # per-channel bias gradient: two passes
    ([1], None, [40000], None),                          # everything into one element
    ([50], [3], [700, 50], [64, 1]),                     # strided destination, padded rows
    ([33, 1], None, [33, 900], [1, 33]),                 # y is a transposed view
    ([4, 1, 5], None, [4, 1000, 5], None),               # reduced axis in the middle
    ([500, 40], [0, 1], [500, 40], None),                # a destination axis of stride 0 is a broadcast axis
    ([12, 1, 1], None, [40, 12, 7, 7], None),            # short innermost group: the batch axis is reduced first
]


@pytest.mark.parametrize("code", [capi.F32, capi.F64, capi.I32, capi.I64, capi.I16, capi.I8, capi.U8])
def test_binary_accum_staged_sum(P, code):
    rng = np.random.default_rng(81)
    for dshape, dstrides, yshape, ystrides in STAGED_LAYOUTS:
        y_elems = 1 + sum((s - 1) * st for s, st in zip(yshape, ystrides)) if ystrides else int(np.prod(yshape))
        d_elems = 1 + sum((s - 1) * st for s, st in zip(dshape, dstrides)) if dstrides else int(np.prod(dshape))
        if code in FLOATS:
            yv, dv = (rng.random(y_elems) + 0.5).astype(NP[code]), rng.random(d_elems).astype(NP[code])
        else:
            yv, dv = values(rng, code, y_elems, -100, 100), values(rng, code, d_elems, -100, 100)
        y, d = P.buf(yv), P.buf(dv)
        for ya, rev in ((1.0, False), (3.0, True)):
            k = P.run(H.binary_accum, View(d, dshape, dstrides), 1.0, View(y, yshape, ystrides), ya, "+", reverse=rev,
                      requires_cas=True)
            assert k == "accum_staged_sum", (k, dshape, yshape)
            what = f"staged accum {dshape}<-{yshape} ya={ya}"
            if code in FLOATS:
                compare(d, what, tol=1e-4 if code == capi.F32 else 1e-12)
            else:
                compare(d, what)                              # integer sums wrap identically
            if code == capi.F32:
                # The bar above is the reference's own (verify/tensor.clj:189-191): its serial float chain drifts.
                # What the kernel stores is pinned against the sum itself: the same call on double copies of the
                # operands through the oracle (a serial double chain, good to 1e-13 here).  The kernel leaves what
                # unary-reduce! :sum passes followed by binary-op! :+ would: sums formed in double, rounded to float
                # once per pass (at most two) and once more by the add; all terms are positive here, so three
                # half units in the last place bound it.
                y64, d64 = P.buf(yv.astype(np.float64)), P.buf(dv.astype(np.float64))
                H.binary_accum(H.ORACLE, View(d64, dshape, dstrides), 1.0, View(y64, yshape, ystrides), ya, "+", reverse=rev,
                               requires_cas=True)
                got = d.download().astype(np.float64)
                assert np.all(np.abs(got - d64.host) <= 1.8e-7 * np.abs(d64.host)), what
            d.reset()


@pytest.mark.parametrize("code", [capi.F32, capi.F64, capi.I32, capi.I64, capi.I8])
@pytest.mark.parametrize("op", ["max", "min"])
def test_binary_accum_staged_max_min(P, code, op):
    """:max / :min into a broadcast destination: the updates are reduced first and one step per
    destination element follows; elements whose reduction is a NaN or a zero walk their updates
    serially, because there the order decides (a NaN restarts or freezes the chain, +0 ties -0).
    Bit-exact against the serial loop either way."""
    rng = np.random.default_rng(82)
    for dshape, dstrides, yshape, ystrides in STAGED_LAYOUTS:
        y_elems = 1 + sum((s - 1) * st for s, st in zip(yshape, ystrides)) if ystrides else int(np.prod(yshape))
        d_elems = 1 + sum((s - 1) * st for s, st in zip(dshape, dstrides)) if dstrides else int(np.prod(dshape))
        yv, dv = values(rng, code, y_elems, -100, 100), values(rng, code, d_elems, -100, 100)
        if code in FLOATS:
            # hazards: NaNs in y and in the destination, destinations whose extreme is a zero of either sign
            yv[rng.integers(0, y_elems, max(1, y_elems // 5000))] = np.nan
            dv[::7] = np.nan
            zero_cols = np.zeros(y_elems, bool)
            zero_cols[rng.integers(0, y_elems, y_elems // 3)] = True
            sign = -1.0 if op == "max" else 1.0
            yv = np.where(zero_cols, np.where(rng.random(y_elems) < 0.5, 0.0, -0.0), sign * np.abs(yv)).astype(NP[code])
            yv[rng.integers(0, y_elems, y_elems // 2)] = (rng.standard_normal(y_elems // 2) * 3).astype(NP[code])
            dv[1::5] = -0.0
        y, d = P.buf(yv), P.buf(dv)
        alphas = ((1.0, False), (1.0, True), (0.5, False), (-2.0, True)) if code in FLOATS else ((1.0, False), (1.0, True))
        for ya, rev in alphas:
            k = P.run(H.binary_accum, View(d, dshape, dstrides), 1.0, View(y, yshape, ystrides), ya, op, reverse=rev,
                      requires_cas=True)
            assert k == "accum_staged_extreme", (k, dshape, yshape)
            compare(d, f"staged {op} {dshape}<-{yshape} ya={ya} reverse={rev}")
            d.reset()
        if code not in FLOATS:
            # a multiplier on integer updates keeps the serial chain: narrowing after every step does not
            # commute with max / min
            k = P.run(H.binary_accum, View(d, dshape, dstrides), 1.0, View(y, yshape, ystrides), 3.0, op, requires_cas=True)
            assert k == "accum_owner" or k.startswith("accum_stream"), k
            compare(d, f"owner {op} {dshape}<-{yshape} ya=3")
        k = P.run(H.binary_accum, View(d, dshape, dstrides), 2.0, View(y, yshape, ystrides), 1.0, op, requires_cas=True)
        assert k == "accum_owner" or k.startswith("accum_stream"), k
        compare(d, f"owner {op} {dshape}<-{yshape} dest_alpha=2")


@pytest.mark.parametrize("code", [capi.F32, capi.I32, capi.F64, capi.I16])
def test_scatter_add_through_duplicate_indexes(P, code):
    # center-loss use case (src/cortex/verify/tensor.clj:1162-1174)
    mat = P.buf(np.tile(np.arange(9), 2).astype(NP[code]))
    idx = P.buf(np.array([0, 1, 0, 2, 1], np.int32))
    centers = View(mat, [5, 3], [3, 1], index=[idx, None])
    batch = P.buf(np.zeros(15, NP[code]))
    P.run(H.assign, View(batch, [5, 3]), centers)
    compare(batch, "gather")
    assert batch.host.tolist() == [0, 1, 2, 3, 4, 5, 0, 1, 2, 6, 7, 8, 3, 4, 5]
    k = P.run(H.binary_accum, centers, 1.0, View(batch, [5, 3]), 1.0, "+", reverse=True, requires_cas=True)
    compare(mat, f"scatter-add ({k})")
    assert k == "accum_grouped"
    assert mat.host[:9].tolist() == [0, 3, 6, 9, 12, 15, 12, 14, 16]


@pytest.mark.parametrize("code", [capi.F32, capi.I32])
def test_indirect_dimension_of_one_element(P, code):
    """An index tensor of a single element still selects its row (a dimension of extent 1 is
    otherwise skipped by the address functions)."""
    table = P.buf(np.arange(12).astype(NP[code]))
    idx = P.buf(np.array([2], np.int32))
    row = View(table, [1, 4], [4, 1], index=[idx, None])
    got = P.buf(np.zeros(4, NP[code]))
    P.run(H.assign, View(got, [1, 4]), row)
    compare(got, "gather of one row")
    assert got.host.tolist() == [8, 9, 10, 11]
    P.run(H.binary_op, row, View(got, [1, 4]), 1.0, View(got, [1, 4]), 1.0, "+")      # scatter back twice the row
    compare(table, "scatter into one row")
    assert table.host.tolist() == [0, 1, 2, 3, 4, 5, 6, 7, 16, 18, 20, 22]
    P.run(H.binary_accum, row, 1.0, View(got, [1, 4]), 1.0, "+", reverse=True, requires_cas=True)
    compare(table, "scatter-add into one row")
    # broadcast over a batch: the one selected row against three rows
    out = P.buf(np.zeros(12, NP[code]))
    P.run(H.binary_op, View(out, [3, 4]), View(table, [3, 4]), 1.0, row, 1.0, "+")
    compare(out, "one indexed row broadcast over three")


# ------------------------------------------------------------------ reductions

def reduce_scale(x64, axis, op, alpha):
    v = np.abs(x64 * alpha)
    if op in ("magnitude-squared",):
        return (v * v).sum(axis=axis)
    return v.sum(axis=axis) if op in ("sum", "mean", "magnitude") else v.max(axis=axis)


@pytest.mark.parametrize("code", H.ALL_DTYPES)
@pytest.mark.parametrize("shape", [(5, 10), (33, 64), (17, 257), (9, 2048), (300, 16), (2, 3, 40), (3, 40000), (1, 100003),
                                   (40, 4), (1000, 8), (21, 32), (19, 100), (13, 200), (11, 500), (7, 1000)],
                         ids=str)
def test_reduce_last_axis_and_transposed(P, code, shape):
    rng = np.random.default_rng(9)
    n = int(np.prod(shape))
    x = values(rng, code, n, -11, 11)
    xb = P.buf(x)
    lead = int(np.prod(shape[:-1]))
    for alpha in (1.0, 2.0):
        for op in capi.REDUCE_OPS:
            out = P.buf(np.zeros(lead, NP[code]))
            k = P.run(H.unary_reduce, View(out, list(shape[:-1]) + [1]), alpha, View(xb, list(shape)), op)
            check_reduce(out, x.reshape(lead, shape[-1]).astype(np.float64), 1, op, alpha, code, f"rows {shape} ({k})")
            if len(shape) == 2:  # the other axis, through a transposed view
                out2 = P.buf(np.zeros(shape[1], NP[code]))
                k = P.run(H.unary_reduce, View(out2, [shape[1], 1]), alpha, View(xb, list(shape)).transpose([1, 0]), op)
                check_reduce(out2, x.reshape(shape).astype(np.float64), 0, op, alpha, code, f"cols {shape} ({k})")


def check_reduce(out, x64, axis, op, alpha, code, what):
    if code not in FLOATS:
        compare(out, what)            # integer reductions are exact in any order
        return
    got, want = out.download().astype(np.float64), out.host.astype(np.float64)
    if op in ("max", "min"):
        H.assert_bit_exact(out.download(), out.host, what)
        return
    # relative to the sum of magnitudes: a sum of N(0,1) values can land anywhere near zero
    scale = reduce_scale(x64, axis, op, alpha)
    if op == "mean":
        scale = scale / x64.shape[axis]
    if op == "magnitude":
        scale = np.sqrt(reduce_scale(x64, axis, "magnitude-squared", alpha))
    tol = REL_TOL if code == capi.F32 else REL_TOL_F64
    assert np.all(np.abs(got - want) <= tol * scale + 0.0), (what, np.max(np.abs(got - want) / scale))


def test_reduce_kernel_selection(P):
    rng = np.random.default_rng(10)
    x = P.buf(rng.standard_normal(64 * 4096).astype(np.float32))
    out = P.buf(np.zeros(4096, np.float32))
    wide = P.buf(rng.standard_normal(2048 * 8192).astype(np.float32))
    assert P.run(H.unary_reduce, View(out, [2048, 1]), 1.0, View(wide, [2048, 8192]), "sum") == "reduce_row512_vec"
    compare(out, "rows of 32 KiB", tol=2e-6)
    assert P.run(H.unary_reduce, View(out, [64, 1]), 1.0, View(x, [64, 4096]), "sum") == "reduce_row256_vec"
    compare(out, "rows of 16 KiB, a small tensor", tol=2e-6)
    assert P.run(H.unary_reduce, View(out, [128, 1]), 1.0, View(x, [128, 2048]), "sum") == "reduce_row256_vec"
    compare(out, "rows of 8 KiB", tol=2e-6)
    assert P.run(H.unary_reduce, View(out, [1024, 1]), 1.0, View(x, [1024, 256]), "sum") == "reduce_row_small_vec"
    assert P.run(H.unary_reduce, View(out, [4096, 1]), 1.0, View(x, [4096, 63]), "sum") == "reduce_row_small"
    compare(out, "unaligned short rows", tol=2e-6)
    assert P.run(H.unary_reduce, View(out, [4096, 1]), 1.0, View(x, [64, 4096]).transpose([1, 0]), "sum") == "reduce_col_vec"
    idx = P.buf(np.arange(63, -1, -1).astype(np.int32))
    k = P.run(H.unary_reduce, View(out, [64, 1]), 1.0, View(x, [64, 64], [4096, 1], index=[idx, None]), "max")
    assert k == "reduce_any"
    compare(out, "indexed reduce")


@pytest.mark.parametrize("code", [capi.F32, capi.F64, capi.I8, capi.I32])
@pytest.mark.parametrize("rows,cols", [(16, 1 << 20), (1, 1 << 20), (128, 300000), (7, 262147), (129, 300000)], ids=str)
def test_few_rows_under_many_columns(P, code, rows, cols):
    """Column reductions of few rows ([16, 2^20] summed over the 16): a lane owns its columns and
    walks the rows in the reference's order (no segments, no second launch) up to 128 rows; column
    counts off the vector grid, one row, and one row more than the kernel takes."""
    rng = np.random.default_rng(12)
    x = values(rng, code, rows * cols, -9, 9)
    xb = P.buf(x)
    for op in ("sum", "max", "magnitude-squared", "mean"):
        out = P.buf(np.zeros(cols, NP[code]))
        k = P.run(H.unary_reduce, View(out, [cols, 1]), 1.0, View(xb, [rows, cols]).transpose([1, 0]), op)
        check_reduce(out, x.reshape(rows, cols).astype(np.float64), 0, op, 1.0, code, f"thin cols {(rows, cols)} {op} ({k})")
        vmax = 16 // x.itemsize
        vec = vmax if cols % vmax == 0 else 1
        if rows == 1:
            pass                                              # nothing to reduce: the planner sees rows of one element
        elif rows <= 128 and -(-cols // (256 * vec)) >= 1024:   # columns enough for four blocks per compute unit
            assert k == ("reduce_col_thin_vec" if vec > 1 else "reduce_col_thin"), k
        else:
            assert k.startswith("reduce_col") and "thin" not in k, k
    # kept axes on both sides of the reduced one: [3, 5, 400000] summed over the 5
    if code == capi.F32:
        b3 = P.buf(values(rng, code, 3 * 5 * 400000, -9, 9))
        out = P.buf(np.zeros(3 * 400000, NP[code]))
        k = P.run(H.unary_reduce, View(out, [3, 400000, 1]), 1.0, View(b3, [3, 5, 400000]).transpose([0, 2, 1]), "sum")
        assert k == "reduce_col_thin_vec", k
        check_reduce(out, np.moveaxis(b3.init.reshape(3, 5, 400000).astype(np.float64), 1, 2).reshape(3 * 400000, 5), 1, "sum",
                     1.0, code, "thin cols with an outer kept axis")
        # the unit-stride kept axis first in the output's order: [400000, 3] results from a [3, 5, 400000] buffer
        out = P.buf(np.zeros(3 * 400000, NP[code]))
        k = P.run(H.unary_reduce, View(out, [400000, 3, 1]), 1.0, View(b3, [3, 5, 400000]).transpose([2, 0, 1]), "max")
        assert k == "reduce_col_thin_vec", k
        check_reduce(out, np.transpose(b3.init.reshape(3, 5, 400000), (2, 0, 1)).reshape(400000 * 3, 5).astype(np.float64), 1,
                     "max", 1.0, code, "thin cols, unit axis first in the output")


@pytest.mark.parametrize("code", FLOATS)
def test_extremes_of_a_large_tensor_under_a_multiplier(P, code):
    """:max / :min with a multiplier other than 1 on 64 MiB and more: the multiplier-free kernel runs on
    the raw values (the opposite extreme for a negative multiplier) and its results are multiplied, which
    must leave the reference's bits: rows with NaN, infinities of both signs, zeros of both signs, a row
    whose extreme overflows the type once multiplied."""
    rng = np.random.default_rng(14)
    rows, cols = 4096, 4096 if code == capi.F32 else 2048
    x = rng.standard_normal((rows, cols)).astype(NP[code])
    x[0, 100] = np.nan
    x[1, 7], x[2, 9] = np.inf, -np.inf
    x[3, :] = 0.0
    x[3, ::3] = -0.0
    x[4, :] = -0.0
    x[5, 11] = np.finfo(NP[code]).max
    x[6, 13] = -np.finfo(NP[code]).max
    xb = P.buf(x)
    for alpha in (0.5, -2.0, 3.0, -1.0):
        for op in ("max", "min"):
            out = P.buf(np.zeros(rows, NP[code]))
            P.run(H.unary_reduce, View(out, [rows, 1]), alpha, View(xb, [rows, cols]), op)
            with np.errstate(all="ignore"):
                H.assert_bit_exact(out.download(), out.host, f"{op} of rows under {alpha}")
            out2 = P.buf(np.zeros(cols, NP[code]))
            P.run(H.unary_reduce, View(out2, [cols, 1]), alpha, View(xb, [rows, cols]).transpose([1, 0]), op)
            H.assert_bit_exact(out2.download(), out2.host, f"{op} of columns under {alpha}")


def test_reduce_nan_propagates_and_signed_zero(P):
    x = np.zeros((4, 512), np.float32)
    x[0, 100] = np.nan
    x[1, :] = -0.0
    x[2, ::2] = -0.0
    x[3, :] = -1.0
    xb, out = P.buf(x), P.buf(np.zeros(4, np.float32))
    for op in ("max", "min"):
        P.run(H.unary_reduce, View(out, [4, 1]), 1.0, View(xb, [4, 512]), op)
        H.assert_bit_exact(out.download(), out.host, op)
        out2 = P.buf(np.zeros(512, np.float32))
        P.run(H.unary_reduce, View(out2, [512, 1]), 1.0, View(xb, [4, 512]).transpose([1, 0]), op)
        H.assert_bit_exact(out2.download(), out2.host, op + " columns")


# ------------------------------------------------------------------ optimizers

@pytest.mark.parametrize("code", FLOATS)
@pytest.mark.parametrize("n,offsets", [(1, (0, 0)), (4099, (0, 0)), (1000, (4, 4)), (1001, (1, 3)), (65536 + 7, (2, 2))])
def test_adam_and_adadelta_bit_exact(P, code, n, offsets):
    rng = np.random.default_rng(12)
    dt = NP[code]
    p = P.buf(rng.uniform(-0.05, 0.05, n).astype(dt))
    g = P.buf((rng.standard_normal(n) * 1e-3).astype(dt))
    # m and v live at an element offset inside a larger flat state buffer
    m = P.buf((rng.standard_normal(n + 8) * 1e-4).astype(dt))
    v = P.buf((rng.random(n + 8) * 1e-6).astype(dt))
    Vm, Vv = View(m, [n], offset=offsets[0]), View(v, [n], offset=offsets[1])
    pb1 = pb2 = 1.0
    for step in range(3):
        pb1, pb2 = pb1 * 0.9, pb2 * 0.999
        k = P.run(H.adam_step, 1e-3, 0.9, 0.999, 1e-8, pb1, pb2, 0.5, View(g, [n]), View(p, [n]), Vm, Vv, n)
        for name, b in (("params", p), ("m", m), ("v", v)):
            compare(b, f"adam {name} step {step} ({k})")
    for step in range(3):
        k = P.run(H.adadelta_step, 0.05, 1e-6, Vm, Vv, 0.7, View(g, [n]), View(p, [n]), n)
        for name, b in (("params", p), ("grad-accum", m), ("dx-accum", v)):
            compare(b, f"adadelta {name} step {step} ({k})")


# ------------------------------------------------------------------ errors

def test_invalid_arguments_are_reported(P):
    import ctypes as C
    d = P.buf(np.zeros(4, np.float32))
    dims = capi.make_dims([4], [1])
    with pytest.raises(capi.CortexHipError, match="unknown datatype"):
        capi.call("ct_assign_constant", None, d.dev, C.byref(dims), 42, 1.0, 4)
    with pytest.raises(capi.CortexHipError, match="unknown unary"):
        capi.call("ct_unary_op", None, d.dev, C.byref(dims), d.dev, C.byref(dims), 1.0, 99, capi.F32, 4)
    with pytest.raises(capi.CortexHipError, match="unknown binary"):
        capi.call("ct_binary_op", None, d.dev, C.byref(dims), d.dev, C.byref(dims), 1.0, d.dev, C.byref(dims), 1.0, 4, 77, capi.F32)
    with pytest.raises(capi.CortexHipError, match="null"):
        capi.call("ct_binary_op", None, d.dev, C.byref(dims), None, C.byref(dims), 1.0, d.dev, C.byref(dims), 1.0, 4, 0, capi.F32)
    bad = capi.CtDims()
    bad.ndim = 9
    with pytest.raises(capi.CortexHipError, match="rank"):
        capi.call("ct_assign_constant", None, d.dev, C.byref(bad), capi.F32, 1.0, 4)
    with pytest.raises(capi.CortexHipError, match="float or double"):
        capi.call("ct_adam_step", None, capi.I32, 1e-3, 0.9, 0.999, 1e-8, 0.9, 0.999, 1.0, d.dev, d.dev, d.dev, d.dev, 4)
    with pytest.raises(capi.CortexHipError, match="permutation"):
        capi.call("ct_ternary_op_constant_constant", None, d.dev, C.byref(dims), d.dev, C.byref(dims), 1.0, 1.0, 2.0, 4, 0,
                  capi.arg_idx([0, 0, 1]), capi.F32)
    # empty work is a no-op
    capi.call("ct_assign_constant", None, d.dev, C.byref(dims), capi.F32, 1.0, 0)


def test_streams_and_events(P):
    import ctypes as C
    s = C.c_void_p()
    capi.call("ct_stream_create", C.byref(s))
    d = P.buf(np.zeros(1 << 20, np.float32))
    capi.call("ct_memset", s, d.dev, capi.F32, 2.5, 1 << 20)
    e = C.c_void_p()
    capi.call("ct_event_record", C.byref(e), s)
    capi.call("ct_stream_wait_event", None, e)
    capi.call("ct_event_sync", e)
    assert np.all(d.download() == 2.5)
    capi.call("ct_event_destroy", e)
    capi.call("ct_stream_destroy", s)
    free, total = C.c_size_t(), C.c_size_t()
    capi.call("ct_memory_info", C.byref(free), C.byref(total))
    assert 0 < free.value <= total.value


# ------------------------------------------------------------------ activation-gradient!, softmax

@pytest.mark.parametrize("code", FLOATS)
@pytest.mark.parametrize("op", ["logistic", "tanh", "relu"])
def test_activation_gradient_bit_exact(P, code, op):
    rng = np.random.default_rng(30)
    n = 4099
    o = values(rng, code, n)
    o[:4] = [0.0, -0.0, np.nan, 1.0]
    out, grad = P.buf(o), P.buf(values(rng, code, n))
    ig = P.buf(np.zeros(n, NP[code]))
    k = P.run(H.activation_gradient, View(ig, [n]), View(grad, [n]), View(out, [n]), op, n)
    compare(ig, f"activation-gradient {op} ({k})")
    # in place over the gradient, and with a transposed output view
    P.run(H.activation_gradient, View(grad, [n]), View(grad, [n]), View(out, [n]), op, n)
    compare(grad, f"activation-gradient {op} in place")
    m = 96
    o2, g2, i2 = P.buf(values(rng, code, m * m)), P.buf(values(rng, code, m * m)), P.buf(np.zeros(m * m, NP[code]))
    k = P.run(H.activation_gradient, View(i2, [m, m]), View(g2, [m, m]), View(o2, [m, m]).transpose([1, 0]), op, m * m)
    compare(i2, f"activation-gradient {op} transposed ({k})")


SOFTMAX_SHAPES = [(5, 1), (9, 3), (300, 10), (64, 16), (33, 40), (17, 100), (12, 200), (9, 500), (5, 1000), (3, 3000),
                  (2, 5001), (2, 70000), (3, 9000), (2, 16384), (2, 12292), (1500, 10), (1025, 21), (2048, 9), (1100, 31), (1024, 15)]


@pytest.mark.parametrize("code", FLOATS)
@pytest.mark.parametrize("shape", SOFTMAX_SHAPES, ids=str)
def test_softmax_rows(P, code, shape):
    rng = np.random.default_rng(31)
    rows, k = shape
    x = P.buf((rng.standard_normal(rows * k) * 4).astype(NP[code]))
    out = P.buf(np.zeros(rows * k, NP[code]))
    tol = 2e-6 if code == capi.F32 else 1e-12
    kern = P.run(H.softmax, View(out, [rows, k]), View(x, [rows, k]))
    compare(out, f"softmax {shape} ({kern})", tol=tol)
    if rows >= 1024 and k >= 8 and k * x.init.itemsize <= 128 and k % (16 // x.init.itemsize):
        assert kern == "softmax_short_rows"       # many dense short rows that are no whole number of vectors
    else:
        assert kern == "softmax_lane" if k < 8 else kern in ("softmax_wave", "softmax_wave_vec", "softmax_block", "softmax_block_reg")
    P.run(H.softmax, View(x, [rows, k]), View(x, [rows, k]))     # in place
    compare(x, f"softmax {shape} in place", tol=tol)


# shape [batch, channels, height, width] (or one image), window, k, alpha, beta
LRN_CASES = [((2, 3, 2, 2), 1, 1.0, 1.0, 1.0), ((2, 3, 2, 2), 2, 1.0, 1.0, 1.0), ((2, 3, 2, 2), 3, 1.0, 1.0, 1.0),
             ((3, 96, 8, 8), 5, 2.0, 1e-4, 0.75), ((2, 70, 7, 9), 5, 2.0, 1e-2, 0.75), ((1, 33, 5, 4), 4, 1.0, 0.5, 0.5),
             ((2, 40, 16, 16), 16, 1.5, 0.3, 0.6), ((2, 5, 3, 3), 16, 1.0, 1.0, 1.0), ((4, 64, 1, 1), 9, 1.0, 0.1, 2.0),
             ((37, 12, 12), 6, 1.0, 1.0, 0.75), ((2, 65, 10, 26), 7, 1e-3, 5.0, 0.9), ((1, 1, 4, 4), 3, 2.0, 1.0, 0.75)]


@pytest.mark.parametrize("code", FLOATS)
@pytest.mark.parametrize("case", LRN_CASES, ids=str)
def test_lrn_forward_and_backward(P, code, case):
    """Local response normalization against the oracle: the reference's own small cases, windows of
    every parity up to 16 (wider than the channel count included), channel counts off the 32-channel
    blocks, planes that are and are not whole vectors, one-image rank-3 tensors.  The float kernels
    take the power through the hardware exp2 / log2 and the reciprocal: 4e-6 of the result, relative to
    the larger of the two terms of the gradient; double tensors 1e-12."""
    shape, n, k, alpha, beta = case
    rng = np.random.default_rng(61)
    count = int(np.prod(shape))
    x = P.buf((rng.standard_normal(count) * 3).astype(NP[code]))
    dy = P.buf(rng.standard_normal(count).astype(NP[code]))
    y = P.buf(np.zeros(count, NP[code]))
    dx = P.buf(np.zeros(count, NP[code]))
    tol = 4e-6 if code == capi.F32 else 1e-12
    kern = P.run(H.lrn_forward, View(y, shape), View(x, shape), n, k, alpha, beta)
    plane = int(np.prod(shape[-2:]))
    assert kern == ("lrn_forward_vec" if plane % (16 // x.init.itemsize) == 0 else "lrn_forward")
    compare(y, f"lrn forward {case}", tol=tol)
    y.upload(y.host)   # both sides differentiate the same stored output
    kern = P.run(H.lrn_backward, View(dx, shape), View(y, shape), View(x, shape), View(dy, shape), n, k, alpha, beta)
    assert kern == ("lrn_backward_vec" if plane % (16 // x.init.itemsize) == 0 else "lrn_backward")
    assert_lrn_gradient(dx, x, y, dy, case, tol)


def assert_lrn_gradient(dx, x, y, dy, case, tol):
    """The gradient is a difference of two terms, dy s^-beta and (2 alpha beta / n) x sum(dy y / s):
    the bar is `tol` of the sum of their magnitudes, formed here in double."""
    shape, n, k, alpha, beta = case
    got, want = dx.download().astype(np.float64), dx.host.astype(np.float64)
    xs = x.host.astype(np.float64).reshape((-1,) + tuple(shape[-3:]))
    ys, gs = y.host.astype(np.float64).reshape(xs.shape), dy.host.astype(np.float64).reshape(xs.shape)
    behind = (n - 1) // 2
    ahead = n - 1 - behind
    with np.errstate(over="ignore", invalid="ignore"):
        sq = np.pad(xs * xs, ((0, 0), (behind, ahead), (0, 0), (0, 0)))
        scale = k + alpha / n * sum(sq[:, w:w + xs.shape[1]] for w in range(n))
        ratio = np.pad(np.abs(gs * ys) / scale, ((0, 0), (behind, ahead), (0, 0), (0, 0)))
        cross = sum(ratio[:, w:w + xs.shape[1]] for w in range(n))
        bar = tol * (np.abs(gs) * scale ** -beta + 2 * alpha * beta / n * np.abs(xs) * cross)
    tiny = float(np.finfo(dx.host.dtype).smallest_subnormal)
    worst = np.max(np.abs(got - want) / (bar.reshape(-1) + 2 * tiny))
    assert worst <= 1.0, f"lrn backward {case}: {worst * tol} of the terms' magnitudes"


@pytest.mark.parametrize("code", FLOATS)
def test_lrn_wide_range(P, code):
    """Inputs from 1e-20 to 1e20 in neighbouring channels, a large beta and a tiny k: the scales run
    from 1e-5 to past the float range (where the float kernels leave their hardware exp2 / log2 path
    for the double one), and the window sums must not carry a large neighbour's error into a window
    of small values.  NaN and infinite inputs give what the double evaluation gives.  The backward pass
    is run over twelve orders of magnitude (see below)."""
    rng = np.random.default_rng(63)
    b, c, h, w = 2, 24, 4, 4
    tol = 4e-6 if code == capi.F32 else 1e-12
    mags = 10.0 ** rng.integers(-20, 21, (b, c, 1, 1)).astype(np.float64)
    v = (rng.standard_normal((b, c, h, w)) * mags).astype(NP[code])
    for n, k, alpha, beta in ((5, 1e-5, 1.0, 0.75), (3, 2.0, 1e-4, 3.0), (8, 1.0, 10.0, 0.5)):
        x = P.buf(v.reshape(-1))
        y = P.buf(np.zeros(v.size, NP[code]))
        P.run(H.lrn_forward, View(y, [b, c, h, w]), View(x, [b, c, h, w]), n, k, alpha, beta)
        compare(y, f"lrn forward wide range n {n} beta {beta}", tol=tol, denormal_ulps=2)
    # The backward pass keeps dy y / s of every channel in the tensor's type: for float tensors the
    # range of neighbouring channels is held to twelve orders of magnitude here, so that no such
    # quotient leaves the float range while its product with a neighbour's x still counts.
    mags = 10.0 ** rng.integers(-6, 7, (b, c, 1, 1)).astype(np.float64)
    v = (rng.standard_normal((b, c, h, w)) * mags).astype(NP[code])
    for n, k, alpha, beta in ((5, 1e-5, 1.0, 0.75), (3, 2.0, 1e-4, 3.0), (8, 1.0, 10.0, 0.5)):
        x = P.buf(v.reshape(-1))
        y = P.buf(np.zeros(v.size, NP[code]))
        P.run(H.lrn_forward, View(y, [b, c, h, w]), View(x, [b, c, h, w]), n, k, alpha, beta)
        y.upload(y.host)
        dy = P.buf(rng.standard_normal(v.size).astype(NP[code]))
        dx = P.buf(np.zeros(v.size, NP[code]))
        P.run(H.lrn_backward, View(dx, [b, c, h, w]), View(y, [b, c, h, w]), View(x, [b, c, h, w]), View(dy, [b, c, h, w]),
              n, k, alpha, beta)
        assert_lrn_gradient(dx, x, y, dy, ([b, c, h, w], n, k, alpha, beta), tol)
    special = v.copy()
    special[0, 3, 1, 1] = np.nan
    special[0, 9, 2, 2] = np.inf
    special[1, 5, 0, 3] = -np.inf
    x = P.buf(special.reshape(-1))
    y = P.buf(np.zeros(v.size, NP[code]))
    P.run(H.lrn_forward, View(y, [b, c, h, w]), View(x, [b, c, h, w]), 5, 2.0, 1e-4, 0.75)
    compare(y, "lrn forward with NaN and infinities", tol=tol, denormal_ulps=2)


@pytest.mark.parametrize("code", FLOATS)
def test_lrn_strided_tensors_and_errors(P, code):
    """Every tensor with its own strides (padded planes, padded channels, a transposed plane), which
    takes the one-element-per-lane kernels, and the calls the library refuses."""
    rng = np.random.default_rng(62)
    b, c, h, w = 2, 35, 6, 8
    tol = 4e-6 if code == capi.F32 else 1e-12
    big = b * (c + 2) * (h + 1) * (w + 3)
    x = P.buf((rng.standard_normal(big) * 2).astype(NP[code]))
    y = P.buf(np.zeros(big, NP[code]))
    dy = P.buf(rng.standard_normal(b * c * h * w).astype(NP[code]))
    dx = P.buf(np.zeros(b * c * h * w, NP[code]))
    xv = View(x, [b, c, h, w], [(c + 2) * (h + 1) * (w + 3), (h + 1) * (w + 3), w + 3, 1], offset=5)
    yv = View(y, [b, c, h, w], [(c + 1) * h * w + 7, h * w, 1, h])       # planes stored column by column
    kern = P.run(H.lrn_forward, yv, xv, 5, 2.0, 1e-2, 0.75)
    assert kern == "lrn_forward"
    compare(y, "lrn forward strided", tol=tol)
    y.upload(y.host)
    kern = P.run(H.lrn_backward, View(dx, [b, c, h, w]), yv, xv, View(dy, [b, c, h, w]), 5, 2.0, 1e-2, 0.75)
    assert kern == "lrn_backward"
    compare(dx, "lrn backward strided", tol=2e-4 if code == capi.F32 else 1e-10)
    shape = [b, c, h, w]
    for bad, text in (((View(y, [b, c, h, w]), View(x, [b, c, h * w]), 5, 2.0, 1e-4, 0.75), "shapes must match"),
                      ((View(y, [b * c, h * w]), View(x, [b * c, h * w]), 5, 2.0, 1e-4, 0.75), "at least rank 3"),
                      ((View(y, shape), View(x, shape), 0, 2.0, 1e-4, 0.75), "outside [1, 16]"),
                      ((View(y, shape), View(x, shape), 17, 2.0, 1e-4, 0.75), "outside [1, 16]"),
                      ((View(y, shape), View(x, shape), 5, 0.0, 1e-4, 0.75), "below 1e-5"),
                      ((View(x, shape), View(x, shape), 5, 2.0, 1e-4, 0.75), "may not be the input")):
        with pytest.raises(capi.CortexHipError, match=re.escape(text)):
            H.lrn_forward(P.hip, *bad)
    g = View(dy, shape)
    for dest in (g, View(y, shape), View(x, shape)):   # an in-place gradient would race with the neighbours' reads
        with pytest.raises(capi.CortexHipError, match=re.escape("may not be one of the tensors read")):
            H.lrn_backward(P.hip, dest, View(y, shape), View(x, shape), g, 5, 2.0, 1e-4, 0.75)


@pytest.mark.parametrize("code", FLOATS)
def test_softmax_wide_range(P, code):
    """Rows whose entries lie hundreds below the maximum (exponentials in the denormal range and
    below it) and rows with infinities and NaN: the float kernels' hardware-exp2 path hands the
    far tail to the library routine, and special values behave as java.lang.Math.exp does."""
    rng = np.random.default_rng(33)
    tol = 2e-6 if code == capi.F32 else 1e-12
    for rows, k in ((64, 16), (40, 1000), (300, 10), (7, 5000)):
        v = (rng.standard_normal(rows * k) * 40).astype(NP[code])
        v[::7] -= 60
        x = P.buf(v)
        out = P.buf(np.zeros(rows * k, NP[code]))
        kern = P.run(H.softmax, View(out, [rows, k]), View(x, [rows, k]))
        compare(out, f"softmax wide range {(rows, k)} ({kern})", tol=tol, denormal_ulps=2)
    rows, k = 8, 12
    v = rng.standard_normal(rows * k).astype(NP[code]).reshape(rows, k)
    v[0, 3] = -np.inf
    v[1, :] = -np.inf          # 0 / 0 throughout
    v[2, 5] = np.inf           # inf - inf
    v[3, 0] = np.nan
    v[4, 1], v[4, 2] = -np.inf, 100.0
    x = P.buf(v.reshape(-1))
    out = P.buf(np.zeros(rows * k, NP[code]))
    for shape, spatial in (([rows, k], False), ([1, rows, k], False)):
        kern = P.run(H.softmax, View(out, shape), View(x, shape), spatial)
        compare(out, f"softmax special values ({kern})", tol=tol)
    xs = P.buf(np.ascontiguousarray(v.T).reshape(-1))      # the same rows along the channel axis
    outs = P.buf(np.zeros(rows * k, NP[code]))
    kern = P.run(H.softmax, View(outs, [1, k, rows]), View(xs, [1, k, rows]), True)
    compare(outs, f"softmax-spatial special values ({kern})", tol=tol)


@pytest.mark.parametrize("code", FLOATS)
def test_softmax_layouts(P, code):
    rng = np.random.default_rng(32)
    tol = 2e-6 if code == capi.F32 else 1e-12
    # spatial: [batch, channels, elements], softmax across channels
    b, c, e = 3, 21, 130
    x = P.buf((rng.standard_normal(b * c * e) * 3).astype(NP[code]))
    out = P.buf(np.zeros(b * c * e, NP[code]))
    kern = P.run(H.softmax, View(out, [b, c, e]), View(x, [b, c, e]), True)
    compare(out, f"softmax-spatial ({kern})", tol=tol)
    assert kern in ("softmax_lane", "softmax_lane_vec")         # 130 positions: pairs of doubles, single floats
    c2 = 70                                       # more channels than the four-positions-per-lane form holds
    x2, out2 = P.buf((rng.standard_normal(2 * c2 * 90) * 3).astype(NP[code])), P.buf(np.zeros(2 * c2 * 90, NP[code]))
    kern2 = P.run(H.softmax, View(out2, [2, c2, 90]), View(x2, [2, c2, 90]), True)
    compare(out2, f"softmax-spatial wide ({kern2})", tol=tol)
    # parked in LDS while the rows of one wave fit 32 KiB, else the loop form
    lds_fits = lambda ch: ch * 64 * x.init.itemsize <= 32768
    assert kern2 == ("softmax_lane_lds" if lds_fits(c2) else "softmax_lane_loop_vec")
    got = out.download().reshape(b, c, e).astype(np.float64)
    assert np.allclose(got.sum(axis=1), 1.0, atol=1e-5)
    # position counts that allow 128-bit accesses across neighbouring positions
    for (b3, c3, e3), want_kernel in (((3, 21, 132), "softmax_lane_vec"), ((2, 5, 64), "softmax_lane_vec"),
                                     ((2, 13, 64), "softmax_lane_vec"), ((2, 30, 64), "softmax_lane_vec"),
                                     ((2, 64, 96), "softmax_lane_lds"),
                                     ((2, 70, 97), "softmax_lane_lds" if lds_fits(70) else "softmax_lane_loop"),
                                     ((2, 300, 96), "softmax_lane_loop_vec"), ((2, 300, 97), "softmax_lane_loop")):
        n3 = b3 * c3 * e3
        x3, out3 = P.buf((rng.standard_normal(n3) * 3).astype(NP[code])), P.buf(np.zeros(n3, NP[code]))
        kern3 = P.run(H.softmax, View(out3, [b3, c3, e3]), View(x3, [b3, c3, e3]), True)
        compare(out3, f"softmax-spatial {(b3, c3, e3)} ({kern3})", tol=tol)
        assert kern3 == want_kernel
        P.run(H.softmax, View(x3, [b3, c3, e3]), View(x3, [b3, c3, e3]), True)
        compare(x3, f"softmax-spatial {(b3, c3, e3)} in place", tol=tol)
    # eltwise on three dimensions
    kern = P.run(H.softmax, View(out, [b, c, e]), View(x, [b, c, e]))
    compare(out, f"softmax 3-d eltwise ({kern})", tol=tol)
    # pitched rows in place: select :all (range 2 10) of a [5, 10] matrix (verify/tensor.clj:611-620)
    m = P.buf(np.tile(np.arange(10), 5).astype(NP[code]))
    sel = View(m, [5, 8], [10, 1], offset=2)
    P.run(H.softmax, sel, sel)
    compare(m, "softmax pitched in place", tol=tol)
    # NaN poisons its row only; infinities of one sign
    y = (rng.standard_normal(4 * 50)).astype(NP[code])
    y[7] = np.nan
    y[60] = np.inf
    yb, ob = P.buf(y), P.buf(np.zeros(200, NP[code]))
    P.run(H.softmax, View(ob, [4, 50]), View(yb, [4, 50]))
    compare(ob, "softmax with NaN and inf rows", tol=tol)


def test_softmax_and_activation_gradient_errors(P):
    x = P.buf(np.zeros(16, np.float32))
    xi = P.buf(np.zeros(16, np.int32))
    with pytest.raises(capi.CortexHipError, match="float and double"):
        H.softmax(P.hip, View(xi, [4, 4]), View(xi, [4, 4]))
    with pytest.raises(capi.CortexHipError, match="2 or 3 dimensions"):
        H.softmax(P.hip, View(x, [16]), View(x, [16]))
    with pytest.raises(capi.CortexHipError, match="do not match"):
        H.softmax(P.hip, View(x, [4, 4]), View(x, [2, 8]))
    with pytest.raises(capi.CortexHipError, match="float and double"):
        H.activation_gradient(P.hip, View(xi, [16]), View(xi, [16]), View(xi, [16]), "relu", 16)


# ------------------------------------------------------------------ batch normalization
# Layouts: (batch, channels) is the eltwise form, (batch, channels, elements) the spatial one.
# They cover both statistics kernels (rows of at least 128 bytes are walked row style), vector
# and scalar accesses, table-per-window and table-of-all-channels apply passes, and tails.
BN_SHAPES = [(4, 3), (128, 1000), (37, 130), (1000, 64), (5, 4099), (2, 3, 4), (8, 16, 196), (4, 5, 49),
             (3, 7, 1024), (16, 3, 4100), (2, 2, 31), (70, 33, 8), (2, 3000, 4), (33, 6, 1000), (1, 4, 64),
             (6, 10, 1023), (3, 4, 35), (9, 3, 50), (5, 3, 257), (2, 7, 513)]


def bn_close(buf, what, code, scale_by=None):
    """|got - want| <= tol * max|want|: the sums are taken in another order than the CPU
    backend's left-to-right walk, so values that cancel are compared on the tensor's scale."""
    tol = REL_TOL if code == capi.F32 else REL_TOL_F64
    got, want = buf.download().astype(np.float64), buf.host.astype(np.float64)
    scale = np.max(np.abs(want)) if scale_by is None else scale_by
    err = np.max(np.abs(got - want))
    assert err <= tol * max(scale, 1e-30), f"{what}: max abs err {err} on scale {scale}"


def bn_setup(P, rng, code, shape):
    b, c = shape[0], shape[1]
    e = shape[2] if len(shape) == 3 else None
    n = b * c * (e or 1)
    f = NP[code]
    t = dict(
        x=P.buf((rng.standard_normal(n) * 2 + 5).astype(f)), out=P.buf(np.zeros(n, f)),
        og=P.buf(rng.standard_normal(n).astype(f)), ig=P.buf(np.zeros(n, f)),
        means=P.buf(rng.standard_normal(c).astype(f)), variances=P.buf(rng.uniform(0, 3, c).astype(f)),
        rmeans=P.buf(rng.standard_normal(c).astype(f)), rvars=P.buf(rng.uniform(0.5, 2, c).astype(f)),
        scale=P.buf(rng.uniform(0.5, 1.5, c).astype(f)), bias=P.buf(rng.standard_normal(c).astype(f)),
        sg=P.buf(np.zeros(c, f)), bg=P.buf(np.zeros(c, f)))
    V = {k: View(v, [v.init.size]) for k, v in t.items()}
    return t, V, (b, c, e)


@pytest.mark.parametrize("code", FLOATS)
@pytest.mark.parametrize("shape", BN_SHAPES, ids=str)
def test_batch_normalize(P, code, shape):
    rng = np.random.default_rng(40)
    t, V, (b, c, e) = bn_setup(P, rng, code, shape)
    t["variances"].init[0] = 0.0          # the reference's edge case
    t["variances"].reset()
    k = P.run(H.batch_normalize, V["out"], V["x"], V["means"], V["variances"], V["scale"], V["bias"], 1e-2, b, c, e)
    compare(t["out"], f"batch-normalize {shape} ({k})")      # elementwise in the CPU backend's order: bit-exact
    P.run(H.batch_normalize, V["x"], V["x"], V["means"], V["variances"], V["scale"], V["bias"], 1e-2, b, c, e)
    compare(t["x"], f"batch-normalize {shape} in place")


@pytest.mark.parametrize("code", FLOATS)
def test_batch_normalize_large_rows(P, code):
    """From 32 MiB on, the plain normalization of long rows writes its channel constants in a
    launch of their own and reads them per row; the rows here end inside blocks."""
    shape = (8, 64, 16400)
    rng = np.random.default_rng(44)
    t, V, (b, c, e) = bn_setup(P, rng, code, shape)
    P.run(H.batch_normalize, V["out"], V["x"], V["means"], V["variances"], V["scale"], V["bias"], 1e-2, b, c, e)
    compare(t["out"], f"batch-normalize {shape}")
    P.run(H.batch_normalize, V["x"], V["x"], V["means"], V["variances"], V["scale"], V["bias"], 1e-2, b, c, e)
    compare(t["x"], f"batch-normalize {shape} in place")


@pytest.mark.parametrize("code", FLOATS)
@pytest.mark.parametrize("shape", BN_SHAPES, ids=str)
def test_batch_normalize_update_and_gradients(P, code, shape):
    rng = np.random.default_rng(41)
    t, V, (b, c, e) = bn_setup(P, rng, code, shape)
    x64 = t["x"].init.astype(np.float64)
    k = P.run(H.batch_normalize_update_and_apply, V["out"], V["x"], V["means"], V["variances"], V["rmeans"],
              V["rvars"], 0.8, V["scale"], V["bias"], 1e-3, b, c, e)
    one_launch = b * (e or 1) <= 4096 and b * c * (e or 1) <= 1 << 21     # a channel fits a block's registers
    assert k == ("bn_update_small" if one_launch else
                 "bn_update_row" if (e or 1) * t["x"].init.itemsize >= 128 else "bn_update_col")
    what = f"batch-normalize-update-and-apply {shape} ({k})"
    bn_close(t["means"], what + " batch means", code, scale_by=np.max(np.abs(x64)))
    bn_close(t["variances"], what + " batch variances", code)
    bn_close(t["rmeans"], what + " running means", code, scale_by=np.max(np.abs(x64)))
    bn_close(t["rvars"], what + " running variances", code)
    bn_close(t["out"], what + " output", code)
    # the gradient takes the statistics as given: hand both sides the oracle's
    for name in ("means", "variances"):
        t[name].upload(t[name].host)
    k = P.run(H.batch_normalize_gradients, V["ig"], V["sg"], V["bg"], V["og"], V["out"], V["x"], V["means"],
              V["variances"], V["scale"], V["bias"], 1e-3, b, c, e)
    assert (k == "bn_gradients_small") == one_launch, k
    what = f"batch-normalize-gradients {shape} ({k})"
    og64 = np.abs(t["og"].init.astype(np.float64))
    per_channel = og64.reshape(b, c, e or 1).sum(axis=(0, 2)).max()
    bn_close(t["bg"], what + " bias gradient", code, scale_by=per_channel)
    bn_close(t["sg"], what + " scale gradient", code, scale_by=per_channel * 4)
    bn_close(t["ig"], what + " input gradient", code, scale_by=np.max(og64))
    # in place over the output gradient
    P.run(H.batch_normalize_gradients, V["og"], V["sg"], V["bg"], V["og"], V["out"], V["x"], V["means"],
          V["variances"], V["scale"], V["bias"], 1e-3, b, c, e)
    bn_close(t["og"], what + " input gradient in place", code, scale_by=np.max(og64))


def test_batch_normalize_offset_mean_and_misaligned(P):
    """A channel far from zero (mean 1000, deviation 0.01) and buffers that start
    off a 16-byte boundary."""
    rng = np.random.default_rng(42)
    b, c, e = 6, 5, 100
    n = b * c * e
    x = (rng.standard_normal(n) * 0.01 + 1000).astype(np.float32)
    xb, ob = P.buf(np.concatenate([[0], x]).astype(np.float32)), P.buf(np.zeros(n + 3, np.float32))
    stats = [P.buf(np.ones(c + 1, np.float32)) for _ in range(6)]
    sv = [View(s, [c], offset=1) for s in stats]
    P.run(H.batch_normalize_update_and_apply, View(ob, [n], offset=3), View(xb, [n], offset=1), sv[0], sv[1], sv[2],
          sv[3], 0.5, sv[4], sv[5], 1e-4, b, c, e)
    bn_close(stats[0], "offset mean: batch means", capi.F32)
    bn_close(stats[1], "offset mean: batch variances", capi.F32)
    bn_close(ob, "offset mean: output", capi.F32)


def test_batch_normalize_errors(P):
    x = P.buf(np.zeros(16, np.float32))
    xi = P.buf(np.zeros(16, np.int32))
    v = View(x, [16])
    with pytest.raises(capi.CortexHipError, match="float and double"):
        H.batch_normalize(P.hip, View(xi, [16]), View(xi, [16]), View(xi, [16]), View(xi, [16]), View(xi, [16]),
                          View(xi, [16]), 1e-2, 4, 4)
    with pytest.raises(capi.CortexHipError, match="positive"):
        H.batch_normalize(P.hip, v, v, v, v, v, v, 1e-2, 0, 4)


# ------------------------------------------------------------------ rand!

@pytest.mark.parametrize("n", [1, 3, 4, 1003, 70001, 1 << 20])
def test_rand_matches_oracle_stream(P, n):
    buf = P.buf(np.zeros(n + 1, np.float32))
    for view in (View(buf, [n]), View(buf, [n], offset=1)):          # aligned and off the 16-byte grid
        k = P.run(H.rand, view, n, "flat", -2.0, 3.0, 0xC0FFEE123, 5)
        compare(buf, f"rand flat n={n} ({k})")                       # integer work and one exact product: bit-exact
        k = P.run(H.rand, view, n, "gaussian", 1.0, 9.0, 0xC0FFEE123, 6)
        got, want = buf.download().astype(np.float64), buf.host.astype(np.float64)
        # Box-Muller in float: log, sqrt, cos and sin of the device library against the host's
        assert np.max(np.abs(got - want)) <= 3 * 2e-6 * 6, f"rand gaussian n={n} ({k})"


def test_rand_errors(P):
    x = P.buf(np.zeros(8, np.float64))
    with pytest.raises(capi.CortexHipError, match="floating point buffers"):
        H.rand(P.hip, View(x, [8]), 8, "flat", 0, 1, 1, 0)
    y = P.buf(np.zeros(8, np.float32))
    with pytest.raises(capi.CortexHipError, match="Minimum must be less"):
        H.rand(P.hip, View(y, [8]), 8, "flat", 1, 1, 1, 0)


# ------------------------------------------------------------------ gemm! (rocBLAS), gemv!
# The vendor library sums in the tensor's own precision and in its own order; the oracle keeps a
# double accumulator.  Bar: |got - want| <= tol * (|alpha| sum |a||b| + |beta c|) with
# tol = 1e-5 for float (k up to 512 terms of 2^-24 relative error each) and 1e-13 for double.

# ------------------------------------------------------------------ convolution
# (batch, in channels, out channels, height, width, kw, kh, px, py, sx, sy)
CONV_CASES = [
    (3, 4, 3, 4, 4, 3, 3, 0, 0, 1, 1),       # the reference's own test geometry
    (2, 3, 5, 9, 11, 3, 3, 1, 1, 1, 1),      # 27 cells per row: cell-by-cell stores
    (2, 4, 6, 12, 10, 3, 3, 1, 1, 2, 2),     # 36 cells per row: 16-byte stores
    (1, 2, 3, 8, 8, 2, 2, 0, 0, 2, 2),
    (2, 1, 4, 7, 9, 5, 3, 2, 1, 2, 1),       # rectangular window
    (1, 8, 16, 14, 14, 1, 1, 0, 0, 1, 1),    # 1 x 1: the unrolled matrix is the transposed input
    (4, 16, 32, 28, 28, 3, 3, 1, 1, 1, 1),
    (2, 2, 3, 100, 130, 3, 3, 1, 1, 1, 1),   # 13000 positions: the weight gradient in three pieces
    (1, 2, 2, 9, 11, 5, 5, 2, 2, 1, 1),
    (2, 3, 4, 10, 14, 3, 3, 0, 0, 1, 1),     # unit stride, rows of whole 16-byte pieces: one load per piece
    (1, 2, 2, 12, 12, 3, 3, 1, 1, 1, 2),
]


def unrolled_matches(work, batch, n_rows, n_cols, what):
    """The library keeps an image's unrolled matrix as [cells, positions], the oracle (like the
    reference's CPU backend) as [positions, cells]; whatever follows the matrices must be untouched."""
    n = batch * n_rows * n_cols
    got, want = work.download(), work.host
    H.assert_bit_exact(np.ascontiguousarray(got[:n].reshape(batch, n_cols, n_rows).transpose(0, 2, 1)),
                       want[:n].reshape(batch, n_rows, n_cols), what)
    H.assert_bit_exact(got[n:], want[n:], what + " (slack)")


@pytest.mark.parametrize("code", FLOATS)
@pytest.mark.parametrize("case", CONV_CASES, ids=str)
def test_convolution(P, code, case):
    batch, cin, cout, h, w, kw, kh, px, py, sx, sy = case
    oh, ow = (h + 2 * py - kh) // sy + 1, (w + 2 * px - kw) // sx + 1
    n_cols, n_rows = cin * kh * kw, oh * ow
    rng = np.random.default_rng(55)
    desc = H.conv_desc(cin, cout, kw, kh, px, py, sx, sy)
    geom = (desc, batch, h, w, oh, ow)
    inp = P.buf(values(rng, code, batch * cin * h * w))
    weights = P.buf(values(rng, code, cout * n_cols) / 8)
    out = P.buf(values(rng, code, batch * cout * n_rows))            # overwritten (alpha 0), then added onto
    work = P.buf(np.full(batch * n_rows * n_cols + 5, 7.0, NP[code]))
    og = P.buf(values(rng, code, batch * cout * n_rows))
    wg = P.buf(values(rng, code, cout * n_cols))
    ig = P.buf(values(rng, code, batch * cin * h * w))
    V = lambda b: View(b, [b.init.size])
    tol = 2e-5 if code == capi.F32 else 1e-12

    def close(buf, scale, what):
        got, want = buf.download().astype(np.float64), buf.host.astype(np.float64)
        assert np.all(np.abs(got - want) <= tol * scale), f"{what} {case}: {np.abs(got - want).max()} vs {tol * scale}"

    x64, w64, g64 = (b.init.astype(np.float64) for b in (inp, weights, og))
    P.run(H.convolution, "forward", V(out), 0.0, V(inp), V(weights), V(work), *geom)
    unrolled_matches(work, batch, n_rows, n_cols, f"unrolled input {case}")   # a copy: bit-exact, the slack untouched
    scale = np.abs(w64).max() * np.abs(x64).max() * n_cols
    close(out, scale, "convolution-forward")
    P.run(H.convolution, "forward", V(out), 0.5, V(inp), V(weights), V(work), *geom)
    close(out, 2 * scale, "convolution-forward onto half the output")
    P.run(H.convolution, "backward_weights", V(wg), 0.0, V(og), V(inp), V(work), *geom)
    close(wg, np.abs(g64).max() * np.abs(x64).max() * n_rows * batch, "convolution-backward-weights")
    P.run(H.convolution, "backward_weights", V(wg), 1.0, V(og), V(inp), V(work), *geom)
    close(wg, 2 * np.abs(g64).max() * np.abs(x64).max() * n_rows * batch, "convolution-backward-weights, accumulated")
    P.run(H.convolution, "backward_data", V(ig), 0.0, V(og), V(weights), V(work), *geom)
    close(ig, np.abs(g64).max() * np.abs(w64).max() * cout * kh * kw, "convolution-backward-data")


def test_convolution_roll_back_is_bit_exact(P):
    """With integer-valued operands every product and sum is exact, so the input gradient must
    agree to the bit whatever order the gemm sums in; the gather then adds windows in the
    reference's order."""
    rng = np.random.default_rng(56)
    V = lambda b: View(b, [b.init.size])
    for h, w, k in ((10, 9, 3), (10, 12, 3), (8, 16, 5), (6, 8, 1)):      # rows of whole 16-byte pieces or not
        batch, cin, cout, pad = 2, 3, 4, k // 2
        oh, ow = h, w                                                   # "same" padding, stride 1
        desc = H.conv_desc(cin, cout, k, k, pad, pad, 1, 1)
        og = P.buf(rng.integers(-3, 4, batch * cout * oh * ow).astype(np.float32))
        weights = P.buf(rng.integers(-3, 4, cout * cin * k * k).astype(np.float32))
        work = P.buf(np.zeros(batch * oh * ow * cin * k * k, np.float32))
        ig = P.buf(np.ones(batch * cin * h * w, np.float32))
        P.run(H.convolution, "backward_data", V(ig), 0.0, V(og), V(weights), V(work), desc, batch, h, w, oh, ow)
        unrolled_matches(work, batch, oh * ow, cin * k * k, f"unrolled gradient {h}x{w} k{k}")
        compare(ig, f"input gradient {h}x{w} k{k}")


def test_convolution_errors(P):
    b = P.buf(np.zeros(4096, np.float32))
    v = View(b, [4096])
    good = H.conv_desc(2, 3, 3, 3, 0, 0, 1, 1)
    with pytest.raises(capi.CortexHipError, match="workspace"):
        H.convolution(P.hip, "forward", v, 0.0, v, v, View(b, [10]), good, 1, 6, 6, 4, 4)
    with pytest.raises(capi.CortexHipError, match="beyond the padded input"):
        H.convolution(P.hip, "forward", v, 0.0, v, v, v, good, 1, 6, 6, 5, 5)
    with pytest.raises(capi.CortexHipError):
        H.convolution(P.hip, "forward", v, 0.0, v, v, v, H.conv_desc(0, 3, 3, 3, 0, 0, 1, 1), 1, 6, 6, 4, 4)
    ints = P.buf(np.zeros(4096, np.int32))
    with pytest.raises(capi.CortexHipError, match="float and double"):
        H.convolution(P.hip, "forward", View(ints, [4096]), 0.0, v, v, v, good, 1, 6, 6, 4, 4)


# ------------------------------------------------------------------ pooling
# (batch, channels, height, width, kw, kh, px, py, sx, sy, dimension-op)
POOL_CASES = [
    (2, 4, 4, 4, 3, 3, 1, 1, 2, 2, "floor"),       # the reference's own test geometry
    (3, 5, 17, 23, 3, 3, 1, 1, 2, 2, "ceil"),      # ragged, windows running past the padding
    (2, 3, 32, 32, 2, 2, 0, 0, 2, 2, "floor"),     # disjoint windows
    (2, 3, 9, 9, 2, 2, 1, 1, 1, 1, "ceil"),        # every input under four windows
    (1, 2, 30, 19, 5, 3, 2, 1, 3, 2, "ceil"),      # rectangular window, stride and padding
    (2, 2, 13, 13, 3, 3, 0, 0, 1, 1, "floor"),     # nine windows per input
    (1, 3, 11, 14, 2, 2, 0, 0, 3, 3, "ceil"),      # stride beyond the window: inputs under no window
    (1, 1, 5, 7, 7, 5, 3, 2, 1, 1, "floor"),       # window as large as the image
    (4, 8, 56, 56, 3, 3, 1, 1, 2, 2, "floor"),
    (1, 1, 1, 1, 1, 1, 0, 0, 1, 1, "floor"),
    (2, 3, 120, 100, 3, 3, 1, 1, 2, 2, "floor"),   # planes beyond the LDS budget: bands of rows
    (1, 2, 131, 97, 3, 3, 1, 1, 2, 2, "ceil"),
    (2, 2, 90, 90, 2, 2, 0, 0, 2, 2, "floor"),
    (1, 3, 75, 110, 3, 3, 1, 1, 1, 1, "floor"),
    (1, 2, 100, 70, 5, 4, 2, 1, 2, 3, "ceil"),
    (2, 2, 10, 10, 3, 3, 0, 0, 2, 2, "ceil"),      # the last windows reach beyond the padded input
    (3, 4, 20, 20, 3, 3, 1, 1, 1, 1, "floor"),     # several small padded planes per block
    (1, 1, 9, 2000, 3, 3, 1, 1, 2, 2, "floor"),    # rows beyond it: the direct kernels
    (1, 1, 40, 300, 17, 17, 8, 8, 1, 1, "floor"),  # a window too large for the reciprocal table
]


def pool_out_dim(n, pad, k, stride, op):
    partial = (n + 2.0 * pad - k) / stride
    return int((np.floor(partial) if op == "floor" else np.ceil(partial)) + 1)


@pytest.mark.parametrize("code", FLOATS)
@pytest.mark.parametrize("op", list(capi.POOL_OPS))
@pytest.mark.parametrize("case", POOL_CASES, ids=str)
def test_pooling_bit_exact(P, code, op, case):
    batch, channels, h, w, kw, kh, px, py, sx, sy, dim_op = case
    oh, ow = pool_out_dim(h, py, kh, sy, dim_op), pool_out_dim(w, px, kw, sx, dim_op)
    rng = np.random.default_rng(50)
    n_in, n_out = batch * channels * h * w, batch * channels * oh * ow
    # small integers: ties inside a window decide which inputs the max gradient reaches
    x = rng.integers(-4, 5, n_in).astype(NP[code]) if op == "max" else values(rng, code, n_in)
    if n_in > 8:
        x[:3] = [np.nan, -0.0, 0.0]
    inp, out = P.buf(x), P.buf(values(rng, code, n_out))       # avg-exc-pad adds onto the output
    og, ig = P.buf(values(rng, code, n_out)), P.buf(values(rng, code, n_in))  # the gradient is added onto
    desc = H.pool_desc(kw, kh, px, py, sx, sy, op)
    geom = (desc, batch, channels, h, w, oh, ow)
    k = P.run(H.pooling_forward, View(out, [n_out]), View(inp, [n_in]), *geom)
    assert k.startswith("pool_forward")
    compare(out, f"pooling-forward {op} {case}")
    k = P.run(H.pooling_backward, View(ig, [n_in]), View(inp, [n_in]), View(out, [n_out]), View(og, [n_out]), *geom)
    assert k.startswith("pool_backward")
    compare(ig, f"pooling-backward {op} {case}")


def test_pooling_first_tap_outside_padded_input(P):
    """A stride that carries the last window past the padded input leaves no first tap to
    reset the value: max and avg continue from what the output held (impl.clj:84-96)."""
    rng = np.random.default_rng(51)
    for op in capi.POOL_OPS:
        h = w = 5
        oh = ow = 4                      # the caller's output is larger than the formula's
        x, prev = values(rng, capi.F32, h * w), values(rng, capi.F32, oh * ow)
        inp, out = P.buf(x), P.buf(prev)
        desc = H.pool_desc(2, 2, 0, 0, 2, 2, op)
        P.run(H.pooling_forward, View(out, [oh * ow]), View(inp, [h * w]), desc, 1, 1, h, w, oh, ow)
        compare(out, f"pooling-forward {op} with windows beyond the input")
        og, ig = P.buf(values(rng, capi.F32, oh * ow)), P.buf(np.zeros(h * w, np.float32))
        P.run(H.pooling_backward, View(ig, [h * w]), View(inp, [h * w]), View(out, [oh * ow]), View(og, [oh * ow]),
              desc, 1, 1, h, w, oh, ow)
        compare(ig, f"pooling-backward {op} with windows beyond the input")


def test_pooling_errors(P):
    b = P.buf(np.zeros(64, np.float32))
    v = View(b, [64])
    good = H.pool_desc(2, 2, 0, 0, 2, 2, "max")
    for desc, dtype_buf in ((H.pool_desc(0, 2, 0, 0, 2, 2, "max"), b), (H.pool_desc(2, 2, 0, 0, 0, 2, "max"), b),
                            (H.pool_desc(2, 2, -1, 0, 2, 2, "max"), b)):
        with pytest.raises(capi.CortexHipError):
            H.pooling_forward(P.hip, v, v, desc, 1, 1, 4, 4, 2, 2)
    ints = P.buf(np.zeros(64, np.int32))
    with pytest.raises(capi.CortexHipError, match="pooling op"):
        H.pooling_forward(P.hip, View(ints, [64]), View(ints, [64]), good, 1, 1, 4, 4, 2, 2)
    with pytest.raises(capi.CortexHipError, match="negative"):
        H.pooling_forward(P.hip, v, v, good, -1, 1, 4, 4, 2, 2)
    H.pooling_forward(P.hip, v, v, good, 0, 1, 4, 4, 2, 2)    # an empty batch is no error


GEMM_CASES = [(5, 7, 4, 9, 8, 6), (64, 64, 64, 64, 64, 64), (33, 129, 65, 140, 70, 70), (256, 512, 128, 512, 512, 128),
              (1, 300, 1, 300, 300, 1)]


@pytest.mark.parametrize("code", FLOATS)
@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("case", GEMM_CASES, ids=str)
def test_gemm(P, code, ta, tb, case):
    M, K, N, lda, ldb, ldc = case
    rng = np.random.default_rng(70)
    f = NP[code]
    a_rows, a_cols = (K, M) if ta else (M, K)
    b_rows, b_cols = (N, K) if tb else (K, N)
    lda, ldb = max(lda, a_cols), max(ldb, b_cols)
    a, b, c = (rng.standard_normal(s).astype(f) for s in ((a_rows, lda), (b_rows, ldb), (M, ldc)))
    ba, bb, bc = P.buf(a), P.buf(b), P.buf(c)
    va, vb, vc = (View(bf, [bf.init.size]) for bf in (ba, bb, bc))
    A, B = np.abs(a[:, :a_cols].astype(np.float64)), np.abs(b[:, :b_cols].astype(np.float64))
    for alpha, beta in ((1.0, 0.0), (1.5, -0.5)):
        P.run(H.gemm, vc, ldc, ta, tb, alpha, va, M, K, lda, vb, N, ldb, beta)
        bound = np.zeros((M, ldc))
        bound[:, :N] = abs(alpha) * ((A.T if ta else A) @ (B.T if tb else B)) + abs(beta) * np.abs(c[:, :N]) + 1e-30
        tol = 1e-5 if code == capi.F32 else 1e-13
        got, want = bc.download().astype(np.float64).reshape(M, ldc), bc.host.astype(np.float64).reshape(M, ldc)
        assert np.all(np.abs(got - want) <= tol * bound + 0.0), f"gemm {case} ta={ta} tb={tb}: {np.max(np.abs(got - want))}"
        assert np.array_equal(got[:, N:], c[:, N:].astype(np.float64))      # row padding untouched
        bc.reset()


# gemv! is the library's own pair of reductions with double accumulators: it differs from the
# oracle only in the order of the double additions, so the bar is the reductions' (2e-6 / 1e-12
# of the sum of magnitudes), and what lies between the strided elements of y must stay untouched.
GEMV_CASES = [(6, 5, 8, 3, 2), (300, 257, 257, 1, 1), (64, 1000, 1024, 1, 5), (2000, 64, 64, 1, 1), (3, 5000, 5000, 1, 1),
              (1500, 260, 264, 2, 1), (700, 1028, 1028, 1, 1), (1, 1, 1, 1, 1), (129, 12, 12, 1, 3)]


@pytest.mark.parametrize("code", FLOATS)
@pytest.mark.parametrize("ta", [False, True])
def test_gemv(P, code, ta):
    rng = np.random.default_rng(71)
    f = NP[code]
    for rows, cols, lda, incx, incy in GEMV_CASES:
        n_in, n_out = (rows, cols) if ta else (cols, rows)
        a, x, y = (rng.standard_normal(s).astype(f) for s in ((rows, lda), n_in * incx, n_out * incy))
        ba, bx, by = P.buf(a), P.buf(x), P.buf(y)
        va, vx, vy = (View(bf, [bf.init.size]) for bf in (ba, bx, by))
        k = P.run(H.gemv, vy, incy, ta, 2.0, va, rows, cols, lda, vx, incx, 0.25)
        assert k.startswith("gemv_cols" if ta else "gemv_rows"), k
        A = np.abs(a[:, :cols].astype(np.float64))
        bound = np.zeros(n_out * incy)
        bound[::incy] = 2.0 * ((A.T if ta else A) @ np.abs(x[::incx].astype(np.float64))) + 0.25 * np.abs(y[::incy])
        tol = 2e-6 if code == capi.F32 else 1e-12
        got, want = by.download().astype(np.float64), by.host.astype(np.float64)
        assert np.all(np.abs(got - want) <= tol * bound), f"gemv {(rows, cols)} ta={ta}: {np.max(np.abs(got - want))}"
        # beta = 0 overwrites whatever y held, NaN included
        by.init[::incy] = np.nan
        by.reset()
        P.run(H.gemv, vy, incy, ta, 1.0, va, rows, cols, lda, vx, incx, 0.0)
        got, want = by.download().astype(np.float64), by.host.astype(np.float64)
        assert not np.isnan(got[::incy]).any()
        assert np.all(np.abs(got - want) <= tol * bound), f"gemv beta 0 {(rows, cols)} ta={ta}"


def test_gemm_errors(P):
    x = P.buf(np.zeros(16, np.float32))
    xi = P.buf(np.zeros(16, np.int32))
    v = View(x, [16])
    with pytest.raises(capi.CortexHipError, match="float and double"):
        H.gemm(P.hip, View(xi, [16]), 4, False, False, 1, View(xi, [16]), 4, 4, 4, View(xi, [16]), 4, 4, 0)
    with pytest.raises(capi.CortexHipError, match="column stride"):
        H.gemm(P.hip, v, 2, False, False, 1, v, 4, 4, 4, v, 4, 4, 0)


# ------------------------------------------------------------------ vector kernel: rows at least a block wide
# Blocks of 256 vectors that start in one row and end in the next, with one, two and three outer axes.

@pytest.mark.parametrize("code", [capi.F32, capi.F64, capi.I16])
def test_wide_rows_crossing_blocks(P, code):
    rng = np.random.default_rng(90)
    f = NP[code]
    for shape, y_shape in (((5, 1200), (1200,)), ((5, 1200), (5, 1)), ((3, 5, 1208), (5, 1)), ((2, 3, 2, 1300), (3, 1, 1)),
                           ((2, 2, 3, 2, 1100), (2, 1, 1, 1))):
        n = int(np.prod(shape))
        x, y = P.buf(values(rng, code, n)), P.buf(values(rng, code, int(np.prod(y_shape))))
        d = P.buf(np.zeros(n, f))
        k = P.run(H.binary_op, View(d, shape), View(x, shape), 1.0, View(y, y_shape), 1.0, "+")
        assert k == "vec"
        compare(d, f"binary-op! :+ {shape} + {y_shape}")
        # pitched rows (a sub-matrix) keep two outer axes apart
        pitch = shape[-1] + 8
        rows = n // shape[-1]
        xp = P.buf(values(rng, code, rows * pitch))
        k = P.run(H.binary_op, View(d, [rows, shape[-1]]), View(xp, [rows, shape[-1]], [pitch, 1]), 1.0,
                  View(y, [1]), 2.0, "*")
        compare(d, f"binary-op! :* pitched {shape}")


@pytest.mark.parametrize("code", [capi.F32, capi.F64, capi.I8])
def test_tile_super_tiles(P, code):
    """Transposed views large enough for several super-tiles of the tile kernel's block order,
    with tile counts that do not divide into them and an outer axis on top."""
    rng = np.random.default_rng(91)
    f = NP[code]
    for outer, a, b in ((1, 2100, 300), (3, 2100, 140), (2, 90, 2200)):
        n = outer * a * b
        x, y, z = (P.buf(values(rng, code, n)) for _ in range(3))
        d = P.buf(np.zeros(n, f))
        dest = View(d, [outer, a, b])
        tr = lambda buf: View(buf, [outer, b, a]).transpose([0, 2, 1])
        k = P.run(H.ternary_op, dest, tr(x), 1.0, tr(y), 1.0, tr(z), 1.0)
        assert k == "tile"
        compare(d, f"select, three transposed {(outer, a, b)}")
        k = P.run(H.binary_op, dest, tr(x), 1.0, View(y, [outer, a, b]), 1.0, "+")
        assert k == "tile_wide_a"
        compare(d, f"x^T + y {(outer, a, b)}")
        k = P.run(H.unary_op, dest, tr(x), 1.0, "-")
        assert k == "tile"
        compare(d, f"negated transpose {(outer, a, b)}")


def test_flat_call_longer_than_one_launch():
    """A flat call of more than 2^30 vectors (16 GiB of bytes) is walked in pieces."""
    import ctypes as C
    n = (1 << 34) + 4096 + 5
    free, total = C.c_size_t(), C.c_size_t()
    capi.call("ct_memory_info", C.byref(free), C.byref(total))
    if free.value < 2 * n + (1 << 30):
        pytest.skip("needs 33 GiB of free device memory")
    a, b = C.c_void_p(), C.c_void_p()
    capi.call("ct_malloc", C.byref(a), n)
    capi.call("ct_malloc", C.byref(b), n)
    try:
        dims1 = capi.make_dims([n], [1])
        capi.call("ct_memset", None, a, capi.I8, 7.0, n)
        capi.call("ct_binary_op_constant", None, b, C.byref(dims1), a, C.byref(dims1), 1.0, 5.0, n, capi.BINARY_OPS["+"], 0,
                  capi.I8)
        capi.call("ct_stream_sync", None)
        assert capi.last_kernel() == "vec"
        for start in (0, (1 << 34) - 2048, (1 << 34) - 8, n - 4096):
            out = np.zeros(4096 if start + 4096 <= n else n - start, np.int8)
            capi.call("ct_memcpy_async", out.ctypes.data, b.value + start, out.nbytes, capi.COPY_D2H, None)
            capi.call("ct_stream_sync", None)
            assert np.all(out == 12), (start, out[:16])
    finally:
        capi.call("ct_free", a)
        capi.call("ct_free", b)


@pytest.mark.parametrize("rows,cols", [((1 << 15) + 3, 1 << 17), (2, (1 << 31) + 48)], ids=["many_rows", "two_long_rows"])
def test_rows_and_columns_call_beyond_32_bit_indexing(rows, cols):
    """A byte matrix of 2^31 elements or more plus a bias row: more than the kernels' 32-bit indices
    count, so the call is cut along its slowest axis into pieces of at most 2^30 elements (8192 rows of
    2^17; a row longer than that is cut again along the row).  Rows at the start, on both sides of piece
    boundaries and at the end are copied back and compared, and the pieces run on the vector kernel."""
    import ctypes as C
    n = rows * cols
    free, total = C.c_size_t(), C.c_size_t()
    capi.call("ct_memory_info", C.byref(free), C.byref(total))
    if free.value < 2 * n + (2 << 30):
        pytest.skip("needs %d GiB of free device memory" % ((2 * n >> 30) + 2))
    a, b, bias = C.c_void_p(), C.c_void_p(), C.c_void_p()
    capi.call("ct_malloc", C.byref(a), n)
    capi.call("ct_malloc", C.byref(b), n)
    capi.call("ct_malloc", C.byref(bias), cols)
    try:
        host_bias = (np.arange(cols) % 11).astype(np.int8)
        capi.call("ct_memcpy_async", bias, host_bias.ctypes.data, cols, capi.COPY_H2D, None)
        capi.call("ct_memset", None, a, capi.I8, 7.0, n)
        capi.call("ct_memset", None, b, capi.I8, 0.0, n)
        full, row = capi.make_dims([rows, cols], [cols, 1]), capi.make_dims([cols], [1])
        capi.call("ct_binary_op", None, b, C.byref(full), a, C.byref(full), 1.0, bias, C.byref(row), 1.0, n,
                  capi.BINARY_OPS["+"], capi.I8)
        capi.call("ct_stream_sync", None)
        assert capi.last_kernel() == "vec"
        want = (7 + host_bias).astype(np.int8)
        picks = {0, 1, 8191, 8192, 8193, 16384, rows // 2 - 1, rows // 2, rows - 8193, rows - 1}
        for r in sorted(p for p in picks if 0 <= p < rows):
            out = np.zeros(cols, np.int8)
            capi.call("ct_memcpy_async", out.ctypes.data, b.value + r * cols, cols, capi.COPY_D2H, None)
            capi.call("ct_stream_sync", None)
            assert np.array_equal(out, want), (r, np.flatnonzero(out != want)[:8])
    finally:
        for p in (a, b, bias):
            capi.call("ct_free", p)


# ------------------------------------------------------------------ threads and streams

def test_threads_on_their_own_streams(P):
    """Several host threads drive their own streams at once, as cortex's training threads do
    (src/cortex/verify/nn/train.clj:211-236): every call that keeps state outside its
    arguments is in the mix (stream scratch of the split reductions, the staged sum-accumulate
    and batch normalization; the per-thread rocBLAS handle; the thread-local error text)."""
    import ctypes as C
    import threading

    rng = np.random.default_rng(100)
    n_threads, rounds = 4, 6
    r, c = 600, 520
    work = []
    for t in range(n_threads):
        x = P.buf(rng.standard_normal(r * c).astype(np.float32))
        w = dict(x=x, col=P.buf(np.zeros(c, np.float32)), row=P.buf(np.zeros(r, np.float32)),
                 acc=P.buf(rng.standard_normal(c).astype(np.float32)), out=P.buf(np.zeros(r * c, np.float32)),
                 stats=[P.buf(rng.uniform(0.5, 1.5, c).astype(np.float32)) for _ in range(6)],
                 gemm=P.buf(np.zeros(c * c, np.float32)))
        work.append(w)

    def run_all(side, w):
        V = lambda b, shape=None: View(b, shape or [b.init.size])
        H.unary_reduce(side, View(w["col"], [c, 1]), 1.0, View(w["x"], [c, r], [1, c]), "sum")      # column reduce: partials
        H.unary_reduce(side, View(w["row"], [r, 1]), 1.0, View(w["x"], [r, c]), "max")
        H.binary_accum(side, View(w["acc"], [c]), 1.0, View(w["x"], [r, c]), 1.0, "+")              # staged sum
        st = w["stats"]
        H.batch_normalize_update_and_apply(side, V(w["out"]), V(w["x"]), V(st[0]), V(st[1]), V(st[2]), V(st[3]), 0.9,
                                           V(st[4]), V(st[5]), 1e-3, r, c)
        H.gemm(side, V(w["gemm"]), c, True, False, 1.0, V(w["x"]), c, r, c, V(w["x"]), c, c, 0.0)    # x^T x

    for w in work:                                  # expected values, serially on the oracle
        for _ in range(rounds):
            run_all(H.ORACLE, w)

    errors = []

    def worker(w):
        try:
            side = H.gpu_side()
            s = C.c_void_p()
            capi.call("ct_set_device", 0)
            capi.call("ct_stream_create", C.byref(s))
            side.stream = s
            for _ in range(rounds):
                run_all(side, w)
            with pytest.raises(capi.CortexHipError, match="float and double"):   # this thread's own error text
                H.softmax(side, View(P_int, [4, 4]), View(P_int, [4, 4]))
            capi.call("ct_stream_destroy", s)
        except BaseException as exc:  # noqa: BLE001 -- reported in the main thread
            errors.append(exc)

    P_int = P.buf(np.zeros(16, np.int32))
    threads = [threading.Thread(target=worker, args=(w,)) for w in work]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for i, w in enumerate(work):
        x64 = np.abs(w["x"].init.astype(np.float64))
        bn_close(w["col"], f"thread {i} column sum", capi.F32, scale_by=x64.sum(axis=None) / c)
        compare(w["row"], f"thread {i} row max")
        bn_close(w["acc"], f"thread {i} accumulated sum", capi.F32, scale_by=rounds * x64.reshape(r, c).sum(axis=0).max())
        bn_close(w["out"], f"thread {i} batch-normalized output", capi.F32)
        got, want = w["gemm"].download().astype(np.float64), w["gemm"].host.astype(np.float64)
        assert np.max(np.abs(got - want)) <= 1e-5 * (x64.reshape(r, c) ** 2).sum(axis=0).max()


def test_thread_exit_releases_blas_handles(P):
    """A host thread's rocBLAS handle (and the device workspace behind it) goes away with the
    thread: a pool that retires threads must not shrink the free device memory thread by thread."""
    import ctypes as C
    import threading

    rng = np.random.default_rng(101)
    m = 64
    a = P.buf(rng.standard_normal(m * m).astype(np.float32))
    out = P.buf(np.zeros(m * m, np.float32))
    errors = []

    def worker():
        try:
            side = H.gpu_side()
            s = C.c_void_p()
            capi.call("ct_set_device", 0)
            capi.call("ct_stream_create", C.byref(s))
            side.stream = s
            V = lambda b: View(b, [b.init.size])
            H.gemm(side, V(out), m, False, False, 1.0, V(a), m, m, m, V(a), m, m, 0.0)
            capi.call("ct_stream_sync", s)
            capi.call("ct_stream_destroy", s)
        except BaseException as exc:  # noqa: BLE001 -- reported in the main thread
            errors.append(exc)

    def free_bytes():
        free, total = C.c_size_t(), C.c_size_t()
        capi.call("ct_memory_info", C.byref(free), C.byref(total))
        return free.value

    def one_thread():
        t = threading.Thread(target=worker)
        t.start()
        t.join()

    one_thread()                      # whatever the first use of the library allocates for good
    before = free_bytes()
    for _ in range(12):
        one_thread()
    assert not errors, errors
    lost = before - free_bytes()
    assert lost < (8 << 20), f"{lost} bytes of device memory did not come back after 12 threads"
