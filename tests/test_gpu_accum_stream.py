"""binary-accum! into a broadcast destination with operations and multipliers that have no staged form
(anything but :+ / :max / :min with dest_alpha 1): the streamed kernels, in which a block stages the
updates of a strip of destination elements through LDS and one lane per destination element applies
them in increasing e (src/cortex/compute/cpu/tensor_math.clj:386-420).  Every step rounds to the tensor's
datatype, so the bar is bit-exact against the serial loop of the oracle, for every datatype."""
import numpy as np
import pytest

import harness as H
from cortex_amd import capi
from harness import View

pytestmark = pytest.mark.gpu

NP = H.NP_DTYPES
FLOATS = (capi.F32, capi.F64)


@pytest.fixture()
def P(pair_factory):
    with pair_factory() as pair:
        yield pair


def exact(buf, what):
    H.assert_bit_exact(buf.download(), buf.host, what)


# (destination shape, destination strides, y shape, y strides, arrangement the streamed kernel sees)
#   "chains": neighbouring destination elements are neighbours in y (rows summed into a vector)
#   "steps":  a destination element's updates are contiguous in y (each row into one element)
LAYOUTS = [
    ([96], None, [400, 96], None, "chains"),                    # three full strips of floats, four tiles
    ([208], None, [3000, 208], None, "chains"),                 # a partial last strip, more tiles than are kept in flight
    ([4, 1, 64], None, [4, 700, 64], None, "chains"),           # a kept axis outside the broadcast one
    ([48], [3], [700, 48], [64, 1], "chains"),                  # strided destination, padded rows of y
    ([32, 1], None, [32, 900], [1, 32], "chains"),              # y is a transposed view
    ([16], None, [129, 16], None, "chains"),                    # one row more than a tile
    ([300, 1], None, [300, 160], None, "steps"),                # each row into one element
    ([6, 1, 1], None, [8, 6, 24, 24], None, "steps"),           # per-channel accumulate over batch and pixels
    ([1], None, [40000], None, "steps"),                        # one chain over everything
    ([7, 1], None, [7, 5008], None, "steps"),                   # long rows: more tiles than are kept in flight
    ([3, 5, 1], [40, 8, 1], [3, 5, 1040], None, "steps"),       # two kept axes, strided destination
    ([40, 1], None, [40, 144], [160, 1], "steps"),              # padded rows
]


def chain_values(rng, code, n):
    """Updates that keep a chain of products, quotients or sums inside the type's range for thousands of steps."""
    if code in FLOATS:
        return (1.0 + 0.05 * rng.standard_normal(n)).astype(NP[code])
    v = rng.integers(-9, 10, n)
    return np.where(v == 0, 3, v).astype(NP[code])


def ops_for(code):
    if code in FLOATS:
        return [("*", 1.0, 1.0, False), ("/", 1.0, 1.0, False), ("/", 1.0, -1.0, True), ("-", 1.0, 1.0, True),
                ("+", 0.9, 1.0, False), ("*", 1.0, 0.5, True), ("min", 0.5, 1.0, False), ("max", 2.0, -1.0, True),
                (">=", 1.0, 1.0, False), ("+", -1.0, 2.0, False), ("-", 0.5, 2.0, True), ("-", 0.75, -0.5, False),
                ("+", 0.9, 3.0, True)]
    return [("*", 1.0, 1.0, False), ("/", 1.0, 1.0, False), ("-", 1.0, 1.0, True), ("+", 3.0, 1.0, False),
            ("bit-xor", 1.0, 1.0, False), ("bit-and", 1.0, 7.0, True), ("max", 1.0, 3.0, False), ("<", 1.0, 1.0, True)]


@pytest.mark.parametrize("code", H.ALL_DTYPES)
def test_streamed_chains_are_serial_exact(P, code):
    rng = np.random.default_rng(91)
    for dshape, dstrides, yshape, ystrides, arrangement in LAYOUTS:
        y_elems = 1 + sum((s - 1) * st for s, st in zip(yshape, ystrides)) if ystrides else int(np.prod(yshape))
        d_elems = 1 + sum((s - 1) * st for s, st in zip(dshape, dstrides)) if dstrides else int(np.prod(dshape))
        y = P.buf(chain_values(rng, code, y_elems))
        d = P.buf(chain_values(rng, code, d_elems))
        for op, da, ya, rev in ops_for(code):
            k = P.run(H.binary_accum, View(d, dshape, dstrides), da, View(y, yshape, ystrides), ya, op, reverse=rev,
                      requires_cas=True)
            exact(d, f"{op} da={da} ya={ya} reverse={rev} {dshape}<-{yshape} ({k})")
            want = "accum_stream" + ("_steps" if arrangement == "steps" else "")
            plain = code == capi.F32 and da == 1.0 and abs(ya) == 1.0
            assert k == want + ("_plain" if plain else ""), (k, want, dshape, yshape)
            d.reset()


@pytest.mark.parametrize("code", FLOATS)
def test_streamed_chains_with_nan_infinity_and_signed_zero(P, code):
    """The order of the updates decides what a NaN, an infinity or a zero of either sign leaves behind."""
    rng = np.random.default_rng(92)
    rows, cols = 1500, 64
    yv = (rng.standard_normal(rows * cols) * 3).astype(NP[code])
    yv[rng.integers(0, rows * cols, 40)] = np.nan
    yv[rng.integers(0, rows * cols, 40)] = np.inf
    yv[rng.integers(0, rows * cols, 40)] = -np.inf
    yv[rng.integers(0, rows * cols, 4000)] = 0.0
    yv[rng.integers(0, rows * cols, 4000)] = -0.0
    y = P.buf(yv)
    dv = rng.standard_normal(cols).astype(NP[code])
    dv[::9] = -0.0
    d = P.buf(dv)
    for op, da, ya, rev in (("max", 0.5, 0.5, False), ("min", 2.0, 1.0, True), ("*", 1.0, 1.0, False), ("/", 1.0, 1.0, True),
                            ("+", 0.5, 1.0, False), ("<=", 1.0, 1.0, False)):
        k = P.run(H.binary_accum, View(d, [cols]), da, View(y, [rows, cols]), ya, op, reverse=rev, requires_cas=True)
        exact(d, f"{op} da={da} ya={ya} reverse={rev} with special values ({k})")
        assert k.startswith("accum_stream"), k
        d.reset()
    # the same updates as rows: steps unit-stride
    d2 = P.buf(rng.standard_normal(cols).astype(NP[code]))
    for op, da, ya, rev in (("*", 1.0, 1.0, False), ("min", 2.0, 1.0, True), ("-", 1.0, 1.0, True)):
        k = P.run(H.binary_accum, View(d2, [cols, 1]), da, View(y, [cols, rows]), ya, op, reverse=rev, requires_cas=True)
        exact(d2, f"{op} rows with special values ({k})")
        assert k.startswith("accum_stream_steps"), k
        d2.reset()


@pytest.mark.parametrize("code", [capi.I32, capi.I8])
def test_streamed_integer_division_by_zero(P, code):
    """A zero among the divisors stores 0 for that step, as everywhere in the library; with debug-sync on the call
    reports it."""
    rng = np.random.default_rng(93)
    rows, cols = 400, 64
    yv = chain_values(rng, code, rows * cols)
    y = P.buf(yv)
    d = P.buf((rng.integers(1, 100, cols)).astype(NP[code]))
    k = P.run(H.binary_accum, View(d, [cols]), 1.0, View(y, [rows, cols]), 1.0, "/", requires_cas=True)
    assert k == "accum_stream", k
    exact(d, "integer division chain")
    yv = yv.copy()
    yv[77 * cols + 5] = 0
    y0 = P.buf(yv)
    d.reset()
    with pytest.raises(H.OracleError, match="Divide by zero"):
        H.binary_accum(H.ORACLE, View(d, [cols]), 1.0, View(y0, [rows, cols]), 1.0, "/", requires_cas=True)
    with pytest.raises(capi.CortexHipError, match="Divide by zero"):
        H.binary_accum(P.hip, View(d, [cols]), 1.0, View(y0, [rows, cols]), 1.0, "/", requires_cas=True)
    want = d.init.astype(np.int64).copy()
    for r in range(rows):                       # Java's long division truncates toward zero; a zero divisor leaves 0
        row = yv[r * cols:(r + 1) * cols].astype(np.int64)
        safe = np.where(row == 0, 1, row)
        q = np.abs(want) // np.abs(safe) * np.sign(want) * np.sign(safe)
        want = np.where(row == 0, 0, q)
    assert np.array_equal(d.download(), want.astype(NP[code]))


def test_short_chains_keep_the_lane_per_element_kernel(P):
    """Few updates per destination element, or very many destination elements: one lane per element has
    lanes enough and reads neighbouring addresses."""
    rng = np.random.default_rng(94)
    y = P.buf(chain_values(rng, capi.F32, 64 * 4096))
    d = P.buf(chain_values(rng, capi.F32, 4096))
    k = P.run(H.binary_accum, View(d, [4096]), 1.0, View(y, [64, 4096]), 1.0, "*", requires_cas=True)
    assert k == "accum_owner", k
    exact(d, "64 updates per element")


@pytest.mark.parametrize("seed", [301, 302])
def test_random_broadcast_destinations(pair_factory, seed):
    """A seeded sweep over destination and update layouts (dense, padded rows, permuted views, strided and
    stride-0 destinations), every datatype, operations and multipliers of either sign, operands in either
    order: whichever kernel takes the call (one lane per element, staged, streamed), the destination must hold
    what the serial loop leaves, bit for bit; only a float :+ with dest_alpha 1 keeps the reference's 1e-4."""
    rng = np.random.default_rng(seed)
    kernels = {}

    def fill(n, dt):
        if np.issubdtype(dt, np.floating):
            return (1.0 + 0.02 * rng.standard_normal(n)).astype(dt)
        v = rng.integers(-3, 4, n)
        return np.where(v == 0, 1, v).astype(dt)

    for it in range(500):
        with pair_factory() as P:
            code = int(rng.choice(H.ALL_DTYPES))
            dt = NP[code]
            nd = int(rng.integers(2, 5))
            yshape = [int(rng.choice([1, 2, 3, 5, 8, 17, 33, 64, 130, 257, 700])) for _ in range(nd)]
            while np.prod(yshape) > 400_000:
                yshape[int(np.argmax(yshape))] //= 2
            dshape = [s if rng.random() < 0.4 else 1 for s in yshape]
            mode = int(rng.integers(0, 3))
            ystr = None
            if mode == 1:
                pad, run, ystr = int(rng.choice([0, 1, 4, 16])), 1, [0] * nd
                for d in reversed(range(nd)):
                    ystr[d] = run
                    run *= yshape[d] + (pad if d == nd - 1 else 0)
            elif mode == 2:
                run, ystr = 1, [0] * nd
                for d in rng.permutation(nd):
                    ystr[d] = run
                    run *= yshape[d]
            y_elems = 1 + sum((s - 1) * st for s, st in zip(yshape, ystr)) if ystr else int(np.prod(yshape))
            dstr = None
            if rng.random() < 0.3:
                mult, run, dstr = int(rng.choice([2, 3])), 1, [0] * nd
                for d in reversed(range(nd)):
                    dstr[d] = run * mult if dshape[d] > 1 else (0 if rng.random() < 0.5 else run * mult)
                    run *= dshape[d]
            d_elems = 1 + sum((s - 1) * st for s, st in zip(dshape, dstr)) if dstr else int(np.prod(dshape))
            floating = code in FLOATS
            ops = ["*", "/", "-", "+", "max", "min", ">=", "eq"] if floating else ["*", "-", "+", "bit-xor", "bit-and", "max", "<"]
            op = str(rng.choice(ops))
            da = float(rng.choice([1.0, 1.0, 0.9, -1.0, 2.0] if floating else [1.0, 1.0, 3.0, -1.0]))
            ya = float(rng.choice([1.0, 1.0, -1.0, 0.5] if floating else [1.0, -1.0, 2.0]))
            rev = bool(rng.integers(0, 2))
            y = View(P.buf(fill(y_elems, dt)), yshape, ystr)
            d = P.buf(fill(d_elems, dt))
            what = f"case {it}: {op} dtype {code} y {yshape} {ystr} dest {dshape} {dstr} da={da} ya={ya} reverse={rev}"
            k = P.run(H.binary_accum, View(d, dshape, dstr), da, y, ya, op, reverse=rev, requires_cas=True)
            kernels[k] = kernels.get(k, 0) + 1
            if k == "accum_staged_sum" and floating:
                reps = np.prod(yshape) / max(1, np.prod(dshape))
                got, want = d.download().astype(np.float64), d.host.astype(np.float64)
                assert np.all(np.abs(got - want) <= 1e-4 * (np.abs(want) + reps)), what
            else:
                H.assert_bit_exact(d.download(), d.host, what + f" ({k})")
    streamed = sum(v for k, v in kernels.items() if k.startswith("accum_stream"))
    assert streamed >= 40 and kernels.get("accum_owner", 0) >= 100, kernels
