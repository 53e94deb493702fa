"""Randomized parity of the elementwise path: random ranks, broadcast and commensurate operand
shapes, permuted storage orders, padded rows, offsets and indirectly addressed dimensions, the
library against the CPU oracle to the bit.  Seeds are fixed; every case prints nothing unless
it fails, and then names its seed, datatype and views.  Needs a GPU."""
import numpy as np
import pytest

import harness as H
from cortex_amd import capi
from harness import View

pytestmark = pytest.mark.gpu

CODES = [capi.F32, capi.F32, capi.F64, capi.I32, capi.I16, capi.I64, capi.I8, capi.U8]


@pytest.fixture()
def P(pair_factory):
    with pair_factory() as pair:
        yield pair


def fill(rng, n, code):
    dt = H.NP_DTYPES[code]
    if np.issubdtype(dt, np.floating):
        return (rng.standard_normal(n) * 3).astype(dt)
    info = np.iinfo(dt)
    return rng.integers(max(-50, info.min), min(50, info.max) + 1, n).astype(dt)


def random_view(P, rng, max_shape, code, dest=False):
    """A view over a fresh buffer whose shape divides max_shape (equals it for a destination)."""
    shape = list(max_shape)
    if not dest:
        for d in range(len(shape)):
            r = rng.random()
            if r < 0.3:
                shape[d] = 1
            elif r < 0.4:
                shape[d] = int(rng.choice([v for v in range(1, max_shape[d] + 1) if max_shape[d] % v == 0]))
        if rng.random() < 0.3:
            shape = shape[int(rng.integers(0, len(shape))):]       # fewer dimensions than the destination
    nd = len(shape)
    order = list(rng.permutation(nd)) if rng.random() < 0.4 else list(range(nd))   # storage order, slowest first
    strides, run = [0] * nd, 1
    for pos, d in enumerate(reversed(order)):
        strides[d] = run
        run *= shape[d]
        if pos == 0 and rng.random() < 0.3:
            run += int(rng.integers(1, 5))                          # padded rows
    offset = int(rng.integers(0, 5)) if rng.random() < 0.4 else 0
    size = offset + sum((s - 1) * st for s, st in zip(shape, strides)) + 1
    return View(P.buf(fill(rng, size, code)), shape, strides, offset)


def indexed_view(P, rng, shape, code, unique):
    """A view of `shape` into a larger table; about half of its dimensions go through index tensors."""
    table_shape, index = [], []
    for extent in shape:
        if rng.random() < 0.5:
            rows = extent + int(rng.integers(0, 6))
            idx = rng.permutation(rows)[:extent] if unique else rng.integers(0, rows, extent)
            table_shape.append(rows)
            index.append(P.buf(idx.astype(np.int32)))
        else:
            table_shape.append(extent)
            index.append(None)
    strides, run = [0] * len(shape), 1
    for d in reversed(range(len(shape))):
        strides[d] = run
        run *= table_shape[d]
    return View(P.buf(fill(rng, int(np.prod(table_shape)), code)), shape, strides, 0, index)


def random_max_shape(rng):
    nd = int(rng.integers(1, 5))
    shape = [int(rng.choice([1, 2, 3, 4, 5, 7, 8, 16, 33, 64, 100])) for _ in range(nd)]
    if rng.random() < 0.2:
        shape[-1] = int(rng.choice([256, 1000, 4096]))
    while np.prod(shape) > 500_000:
        shape[int(rng.integers(0, nd))] = 2
    return shape


@pytest.mark.parametrize("seed", range(4))
def test_random_views(P, seed):
    rng = np.random.default_rng(1000 + seed)
    for case in range(60):
        code = CODES[int(rng.integers(0, len(CODES)))]
        max_shape = random_max_shape(rng)
        dest = random_view(P, rng, max_shape, code, dest=True)
        kind = int(rng.integers(0, 6))
        scalar = float(rng.choice([2.0, -3.0, 0.0, 1.5]))
        bop = ["+", "*", "max", "min", "-", ">", "eq"][int(rng.integers(0, 7))]
        if kind == 0:
            k = P.run(H.binary_op, dest, random_view(P, rng, max_shape, code), 1.0, random_view(P, rng, max_shape, code),
                      float(rng.choice([1.0, -1.0, 2.0])), bop)
        elif kind == 1:
            k = P.run(H.unary_op, dest, random_view(P, rng, max_shape, code), float(rng.choice([1.0, 2.0])),
                      ["floor", "-", "noop", "ceil"][int(rng.integers(0, 4))])
        elif kind == 2:
            k = P.run(H.ternary_op, dest, random_view(P, rng, max_shape, code), 1.0,
                      random_view(P, rng, max_shape, code), 1.0, random_view(P, rng, max_shape, code), 1.0)
        elif kind == 3:
            k = P.run(H.assign, dest, random_view(P, rng, max_shape, CODES[int(rng.integers(0, len(CODES)))]))
        elif kind == 4:
            k = P.run(H.binary_op_constant, dest, random_view(P, rng, max_shape, code), 1.0, scalar, bop,
                      reverse=bool(rng.integers(0, 2)))
        else:
            k = P.run(H.binary_op, dest, dest, 1.0, random_view(P, rng, max_shape, code), 1.0, bop)   # in place
        H.assert_bit_exact(dest.buf.download(), dest.buf.host,
                           f"seed {seed} case {case} kind {kind} {bop} dtype {code} max-shape {max_shape} ({k})")
        P.close()


@pytest.mark.parametrize("seed", range(3))
def test_random_indirect_dimensions(P, seed):
    rng = np.random.default_rng(2000 + seed)
    for case in range(60):
        code = [capi.F32, capi.F64, capi.I32, capi.I16, capi.I64][int(rng.integers(0, 5))]
        shape = [int(rng.choice([1, 1, 2, 3, 5, 8, 16, 40])) for _ in range(int(rng.integers(1, 4)))]
        kind = int(rng.integers(0, 3))
        if kind == 0:      # gather through indexed inputs
            dest = View(P.buf(np.zeros(int(np.prod(shape)), H.NP_DTYPES[code])), shape)
            P.run(H.binary_op, dest, indexed_view(P, rng, shape, code, False), 1.0,
                  indexed_view(P, rng, shape, code, False), 1.0, "+")
        elif kind == 1:    # scatter through distinct indexes
            dest = indexed_view(P, rng, shape, code, True)
            P.run(H.assign, dest, indexed_view(P, rng, shape, code, False))
        else:              # an indexed operand broadcast against a larger one
            big = [int(rng.choice([2, 3, 4]))] + shape
            dest = View(P.buf(np.zeros(int(np.prod(big)), H.NP_DTYPES[code])), big)
            P.run(H.binary_op, dest, View(P.buf(fill(rng, int(np.prod(big)), code)), big), 1.0,
                  indexed_view(P, rng, shape, code, False), 1.0, "*")
        H.assert_bit_exact(dest.buf.download(), dest.buf.host, f"seed {seed} case {case} kind {kind} dtype {code} {shape}")
        P.close()
