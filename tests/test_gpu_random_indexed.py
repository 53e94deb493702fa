"""Seeded random sweeps of the two kernel families for indexed rows and planar <-> interleaved
layouts against the CPU oracle, bit-exact: accumulation into destinations with one indexed axis
(random rank, position of the indexed axis, padded rows, offsets, broadcast y, every op and
datatype) and assign! between planar and interleaved images (random datatype pairs, 2-5 channels,
padded rows, offsets)."""
import numpy as np
import pytest

import harness as H
from cortex_amd import capi
from harness import View

pytestmark = pytest.mark.gpu
NP = H.NP_DTYPES
ACC_CODES = [capi.F32, capi.F64, capi.I32, capi.I64, capi.I16, capi.I8, capi.U8]
OPS = ["+", "-", "*", "max", "min", "bit-xor", "/", "eq", ">"]


def fill(rng, n, dt, nonzero=False):
    if np.issubdtype(dt, np.floating):
        v = (rng.standard_normal(n) * 2).astype(dt)
        return np.where(np.abs(v) < 0.05, 0.5, v).astype(dt) if nonzero else v
    v = rng.integers(-9 if np.dtype(dt).kind == "i" else 0, 10, n).astype(dt)
    return np.where(v == 0, 3, v).astype(dt) if nonzero else v


def same_bits(got, want):
    if got.dtype.kind == "f":
        return bool(np.all((got == want) | ((got != got) & (want != want))))
    return bool(np.array_equal(got, want))


@pytest.mark.parametrize("seed", [101, 102, 103])
def test_random_accumulate_into_an_indexed_axis(pair_factory, seed):
    rng = np.random.default_rng(seed)
    kernels = {}
    with pair_factory() as P:
        for it in range(120):
            code = int(rng.choice(ACC_CODES))
            dt = NP[code]
            nd = int(rng.integers(1, 4))
            shape = [int(rng.choice([1, 2, 3, 4, 8, 16, 33, 64])) for _ in range(nd)]
            gi = int(rng.integers(0, nd))
            shape[gi] = int(rng.choice([1, 2, 5, 40, 300, 9000 if rng.random() < 0.3 else 77]))
            if rng.random() < 0.4 and gi != nd - 1:
                shape[-1] = int(rng.choice([4, 8, 16, 128]))
            while np.prod(shape) > 400_000:
                j = int(rng.integers(0, nd))
                shape[j] = max(1, shape[j] // 2)
            extent = int(rng.integers(1, shape[gi] + 3))
            table_shape = list(shape)
            table_shape[gi] = extent
            pad = int(rng.choice([0, 0, 4, 3]))
            strides, run = [0] * nd, 1
            for d in reversed(range(nd)):
                strides[d] = run
                run *= table_shape[d]
                if d == nd - 1:
                    run += pad
            off = int(rng.choice([0, 0, 4, 1]))
            idx = P.buf(rng.integers(0, extent, shape[gi]).astype(np.int32))
            op = str(rng.choice(OPS))
            if op == "bit-xor" and np.issubdtype(dt, np.floating):
                op = "+"
            table = P.buf(fill(rng, run + off, dt, nonzero=(op == "/")))
            index = [None] * nd
            index[gi] = idx
            dest = View(table, shape, strides, off, index)
            yshape = [s if rng.random() < 0.8 else 1 for s in shape]
            y = View(P.buf(fill(rng, int(np.prod(yshape)), dt, nonzero=(op == "/"))), yshape)
            da = float(rng.choice([1.0, 1.0, 0.5, 2.0])) if op != "/" else 1.0
            ya = float(rng.choice([1.0, -1.0, 2.0]))
            rev = bool(rng.integers(0, 2))
            what = f"case {it}: {op} dtype {code} shape {shape} indexed axis {gi} extent {extent} pad {pad} offset {off} " \
                   f"y {yshape} dest_alpha {da} y_alpha {ya} reverse {rev}"
            try:
                k = P.run(H.binary_accum, dest, da, y, ya, op, reverse=rev, requires_cas=True)
            except (capi.CortexHipError, H.OracleError) as err:
                assert "Divide by zero" in str(err), what      # an integer quotient reached zero on the way
                table.reset()
                continue
            assert same_bits(table.download(), table.host), f"{what} ({k})"
            kernels[k] = kernels.get(k, 0) + 1
            if it % 40 == 39:
                P.close()
    assert set(kernels) <= {"accum_grouped", "accum_grouped_vec"}, kernels
    assert kernels.get("accum_grouped_vec", 0) > 0


@pytest.mark.parametrize("seed", [201, 202])
def test_random_planar_and_interleaved_assigns(pair_factory, seed):
    rng = np.random.default_rng(seed)
    kernels = {}
    with pair_factory() as P:
        for it in range(150):
            src, dst = int(rng.choice(H.ALL_DTYPES)), int(rng.choice(H.ALL_DTYPES))
            c = int(rng.choice([2, 3, 4, 5]))
            n, h = int(rng.choice([1, 2, 5])), int(rng.choice([1, 3, 8, 17]))
            w = int(rng.choice([4, 15, 16, 64, 100, 256]))
            extra = int(rng.choice([0, 0, 4, 5]))
            off = int(rng.choice([0, 0, 4, 1]))
            wp = w + extra
            count = n * c * h * wp + off + 8
            st, dt = NP[src], NP[dst]
            data = (rng.standard_normal(count) * 100).astype(st) if np.issubdtype(st, np.floating) else \
                rng.integers(-100, 101, count).astype(st)
            a, o = P.buf(data), P.buf(np.zeros(count, dt))
            if rng.integers(0, 2) == 0:   # planar (rows possibly padded) <- interleaved
                dest = View(o, [n, c, h, w], [c * h * wp, h * wp, wp, 1], offset=off)
                source = View(a, [n, c, h, w], [h * w * c, 1, w * c, c])
            else:                         # interleaved <- planar (rows possibly padded)
                dest = View(o, [n, h, w, c])
                source = View(a, [n, h, w, c], [c * h * wp, wp, 1, h * wp], offset=off)
            k = P.run(H.assign, dest, source)
            assert same_bits(o.download(), o.host), \
                f"case {it}: {src}->{dst} n {n} c {c} h {h} w {w} row padding {extra} offset {off} ({k})"
            kernels[k] = kernels.get(k, 0) + 1
            if it % 50 == 49:
                P.close()
    assert kernels.get("lace", 0) > 0 and kernels.get("lace1", 0) > 0, kernels
