"""Seeded random sweep of calls over rows that sit off the 16-byte grid, at sizes that take the
vector kernels (ew_ragged_kernel, ew_vecu_kernel) rather than the one-element-per-lane forms the
small random-view sweeps reach: random datatype, row length, pitch, offset, number of outer axes,
per-row / bias-row / constant / dense second operands, in place or not, every binary op, select and
conversions.  Against the CPU oracle, bit for bit."""
import numpy as np
import pytest

import harness as H
from cortex_amd import capi
from harness import View

pytestmark = pytest.mark.gpu
NP = H.NP_DTYPES
CODES = [capi.F32, capi.F64, capi.I32, capi.I64, capi.I16, capi.I8, capi.U8]
OPS = ["+", "-", "*", "max", "min", "bit-and", "/", "eq", "<="]


def fill(rng, n, dt, nonzero=False):
    if np.issubdtype(dt, np.floating):
        v = (rng.standard_normal(n) * 2).astype(dt)
        return np.where(np.abs(v) < 0.05, 0.5, v).astype(dt) if nonzero else v
    v = rng.integers(-9 if np.dtype(dt).kind == "i" else 0, 10, n).astype(dt)
    return np.where(v == 0, 3, v).astype(dt) if nonzero else v


@pytest.mark.parametrize("seed", [201, 202, 203])
def test_random_rows_off_the_vector_grid(pair_factory, seed):
    rng = np.random.default_rng(seed)
    kernels = {}
    with pair_factory() as P:
        for it in range(90):
            code = int(rng.choice(CODES))
            dt = NP[code]
            vmax = 16 // dt().itemsize
            width = int(rng.integers(vmax, 6 * vmax + 40))
            outer = [int(rng.choice([1, 2, 3, 7, 24, 130])) for _ in range(int(rng.integers(1, 4)))]
            while np.prod(outer) * width < 6000:
                outer[int(rng.integers(0, len(outer)))] *= 3
            while np.prod(outer) * width > 600_000:
                j = int(np.argmax(outer))
                outer[j] = max(1, outer[j] // 2)
            shape = outer + [width]
            dense = rng.random() < 0.5
            pitch = width if dense else width + int(rng.choice([0, 1, 3, 4, vmax]))
            offset = 0 if dense and rng.random() < 0.7 else int(rng.choice([0, 1, 3, vmax]))
            strides, run = [0] * len(shape), 1
            for d in reversed(range(len(shape))):
                strides[d] = run
                run = run * shape[d] if d != len(shape) - 1 else pitch
            span = strides[0] * shape[0] + offset + 8
            op = str(rng.choice(OPS))
            if op == "bit-and" and np.issubdtype(dt, np.floating):
                op = "-"
            big = lambda buf: View(buf, shape, strides, offset)
            x = P.buf(fill(rng, span, dt))
            dest = x if rng.random() < 0.3 else P.buf(np.zeros(span, dt))
            kind = str(rng.choice(["dense", "per-row", "bias-row", "constant", "channel"]))
            if kind == "channel" and len(shape) < 3:
                kind = "per-row"
            nz = op == "/"
            if kind == "dense":
                y = big(P.buf(fill(rng, span, dt, nonzero=nz)))
            elif kind == "per-row":
                y = View(P.buf(fill(rng, int(np.prod(outer)), dt, nonzero=nz)), outer + [1])
            elif kind == "bias-row":
                y = View(P.buf(fill(rng, width, dt, nonzero=nz)), [width])
            elif kind == "channel":
                y = View(P.buf(fill(rng, shape[-2], dt, nonzero=nz)), [shape[-2], 1])
            else:
                y = None
            xa, ya = float(rng.choice([1.0, -1.0, 2.0])), float(rng.choice([1.0, 1.0, 3.0]))
            what = f"case {it}: {op} dtype {code} shape {shape} strides {strides} offset {offset} second operand {kind} " \
                   f"alphas {xa} {ya} in place {dest is x}"
            try:
                if y is None:
                    k = P.run(H.binary_op_constant, big(dest), big(x), xa, 3.0, op, reverse=bool(rng.integers(0, 2)))
                elif rng.random() < 0.2 and kind != "dense":
                    k = P.run(H.ternary_op, big(dest), y, 1.0, big(x), xa, y, ya)
                else:
                    k = P.run(H.binary_op, big(dest), big(x), xa, y, ya, op)
            except (capi.CortexHipError, H.OracleError) as err:
                assert "Divide by zero" in str(err), what
                continue
            kernels[k] = kernels.get(k, 0) + 1
            H.assert_bit_exact(dest.download(), dest.host, what + f" ({k})")
            # a conversion out of the same rows
            other = NP[int(rng.choice(CODES))]
            conv = P.buf(np.zeros(int(np.prod(shape)), other))
            k = P.run(H.assign, View(conv, shape), big(dest))
            kernels[k] = kernels.get(k, 0) + 1
            H.assert_bit_exact(conv.download(), conv.host, what + f" then assign to {other.__name__} ({k})")
    assert kernels.get("vecu", 0) > 10 and kernels.get("ragged", 0) > 5, kernels
