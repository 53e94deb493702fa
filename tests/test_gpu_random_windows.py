"""Randomized parity of the windowed methods: pooling over random geometries (windows 1-5,
rectangular, strides 1-3, both rounding rules, three pool ops, both directions) bit-exact
against the CPU oracle, convolution with integer-valued operands (every product and sum
exact, so the three methods must agree to the bit whatever order the products sum in).
Seeds are fixed.  Needs a GPU."""
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


def out_dim(n, pad, k, stride, op):
    v = (n + 2.0 * pad - k) / stride
    return int((np.floor(v) if op == "floor" else np.ceil(v)) + 1)


@pytest.mark.parametrize("seed", range(3))
def test_random_pooling_geometries(P, seed):
    rng = np.random.default_rng(3000 + seed)
    for case in range(50):
        code = capi.F32 if rng.random() < 0.7 else capi.F64
        dt = H.NP_DTYPES[code]
        if rng.random() < 0.7:
            kw = kh = int(rng.integers(1, 5))
        else:
            kw, kh = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        px, py = int(rng.integers(0, kw)), int(rng.integers(0, kh))
        sx, sy = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        h, w = int(rng.integers(max(1, kh - 2 * py), 90)), int(rng.integers(max(1, kw - 2 * px), 150))
        if rng.random() < 0.3:
            w = (w + 3) // 4 * 4
        batch, channels = int(rng.integers(1, 4)), int(rng.integers(1, 6))
        dim_op = "floor" if rng.random() < 0.5 else "ceil"
        oh, ow = out_dim(h, py, kh, sy, dim_op), out_dim(w, px, kw, sx, dim_op)
        if oh < 1 or ow < 1:
            continue
        op = ["max", "avg", "avg-exc-pad"][int(rng.integers(0, 3))]
        n_in, n_out = batch * channels * h * w, batch * channels * oh * ow
        x = rng.integers(-4, 5, n_in).astype(dt) if op == "max" else (rng.standard_normal(n_in) * 3).astype(dt)
        inp, out = P.buf(x), P.buf(rng.standard_normal(n_out).astype(dt))
        og, ig = P.buf(rng.standard_normal(n_out).astype(dt)), P.buf(rng.standard_normal(n_in).astype(dt))
        geom = (H.pool_desc(kw, kh, px, py, sx, sy, op), batch, channels, h, w, oh, ow)
        what = f"seed {seed} case {case} {op} dtype {code} [{batch},{channels},{h},{w}] window {kw}x{kh} pad {px},{py} " \
               f"stride {sx},{sy} {dim_op}"
        k = P.run(H.pooling_forward, View(out, [n_out]), View(inp, [n_in]), *geom)
        H.assert_bit_exact(out.download(), out.host, f"forward {what} ({k})")
        k = P.run(H.pooling_backward, View(ig, [n_in]), View(inp, [n_in]), View(out, [n_out]), View(og, [n_out]), *geom)
        H.assert_bit_exact(ig.download(), ig.host, f"backward {what} ({k})")
        P.close()


@pytest.mark.parametrize("seed", range(2))
def test_random_convolution_geometries(P, seed):
    rng = np.random.default_rng(4000 + seed)
    V = lambda b: View(b, [b.init.size])
    for case in range(25):
        dt = np.float32
        k = int(rng.integers(1, 6))
        pad, stride = int(rng.integers(0, k)), int(rng.integers(1, 3))
        h, w = int(rng.integers(k, 40)), int(rng.integers(k, 60))
        if rng.random() < 0.4:
            w = (w + 3) // 4 * 4
        batch, cin, cout = int(rng.integers(1, 4)), int(rng.integers(1, 9)), int(rng.integers(1, 9))
        oh, ow = (h + 2 * pad - k) // stride + 1, (w + 2 * pad - k) // stride + 1
        n_cols, n_rows = cin * k * k, oh * ow
        geom = (H.conv_desc(cin, cout, k, k, pad, pad, stride, stride), batch, h, w, oh, ow)
        inp = P.buf(rng.integers(-3, 4, batch * cin * h * w).astype(dt))
        weights = P.buf(rng.integers(-3, 4, cout * n_cols).astype(dt))
        og = P.buf(rng.integers(-3, 4, batch * cout * n_rows).astype(dt))
        out, work = P.buf(np.ones(batch * cout * n_rows, dt)), P.buf(np.zeros(batch * n_rows * n_cols, dt))
        wg, ig = P.buf(np.ones(cout * n_cols, dt)), P.buf(np.ones(batch * cin * h * w, dt))
        what = f"seed {seed} case {case} [{batch},{cin}->{cout},{h},{w}] window {k} pad {pad} stride {stride}"
        P.run(H.convolution, "forward", V(out), 0.0, V(inp), V(weights), V(work), *geom)
        P.run(H.convolution, "backward_weights", V(wg), 0.0, V(og), V(inp), V(work), *geom)
        P.run(H.convolution, "backward_data", V(ig), 0.0, V(og), V(weights), V(work), *geom)
        for b, name in ((out, "output"), (wg, "weight gradient"), (ig, "input gradient")):
            H.assert_bit_exact(b.download(), b.host, f"{name} {what}")
        P.close()
