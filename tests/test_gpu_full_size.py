"""The benchmark configurations at their full sizes on the GPU: compared with the
CPU oracle where it finishes in seconds, and through size-independent
properties (closed forms, a checksum of checksums, selection consistency).
Inputs: numpy default_rng(seed), generated in float64 and cast.  Needs a GPU.
"""
import ctypes as C

import numpy as np
import pytest

from cortex_amd import capi
from oracle import binding as ob

pytestmark = pytest.mark.gpu


class Dev:
    """A device array holding a copy of a host array."""

    def __init__(self, host: np.ndarray):
        self.host = np.ascontiguousarray(host).reshape(-1)
        p = C.c_void_p()
        capi.call("ct_malloc", C.byref(p), max(1, self.host.nbytes))
        self.ptr = p.value
        capi.call("ct_memcpy_async", self.ptr, self.host.ctypes.data, self.host.nbytes, capi.COPY_H2D, None)
        capi.call("ct_stream_sync", None)

    def download(self) -> np.ndarray:
        out = np.empty_like(self.host)
        capi.call("ct_stream_sync", None)
        capi.call("ct_memcpy_async", out.ctypes.data, self.ptr, out.nbytes, capi.COPY_D2H, None)
        capi.call("ct_stream_sync", None)
        return out

    def free(self):
        capi.call("ct_free", self.ptr)


@pytest.fixture(autouse=True)
def device():
    capi.call("ct_set_device", 0)
    capi.call("ct_set_debug_sync", 1)
    yield


def dims(shape, strides=None):
    if strides is None:
        strides, m = [], 1
        for s in reversed(shape):
            strides.insert(0, m)
            m *= s
    return capi.make_dims(shape, strides)


def bits_equal(a, b) -> bool:
    return bool(np.array_equal(a.view(f"u{a.itemsize}"), b.view(f"u{b.itemsize}")))


def test_config0_bias_add():
    rng = np.random.default_rng(0)
    x = rng.uniform(-1, 1, (1024, 1024)).astype(np.float32)
    b = rng.uniform(-1, 1, 1024).astype(np.float32)
    dx, db, dd = Dev(x), Dev(b), Dev(np.zeros_like(x))
    capi.call("ct_binary_op", None, dd.ptr, C.byref(dims([1024, 1024])), dx.ptr, C.byref(dims([1024, 1024])), 1.0, db.ptr,
              C.byref(dims([1024])), 1.0, 1024 * 1024, capi.BINARY_OPS["+"], capi.F32)
    got = dd.download().reshape(1024, 1024)
    assert capi.last_kernel() == "vec"
    assert bits_equal(got, x + b[None, :])  # one float add per element is the closed form
    want = np.zeros(1024 * 1024, np.float32)
    ob.call("binary_op", want.ctypes.data, C.byref(dims([1024, 1024])), x.ctypes.data, C.byref(dims([1024, 1024])), 1.0,
            b.ctypes.data, C.byref(dims([1024])), 1.0, 1024 * 1024, capi.BINARY_OPS["+"], capi.F32)
    assert bits_equal(got.reshape(-1), want)
    for t in (dx, db, dd):
        t.free()


def test_config1_transposed_views_8192():
    n = 8192
    hosts = [np.random.default_rng(seed).standard_normal(n * n).astype(np.float32) for seed in (1, 2, 3)]
    devs = [Dev(h) for h in hosts]
    dest = Dev(np.zeros(n * n, np.float32))
    cont, view = dims([n, n]), dims([n, n], [1, n])
    want = np.zeros(n * n, np.float32)
    for op in ("exp", "tanh"):
        capi.call("ct_unary_op", None, dest.ptr, C.byref(cont), devs[0].ptr, C.byref(view), 1.0, capi.UNARY_OPS[op],
                  capi.F32, n * n)
        assert capi.last_kernel() == "tile"
        got = dest.download()
        ob.call("unary_op", want.ctypes.data, C.byref(cont), hosts[0].ctypes.data, C.byref(view), 1.0, capi.UNARY_OPS[op],
                capi.F32, n * n)
        rel = np.abs(got.astype(np.float64) - want) / np.abs(want)
        assert np.nanmax(rel) <= 2e-6, (op, np.nanmax(rel))
        # indexing is exact: element (i, j) of the result comes from element (j, i) of the input
        fn = np.exp if op == "exp" else np.tanh
        sample = fn(hosts[0].reshape(n, n)[::97, ::89].T.astype(np.float64))
        assert np.max(np.abs(got.reshape(n, n)[::89, ::97] - sample) / np.abs(sample)) <= 2e-6
    capi.call("ct_ternary_op", None, dest.ptr, C.byref(cont), devs[0].ptr, C.byref(view), 1.0, devs[1].ptr, C.byref(view),
              1.0, devs[2].ptr, C.byref(view), 1.0, n * n, 0, capi.F32)
    assert capi.last_kernel() == "tile"
    got = dest.download()
    ob.call("ternary_op", want.ctypes.data, C.byref(cont), hosts[0].ctypes.data, C.byref(view), 1.0,
            hosts[1].ctypes.data, C.byref(view), 1.0, hosts[2].ctypes.data, C.byref(view), 1.0, n * n, 0, capi.F32)
    assert bits_equal(got, want)
    # closed form: (x >= 0) ? z : y on the transposed data
    xt, yt, zt = (h.reshape(n, n).T for h in hosts)
    assert bits_equal(got.reshape(n, n), np.where(xt >= 0, zt, yt))
    for t in devs + [dest]:
        t.free()


@pytest.mark.parametrize("code,shape,seed", [(capi.F32, (16384, 4096), 4), (capi.F64, (4096, 4096), 5)])
def test_config2_reductions(code, shape, seed):
    r, c = shape
    dt = np.float32 if code == capi.F32 else np.float64
    x = np.random.default_rng(seed).standard_normal(r * c).astype(dt)
    dx = Dev(x)
    rows_out, cols_out = Dev(np.zeros(r, dt)), Dev(np.zeros(c, dt))
    tol = 2e-6 if code == capi.F32 else 1e-12
    x64 = x.reshape(r, c).astype(np.float64)
    for op in ("sum", "max", "magnitude-squared"):
        capi.call("ct_unary_reduce", None, rows_out.ptr, C.byref(dims([r, 1])), 1.0, dx.ptr, C.byref(dims([r, c])),
                  capi.REDUCE_OPS[op], code)
        k_rows = capi.last_kernel()
        capi.call("ct_unary_reduce", None, cols_out.ptr, C.byref(dims([c, 1])), 1.0, dx.ptr, C.byref(dims([c, r], [1, c])),
                  capi.REDUCE_OPS[op], code)
        k_cols = capi.last_kernel()
        assert k_rows.startswith("reduce_row") and k_cols.startswith("reduce_col"), (k_rows, k_cols)
        got_r, got_c = rows_out.download().astype(np.float64), cols_out.download().astype(np.float64)
        want_r, want_c = np.zeros(r, dt), np.zeros(c, dt)
        ob.call("unary_reduce", want_r.ctypes.data, C.byref(dims([r, 1])), 1.0, x.ctypes.data, C.byref(dims([r, c])),
                capi.REDUCE_OPS[op], code)
        ob.call("unary_reduce", want_c.ctypes.data, C.byref(dims([c, 1])), 1.0, x.ctypes.data,
                C.byref(dims([c, r], [1, c])), capi.REDUCE_OPS[op], code)
        if op == "max":
            assert np.array_equal(got_r, want_r) and np.array_equal(got_c, want_c)
            assert got_r.max() == got_c.max() == x64.max()
            continue
        mag = np.abs(x64) if op == "sum" else x64 * x64
        assert np.all(np.abs(got_r - want_r) <= tol * mag.sum(axis=1)), op
        assert np.all(np.abs(got_c - want_c) <= tol * mag.sum(axis=0)), op
        # checksum of checksums: both directions add up to the same total
        total = mag.sum() if op != "sum" else np.abs(x64).sum()
        assert abs(got_r.sum() - got_c.sum()) <= 4 * tol * total
    for t in (dx, rows_out, cols_out):
        t.free()


def test_config3_adam_and_adadelta_2_28():
    n = 1 << 28
    rng = np.random.default_rng(6)
    p = rng.uniform(-0.05, 0.05, n).astype(np.float32)
    g = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    m = np.zeros(n, np.float32)
    v = np.full(n, 1e-6, np.float32)
    dp, dg, dm, dv = Dev(p), Dev(g), Dev(m), Dev(v)
    pb1 = pb2 = 1.0
    for _ in range(10):
        pb1, pb2 = pb1 * 0.9, pb2 * 0.999
    capi.call("ct_adam_step", None, capi.F32, 1e-3, 0.9, 0.999, 1e-8, pb1, pb2, 1.0, dg.ptr, dp.ptr, dm.ptr, dv.ptr, n)
    assert capi.last_kernel() == "adam_vec"
    ob.call("adam_step", capi.F32, 1e-3, 0.9, 0.999, 1e-8, pb1, pb2, 1.0, g.ctypes.data, p.ctypes.data, m.ctypes.data,
            v.ctypes.data, n)  # the oracle updates p, m, v in place
    for name, dev, want in (("params", dp, p), ("m", dm, m), ("v", dv, v)):
        assert bits_equal(dev.download(), want), name
    # Adadelta on the same parameters and gradients, accumulators 0
    capi.call("ct_memset", None, dm.ptr, capi.F32, 0.0, n)
    capi.call("ct_memset", None, dv.ptr, capi.F32, 0.0, n)
    m[...] = 0
    v[...] = 0
    capi.call("ct_adadelta_step", None, capi.F32, 0.05, 1e-6, dm.ptr, dv.ptr, 1.0, dg.ptr, dp.ptr, n)
    # the Java step is single-threaded; the oracle restates it that way, so check a bounded prefix and suffix
    k = 1 << 22
    got_p, got_m, got_v = dp.download(), dm.download(), dv.download()
    for lo in (0, n // 2 - 12345, n - k):
        sl = slice(lo, lo + k)
        pp, mm, vv, gg = p[sl].copy(), m[sl].copy(), v[sl].copy(), g[sl].copy()
        ob.call("adadelta_step", capi.F32, 0.05, 1e-6, mm.ctypes.data, vv.ctypes.data, 1.0, gg.ctypes.data,
                pp.ctypes.data, k)
        assert bits_equal(got_p[sl], pp) and bits_equal(got_m[sl], mm) and bits_equal(got_v[sl], vv), lo
    for t in (dp, dg, dm, dv):
        t.free()


def test_config4_image_normalise_and_int_to_double():
    shp = [256, 3, 224, 224]
    n = int(np.prod(shp))
    u8 = np.random.default_rng(7).integers(0, 256, n, dtype=np.uint8)
    du8, df, df2 = Dev(u8), Dev(np.zeros(n, np.float32)), Dev(np.zeros(n, np.float32))
    capi.call("ct_assign", None, df.ptr, C.byref(dims(shp)), capi.F32, du8.ptr, C.byref(dims(shp)), capi.U8, n)
    assert capi.last_kernel() == "vec"
    f = df.download()
    assert bits_equal(f, u8.astype(np.float32))  # uint8 -> float32 is exact
    mean = (np.array([0.485, 0.456, 0.406]) * 255).astype(np.float32)
    std = (np.array([0.229, 0.224, 0.225]) * 255).astype(np.float32)
    dmean, dstd = Dev(mean), Dev(std)
    f4 = f.reshape(shp)
    # :- arrives as :+ with y_alpha -1 (src/cortex/tensor.clj:774-777)
    capi.call("ct_binary_op", None, df2.ptr, C.byref(dims(shp)), df.ptr, C.byref(dims(shp)), 1.0, dmean.ptr,
              C.byref(dims([3, 1, 1])), -1.0, n, capi.BINARY_OPS["+"], capi.F32)
    assert capi.last_kernel() == "vec"
    sub = df2.download()
    assert bits_equal(sub.reshape(shp), f4 - mean[None, :, None, None])
    capi.call("ct_binary_op", None, df.ptr, C.byref(dims(shp)), df2.ptr, C.byref(dims(shp)), 1.0, dstd.ptr,
              C.byref(dims([3, 1, 1])), 1.0, n, capi.BINARY_OPS["/"], capi.F32)
    div = df.download()
    assert bits_equal(div.reshape(shp), sub.reshape(shp) / std[None, :, None, None])
    want = np.zeros(n, np.float32)
    ob.call("binary_op", want.ctypes.data, C.byref(dims(shp)), sub.ctypes.data, C.byref(dims(shp)), 1.0, std.ctypes.data,
            C.byref(dims([3, 1, 1])), 1.0, n, capi.BINARY_OPS["/"], capi.F32)
    assert bits_equal(div, want)
    for t in (du8, df, df2, dmean, dstd):
        t.free()

    n = 1 << 26
    i32 = np.random.default_rng(8).integers(-2 ** 31, 2 ** 31, n, dtype=np.int64).astype(np.int32)
    di, dd = Dev(i32), Dev(np.zeros(n, np.float64))
    capi.call("ct_assign", None, dd.ptr, C.byref(dims([n])), capi.F64, di.ptr, C.byref(dims([n])), capi.I32, n)
    assert bits_equal(dd.download(), i32.astype(np.float64))
    di.free()
    dd.free()


def _pool(forward, desc, geom, *ptrs):
    d = capi.make_pool_desc(desc)
    name = "ct_pooling_forward" if forward else "ct_pooling_backward"
    capi.call(name, None, ptrs[0], 0.0, *ptrs[1:], C.byref(d), *geom, capi.F32)
    return capi.last_kernel()


def test_pooling_at_image_batch_size():
    """[32, 64, 224, 224] float (411 MB): 2 x 2 stride 2 max against numpy's window maximum and the
    indicator of the maxima, 3 x 3 pad 1 stride 2 through window-independent properties (an average
    of a constant image is the constant times the fraction of the window inside it; a 1 x 1 window is
    a copy), and the two averages' backward passes as adjoints of their forward passes."""
    batch, channels, h, w = 32, 64, 224, 224
    planes = batch * channels
    rng = np.random.default_rng(70)
    x = rng.standard_normal((planes, h, w), dtype=np.float32)
    xin = Dev(x)

    # 2 x 2 windows that tile the image
    oh, ow = h // 2, w // 2
    desc = {"kernel-width": 2, "kernel-height": 2, "pad-x": 0, "pad-y": 0, "stride-x": 2, "stride-y": 2, "pool-op": "max"}
    geom = (batch, channels, h, w, oh, ow)
    out = Dev(np.zeros(planes * oh * ow, np.float32))
    assert _pool(True, desc, geom, out.ptr, xin.ptr) == "pool_forward_tile2"
    want = x.reshape(planes, oh, 2, ow, 2).max(axis=(2, 4))
    got = out.download().reshape(want.shape)
    assert bits_equal(got, want)
    og = Dev(np.ones(planes * oh * ow, np.float32))
    ig = Dev(np.zeros(planes * h * w, np.float32))
    assert _pool(False, desc, geom, ig.ptr, xin.ptr, out.ptr, og.ptr) == "pool_backward_tile2"
    indicator = (x.reshape(planes, oh, 2, ow, 2) == want[:, :, None, :, None]).astype(np.float32).reshape(-1)
    assert bits_equal(ig.download(), indicator)
    for b in (out, og, ig):
        b.free()

    # a 1 x 1 window is a copy for every pool op (the generic band kernel at full size)
    geom1 = (batch, channels, h, w, h, w)
    for op in ("max", "avg", "avg-exc-pad"):
        desc1 = {"kernel-width": 1, "kernel-height": 1, "pad-x": 0, "pad-y": 0, "stride-x": 1, "stride-y": 1, "pool-op": op}
        out = Dev(np.zeros(planes * h * w, np.float32))
        _pool(True, desc1, geom1, out.ptr, xin.ptr)
        got = out.download()
        if op == "max":
            assert bits_equal(got, x.reshape(-1)), op
        else:       # 0 + -0.0 = +0.0: the averages return a negative zero as a positive one
            assert np.array_equal(got, x.reshape(-1)) and not np.any(np.signbit(got) & (got == 0)), op
        out.free()
    xin.free()

    # 3 x 3, pad 1, stride 2 on a constant image; adjointness on random data at a smaller batch
    oh = ow = (h + 2 - 3) // 2 + 1
    geom3 = (batch, channels, h, w, oh, ow)
    ones = Dev(np.full(planes * h * w, 3.0, np.float32))
    inside_y = np.array([min(2 * o - 1 + 3, h) - max(2 * o - 1, 0) for o in range(oh)], np.float64)
    inside = np.outer(inside_y, inside_y)
    for op, expect in (("max", np.full((oh, ow), 3.0)), ("avg", None), ("avg-exc-pad", np.full((oh, ow), 3.0))):
        desc3 = {"kernel-width": 3, "kernel-height": 3, "pad-x": 1, "pad-y": 1, "stride-x": 2, "stride-y": 2, "pool-op": op}
        out = Dev(np.zeros(planes * oh * ow, np.float32))
        assert _pool(True, desc3, geom3, out.ptr, ones.ptr).startswith("pool_forward")
        got = out.download().reshape(planes, oh, ow)
        assert np.all(got == got[0]), op               # every plane alike
        if expect is None:
            np.testing.assert_allclose(got[0], 3.0 * inside / 9.0, rtol=1e-6)
        else:
            np.testing.assert_allclose(got[0], expect, rtol=1e-6)
        out.free()
    ones.free()
    sub = 256
    xs, gs = x[:sub], rng.standard_normal((sub, oh, ow), dtype=np.float32)
    for op in ("avg", "avg-exc-pad"):
        desc3 = {"kernel-width": 3, "kernel-height": 3, "pad-x": 1, "pad-y": 1, "stride-x": 2, "stride-y": 2, "pool-op": op}
        xi, gi = Dev(xs), Dev(gs)
        out, ig = Dev(np.zeros(sub * oh * ow, np.float32)), Dev(np.zeros(sub * h * w, np.float32))
        g3 = (1, sub, h, w, oh, ow)
        _pool(True, desc3, g3, out.ptr, xi.ptr)
        _pool(False, desc3, g3, ig.ptr, xi.ptr, out.ptr, gi.ptr)
        lhs = np.dot(out.download().astype(np.float64), gs.reshape(-1).astype(np.float64))
        rhs = np.dot(xs.reshape(-1).astype(np.float64), ig.download().astype(np.float64))
        assert abs(lhs - rhs) <= 1e-6 * np.abs(gs).sum(), (op, lhs, rhs)
        for b in (xi, gi, out, ig):
            b.free()


def test_indexed_rows_at_benchmark_size():
    """The row gather and the scatter-add of bench.py's access-pattern section at their full sizes:
    65536 rows of 1024 floats through an index tensor into / out of a [32768, 1024] table.  The gather
    against numpy's fancy indexing; the scatter-add against the oracle's serial loop (bit for bit) and,
    with integer-valued floats whose sums are exact in any order, against numpy's add.at."""
    rows, table_rows, width = 65536, 32768, 1024
    rng = np.random.default_rng(81)
    idx = rng.integers(0, table_rows, rows).astype(np.int32)
    idx[:4096] = 7  # one long run of equal values
    table = rng.standard_normal((table_rows, width)).astype(np.float32)
    upd = rng.integers(-64, 65, (rows, width)).astype(np.float32)
    d_idx, d_table, d_upd = Dev(idx), Dev(table), Dev(upd)
    out = Dev(np.zeros(rows * width, np.float32))
    picked = capi.make_dims([rows, width], [width, 1], [d_idx.ptr, None])
    capi.call("ct_assign", None, out.ptr, C.byref(dims([rows, width])), capi.F32, d_table.ptr, C.byref(picked), capi.F32,
              rows * width)
    assert capi.last_kernel() == "vec"
    assert bits_equal(out.download().reshape(rows, width), table[idx])
    out.free()

    capi.call("ct_binary_accum", None, d_table.ptr, C.byref(picked), 1.0, d_upd.ptr, C.byref(dims([rows, width])), 1.0,
              rows * width, capi.BINARY_OPS["+"], 0, 1, capi.F32)
    assert capi.last_kernel() == "accum_grouped_vec"
    got = d_table.download().reshape(table_rows, width)
    want = table.copy().reshape(-1)
    host_picked = capi.make_dims([rows, width], [width, 1], [idx.ctypes.data, None])
    ob.call("binary_accum", want.ctypes.data, C.byref(host_picked), 1.0, upd.ctypes.data, C.byref(dims([rows, width])), 1.0,
            rows * width, capi.BINARY_OPS["+"], 0, 1, capi.F32)
    assert bits_equal(got.reshape(-1), want)
    # exact arithmetic: integer updates into an integer-valued table sum to the same value in any order
    itable = np.rint(table * 8).astype(np.float32)
    d_itable = Dev(itable)
    capi.call("ct_binary_accum", None, d_itable.ptr, C.byref(picked), 1.0, d_upd.ptr, C.byref(dims([rows, width])), 1.0,
              rows * width, capi.BINARY_OPS["+"], 0, 1, capi.F32)
    sums = itable.astype(np.float64)
    np.add.at(sums, idx, upd.astype(np.float64))
    assert np.array_equal(d_itable.download().reshape(table_rows, width).astype(np.float64), sums)
    for t in (d_idx, d_table, d_upd, d_itable):
        t.free()


def test_planar_and_interleaved_images_at_benchmark_size():
    """[256, 3, 224, 224] planar <-> [256, 224, 224, 3] interleaved, float and u8 -> float: numpy's
    transpose is the closed form, and there and back is the identity."""
    n, c, h, w = 256, 3, 224, 224
    rng = np.random.default_rng(82)
    planar = rng.standard_normal((n, c, h, w)).astype(np.float32)
    d_planar, d_inter, d_back = Dev(planar), Dev(np.zeros(planar.size, np.float32)), Dev(np.zeros(planar.size, np.float32))
    inter_as_planar = dims([n, c, h, w], [h * w * c, 1, w * c, c])  # the interleaved buffer addressed [n, c, y, x]
    cont = dims([n, c, h, w])
    capi.call("ct_assign", None, d_inter.ptr, C.byref(inter_as_planar), capi.F32, d_planar.ptr, C.byref(cont), capi.F32,
              planar.size)
    assert capi.last_kernel() == "lace"
    assert bits_equal(d_inter.download().reshape(n, h, w, c), planar.transpose(0, 2, 3, 1))
    capi.call("ct_assign", None, d_back.ptr, C.byref(cont), capi.F32, d_inter.ptr, C.byref(inter_as_planar), capi.F32,
              planar.size)
    assert capi.last_kernel() == "lace"
    assert bits_equal(d_back.download(), planar.reshape(-1))
    pixels = rng.integers(0, 256, (n, h, w, c)).astype(np.uint8)
    d_pix = Dev(pixels)
    capi.call("ct_assign", None, d_back.ptr, C.byref(cont), capi.F32, d_pix.ptr, C.byref(inter_as_planar), capi.U8,
              planar.size)
    assert capi.last_kernel() == "lace"
    assert bits_equal(d_back.download().reshape(n, c, h, w), pixels.transpose(0, 3, 1, 2).astype(np.float32))
    for t in (d_planar, d_inter, d_back, d_pix):
        t.free()


def test_broadcast_accumulates_at_benchmark_size():
    """[4096] <- max / + over the 16384 rows of a [16384, 4096] float matrix (the staged forms) against
    the oracle's serial chain: bit for bit for :max; for :+ bit for bit on integer-valued data (exact in
    any order) and within 2e-6 of the sum of magnitudes on gaussian data."""
    rows, cols = 16384, 4096
    rng = np.random.default_rng(83)
    y = rng.standard_normal((rows, cols)).astype(np.float32)
    y[5, 17] = np.nan
    y[9, 33] = 0.0
    y[:, 33] = np.minimum(y[:, 33], 0.0)  # a column whose maximum is a zero: the order of +-0 decides
    start = rng.standard_normal(cols).astype(np.float32)
    start[33] = -1.0
    y[0, 33] = -0.0
    d_y = Dev(y)
    row_view, full = dims([rows, cols], [0, 1]), dims([rows, cols])
    for op in ("max", "+"):
        d_acc = Dev(start)
        capi.call("ct_binary_accum", None, d_acc.ptr, C.byref(row_view), 1.0, d_y.ptr, C.byref(full), 1.0, rows * cols,
                  capi.BINARY_OPS[op], 0, 1, capi.F32)
        kernel = capi.last_kernel()
        got = d_acc.download()
        want = start.copy()
        ob.call("binary_accum", want.ctypes.data, C.byref(row_view), 1.0, y.ctypes.data, C.byref(full), 1.0, rows * cols,
                capi.BINARY_OPS[op], 0, 1, capi.F32)
        if op == "max":
            assert kernel == "accum_staged_extreme", kernel
            assert bits_equal(got, want)
        else:
            assert kernel == "accum_staged_sum", kernel
            scale = np.abs(start.astype(np.float64)) + np.abs(np.nan_to_num(y.astype(np.float64))).sum(axis=0)
            ok = np.abs(got.astype(np.float64) - want) <= 2e-6 * scale
            assert np.all(ok | (np.isnan(got) & np.isnan(want)))
            # and against the sum itself.  The kernel leaves what unary-reduce! :sum followed by binary-op! :+ would:
            # the column's sum (formed in double) rounded to float, added to the start, rounded again.  Half a unit
            # in the last place for each rounding, plus what 16384 double additions can lose relative to the
            # magnitudes they add
            col_sum = y.astype(np.float64).sum(axis=0)
            exact = start.astype(np.float64) + col_sum
            near = np.abs(got.astype(np.float64) - exact) <= 6.0e-8 * (np.abs(col_sum) + np.abs(exact)) + 1e-11 * scale
            assert np.all(near | (np.isnan(got) & np.isnan(exact)))
        d_acc.free()
    whole = rng.integers(-8, 9, (rows, cols)).astype(np.float32)
    d_whole, d_acc = Dev(whole), Dev(np.zeros(cols, np.float32))
    capi.call("ct_binary_accum", None, d_acc.ptr, C.byref(row_view), 1.0, d_whole.ptr, C.byref(full), 1.0, rows * cols,
              capi.BINARY_OPS["+"], 0, 1, capi.F32)
    assert np.array_equal(d_acc.download().astype(np.float64), whole.astype(np.float64).sum(axis=0))
    for t in (d_y, d_whole, d_acc):
        t.free()


def test_streamed_accumulates_at_benchmark_size():
    """[4096] <- the 16384 rows of a [16384, 4096] float matrix under operations that only the serial order
    defines (:*, :/ reversed, :- reversed, :+ under a destination multiplier of 0.9): bit for bit against the
    oracle's chain e = 0 .. n-1 (src/cortex/compute/cpu/tensor_math.clj:386-420)."""
    rows, cols = 16384, 4096
    rng = np.random.default_rng(84)
    y = (1.0 + 0.01 * rng.standard_normal((rows, cols))).astype(np.float32)
    y[77, 5] = np.nan
    y[4000, 9] = 0.0
    y[9000, 9] = -0.0
    start = rng.standard_normal(cols).astype(np.float32)
    d_y = Dev(y)
    row_view, full = dims([rows, cols], [0, 1]), dims([rows, cols])
    for op, dest_alpha, y_alpha, reverse, kernel in (("*", 1.0, 1.0, 0, "accum_stream_plain"), ("/", 1.0, 1.0, 1, "accum_stream_plain"),
                                                     ("-", 1.0, 1.0, 1, "accum_stream_plain"), ("+", 0.9, 1.0, 0, "accum_stream"),
                                                     ("max", 0.999, 0.5, 0, "accum_stream")):
        d_acc = Dev(start)
        capi.call("ct_binary_accum", None, d_acc.ptr, C.byref(row_view), dest_alpha, d_y.ptr, C.byref(full), y_alpha, rows * cols,
                  capi.BINARY_OPS[op], reverse, 1, capi.F32)
        assert capi.last_kernel() == kernel, (op, capi.last_kernel())
        want = start.copy()
        ob.call("binary_accum", want.ctypes.data, C.byref(row_view), dest_alpha, y.ctypes.data, C.byref(full), y_alpha, rows * cols,
                capi.BINARY_OPS[op], reverse, 1, capi.F32)
        assert bits_equal(d_acc.download(), want), op
        d_acc.free()
    # each row into one element: the chains lie along the unit-stride axis
    col_view = dims([cols, rows], [1, 0])
    yt = dims([cols, rows])
    d_acc = Dev(start)
    capi.call("ct_binary_accum", None, d_acc.ptr, C.byref(col_view), 1.0, d_y.ptr, C.byref(yt), 1.0, rows * cols,
              capi.BINARY_OPS["*"], 0, 1, capi.F32)
    assert capi.last_kernel() == "accum_stream_steps_plain", capi.last_kernel()
    want = start.copy()
    ob.call("binary_accum", want.ctypes.data, C.byref(col_view), 1.0, y.ctypes.data, C.byref(yt), 1.0, rows * cols,
            capi.BINARY_OPS["*"], 0, 1, capi.F32)
    assert bits_equal(d_acc.download(), want)
    for t in (d_y, d_acc):
        t.free()


def test_blocks_of_a_wider_matrix_at_benchmark_size():
    """ct/submatrix at the benchmark's sizes (tensor.clj:490-513): a [65536, 999] block of a pitch-1024 float
    matrix copied out and written back (calls large enough for the stores to bypass the caches), rows of 10 out
    of a pitch of 16 gathered into a dense matrix, and a block converted to double on the way.  numpy's slices
    are the closed form; what lies between the rows of a pitched destination must stay as it was."""
    rows, width, pitch = 65536, 999, 1024
    rng = np.random.default_rng(85)
    wide = rng.standard_normal((rows, pitch)).astype(np.float32)
    d_wide, d_block = Dev(wide), Dev(np.zeros(rows * width, np.float32))
    pitched, dense = dims([rows, width], [pitch, 1]), dims([rows, width])
    capi.call("ct_assign", None, d_block.ptr, C.byref(dense), capi.F32, d_wide.ptr, C.byref(pitched), capi.F32, rows * width)
    assert capi.last_kernel() == "ragged", capi.last_kernel()
    assert bits_equal(d_block.download().reshape(rows, width), wide[:, :width])
    fresh = rng.standard_normal((rows, width)).astype(np.float32)
    d_fresh = Dev(fresh)
    capi.call("ct_assign", None, d_wide.ptr, C.byref(pitched), capi.F32, d_fresh.ptr, C.byref(dense), capi.F32, rows * width)
    assert capi.last_kernel() == "vecu", capi.last_kernel()
    want = wide.copy()
    want[:, :width] = fresh
    assert bits_equal(d_wide.download().reshape(rows, pitch), want)
    # a block that starts one element into the rows: nothing of it lies on the 16-byte grid
    off_rows = rows - 1
    d_block2 = Dev(np.zeros(off_rows * width, np.float32))
    capi.call("ct_assign", None, d_block2.ptr, C.byref(dims([off_rows, width])), capi.F32, d_wide.ptr + 4 * 21,
              C.byref(dims([off_rows, width], [pitch, 1])), capi.F32, off_rows * width)
    flat = want.reshape(-1)
    expect = np.lib.stride_tricks.as_strided(flat[21:], (off_rows, width), (4 * pitch, 4))
    assert bits_equal(d_block2.download().reshape(off_rows, width), np.ascontiguousarray(expect))
    d_double = Dev(np.zeros(rows * width, np.float64))
    capi.call("ct_assign", None, d_double.ptr, C.byref(dense), capi.F64, d_wide.ptr, C.byref(pitched), capi.F32, rows * width)
    assert bits_equal(d_double.download().reshape(rows, width), want[:, :width].astype(np.float64))
    for t in (d_block, d_fresh, d_block2, d_double):
        t.free()
    short_rows, short_w, short_pitch = 1 << 22, 10, 16
    d_short = Dev(np.zeros(short_rows * short_w, np.float32))
    capi.call("ct_assign", None, d_short.ptr, C.byref(dims([short_rows, short_w])), capi.F32, d_wide.ptr,
              C.byref(dims([short_rows, short_w], [short_pitch, 1])), capi.F32, short_rows * short_w)
    assert capi.last_kernel() == "span", capi.last_kernel()
    assert bits_equal(d_short.download().reshape(short_rows, short_w), want.reshape(short_rows, short_pitch)[:, :short_w])
    for t in (d_wide, d_short):
        t.free()


def test_matrix_of_2_31_elements_built_and_reduced():
    """A float matrix of 65536 x 32768 (2^31 elements, 8 GiB: one element more than a 32-bit index
    counts) is built on the device as column[r] + row[c] (r % 5 and c % 7, so that every sum below is an
    integer under 2^24 and exact in any order), then summed along its rows and, through the transposed
    view, along its columns; both results are compared with their closed forms.  The build runs as
    pieces on the vector kernel, the sums on the row and column kernels."""
    rows, cols = 1 << 16, 1 << 15
    n = rows * cols
    free, total = C.c_size_t(), C.c_size_t()
    capi.call("ct_memory_info", C.byref(free), C.byref(total))
    if free.value < 4 * n + (2 << 30):
        pytest.skip("needs 10 GiB of free device memory")
    col_vals = (np.arange(rows) % 5).astype(np.float32)
    row_vals = (np.arange(cols) % 7).astype(np.float32)
    d_col, d_row = Dev(col_vals), Dev(row_vals)
    d_rsum, d_csum = Dev(np.zeros(rows, np.float32)), Dev(np.zeros(cols, np.float32))
    big = C.c_void_p()
    capi.call("ct_malloc", C.byref(big), 4 * n)
    try:
        full = dims([rows, cols])
        capi.call("ct_binary_op", None, big, C.byref(full), d_col.ptr, C.byref(dims([rows, 1])), 1.0, d_row.ptr,
                  C.byref(dims([cols])), 1.0, n, capi.BINARY_OPS["+"], capi.F32)
        assert capi.last_kernel() == "vec"
        capi.call("ct_unary_reduce", None, d_rsum.ptr, C.byref(dims([rows, 1])), 1.0, big, C.byref(full),
                  capi.REDUCE_OPS["sum"], capi.F32)
        assert capi.last_kernel() == "reduce_row512_vec"
        capi.call("ct_unary_reduce", None, d_csum.ptr, C.byref(dims([cols, 1])), 1.0, big,
                  C.byref(dims([cols, rows], [1, cols])), capi.REDUCE_OPS["sum"], capi.F32)
        assert capi.last_kernel() == "reduce_col_vec"
        want_r = cols * col_vals.astype(np.float64) + row_vals.astype(np.float64).sum()
        want_c = rows * row_vals.astype(np.float64) + col_vals.astype(np.float64).sum()
        assert np.array_equal(d_rsum.download().astype(np.float64), want_r)
        assert np.array_equal(d_csum.download().astype(np.float64), want_c)
    finally:
        capi.call("ct_free", big)
        for t in (d_col, d_row, d_rsum, d_csum):
            t.free()


def test_indexed_rows_of_2_31_bytes_gathered_and_scattered():
    """65541 rows of 32768 bytes picked from a [1000, 32768] table through an index tensor (2^31 + 163840
    elements): the gather runs as pieces of 32768 rows whose index pointers advance with them, and rows
    on both sides of the piece boundaries are compared with the table.  The gathered rows are then
    scatter-added into a zeroed table through the same index: row t ends as (its number of
    occurrences) x (table row t) in wrapping byte arithmetic, whatever the order."""
    rows, table_rows, width = (1 << 16) + 5, 1000, 1 << 15
    n = rows * width
    free, total = C.c_size_t(), C.c_size_t()
    capi.call("ct_memory_info", C.byref(free), C.byref(total))
    if free.value < n + (2 << 30):
        pytest.skip("needs 4 GiB of free device memory")
    idx = ((np.arange(rows, dtype=np.int64) * 7) % table_rows).astype(np.int32)
    table = ((np.arange(table_rows)[:, None] + np.arange(width)[None, :]) % 100).astype(np.int8)
    d_idx, d_table, d_sums = Dev(idx), Dev(table), Dev(np.zeros(table_rows * width, np.int8))
    out = C.c_void_p()
    capi.call("ct_malloc", C.byref(out), n)
    try:
        picked = capi.make_dims([rows, width], [width, 1], [d_idx.ptr, None])
        capi.call("ct_assign", None, out, C.byref(dims([rows, width])), capi.I8, d_table.ptr, C.byref(picked), capi.I8, n)
        assert capi.last_kernel() == "vec"
        for r in (0, 1, 32767, 32768, 32769, 65535, 65536, rows - 1):
            got = np.zeros(width, np.int8)
            capi.call("ct_memcpy_async", got.ctypes.data, out.value + r * width, width, capi.COPY_D2H, None)
            capi.call("ct_stream_sync", None)
            assert np.array_equal(got, table[idx[r]]), r
        capi.call("ct_binary_accum", None, d_sums.ptr, C.byref(picked), 1.0, out, C.byref(dims([rows, width])), 1.0, n,
                  capi.BINARY_OPS["+"], 0, 1, capi.I8)
        assert capi.last_kernel() == "accum_grouped_vec"
        counts = np.bincount(idx, minlength=table_rows).astype(np.int64)
        want = (counts[:, None] * table.astype(np.int64)).astype(np.int8)
        assert np.array_equal(d_sums.download().reshape(table_rows, width), want)
    finally:
        capi.call("ct_free", out)
        for t in (d_idx, d_table, d_sums):
            t.free()


def test_lrn_at_benchmark_size():
    """lrn-forward! and lrn-backward! on bench.py's [64, 256, 56, 56] float tensor (n 5, k 2, alpha 1e-4,
    beta 0.75: the reference's defaults) against the oracle; alpha 1e-2 as well so that the window sums
    weigh as much as k.  Forward within 4e-6 of the result; backward within 4e-6 of the magnitudes of
    its two terms (bounded here by |dy| s^-beta + 2 alpha beta |x| max|dy y| / k)."""
    shape = [64, 256, 56, 56]
    count = int(np.prod(shape))
    rng = np.random.default_rng(91)
    x = (rng.standard_normal(count, dtype=np.float32) * 4).astype(np.float32)
    dy = rng.standard_normal(count, dtype=np.float32)
    d_x, d_dy = Dev(x), Dev(dy)
    d_y, d_dx = Dev(np.zeros(count, np.float32)), Dev(np.zeros(count, np.float32))
    dm = dims(shape)
    try:
        for alpha in (1e-4, 1e-2):
            capi.call("ct_lrn_forward", None, d_y.ptr, C.byref(dm), d_x.ptr, C.byref(dm), 5, 2.0, alpha, 0.75, capi.F32)
            assert capi.last_kernel() == "lrn_forward_vec"
            want_y = np.zeros(count, np.float32)
            ob.call("lrn_forward", want_y.ctypes.data, C.byref(dm), x.ctypes.data, C.byref(dm), 5, 2.0, alpha, 0.75, capi.F32)
            got_y = d_y.download()
            assert np.all(np.abs(got_y.astype(np.float64) - want_y) <= 4e-6 * np.abs(want_y.astype(np.float64)))
            d_y.host[:] = want_y   # both sides differentiate the same stored output
            capi.call("ct_memcpy_async", d_y.ptr, want_y.ctypes.data, want_y.nbytes, capi.COPY_H2D, None)
            capi.call("ct_lrn_backward", None, d_dx.ptr, C.byref(dm), d_y.ptr, C.byref(dm), d_x.ptr, C.byref(dm), d_dy.ptr,
                      C.byref(dm), 5, 2.0, alpha, 0.75, capi.F32)
            assert capi.last_kernel() == "lrn_backward_vec"
            want_dx = np.zeros(count, np.float32)
            ob.call("lrn_backward", want_dx.ctypes.data, C.byref(dm), want_y.ctypes.data, C.byref(dm), x.ctypes.data,
                    C.byref(dm), dy.ctypes.data, C.byref(dm), 5, 2.0, alpha, 0.75, capi.F32)
            got_dx = d_dx.download().astype(np.float64)
            bar = 4e-6 * (np.abs(dy.astype(np.float64)) + 2 * alpha * 0.75 * np.abs(x.astype(np.float64)) *
                          float(np.max(np.abs(dy.astype(np.float64) * want_y))) / 2.0)
            assert np.all(np.abs(got_dx - want_dx) <= bar)
    finally:
        for t in (d_x, d_dy, d_y, d_dx):
            t.free()
