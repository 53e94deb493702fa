"""Rows that are no whole number of 16-byte vectors under dense operands (ew_ragged_kernel): a
per-channel bias on 7 x 7 images (src/cortex/compute/nn/layers.clj:313-318), a per-row scale of
ten-class rows (src/cortex/tensor.clj:1618-1644), a bias row on ten columns
(src/cortex/compute/nn/backend.clj:109).  Against the oracle, bit for bit."""
import numpy as np
import pytest

import harness as H
from cortex_amd import capi
from harness import View

pytestmark = pytest.mark.gpu
NP = H.NP_DTYPES


@pytest.fixture()
def P(pair_factory):
    with pair_factory() as pair:
        yield pair


def values(rng, code, n):
    if code in (capi.F32, capi.F64):
        return (rng.standard_normal(n) * 3).astype(NP[code])
    info = np.iinfo(NP[code])
    return rng.integers(max(info.min, -90), min(info.max, 90) + 1, n).astype(NP[code])


def exact(buf, what):
    H.assert_bit_exact(buf.download(), buf.host, what)


@pytest.mark.parametrize("code", [capi.F32, capi.F64, capi.I32, capi.I8, capi.U8, capi.I64])
def test_channel_bias_on_odd_images(P, code):
    rng = np.random.default_rng(91)
    vmax = 16 // NP[code]().itemsize
    for batch, channels, pixels in ((9, 24, 49), (3, 5, 7 * 7 * 9), (2, 3, 4099), (16, 37, 25)):
        n = batch * channels * pixels
        x = P.buf(values(rng, code, n))
        bias = P.buf(values(rng, code, channels))
        d = P.buf(np.zeros(n, NP[code]))
        shape = [batch, channels, pixels]
        k = P.run(H.binary_op, View(d, shape), View(x, shape), 1.0, View(bias, [channels, 1]), 1.0, "+")
        exact(d, f"channel bias {shape} ({k})")
        want = "ragged" if pixels >= vmax and pixels % vmax and n >= 4096 else None
        if want:
            assert k == want, (k, shape)
        # in place, with multipliers, and the bias on the left
        k = P.run(H.binary_op, View(x, shape), View(bias, [channels, 1]), 2.0, View(x, shape), -1.0, "*")
        exact(x, f"in place {shape} ({k})")


@pytest.mark.parametrize("code", [capi.F32, capi.F64, capi.I16])
def test_per_row_scale_and_bias_row_on_short_rows(P, code):
    rng = np.random.default_rng(92)
    vmax = 16 // NP[code]().itemsize
    for rows, cols in ((1000, 10), (4097, 9), (513, 33), (77, 101)):
        if cols < vmax:
            continue
        n = rows * cols
        x = P.buf(values(rng, code, n))
        per_row = P.buf(values(rng, code, rows) + NP[code](1))
        bias = P.buf(values(rng, code, cols))
        d = P.buf(np.zeros(n, NP[code]))
        k = P.run(H.binary_op, View(d, [rows, cols]), View(x, [rows, cols]), 1.0, View(per_row, [rows, 1]), 1.0, "*")
        exact(d, f"per-row scale [{rows},{cols}] ({k})")
        if n >= 4096 and cols % vmax:
            assert k == "ragged", k
        k = P.run(H.binary_op, View(d, [rows, cols]), View(x, [rows, cols]), 1.0, View(bias, [cols]), 1.0, "+")
        exact(d, f"bias row [{rows},{cols}] ({k})")
        if n >= 4096 and cols % vmax:
            assert k == "ragged", k
        # select with a per-row condition, a dense operand and a bias row
        k = P.run(H.ternary_op, View(d, [rows, cols]), View(per_row, [rows, 1]), 1.0, View(x, [rows, cols]), 1.0,
                  View(bias, [cols]), 1.0)
        exact(d, f"select [{rows},{cols}] ({k})")
        # constants and conversions ride along
        k = P.run(H.binary_op_constant, View(d, [rows, cols]), View(x, [rows, cols]), 1.0, 3.0, "+")
        exact(d, f"constant [{rows},{cols}] ({k})")


def test_three_outer_axes_and_mixed_widths(P):
    rng = np.random.default_rng(93)
    shape = [4, 6, 5, 45]                      # [n, c, h, w-ish] with a [c, 1, 1] operand
    n = int(np.prod(shape))
    x = P.buf(values(rng, capi.F32, n))
    scale = P.buf(values(rng, capi.F32, 6))
    d = P.buf(np.zeros(n, np.float32))
    k = P.run(H.binary_op, View(d, shape), View(x, shape), 1.0, View(scale, [6, 1, 1]), 1.0, "/")
    exact(d, f"channel divide {shape} ({k})")
    assert k == "ragged", k
    # u8 image to float with rows of 45 bytes: the vector is four floats wide
    pix = P.buf(rng.integers(0, 256, n).astype(np.uint8))
    k = P.run(H.assign, View(d, shape), View(pix, shape))
    exact(d, f"assign u8 -> f32 {shape} ({k})")


@pytest.mark.parametrize("code", [capi.F32, capi.F64, capi.I16, capi.I8, capi.I64])
def test_rows_off_the_vector_grid(P, code):
    """Odd-width blocks of a pitched matrix (ct/submatrix, src/cortex/tensor.clj:490-513), sub-buffers that start at
    an odd element, rows one element longer than a vector: vectors that start anywhere (ew_vecu_kernel)."""
    rng = np.random.default_rng(94)
    vmax = 16 // NP[code]().itemsize
    for rows, width, pitch, offset in ((70, 999, 1024, 0), (129, 67, 80, 3), (4100, vmax + 1, vmax + 3, 1), (33, 200, 200, 5)):
        if width < vmax:
            continue
        n = rows * width
        src = P.buf(values(rng, code, rows * pitch + offset + 8))
        other = P.buf(values(rng, code, rows * pitch + offset + 8))
        dense = P.buf(np.zeros(n, NP[code]))
        pitched = P.buf(values(rng, code, rows * pitch + offset + 8))
        sub = lambda b: View(b, [rows, width], [pitch, 1], offset=offset)
        k = P.run(H.assign, View(dense, [rows, width]), sub(src))
        exact(dense, f"copy out of a pitched block [{rows},{width}]/{pitch}+{offset} ({k})")
        # a dense destination takes aligned vectors that may straddle a row end when the rows are no whole number of
        # vectors; otherwise each row is walked in vectors that start wherever the row does
        if n >= 4096 and width % vmax and pitch != width:
            assert k == "ragged", (k, rows, width, pitch, offset)
        elif n >= 4096 and (pitch % vmax or offset % vmax):
            assert k == "vecu", (k, rows, width, pitch, offset)
        k = P.run(H.binary_op, sub(pitched), sub(src), 1.0, sub(other), -1.0, "+")
        exact(pitched, f"pitched block minus pitched block ({k})")
        k = P.run(H.binary_op, sub(pitched), sub(pitched), 1.0, View(dense, [rows, width]), 2.0, "max")
        exact(pitched, f"in place against a dense block ({k})")
        per_row = P.buf(values(rng, code, rows))
        k = P.run(H.binary_op, sub(pitched), sub(src), 1.0, View(per_row, [rows, 1]), 1.0, "*")
        exact(pitched, f"pitched block times a per-row value ({k})")
        k = P.run(H.binary_op_constant, sub(pitched), sub(src), 1.0, 3.0, "+")
        exact(pitched, f"pitched block plus a constant ({k})")


def test_conversion_off_the_vector_grid(P):
    rng = np.random.default_rng(95)
    rows, width, pitch = 100, 333, 340
    pix = P.buf(rng.integers(0, 256, rows * pitch + 4).astype(np.uint8))
    out = P.buf(np.zeros(rows * width, np.float32))
    k = P.run(H.assign, View(out, [rows, width]), View(pix, [rows, width], [pitch, 1], offset=1))
    exact(out, f"u8 block to float ({k})")
    assert k == "ragged", k
    back = P.buf(np.zeros(rows * pitch + 4, np.int16))
    k = P.run(H.assign, View(back, [rows, width], [pitch, 1], offset=3), View(out, [rows, width]))
    exact(back, f"float to a pitched short block ({k})")


@pytest.mark.parametrize("pair", [(capi.F32, capi.F32), (capi.U8, capi.F32), (capi.F32, capi.I16), (capi.F64, capi.F32),
                                  (capi.I8, capi.I64)])
def test_short_rows_of_a_small_pitch(P, pair):
    """A dense [rows, w] destination from rows of a pitch of at most 128 bytes (the first ten of every sixteen
    values): a block stages the span of memory that holds its rows through LDS (ew_span_kernel).  assign!, with
    conversion; a last block that is not full, and a width that leaves the padding of the last row unread."""
    src_code, dst_code = pair
    rng = np.random.default_rng(96)
    item = NP[src_code]().itemsize
    for rows, w, pitch in ((150000, 10, 16), (300017, 5, 8), (70001, 19, 128 // item)):
        if pitch * item > 128 or w * 5 > pitch * 4 or pitch <= w:
            continue
        src = P.buf(values(rng, src_code, (rows - 1) * pitch + w))       # the buffer ends with the last row's last value
        out = P.buf(np.zeros(rows * w, NP[dst_code]))
        k = P.run(H.assign, View(out, [rows, w]), View(src, [rows, w], [pitch, 1]))
        exact(out, f"short rows {w} of pitch {pitch}, {rows} rows ({k})")
        assert k == "span", (k, rows, w, pitch)
    # a destination that is not dense, or too small a call, keeps the other kernels
    src = P.buf(values(rng, src_code, 4000 * 16))
    out = P.buf(np.zeros(4000 * 12, NP[dst_code]))
    k = P.run(H.assign, View(out, [4000, 10], [12, 1]), View(src, [4000, 10], [16, 1]))
    exact(out, f"pitched destination ({k})")
    assert k != "span", k
