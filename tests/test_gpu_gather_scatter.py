"""Rows addressed through an index tensor: the vector kernel's gather / scatter form and the
deterministic parallel accumulate into an indexed destination, against the CPU oracle.
Everything here is bit-exact: the accumulate applies each destination element's updates in
increasing e, as the reference's serial loop does (src/cortex/compute/cpu/tensor_math.clj:386-420;
use case src/cortex/loss/center.clj:32-92, src/cortex/verify/tensor.clj:1147-1199)."""
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


def values(rng, code, n, lo=-50, hi=50):
    if code in FLOATS:
        return (rng.standard_normal(n) * 3.0).astype(NP[code])
    info = np.iinfo(NP[code])
    return rng.integers(max(lo, info.min), min(hi, info.max) + 1, n).astype(NP[code])


def exact(buf, what):
    H.assert_bit_exact(buf.download(), buf.host, what)


@pytest.mark.parametrize("code", H.ALL_DTYPES)
@pytest.mark.parametrize("rows,table_rows,width", [(37, 11, 64), (300, 40, 512), (19, 7, 50), (5, 3, 3)])
def test_row_gather_runs_on_the_vector_kernel(P, code, rows, table_rows, width):
    rng = np.random.default_rng(31)
    table = P.buf(values(rng, code, table_rows * width))
    idx = P.buf(rng.integers(0, table_rows, rows).astype(np.int32))
    picked = View(table, [rows, width], [width, 1], index=[idx, None])
    out = P.buf(np.zeros(rows * width, NP[code]))
    k = P.run(H.assign, View(out, [rows, width]), picked)
    exact(out, f"gather ({k})")
    assert k == ("vec" if width % (16 // NP[code]().itemsize) == 0 else "vec1"), k
    # the gathered rows as an operand next to a direct one and a broadcast row
    other = P.buf(values(rng, code, rows * width))
    bias = P.buf(values(rng, code, width))
    k = P.run(H.binary_op, View(out, [rows, width]), picked, 1.0, View(other, [rows, width]), -1.0, "+")
    exact(out, f"gathered - direct ({k})")
    k = P.run(H.ternary_op, View(out, [rows, width]), View(other, [rows, width]), 1.0, picked, 1.0, View(bias, [width]), 1.0)
    exact(out, f"select with a gathered operand ({k})")


@pytest.mark.parametrize("code", [capi.F32, capi.I16, capi.F64])
def test_scatter_assign_and_second_axis_index(P, code):
    rng = np.random.default_rng(32)
    # unique destinations: assign! rows into a permutation of a table
    rows, width = 24, 32
    table = P.buf(values(rng, code, (rows + 3) * width))
    perm = P.buf(rng.permutation(rows + 3)[:rows].astype(np.int32))
    src = P.buf(values(rng, code, rows * width))
    k = P.run(H.assign, View(table, [rows, width], [width, 1], index=[perm, None]), View(src, [rows, width]))
    exact(table, f"scatter assign ({k})")
    assert k == "vec"
    # the index on the second outer axis of a [batch, picks, width] view
    batch, picks, t_rows = 3, 10, 6
    cube = P.buf(values(rng, code, batch * t_rows * width))
    idx = P.buf(rng.integers(0, t_rows, picks).astype(np.int32))
    out = P.buf(np.zeros(batch * picks * width, NP[code]))
    k = P.run(H.assign, View(out, [batch, picks, width]),
              View(cube, [batch, picks, width], [t_rows * width, width, 1], index=[None, idx, None]))
    exact(out, f"gather along the second axis ({k})")
    assert k == "vec"
    # two indexed axes at once
    idx_b = P.buf(np.array([2, 0, 2, 1], np.int32))
    out2 = P.buf(np.zeros(4 * picks * width, NP[code]))
    k = P.run(H.assign, View(out2, [4, picks, width]),
              View(cube, [4, picks, width], [t_rows * width, width, 1], index=[idx_b, idx, None]))
    exact(out2, f"gather along two axes ({k})")
    # an index on the innermost axis keeps the general kernel; permuted storage around an indexed axis
    inner = P.buf(rng.integers(0, width, 16).astype(np.int32))
    out3 = P.buf(np.zeros(rows * 16, NP[code]))
    k = P.run(H.assign, View(out3, [rows, 16]), View(src, [rows, 16], [width, 1], index=[None, inner]))
    exact(out3, f"gather along the innermost axis ({k})")
    assert k == "general"
    deep = P.buf(np.array([1, 0, 1], np.int32))
    big = P.buf(values(rng, code, 2 * 5 * 4 * 8))
    out4 = P.buf(np.zeros(3 * 5 * 4 * 8, NP[code]))
    k = P.run(H.assign, View(out4, [3, 5, 4, 8], [160, 32, 8, 1]).transpose([0, 2, 1, 3]),
              View(big, [3, 5, 4, 8], [160, 32, 8, 1], index=[deep, None, None, None]).transpose([0, 2, 1, 3]))
    exact(out4, f"gather under a permuted view ({k})")


ACCUM_CASES = [
    # rows, classes, width, expected kernel
    (5, 3, 3, "accum_grouped"),
    (700, 13, 64, "accum_grouped_vec"),
    (4096, 1000, 128, "accum_grouped_vec"),
    (20000, 50, 8, "accum_grouped_vec"),      # more index entries than the ranking kernel takes: radix sort
    (9000, 9000, 4, "accum_grouped_vec"),     # no duplicates at all
    (131075, 40000, 4, "accum_grouped_vec"),  # many entries, few duplicates, a count off every power of two
    (300, 1, 20, "accum_grouped_vec"),        # every row lands on one destination row
    (30000, 70000, 4, "accum_grouped_vec"),   # index values beyond 16 bits: a third pass of the radix sort
    (9001, 17000000, 1, "accum_grouped"),     # and beyond 24 bits: the fourth
]


@pytest.mark.parametrize("code", [capi.F32, capi.F64, capi.I32, capi.I8])
@pytest.mark.parametrize("rows,classes,width,kernel", ACCUM_CASES)
def test_accumulate_into_indexed_rows(P, code, rows, classes, width, kernel):
    rng = np.random.default_rng(33)
    vmax = 16 // NP[code]().itemsize
    centers = P.buf(values(rng, code, classes * width))
    if classes >= rows:
        labels = rng.permutation(classes)[:rows]
    else:
        labels = rng.integers(0, classes, rows)
    idx = P.buf(labels.astype(np.int32))
    y = P.buf(values(rng, code, rows * width, -9, 9))
    dest = View(centers, [rows, width], [width, 1], index=[idx, None])
    cases = [("+", 1.0, 1.0, False), ("+", 1.0, 0.5 if code in FLOATS else 3.0, True), ("-", 1.0, 1.0, True),
             ("max", 1.0, 1.0, False), ("min", 1.0, 2.0, True)]
    cases.append(("*", 0.5, 1.0, False) if code in FLOATS else ("bit-xor", 1.0, 1.0, False))
    for op, da, ya, rev in cases:
        k = P.run(H.binary_accum, dest, da, View(y, [rows, width]), ya, op, reverse=rev, requires_cas=True)
        exact(centers, f"accumulate {op} da={da} ya={ya} reverse={rev} rows={rows} classes={classes} ({k})")
        want = kernel if width % vmax == 0 else "accum_grouped"
        assert k == want, (k, want)
        centers.reset()


@pytest.mark.parametrize("code", [capi.F32, capi.I32])
def test_accumulate_indexed_layouts(P, code):
    rng = np.random.default_rng(34)
    rows, classes, width = 60, 7, 16
    idx = P.buf(rng.integers(0, classes, rows).astype(np.int32))
    # y broadcast along the row axis ([rows, 1]) and along the indexed axis ([1, width])
    centers = P.buf(values(rng, code, classes * width))
    dest = View(centers, [rows, width], [width, 1], index=[idx, None])
    per_row = P.buf(values(rng, code, rows, -9, 9))
    k = P.run(H.binary_accum, dest, 1.0, View(per_row, [rows, 1]), 1.0, "+", requires_cas=True)
    exact(centers, f"y one value per row ({k})")
    one_row = P.buf(values(rng, code, width, -9, 9))
    k = P.run(H.binary_accum, dest, 1.0, View(one_row, [width]), 1.0, "+", requires_cas=True)
    exact(centers, f"y one row for every entry ({k})")
    # a kept axis in front of the indexed one, padded rows, an offset
    planes = 3
    pitch = width + 4
    table = P.buf(values(rng, code, planes * classes * pitch + 5))
    y = P.buf(values(rng, code, planes * rows * width, -9, 9))
    dest3 = View(table, [planes, rows, width], [classes * pitch, pitch, 1], offset=4, index=[None, idx, None])
    k = P.run(H.binary_accum, dest3, 1.0, View(y, [planes, rows, width]), 1.0, "+", requires_cas=True)
    exact(table, f"kept axis outside the indexed one ({k})")
    assert k.startswith("accum_grouped"), k
    # columns selected through the index: the kept axis is the slow one
    cols = P.buf(rng.integers(0, width, 40).astype(np.int32))
    grid = P.buf(values(rng, code, 9 * width))
    yc = P.buf(values(rng, code, 9 * 40, -9, 9))
    k = P.run(H.binary_accum, View(grid, [9, 40], [width, 1], index=[None, cols]), 1.0, View(yc, [9, 40]), 1.0, "+",
              requires_cas=True)
    exact(grid, f"indexed columns ({k})")
    assert k == "accum_grouped", k
    # a reduced axis next to the indexed one keeps the serial loop
    small = P.buf(values(rng, code, classes))
    yr = P.buf(values(rng, code, rows * 5, -9, 9))
    k = P.run(H.binary_accum, View(small, [rows, 1], [1, 1], index=[idx, None]), 1.0, View(yr, [rows, 5]), 1.0, "+",
              requires_cas=True)
    exact(small, f"indexed and reduced ({k})")
    assert k == "serial", k
    # rows that overlap in the destination (a sliding window: the row step is half a row): two index values
    # share addresses, so the updates must go one by one, as the reference applies them
    window = P.buf(values(rng, code, (classes + 1) * (width // 2)))
    yw = P.buf(values(rng, code, rows * width, -9, 9))
    k = P.run(H.binary_accum, View(window, [rows, width], [width // 2, 1], index=[idx, None]), 1.0, View(yw, [rows, width]), 1.0,
              "+", requires_cas=True)
    exact(window, f"overlapping indexed rows ({k})")
    assert k == "serial", k
