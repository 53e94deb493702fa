"""Planar <-> interleaved layouts (images as [C,H,W] against [H,W,C], a narrow transpose in
general): assign! with dtype conversion through the lace kernel, bit-exact against the CPU
oracle (reference use: src/cortex/verify/tensor.clj:668-684, 785-805)."""
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
        return (rng.standard_normal(n) * 100.0).astype(NP[code])
    info = np.iinfo(NP[code])
    return rng.integers(info.min, int(info.max) + 1, n, dtype=np.int64).astype(NP[code]) if code != capi.I64 else \
        rng.integers(-2 ** 62, 2 ** 62, n, dtype=np.int64)


PAIRS = [(capi.U8, capi.F32), (capi.F32, capi.F32), (capi.F32, capi.U8), (capi.I16, capi.F64), (capi.F64, capi.I8),
         (capi.I32, capi.I64), (capi.I8, capi.I8), (capi.F64, capi.F64)]


@pytest.mark.parametrize("src,dst", PAIRS)
@pytest.mark.parametrize("channels", [2, 3, 4])
def test_images_between_planar_and_interleaved(P, src, dst, channels):
    rng = np.random.default_rng(41)
    for n, h, w in ((2, 16, 24), (3, 9, 11), (1, 1, 4096)):
        c = channels
        count = n * c * h * w
        data = P.buf(values(rng, src, count))
        out = P.buf(np.zeros(count, NP[dst]))
        # planar destination <- interleaved source
        k = P.run(H.assign, View(out, [n, c, h, w]), View(data, [n, c, h, w], [h * w * c, 1, w * c, c]))
        H.assert_bit_exact(out.download(), out.host, f"planar <- interleaved {n}x{c}x{h}x{w} ({k})")
        widest = max(NP[src]().itemsize, NP[dst]().itemsize)
        assert k == ("lace" if (h * w) % (16 // widest) == 0 else "lace1"), k
        # interleaved destination <- planar source
        k = P.run(H.assign, View(out, [n, h, w, c]), View(data, [n, h, w, c], [c * h * w, w, 1, h * w]))
        H.assert_bit_exact(out.download(), out.host, f"interleaved <- planar {n}x{h}x{w}x{c} ({k})")
        assert k == ("lace" if (h * w) % (16 // widest) == 0 else "lace1"), k


@pytest.mark.parametrize("code", [capi.F32, capi.I16, capi.F64])
def test_lace_layout_variants(P, code):
    rng = np.random.default_rng(42)
    # a narrow transpose: [n,4] <- [4,n] and back
    n = 1000
    a = P.buf(values(rng, code, 4 * n))
    b = P.buf(np.zeros(4 * n, NP[code]))
    k = P.run(H.assign, View(b, [n, 4]), View(a, [4, n]).transpose([1, 0]))
    H.assert_bit_exact(b.download(), b.host, f"[n,4] <- [4,n] ({k})")
    assert k.startswith("lace"), k
    k = P.run(H.assign, View(b, [4, n]), View(a, [n, 4]).transpose([1, 0]))
    H.assert_bit_exact(b.download(), b.host, f"[4,n] <- [n,4] ({k})")
    assert k.startswith("lace"), k
    # padded planes and an offset: the planar side is a window of a larger buffer
    c, h, w, pitch = 3, 8, 32, 40
    big = P.buf(values(rng, code, c * h * pitch + 16))
    inter = P.buf(values(rng, code, h * w * c))
    k = P.run(H.assign, View(big, [c, h, w], [h * pitch, pitch, 1], offset=8), View(inter, [c, h, w], [1, w * c, c]))
    H.assert_bit_exact(big.download(), big.host, f"padded planar <- interleaved ({k})")
    assert k.startswith("lace"), k
    k = P.run(H.assign, View(inter, [h, w, c]), View(big, [h, w, c], [pitch, 1, h * pitch], offset=8))
    H.assert_bit_exact(inter.download(), inter.host, f"interleaved <- padded planar ({k})")
    assert k.startswith("lace"), k
    # pixels with a pitch of four but three used entries are not laced: the general kernel
    rgba = P.buf(values(rng, code, h * w * 4))
    planes = P.buf(np.zeros(3 * h * w, NP[code]))
    k = P.run(H.assign, View(planes, [3, h, w]), View(rgba, [3, h, w], [1, w * 4, 4]))
    H.assert_bit_exact(planes.download(), planes.host, f"three of four interleaved entries ({k})")
    assert k == "general", k
    # five channels are beyond the lace kernel
    five = P.buf(values(rng, code, 5 * 256))
    out5 = P.buf(np.zeros(5 * 256, NP[code]))
    k = P.run(H.assign, View(out5, [5, 256]), View(five, [5, 256], [1, 5]))
    H.assert_bit_exact(out5.download(), out5.host, f"five channels ({k})")
    assert k == "general", k
