"""Host-side shape/stride algebra against the reference's stored vectors
(/root/reference/test/clj/cortex/tensor_dimensions_test.clj:7-51) and the
dimension behaviour its tensor tests rely on."""
import pytest

from cortex_amd import dimensions as d


def strip(x):
    return {"shape": x["shape"], "strides": x["strides"]}


@pytest.mark.parametrize("existing,new_shape,want", [
    (d.dimensions([3, 2, 2], strides=[4, 2, 1]), [6, 2], {"shape": [6, 2], "strides": [2, 1]}),
    (d.dimensions([3, 2, 2], strides=[4, 2, 1]), [3, 4], {"shape": [3, 4], "strides": [4, 1]}),
    (d.dimensions([3, 2, 2], strides=[5, 2, 1]), [3, 4], {"shape": [3, 4], "strides": [5, 1]}),
    ({"shape": [4, 5, 8], "strides": [50, 10, 1]}, [20, 8], {"shape": [20, 8], "strides": [10, 1]}),
    ({"shape": [4, 5, 8], "strides": [50, 10, 1]}, [20, 8, 1, 1], {"shape": [20, 8, 1, 1], "strides": [10, 1, 1, 1]}),
    ({"shape": [4, 5, 8], "strides": [50, 10, 1]}, [1, 1, 20, 8], {"shape": [1, 1, 20, 8], "strides": [200, 200, 10, 1]}),
    ({"shape": [845], "strides": [1]}, [169, 5], {"shape": [169, 5], "strides": [5, 1]}),
    ({"shape": [10, 1, 18, 2], "strides": [36, 36, 2, 1]}, [10, 4, 9], {"shape": [10, 4, 9], "strides": [36, 9, 1]}),
    ({"shape": [13, 13, 5, 1], "strides": [1625, 125, 25, 1]}, [845, 1], {"shape": [845, 1], "strides": [25, 1]}),
    ({"shape": [1], "strides": [1]}, [1, 1], {"shape": [1, 1], "strides": [1, 1]}),
])
def test_in_place_reshape_reference_vectors(existing, new_shape, want):
    assert strip(d.in_place_reshape(existing, new_shape)) == want


def test_dimensions_default_strides_and_validation():
    assert d.dimensions([2, 3, 4])["strides"] == [12, 4, 1]
    assert d.dimensions([3, 4], strides=[8, 1])["strides"] == [8, 1]
    with pytest.raises(d.DimensionError):
        d.dimensions([3, 4], strides=[2, 1])  # stride too small for the element count


def test_dense_and_access_increasing():
    assert d.dense({"shape": [3, 3], "strides": [3, 1]})
    assert not d.dense({"shape": [3, 2], "strides": [3, 1]})          # pitched rows
    assert d.dense({"shape": [3], "strides": [1]}) and not d.dense({"shape": [3], "strides": [3]})
    assert d.dense({"shape": [3, 1, 1], "strides": [1, 1, 1]})
    t = d.transpose({"shape": [4, 4, 3], "strides": [12, 3, 1]}, [2, 0, 1])
    assert t == {"shape": [3, 4, 4], "strides": [1, 12, 3]}
    assert d.dense(t) and not d.access_increasing(t)


def test_max_shape_pads_like_the_reference():
    r = d.dimension_seq_to_max_shape({"shape": [2, 3, 3], "strides": [9, 3, 1]}, {"shape": [3, 1], "strides": [1, 1]})
    assert r["max-shape"] == [2, 3, 3]
    assert r["dimensions"][1] == {"shape": [1, 3, 1], "strides": [3, 1, 1]}


def test_select_offsets_and_strides():
    base = {"shape": [2, 3, 3], "strides": [9, 3, 1]}
    r = d.select(base, d.ALL, d.ALL, [1, 2])
    assert r == {"dimensions": {"shape": [2, 3, 2], "strides": [9, 3, 1]}, "elem-offset": 1}
    r = d.select(base, 1, d.ALL, 2)
    assert r == {"dimensions": {"shape": [3], "strides": [3]}, "elem-offset": 11}
    r = d.select(base, [1], [1], d.ALL)
    assert r == {"dimensions": {"shape": [1, 1, 3], "strides": [9, 3, 1]}, "elem-offset": 12}
    with pytest.raises(d.DimensionError):
        d.select(base, d.ALL, d.ALL, [2, 1])
    with pytest.raises(d.DimensionError):
        d.select(base, d.ALL, d.ALL, [3])


def test_minimize():
    assert d.minimize({"shape": [4, 1, 5, 8], "strides": [40, 40, 8, 1]}) == {"shape": [160], "strides": [1]}
    assert d.minimize({"shape": [4, 5, 8], "strides": [50, 10, 1]}) == {"shape": [20, 8], "strides": [10, 1]}
    assert d.minimize({"shape": [1, 1], "strides": [1, 1]}) == {"shape": [1], "strides": [1]}
