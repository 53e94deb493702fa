"""Shape / stride algebra of cortex tensors: a Python mirror of
``src/cortex/tensor/dimensions.clj``.

A *dimensions* value is a dict ``{"shape": [...], "strides": [...]}`` with the
slowest-changing dimension first and strides in elements.  A shape entry may be
an index tensor (any object with ``ecount()``) instead of a number; that
dimension is then addressed indirectly (``dimensions.clj:7-9``).

Everything here is host-side integer logic shared by all backends; the device
library re-derives the same address function from the resulting maps.
"""
from __future__ import annotations

from typing import List, Sequence


class DimensionError(ValueError):
    """Stands in for the ``ex-info`` thrown by ``when-not-error``."""

    def __init__(self, message: str, data=None):
        super().__init__(f"{message} {data or {}}")
        self.data = data or {}


def _is_number(x) -> bool:
    return isinstance(x, int) or (hasattr(x, "__index__") and not hasattr(x, "ecount"))


def _entry(shape_entry) -> int:
    """``disambiguate-shape-entry`` (:48-53)."""
    if _is_number(shape_entry):
        return int(shape_entry)
    return int(shape_entry.ecount())


def disambiguate_shape(shape_vec) -> List[int]:
    return [_entry(s) for s in shape_vec]


def direct_shape(shape) -> bool:
    return all(_is_number(s) for s in shape)


def extend_strides(shape, strides) -> List[int]:
    """``extend-strides`` (:75-92): fills missing leading strides row-major."""
    rev_strides = list(reversed(list(strides or [])))
    rev_shape = list(reversed(disambiguate_shape(shape)))
    out: List[int] = []
    for i in range(len(shape)):
        cur = rev_strides[i] if i < len(rev_strides) else None
        if i == 0:
            out.append(cur if cur is not None else 1)
        else:
            out.append(cur if cur is not None else out[i - 1] * rev_shape[i - 1])
    return list(reversed(out))


def dimensions(shape, names=None, strides=None) -> dict:
    """``dimensions`` (:95-118)."""
    strides = extend_strides(shape, strides)
    pairs = sorted(zip(disambiguate_shape(shape), strides), key=lambda p: -p[1])
    max_stride = max([0] + [p[1] for p in pairs])
    elem_count = 1
    for s, _ in pairs[1:]:
        elem_count *= s
    if not elem_count <= max_stride:
        raise DimensionError("Stride appears to be too small for element count",
                             {"max-stride": max_stride, "elem-count": elem_count, "strides": strides, "shape": list(shape)})
    return {"shape": list(shape), "strides": strides, "names": names}


def ecount(dims) -> int:
    n = 1
    for s in disambiguate_shape(dims["shape"]):
        n *= s
    return n


def shape(dims) -> List[int]:
    return disambiguate_shape(dims["shape"])


def to_2d_shape(dims) -> List[int]:
    """``->2d-shape`` (:144-153)."""
    shp = dims["shape"]
    if not shp:
        raise DimensionError("Invalid shape in dimension map", {"shape": shp})
    if len(shp) == 1:
        return [1, _entry(shp[0])]
    if not direct_shape(shp[:-1]):
        raise DimensionError("Index buffers not supported for this operation.")
    n = 1
    for s in shp[:-1]:
        n *= int(s)
    return [n, _entry(shp[-1])]


def to_batch_shape(dims) -> List[int]:
    """``->batch-shape`` (:156-165)."""
    shp = dims["shape"]
    if not shp:
        raise DimensionError("Invalid shape in dimension map", {"shape": shp})
    if len(shp) == 1:
        return [1, _entry(shp[0])]
    if not direct_shape(shp[1:]):
        raise DimensionError("Index buffers not supported for this operation.")
    n = 1
    for s in shp[1:]:
        n *= int(s)
    return [_entry(shp[0]), n]


def dense(dims) -> bool:
    """``dense?`` (:178-191)."""
    shp, strides = dims["shape"], dims["strides"]
    if not direct_shape(shp):
        return False
    if len(shp) == 1:
        return int(strides[0]) == 1
    pairs = [(int(s), int(st)) for s, st in zip(shp, strides) if int(s) != 1]
    pairs.sort(key=lambda p: -p[1])
    if not pairs:
        return False
    rest = 1
    for s, _ in pairs[1:]:
        rest *= s
    return pairs[0][1] == rest


def direct(dims) -> bool:
    return direct_shape(dims["shape"])


def indirect(dims) -> bool:
    return not direct(dims)


def access_increasing(dims) -> bool:
    """``access-increasing?`` (:204-211)."""
    if not direct_shape(dims["shape"]):
        return False
    st = dims["strides"]
    return all(st[i] >= st[i + 1] for i in range(len(st) - 1))


def elem_idx_to_addr(rev_shape, rev_strides, rev_max_shape, arg: int, index_lookup=None) -> int:
    """``elem-idx->addr`` (:226-252).  ``index_lookup(entry, i)`` reads element
    ``i`` of an index tensor; it is only needed for indirect shapes."""
    offset = 0
    for i in range(len(rev_shape)):
        next_max = int(rev_max_shape[i])
        entry = rev_shape[i]
        next_dim = _entry(entry)
        shape_idx = arg % next_dim
        arg //= next_max
        if _is_number(entry):
            offset += int(rev_strides[i]) * shape_idx
        else:
            offset += int(rev_strides[i]) * int(index_lookup(entry, shape_idx))
    return offset


def max_extend_strides(shp, strides, max_count: int) -> List[int]:
    """``max-extend-strides`` (:280-300)."""
    shp = disambiguate_shape(shp)
    mi = 0
    for i in range(1, len(shp)):
        if strides[i] > strides[mi]:
            mi = i
    stride_val = strides[mi] * shp[mi]
    return [stride_val] * (max_count - len(strides)) + list(strides)


def dimension_seq_to_max_shape(*args) -> dict:
    """``dimension-seq->max-shape`` (:326-353)."""
    for a in args:
        if len(a["shape"]) != len(a["strides"]):
            raise DimensionError("Some dimensions have different shape and stride counts", {"args": list(args)})
    max_count = max([0] + [len(a["shape"]) for a in args])
    strides = [max_extend_strides(a["shape"], a["strides"], max_count) for a in args]
    shapes = [[1] * (max_count - len(a["shape"])) + list(a["shape"]) for a in args]
    max_shape = [max([0] + [disambiguate_shape(s)[i] for s in shapes]) for i in range(max_count)]
    return {"max-shape": max_shape,
            "dimensions": [{"shape": s, "strides": st} for s, st in zip(shapes, strides)]}


def minimize(dims) -> dict:
    """``minimize`` (:356-383): strip size-1 dimensions, merge packed neighbours."""
    stripped = [(s, st) for s, st in zip(dims["shape"], dims["strides"]) if not (_is_number(s) and int(s) == 1)]
    if not stripped:
        return {"shape": [1], "strides": [1]}
    rev = list(reversed(stripped))
    out = [rev[0]]
    for (cur_shp, cur_stride), (last_shp, last_stride) in zip(rev[1:], rev[:-1]):
        if _is_number(last_shp) and int(cur_stride) == int(last_shp) * int(last_stride):
            str_shp, str_str = out[-1]
            out[-1] = (int(str_shp) * int(cur_shp), str_str)
        else:
            out.append((cur_shp, cur_stride))
    out.reverse()
    return {"shape": [s for s, _ in out], "strides": [st for _, st in out]}


def in_place_reshape(existing_dims, new_shape: Sequence[int]) -> dict:
    """``in-place-reshape`` (:386-470)."""
    new_shape = list(new_shape)
    new_dims = dimensions(new_shape)
    if not ecount(new_dims) <= ecount(existing_dims):
        raise DimensionError("Reshaped dimensions are larger than tensor",
                             {"tensor-ecount": ecount(existing_dims), "reshape-ecount": ecount(new_dims)})
    if access_increasing(existing_dims) and dense(existing_dims):
        return {"shape": new_shape, "strides": extend_strides(new_shape, [])}
    if access_increasing(existing_dims):
        existing = minimize(existing_dims)
        info = [[int(s), int(st)] for s, st in zip(reversed(existing["shape"]), reversed(existing["strides"]))]
        old_count = len(info)
        max_old_idx = old_count - 1
        rev_shape = list(reversed(new_shape))
        rev_new_strides: List[int] = []
        new_idx = old_idx = 0
        while new_idx < len(new_shape):
            old_dim, old_stride = info[min(old_idx, max_old_idx)]
            new_dim = int(rev_shape[new_idx])
            if not (old_idx < old_count or new_dim == 1):
                raise DimensionError("Ran out of old shape dimensions",
                                     {"old-idx": old_idx, "rev-new-strides": rev_new_strides, "new-dim": new_dim})
            if new_dim == 1:
                last = rev_new_strides[-1] if rev_new_strides else 1
                prev = rev_shape[new_idx - 1] if new_idx >= 1 else 1
                rev_new_strides.append(int(last) * int(prev))
                new_idx += 1
            elif old_dim == new_dim:
                rev_new_strides.append(old_stride)
                new_idx += 1
                old_idx += 1
            elif old_dim < new_dim:
                raise DimensionError("Cannot combine dimensions across padded boundaries",
                                     {"old-dim": old_dim, "new-dim": new_dim})
            else:
                if old_dim % new_dim != 0:
                    raise DimensionError("New dimension not commensurate with old dimension",
                                         {"old-dim": old_dim, "new-dim": new_dim})
                info[old_idx] = [old_dim // new_dim, old_stride * new_dim]
                rev_new_strides.append(old_stride)
                new_idx += 1
        return {"shape": new_shape, "strides": extend_strides(new_shape, list(reversed(rev_new_strides)))}
    raise DimensionError("Cannot (at this point) in-place-reshape transposed or indirect dimensions")


def transpose(dims, reorder_vec: Sequence[int]) -> dict:
    """``transpose`` (:473-484): permutes shape and strides; no data moves."""
    shp, strides = dims["shape"], dims["strides"]
    if len(set(reorder_vec)) != len(shp):
        raise DimensionError("Every dimension must be represented in the reorder vector",
                             {"shape": shp, "reorder-vec": list(reorder_vec)})
    return {"shape": [shp[i] for i in reorder_vec], "strides": [strides[i] for i in reorder_vec]}


ALL = "all"


def select(dims, *args) -> dict:
    """``select`` (:487-569).  Each argument is ``ALL``, a number, an increasing
    list of indexes (a contiguous range) or an index tensor.  Returns
    ``{"dimensions": ..., "elem-offset": n}``."""
    data_shp = shape(dims)
    if len(data_shp) != len(args):
        raise DimensionError("arg count must match shape count", {"shape": data_shp, "args": list(args)})
    shp, strides = dims["shape"], dims["strides"]
    rev_shape = list(reversed(shp))
    rev_strides = list(reversed(strides))
    conv = []
    for dim, arg in zip(shp, args):
        if isinstance(arg, str) and arg == ALL:
            conv.append(list(range(_entry(dim))))
        elif isinstance(arg, (list, tuple, range)):
            arg = list(arg)
            if not all(arg[i] < arg[i + 1] for i in range(len(arg) - 1)):
                raise DimensionError("Argument is not monotonicly increasing", {"argument": arg})
            if not _entry(dim) > max([0] + arg):
                raise DimensionError("Argument out of range of dimension", {"dimension": dim, "argument": arg})
            conv.append(arg)
        elif _is_number(arg):
            conv.append(int(arg))
        elif hasattr(arg, "ecount"):
            if len(arg.shape()) != 1:
                raise DimensionError("Index arguments must be vectors", {"arg-shape": arg.shape()})
            conv.append(arg)
        else:
            raise DimensionError("argument to select of incorrect type", {"arg": arg})
    rev_args = list(reversed(conv))
    products = []
    for item in rev_shape:
        products.append(_entry(item) * (products[-1] if products else 1))
    first_elem_idx = 0
    for arg, prev in zip(rev_args, [None] + products):
        if isinstance(arg, int):
            start = arg
        elif isinstance(arg, list):
            start = arg[0]
        else:
            start = 0  # indirect indexing: relative index 0
        first_elem_idx += (prev or 1) * start
    elem_addr = elem_idx_to_addr(rev_shape, rev_strides, rev_shape, first_elem_idx,
                                 index_lookup=lambda entry, i: 0)
    kept = [(a, st) for a, st in zip(rev_args, rev_strides) if not isinstance(a, int)]
    new_strides = list(reversed([st for _, st in kept]))
    new_shape = list(reversed([len(a) if isinstance(a, list) else a for a, _ in kept]))
    return {"dimensions": {"shape": new_shape, "strides": new_strides}, "elem-offset": elem_addr}
