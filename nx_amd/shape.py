"""Shape inference used to build output templates (reference: nx/lib/nx/shape.ex).

Shapes are tuples of ints.  Axis names are not modelled (every name is None): they never reach a
backend callback's arithmetic.
"""
from __future__ import annotations

import functools

from math import prod


def size(shape) -> int:
    return prod(shape)


def normalize_axis(shape, axis: int) -> int:
    """Nx.Shape.normalize_axis/4 (shape.ex:1110-1143)."""
    rank = len(shape)
    if not isinstance(axis, int):
        raise ValueError(f"axis must be an integer, got {axis!r}")
    if axis < 0 and abs(axis) <= rank:
        return rank + axis
    if 0 <= axis < rank:
        return axis
    raise ValueError(f"given axis ({axis}) invalid for shape with rank {rank}")


def normalize_axes(shape, axes):
    """Nx.Shape.normalize_axes/4 (shape.ex:1145-1164): normalises and rejects duplicates."""
    out = [normalize_axis(shape, a) for a in axes]
    if len(set(out)) != len(out):
        raise ValueError(f"axes {list(axes)!r} must be unique integers between 0 and {len(shape) - 1}")
    return out


def binary_broadcast(left, right):
    """Nx.Shape.binary_broadcast/4 (shape.ex:316-376): numpy-style, right-aligned."""
    left, right = tuple(left), tuple(right)
    if left == right:
        return left
    rank = max(len(left), len(right))
    lp = (1,) * (rank - len(left)) + left
    rp = (1,) * (rank - len(right)) + right
    out = []
    for l, r in zip(lp, rp):
        if l == r or l == 1 or r == 1:
            out.append(max(l, r))
        else:
            raise ValueError(f"cannot broadcast tensor of dimensions {_fmt(left)} to {_fmt(right)}")
    return tuple(out)


def broadcast_strides(shape, out_shape):
    """Element strides of `shape` viewed in `out_shape` (right-aligned), 0 on broadcast axes --
    the index arithmetic behind broadcast_data/2 (binary_backend.ex:228-276)."""
    return list(_broadcast_strides(tuple(shape), tuple(out_shape)))


@functools.lru_cache(maxsize=4096)
def _broadcast_strides(shape, out_shape):
    rank = len(out_shape)
    padded = (1,) * (rank - len(shape)) + shape
    strides, s = [0] * rank, 1
    for a in range(rank - 1, -1, -1):
        strides[a] = 0 if padded[a] == 1 else s
        s *= padded[a]
    return tuple(strides)


def broadcast_axes(shape, new_shape):
    """Nx.Shape.broadcast_axes/2 (shape.ex:1197-1207): default axes = the trailing ones."""
    return list(range(len(new_shape) - len(shape), len(new_shape)))


def broadcast(old_shape, new_shape, axes):
    """Nx.Shape.broadcast!/3 (shape.ex:205-245): validates an explicit-axes broadcast."""
    old_shape, new_shape = tuple(old_shape), tuple(new_shape)
    if len(axes) != len(old_shape):
        raise ValueError("expected length of axes to match rank of shape")
    if len(old_shape) > len(new_shape):
        raise ValueError(f"cannot broadcast tensor of dimensions {_fmt(old_shape)} to {_fmt(new_shape)}")
    for pos, a in enumerate(axes):
        if old_shape[pos] != 1 and old_shape[pos] != new_shape[a]:
            raise ValueError(
                f"cannot broadcast tensor of dimensions {_fmt(old_shape)} to {_fmt(new_shape)} with axes {list(axes)}")
    return new_shape


def contract(shape, axes, keep_axes: bool):
    """Nx.Shape.contract/4 (shape.ex:413-435)."""
    out = []
    for i, d in enumerate(shape):
        if i not in axes:
            out.append(d)
        elif keep_axes:
            out.append(1)
    return tuple(out)


def transpose(shape, perm):
    """Nx.Shape.transpose/3 (shape.ex:612-640)."""
    if sorted(perm) != list(range(len(shape))):
        raise ValueError(f"axes {list(perm)!r} must be a permutation of the tensor axes")
    return tuple(shape[a] for a in perm)


def zip_reduce(s1, c1, s2, c2):
    """Nx.Shape.zip_reduce/6 (shape.ex:484-519)."""
    if len(c1) != len(c2):
        raise ValueError("dot/zip_reduce expects the same number of contraction axes on both sides")
    for a1, a2 in zip(c1, c2):
        if s1[a1] != s2[a2]:
            raise ValueError(
                "dot/zip_reduce expects shapes to be compatible, "
                f"dimension {a1} of left-side ({s1[a1]}) does not equal dimension {a2} of right-side ({s2[a2]})")
    return contract(s1, c1, False) + contract(s2, c2, False)


def dot(s1, c1, b1, s2, c2, b2):
    """Nx.Shape.dot/8 (shape.ex:1801-1911): batch axes lead, then left kept, then right kept."""
    if not b1 and b2:
        raise ValueError("left tensor must be batched if right tensor is batched")
    if b1 and not b2:
        raise ValueError("right tensor must be batched if left tensor is batched")
    valid = list(range(len(b1)))
    if b1 and list(b1) != valid:
        raise ValueError("invalid dot batch axis for the left tensor, batch axes must be successive"
                         f" dimensions starting from 0, got {list(b1)}")
    if b2 and list(b2) != valid:
        raise ValueError("invalid dot batch axis for the right tensor, batch axes must be successive"
                         f" dimensions starting from 0, got {list(b2)}")
    if [s1[a] for a in b1] != [s2[a] for a in b2]:
        raise ValueError("dot batch dimension sizes must match")
    if any(a in c1 for a in b1):
        raise ValueError(f"dot batch axes for left tensor ({list(b1)}) cannot be in contract axes ({list(c1)})")
    if any(a in c2 for a in b2):
        raise ValueError(f"dot batch axes for right tensor ({list(b2)}) cannot be in contract axes ({list(c2)})")
    nb = len(b1)
    batch_dims = tuple(s1[a] for a in b1)
    inner = zip_reduce(tuple(s1[nb:]), [a - nb for a in c1], tuple(s2[nb:]), [a - nb for a in c2])
    return batch_dims + inner


def take(shape, indices_shape, axis: int):
    """Nx.Shape.take/5 (shape.ex:1366-1382)."""
    return tuple(shape[:axis]) + tuple(indices_shape) + tuple(shape[axis + 1:])


def gather(shape, indices_shape, axes):
    """Nx.Shape.gather/3 (shape.ex:1643-1661)."""
    if len(indices_shape) == 0:
        raise ValueError("expected indices rank to be at least 1, got: 0")
    last = indices_shape[-1]
    if last > len(shape):
        raise ValueError(f"expected the last indices dimension size ({last}) to be less than or equal "
                         f"to the tensor rank ({len(shape)})")
    inner = tuple(d for i, d in enumerate(shape) if i not in axes)
    return tuple(indices_shape[:-1]) + inner


def squeeze(shape, axes):
    for a in axes:
        if shape[a] != 1:
            raise ValueError(f"cannot squeeze dimensions whose sizes are not 1, got {shape[a]} for dimension {a}")
    return tuple(d for i, d in enumerate(shape) if i not in axes)


def _fmt(shape) -> str:
    return "{" + ", ".join(str(d) for d in shape) + "}"


fmt = _fmt
