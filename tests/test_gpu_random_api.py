"""Seeded sweeps over the callbacks' argument space rather than over sizes: ranks up to five, contraction and batch
axes in any position and order, reductions over any subset of axes with and without kept axes, `argmax` over the
flattened tensor, `take` / `gather` along any axis with indices of any rank, broadcasting with explicit axes.  Every
case runs on the device and on the CPU oracle and compares bits: float operands hold small integers, so every sum of
products is exact whatever the order of its additions."""
import os

import numpy as np
import pytest

from nx_amd import nx as Nx
from nx_amd import types as T
from support import assert_bits_equal, seed_of
from test_gpu_elementwise import both, rand_raw

pytestmark = pytest.mark.gpu

# HIPNX_SWEEP_OFFSET=n shifts every sweep to cases n, n + 1, ... (the committed run is offset 0)
OFFSET = int(os.environ.get("HIPNX_SWEEP_OFFSET", "0"))
DIMS = [1, 1, 2, 3, 4, 5, 7, 8, 9, 16, 17, 33]


def draw_shape(rng, rank, limit=20000):
    while True:
        shape = tuple(int(rng.choice(DIMS)) for _ in range(rank))
        if int(np.prod(shape, dtype=np.int64)) <= limit:
            return shape


def small_ints(rng, ty, shape, span=3):
    """Values in [-span, span] (from 0 for unsigned types) in the raw representation of `ty`."""
    ty = T.normalize(ty)
    lo = 0 if ty[0] == "u" else -span
    v = rng.integers(lo, span + 1, size=shape)
    if ty == ("bf", 16):
        return (v.astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    return v.astype(T.numpy_dtype(ty))


@pytest.mark.parametrize("case", range(300))
def test_dot_over_random_contraction_and_batch_axes(case, hip, oracle):
    rng = np.random.default_rng(seed_of("api-dot", case + OFFSET))
    nb, nc = int(rng.integers(0, 3)), int(rng.integers(1, 3))
    batch = [int(rng.choice([1, 2, 3, 5])) for _ in range(nb)]
    contract = [int(rng.choice([1, 2, 3, 8, 16, 40, 64, 128])) for _ in range(nc)]
    free1 = [int(rng.choice(DIMS)) for _ in range(int(rng.integers(0, 3)))]
    free2 = [int(rng.choice(DIMS)) for _ in range(int(rng.integers(0, 3)))]

    def operand(free):
        # batch axes lead; the contracted and the free axes follow in a random order
        rest = [("c", i) for i in range(nc)] + [("f", i) for i in range(len(free))]
        order = [rest[i] for i in rng.permutation(len(rest))]
        shape = tuple(batch) + tuple(contract[i] if k == "c" else free[i] for k, i in order)
        pos = {i: nb + order.index(("c", i)) for i in range(nc)}
        return shape, pos

    s1, p1 = operand(free1)
    s2, p2 = operand(free2)
    pairing = rng.permutation(nc).tolist()  # the pairs are given in any order
    c1, c2 = [p1[i] for i in pairing], [p2[i] for i in pairing]
    if rng.random() < 0.3:  # negative axes count from the end
        c1 = [a - len(s1) for a in c1]
    ty, out = [("s8", "s32"), ("s32", None), ("f32", None), ("bf16", None), ("s16", None), ("u8", "u32"), ("f16", None), ("bf16", "f32"),
               ("s64", None), ("f64", None)][int(rng.integers(0, 10))]
    a, b = small_ints(rng, ty, s1), small_ints(rng, ty, s2)
    ha, oa = both(a, ty, hip, oracle)
    hb, ob = both(b, ty, hip, oracle)
    kw = {"out_type": out} if out else {}
    bax = list(range(nb))
    what = f"dot {ty} {s1} c{c1} x {s2} c{c2} batch {bax}"
    assert_bits_equal(Nx.dot(ha, c1, bax, hb, c2, bax, **kw), Nx.dot(oa, c1, bax, ob, c2, bax, **kw), what)


@pytest.mark.parametrize("case", range(300))
def test_reductions_over_random_axis_sets(case, hip, oracle):
    rng = np.random.default_rng(seed_of("api-reduce", case + OFFSET))
    rank = int(rng.integers(1, 6))
    shape = draw_shape(rng, rank)
    ty = ["s32", "u8", "s8", "s64", "f32", "bf16", "f16", "f64", "u16"][int(rng.integers(0, 9))]
    x = small_ints(rng, ty, shape, span=2)
    hx, ox = both(x, ty, hip, oracle)
    axes = None if rng.random() < 0.15 else sorted(rng.choice(rank, size=int(rng.integers(1, rank + 1)), replace=False).tolist())
    if axes is not None and rng.random() < 0.3:
        axes = [a - rank for a in axes]
    keep = bool(rng.integers(0, 2))
    what = f"{ty}{shape} axes {axes} keep {keep}"
    for op in ("sum", "reduce_max", "reduce_min", "all", "any"):
        assert_bits_equal(getattr(Nx, op)(hx, axes=axes, keep_axes=keep), getattr(Nx, op)(ox, axes=axes, keep_axes=keep), f"{op} {what}")
    if int(np.prod(shape)) <= 4096:  # (values up to 2: the product of a long axis still wraps or overflows alike on both sides)
        y = small_ints(rng, ty, shape, span=1)
        hy, oy = both(y, ty, hip, oracle)
        assert_bits_equal(Nx.product(hy, axes=axes, keep_axes=keep), Nx.product(oy, axes=axes, keep_axes=keep), f"product {what}")
    axis = None if rng.random() < 0.2 else int(rng.integers(-rank, rank))
    tie = ["low", "high"][int(rng.integers(0, 2))]
    out_ty = ["s32", "u32", "s64", "u8" if max(shape) <= 200 and int(np.prod(shape)) <= 200 else "s32"][int(rng.integers(0, 4))]
    for op in ("argmax", "argmin"):
        assert_bits_equal(getattr(Nx, op)(hx, axis=axis, tie_break=tie, keep_axis=keep, type=out_ty),
                          getattr(Nx, op)(ox, axis=axis, tie_break=tie, keep_axis=keep, type=out_ty), f"{op} {what} axis {axis} {tie} -> {out_ty}")


@pytest.mark.parametrize("case", range(300))
def test_binary_ops_over_random_ranks_and_numbers(case, hip, oracle):
    rng = np.random.default_rng(seed_of("api-binary", case + OFFSET))
    rank = int(rng.integers(0, 6))
    shape = draw_shape(rng, rank)

    def operand_shape():
        s = [d if rng.random() < 0.65 else 1 for d in shape]
        return tuple(s[int(rng.integers(0, len(s) + 1)):])

    ls, rs = operand_shape(), operand_shape()
    types = ["f32", "bf16", "f16", "f64", "s8", "s16", "s32", "s64", "u8", "u16", "u32"]
    lt, rt = types[int(rng.integers(0, 11))], types[int(rng.integers(0, 11))]
    op = ["add", "subtract", "multiply", "max", "min", "less", "equal", "not_equal", "greater_equal", "logical_and", "logical_or", "logical_xor"][int(rng.integers(0, 12))]
    a, b = rand_raw(rng, lt, ls), rand_raw(rng, rt, rs)
    ha, oa = both(a, lt, hip, oracle)
    hb, ob = both(b, rt, hip, oracle)
    what = f"{op} {lt}{ls} {rt}{rs}"

    def check(on_device, on_oracle, what):
        try:
            want = on_oracle()
        except Exception as e:  # the reference raises where a finite value overflows f16: the device writes infinity
            assert "overflows" in str(e), what
        else:
            assert_bits_equal(on_device(), want, what)

    f = getattr(Nx, op)
    check(lambda: f(ha, hb), lambda: f(oa, ob), what)
    number = [2, -3, 0.5, 1.0, 7, 0.1, 0.044715, -1.0e-3, 3.0e9, 300][int(rng.integers(0, 10))]  # some inexact in every float type, some beyond the narrow integers
    check(lambda: f(ha, number), lambda: f(oa, number), f"{what} with the number {number} on the right")
    check(lambda: f(number, hb), lambda: f(number, ob), f"{what} with the number {number} on the left")


@pytest.mark.parametrize("case", range(300))
def test_take_and_gather_along_random_axes(case, hip, oracle):
    rng = np.random.default_rng(seed_of("api-take", case + OFFSET))
    rank = int(rng.integers(1, 5))
    shape = draw_shape(rng, rank)
    ty = ["u8", "s16", "bf16", "f32", "s64", "f64"][int(rng.integers(0, 6))]
    x = rand_raw(rng, ty, shape)
    hx, ox = both(x, ty, hip, oracle)
    axis = int(rng.integers(-rank, rank))
    n = shape[axis]
    ishape = draw_shape(rng, int(rng.integers(0, 3)), limit=300)
    ity = ["s32", "s64", "u32", "u8", "s8", "u16"][int(rng.integers(0, 6))]
    top = min(n, 127 if ity in ("s8",) else 255 if ity == "u8" else n)
    idx = rng.integers(0, top, size=ishape).astype(T.numpy_dtype(T.normalize(ity)))
    hi, oi = both(idx, ity, hip, oracle)
    assert_bits_equal(Nx.take(hx, hi, axis=axis), Nx.take(ox, oi, axis=axis), f"take {ty}{shape} axis {axis} indices {ity}{ishape}")
    depth = int(rng.integers(1, rank + 1))
    gaxes = rng.choice(rank, size=depth, replace=False).tolist()  # in any order
    lead = draw_shape(rng, int(rng.integers(0, 3)), limit=200)
    gidx = np.stack([rng.integers(0, shape[a], size=lead) for a in gaxes], axis=-1).astype(np.int64 if rng.random() < 0.5 else np.int32)
    gty = "s64" if gidx.dtype == np.int64 else "s32"
    hg, og = both(gidx, gty, hip, oracle)
    assert_bits_equal(Nx.gather(hx, hg, axes=gaxes), Nx.gather(ox, og, axes=gaxes), f"gather {ty}{shape} axes {gaxes} indices {gty}{gidx.shape}")


@pytest.mark.parametrize("case", range(250))
def test_layout_callbacks_over_random_ranks(case, hip, oracle):
    rng = np.random.default_rng(seed_of("api-layout", case + OFFSET))
    rank = int(rng.integers(1, 6))
    shape = draw_shape(rng, rank)
    ty = ["u8", "s16", "bf16", "f32", "s64", "f64", "s8"][int(rng.integers(0, 7))]
    x = rand_raw(rng, ty, shape)
    hx, ox = both(x, ty, hip, oracle)
    perm = rng.permutation(rank).tolist()
    assert_bits_equal(Nx.transpose(hx, perm), Nx.transpose(ox, perm), f"transpose {ty}{shape}{perm}")
    # broadcast with explicit axes: the operand's axes land on an increasing choice of the new shape's axes
    extra = int(rng.integers(0, 3))
    new_rank = rank + extra
    where = sorted(rng.choice(new_rank, size=rank, replace=False).tolist())
    new = [int(rng.choice([1, 2, 3, 4])) for _ in range(new_rank)]
    src = list(shape)
    for k, a in enumerate(where):
        if rng.random() < 0.3:
            src[k] = 1  # a unit axis stretches
            new[a] = int(rng.choice([1, 2, 5]))
        else:
            new[a] = shape[k]
    if int(np.prod(new, dtype=np.int64)) <= 200000:
        y = rand_raw(rng, ty, tuple(src))
        hy, oy = both(y, ty, hip, oracle)
        assert_bits_equal(Nx.broadcast(hy, tuple(new), axes=where), Nx.broadcast(oy, tuple(new), axes=where), f"broadcast {ty}{tuple(src)} -> {tuple(new)} axes {where}")
    to = ["f32", "bf16", "f16", "s32", "s64", "u8", "f64", "s8", "u16", "u32"][int(rng.integers(0, 10))]
    try:
        want = Nx.as_type(ox, to)
    except Exception as e:  # the reference raises where a finite value overflows f16: the device writes infinity
        assert "overflows" in str(e)
    else:
        assert_bits_equal(Nx.as_type(hx, to), want, f"as_type {ty}->{to} {shape}")
    # metadata-only callbacks between two computing ones
    flat = int(np.prod(shape))
    hr, orr = Nx.reshape(Nx.negate(hx), (flat,)), Nx.reshape(Nx.negate(ox), (flat,))
    assert_bits_equal(Nx.abs(hr), Nx.abs(orr), f"reshape {ty}{shape}")
    ones = [i for i, d in enumerate(shape) if d == 1]
    if ones:
        assert_bits_equal(Nx.add(Nx.squeeze(hx, axes=ones), 1), Nx.add(Nx.squeeze(ox, axes=ones), 1), f"squeeze {ty}{shape}{ones}")
