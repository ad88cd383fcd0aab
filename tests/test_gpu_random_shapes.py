"""Seeded sweeps over random shapes: the vector paths of the streaming kernels change with divisibility and
alignment (whole 16-byte vectors or ragged tails, one row or many, operands broadcast along rows or columns,
windows that start off a vector boundary), so every case draws its shape, its broadcast pattern and its
window at random, runs the callback on the device and on the CPU oracle, and compares bits."""
import numpy as np
import pytest

from nx_amd import nx as Nx
from nx_amd import types as T
from support import assert_bits_equal, seed_of
from test_gpu_elementwise import both, rand_raw

import os

pytestmark = pytest.mark.gpu

# HIPNX_SWEEP_OFFSET=n shifts every sweep to cases n, n + 1, ...: other shapes, types and windows than the ones every
# run covers, for an occasional longer hunt (the committed run is offset 0)
OFFSET = int(os.environ.get("HIPNX_SWEEP_OFFSET", "0"))

SIZES = [1, 2, 3, 4, 5, 7, 8, 9, 15, 16, 17, 24, 31, 32, 33, 40, 63, 64, 65, 96, 127, 128, 130, 255, 256, 264]


def draw_shape(rng, rank, limit=70000):
    while True:
        shape = tuple(int(rng.choice(SIZES)) for _ in range(rank))
        if np.prod(shape) <= limit:
            return shape


def broadcastable(rng, shape):
    """A shape that broadcasts to `shape`: some axes set to 1, some leading axes dropped."""
    s = [d if rng.random() < 0.6 else 1 for d in shape]
    drop = int(rng.integers(0, len(s)))
    return tuple(s[drop:]) if rng.random() < 0.4 else tuple(s)


@pytest.mark.parametrize("case", range(300))
def test_exact_binary_ops_on_random_broadcasts(case, hip, oracle):
    rng = np.random.default_rng(seed_of("binary", case + OFFSET))
    rank = int(rng.integers(1, 4))
    shape = draw_shape(rng, rank)
    ls, rs = broadcastable(rng, shape), broadcastable(rng, shape)
    if rng.random() < 0.5:
        ls = shape
    lt, rt = [("f32", "f32"), ("bf16", "bf16"), ("f16", "f16"), ("s32", "s32"), ("s64", "s64"), ("u8", "u8"), ("f32", "bf16"),
              ("s16", "s16"), ("f64", "f64"), ("bf16", "f32"), ("s32", "s64")][int(rng.integers(0, 11))]
    op = ["add", "subtract", "multiply", "max", "min", "less", "equal", "greater_equal", "logical_and"][int(rng.integers(0, 9))]
    a, b = rand_raw(rng, lt, ls), rand_raw(rng, rt, rs)
    ha, oa = both(a, lt, hip, oracle)
    hb, ob = both(b, rt, hip, oracle)
    assert_bits_equal(getattr(Nx, op)(ha, hb), getattr(Nx, op)(oa, ob), f"{op} {lt}{ls} {rt}{rs}")


@pytest.mark.parametrize("case", range(250))
def test_unary_conversions_and_selections_on_random_shapes(case, hip, oracle):
    rng = np.random.default_rng(seed_of("unary", case + OFFSET))
    shape = draw_shape(rng, int(rng.integers(1, 4)))
    ty = ["f32", "bf16", "f16", "s32", "s64", "u8", "f64", "s16"][int(rng.integers(0, 8))]
    x = rand_raw(rng, ty, shape)
    hx, ox = both(x, ty, hip, oracle)
    assert_bits_equal(Nx.negate(hx), Nx.negate(ox), f"negate {ty}{shape}")
    assert_bits_equal(Nx.abs(hx), Nx.abs(ox), f"abs {ty}{shape}")
    to = ["f32", "bf16", "f16", "s32", "s64", "u8", "f64"][int(rng.integers(0, 7))]
    try:
        want = Nx.as_type(ox, to)
    except Exception as e:  # the reference raises where a finite value overflows f16: the device writes infinity
        assert "overflows" in str(e)
    else:
        assert_bits_equal(Nx.as_type(hx, to), want, f"as_type {ty}->{to} {shape}")
    y = rand_raw(rng, ty, shape)
    hy, oy = both(y, ty, hip, oracle)
    hp, op_ = Nx.less(hx, hy), Nx.less(ox, oy)
    assert_bits_equal(Nx.select(hp, hx, hy), Nx.select(op_, ox, oy), f"select {ty}{shape}")


@pytest.mark.parametrize("case", range(250))
def test_exact_reductions_on_random_axes(case, hip, oracle):
    rng = np.random.default_rng(seed_of("reduce", case + OFFSET))
    rank = int(rng.integers(1, 4))
    shape = draw_shape(rng, rank)
    axes = sorted(rng.choice(rank, size=int(rng.integers(1, rank + 1)), replace=False).tolist())
    ty = ["s32", "u8", "s16", "s64", "f32", "bf16", "f16"][int(rng.integers(0, 7))]
    x = rand_raw(rng, ty, shape)
    hx, ox = both(x, ty, hip, oracle)
    assert_bits_equal(Nx.reduce_max(hx, axes=axes), Nx.reduce_max(ox, axes=axes), f"reduce_max {ty}{shape}{axes}")
    assert_bits_equal(Nx.reduce_min(hx, axes=axes), Nx.reduce_min(ox, axes=axes), f"reduce_min {ty}{shape}{axes}")
    if T.is_integer(T.normalize(ty)):
        assert_bits_equal(Nx.sum(hx, axes=axes), Nx.sum(ox, axes=axes), f"sum {ty}{shape}{axes}")
    axis = int(axes[0])
    assert_bits_equal(Nx.argmax(hx, axis=axis), Nx.argmax(ox, axis=axis), f"argmax {ty}{shape}{axis}")
    assert_bits_equal(Nx.argmin(hx, axis=axis, tie_break="high"), Nx.argmin(ox, axis=axis, tie_break="high"), f"argmin {ty}{shape}{axis}")


@pytest.mark.parametrize("case", range(250))
def test_copies_on_random_windows(case, hip, oracle):
    rng = np.random.default_rng(seed_of("copy", case + OFFSET))
    rank = int(rng.integers(1, 4))
    shape = draw_shape(rng, rank)
    ty = ["u8", "s16", "bf16", "f32", "s64"][int(rng.integers(0, 5))]
    x = rand_raw(rng, ty, shape)
    hx, ox = both(x, ty, hip, oracle)
    starts = [int(rng.integers(0, d)) for d in shape]
    lengths = [int(rng.integers(1, d - s + 1)) for d, s in zip(shape, starts)]
    strides = [int(rng.integers(1, 3)) if rng.random() < 0.25 else 1 for _ in shape]
    assert_bits_equal(Nx.slice(hx, starts, lengths, strides=strides), Nx.slice(ox, starts, lengths, strides=strides), f"slice {ty}{shape}")
    rev = sorted(rng.choice(rank, size=int(rng.integers(1, rank + 1)), replace=False).tolist())
    assert_bits_equal(Nx.reverse(hx, axes=rev), Nx.reverse(ox, axes=rev), f"reverse {ty}{shape}{rev}")
    perm = rng.permutation(rank).tolist()
    assert_bits_equal(Nx.transpose(hx, perm), Nx.transpose(ox, perm), f"transpose {ty}{shape}{perm}")
    new = tuple(int(rng.choice([2, 3, 8])) for _ in range(int(rng.integers(0, 2)))) + shape
    assert_bits_equal(Nx.broadcast(hx, new), Nx.broadcast(ox, new), f"broadcast {ty}{shape}->{new}")
    cfg = [(int(rng.integers(-1, 3)), int(rng.integers(-1, 3)), int(rng.integers(0, 2))) for _ in shape]
    if all(d + lo + hi + (d - 1) * it > 0 for d, (lo, hi, it) in zip(shape, cfg)):
        pv_h, pv_o = Nx.tensor(1, type=ty, backend=hip), Nx.tensor(1, type=ty, backend=oracle)
        assert_bits_equal(Nx.pad(hx, pv_h, cfg), Nx.pad(ox, pv_o, cfg), f"pad {ty}{shape}{cfg}")
    assert_bits_equal(Nx.concatenate([hx, hx], axis=rank - 1), Nx.concatenate([ox, ox], axis=rank - 1), f"concatenate {ty}{shape}")


DOT_M = [1, 3, 16, 33, 64, 65, 100, 128, 130, 192, 200, 256, 264, 300, 513]
DOT_N = [1, 8, 16, 40, 64, 72, 128, 136, 256, 264, 320, 520]
DOT_K = [1, 7, 8, 16, 24, 64, 72, 128, 136, 192, 256, 512, 1000, 1024, 4096]


@pytest.mark.parametrize("case", range(200))
def test_dot_on_random_shapes_types_and_layouts(case, hip, oracle):
    """The contraction picks its kernel from the shape (generic, K-inner MFMA, the tiled kernels in four tile
    sizes, the few-rows stream, K in splits, K extended by zeros): random extents, operand layouts, batch counts
    and types against the oracle -- int8 exactly, floats within the accumulation bound."""
    from test_gpu_dot import check_float_dot
    from support import values
    rng = np.random.default_rng(seed_of("dot", case + OFFSET))
    M, N, K = int(rng.choice(DOT_M)), int(rng.choice(DOT_N)), int(rng.choice(DOT_K))
    while M * N * K > 40_000_000:
        M, N, K = int(rng.choice(DOT_M)), int(rng.choice(DOT_N)), int(rng.choice(DOT_K))
    batch = int(rng.choice([1, 1, 1, 2, 3]))
    ty = ["bf16", "f16", "f32", "s8", "f64"][int(rng.integers(0, 5))]
    lk, rk = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))  # K-inner (True) or K-outer operand
    if ty == "s8":
        a = rng.integers(-127, 128, size=(batch, M, K)).astype(np.int8)
        b = rng.integers(-127, 128, size=(batch, K, N)).astype(np.int8)
    else:
        a, b = rand_raw(rng, ty, (batch, M, K), lo=-1, hi=1), rand_raw(rng, ty, (batch, K, N), lo=-1, hi=1)
    la = a if lk else np.ascontiguousarray(a.transpose(0, 2, 1))
    lb = b if not rk else np.ascontiguousarray(b.transpose(0, 2, 1))
    c1, c2 = [2] if lk else [1], [2] if rk else [1]
    kw = {"out_type": "s32"} if ty == "s8" else {}
    hla, ola = both(la, ty, hip, oracle)
    hlb, olb = both(lb, ty, hip, oracle)
    got = Nx.dot(hla, c1, [0], hlb, c2, [0], **kw)
    want = Nx.dot(ola, c1, [0], olb, c2, [0], **kw)
    what = f"dot {ty} batch {batch} {M}x{N}x{K} {'k-inner' if lk else 'k-outer'} {'k-inner' if rk else 'k-outer'}"
    if ty == "s8":
        assert_bits_equal(got, want, what)
    else:
        oa, ob = both(a, ty, hip, oracle)[1], both(b, ty, hip, oracle)[1]
        check_float_dot(got, want, values(oa), values(ob), "bmk,bkn->bmn", K, what)


# ---- the same sweeps at sizes where the kernels change shape: rows longer than a work-group's share (split rows), more
# vectors than one pass of the grid, column reductions under long axes, copies past 2^16 vectors ----------------------------

BIG = [1, 2, 3, 8, 17, 64, 100, 257, 1000, 1024, 4096, 4100, 8191, 32768, 40000, 65536, 70001, 131080, 262144, 1000003]


def draw_big_shape(rng, rank, lo=200_000, hi=5_000_000):
    while True:
        shape = tuple(int(rng.choice(BIG)) for _ in range(rank))
        if lo <= int(np.prod(shape, dtype=np.int64)) <= hi:
            return shape


@pytest.mark.parametrize("case", range(40))
def test_exact_callbacks_on_large_random_shapes(case, hip, oracle):
    rng = np.random.default_rng(seed_of("large", case + OFFSET))
    rank = int(rng.integers(1, 4))
    shape = draw_big_shape(rng, rank)
    ty = ["f32", "bf16", "s32", "u8", "f16", "s16", "s64", "f64"][int(rng.integers(0, 8))]
    x = rand_raw(rng, ty, shape)
    hx, ox = both(x, ty, hip, oracle)
    what = f"{ty}{shape}"
    # element-wise against a broadcast operand, and a conversion
    bs = broadcastable(rng, shape)
    y = rand_raw(rng, ty, bs)
    hy, oy = both(y, ty, hip, oracle)
    op = ["add", "subtract", "multiply", "max", "less", "equal"][int(rng.integers(0, 6))]
    assert_bits_equal(getattr(Nx, op)(hx, hy), getattr(Nx, op)(ox, oy), f"{op} {what} {bs}")
    to = ["f32", "bf16", "s32", "u8", "f64", "s64"][int(rng.integers(0, 6))]
    try:
        want = Nx.as_type(ox, to)
    except Exception as e:
        assert "overflows" in str(e)
    else:
        assert_bits_equal(Nx.as_type(hx, to), want, f"as_type {what} -> {to}")
    # reductions over a random axis set
    axes = sorted(rng.choice(rank, size=int(rng.integers(1, rank + 1)), replace=False).tolist())
    assert_bits_equal(Nx.reduce_max(hx, axes=axes), Nx.reduce_max(ox, axes=axes), f"reduce_max {what}{axes}")
    assert_bits_equal(Nx.reduce_min(hx, axes=axes, keep_axes=True), Nx.reduce_min(ox, axes=axes, keep_axes=True), f"reduce_min {what}{axes}")
    if T.is_integer(T.normalize(ty)):
        assert_bits_equal(Nx.sum(hx, axes=axes), Nx.sum(ox, axes=axes), f"sum {what}{axes}")
    axis = int(axes[-1])
    assert_bits_equal(Nx.argmax(hx, axis=axis), Nx.argmax(ox, axis=axis), f"argmax {what}{axis}")
    assert_bits_equal(Nx.argmin(hx, axis=None, tie_break="high", type="s64"), Nx.argmin(ox, axis=None, tie_break="high", type="s64"), f"argmin {what} flat")
    # copies
    perm = rng.permutation(rank).tolist()
    assert_bits_equal(Nx.transpose(hx, perm), Nx.transpose(ox, perm), f"transpose {what}{perm}")
    starts = [int(rng.integers(0, d)) for d in shape]
    lengths = [int(rng.integers(1, d - s + 1)) for d, s in zip(shape, starts)]
    assert_bits_equal(Nx.slice(hx, starts, lengths), Nx.slice(ox, starts, lengths), f"slice {what}{starts}{lengths}")
    n = shape[axis]
    idx = rng.integers(0, n, size=(int(rng.choice([1, 7, 300])),)).astype(np.int64)
    hi_, oi_ = both(idx, "s64", hip, oracle)
    assert_bits_equal(Nx.take(hx, hi_, axis=axis), Nx.take(ox, oi_, axis=axis), f"take {what} axis {axis}")


DOT_BIG_MN = [1, 16, 33, 64, 100, 128, 192, 256, 300, 512, 768, 1000, 1024, 1536, 2048, 3072, 4096, 11008]
DOT_BIG_K = [64, 128, 136, 512, 784, 1000, 1024, 2048, 4096, 8192, 11008]


@pytest.mark.parametrize("case", range(60))
def test_dot_on_large_random_shapes_against_f64_blas(case, hip):
    """The tile rules of the contraction (256 x 256, 256 x 128, 128 x 128 and 64 x 64 two-group tiles, K in splits, K
    extended by zeros, few rows, few columns) at the sizes that select them.  Operands hold small integers, so every
    partial sum is exact in f32 / s32 and in the f64 product the host's BLAS computes: the device must match it bit for
    bit whatever the order of its additions (bf16 results by truncation, f16 to nearest)."""
    from support import from_numpy
    rng = np.random.default_rng(seed_of("dot-large", case + OFFSET))
    while True:
        M, N, K = int(rng.choice(DOT_BIG_MN)), int(rng.choice(DOT_BIG_MN)), int(rng.choice(DOT_BIG_K))
        batch = int(rng.choice([1, 1, 1, 2, 4]))
        if 50_000_000 <= batch * M * N * K <= 9_000_000_000 and batch * (M + N) * K <= 200_000_000 and batch * M * N <= 40_000_000:
            break
    ty, out = [("s8", "s32"), ("bf16", None), ("bf16", "f32"), ("f16", None), ("f32", None), ("s8", "s32"), ("bf16", None), ("f64", None),
               ("f64", "f32")][int(rng.integers(0, 9))]
    lk, rk = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))  # K-inner (True) or K-outer operand
    span = 127 if ty == "s8" else 3
    a = rng.integers(-span, span + 1, size=(batch, M, K)).astype(np.int8)
    b = rng.integers(-span, span + 1, size=(batch, K, N)).astype(np.int8)
    want = np.matmul(a.astype(np.float64), b.astype(np.float64))  # exact: every sum is far below 2^53

    def raw(v):
        if ty == "s8":
            return v
        if ty == "bf16":
            return (v.astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
        return v.astype(np.float16 if ty == "f16" else np.float64 if ty == "f64" else np.float32)

    la = a if lk else np.ascontiguousarray(a.transpose(0, 2, 1))
    lb = b if not rk else np.ascontiguousarray(b.transpose(0, 2, 1))
    c1, c2 = [2] if lk else [1], [2] if rk else [1]
    kw = {"out_type": out} if out else {}
    got = Nx.dot(from_numpy(raw(la), ty, hip), c1, [0], from_numpy(raw(lb), ty, hip), c2, [0], **kw)
    res = hip.to_numpy(got)
    what = f"dot {ty}->{out or ty} batch {batch} {M}x{N}x{K} {'k-inner' if lk else 'k-outer'} {'k-inner' if rk else 'k-outer'}"
    out_ty = out or ty
    if out_ty == "s32":
        expect = want.astype(np.int64).astype(np.int32)
    elif out_ty == "bf16":
        expect = (want.astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    elif out_ty == "f16":
        with np.errstate(over="ignore"):
            expect = want.astype(np.float32).astype(np.float16)
    else:
        expect = want.astype(np.float64 if out_ty == "f64" else np.float32)
    assert res.shape == expect.shape, what
    same = res.view(np.uint8) == expect.view(np.uint8)
    assert same.all(), f"{what}: {int((~same).sum())} bytes differ"


@pytest.mark.parametrize("case", range(60))
def test_scaled_int8_dot_on_random_shapes(case, hip):
    """The quantised linear layer (dot to s32, as_type f32, multiply by scales) as one callback on the accumulators against
    the three callbacks one after the other: rows from one to several tiles, ragged columns, K in steps of 128, weights
    K-inner or K-outer, batches, every kind of scale; an integer check of the accumulators themselves on top
    (small operands: the s32 sums are exact in numpy's int64)."""
    from nx_amd import defn
    from support import from_numpy, raw
    rng = np.random.default_rng(seed_of("scaled-dot", case + OFFSET))
    m = int(rng.choice([1, 2, 7, 16, 33, 64, 65, 128, 200, 300, 520]))
    n = int(rng.choice([1, 8, 40, 64, 100, 256, 260, 512, 1000, 1100]))
    k = 128 * int(rng.choice([1, 2, 3, 5, 8, 16, 33]))
    batch = int(rng.choice([0, 0, 0, 2, 3]))
    k_outer = bool(rng.integers(0, 2))
    lead = (batch,) if batch else ()
    x = from_numpy(rng.integers(-127, 128, size=lead + (m, k), dtype=np.int8), "s8", hip)
    w = from_numpy(rng.integers(-127, 128, size=lead + ((k, n) if k_outer else (n, k)), dtype=np.int8), "s8", hip)
    kind = ["per_column", "per_row", "one", "constant"][int(rng.integers(0, 4))]
    r = len(lead)
    bx = [0] if batch else []

    def product(xq, wq):
        return Nx.dot(xq, [r + 1], bx, wq, [r] if k_outer else [r + 1], bx, out_type="s32")
    what = f"case {case + OFFSET}: {lead} {m}x{n}x{k} weights {'K-outer' if k_outer else 'K-inner'} scales {kind}"
    if kind == "constant":
        fun, args = (lambda xq, wq: Nx.multiply(Nx.as_type(product(xq, wq), "f32"), 0.0078125)), (x, w)
    else:
        shape = {"per_column": (n,), "per_row": (m, 1), "one": (1, 1)}[kind]
        sc = from_numpy(rng.uniform(1e-3, 1e-2, size=shape).astype(np.float32), "f32", hip)
        fun, args = (lambda xq, wq, s: Nx.multiply(Nx.as_type(product(xq, wq), "f32"), s)), (x, w, sc)
    want = defn.compile(fun, *args)(*args)
    planned = defn.compile(fun, *args, fuse=True)
    assert_bits_equal(planned(*args), want, what)
    # the accumulators, by int64 arithmetic on the host
    xs, ws = raw(x).astype(np.int64), raw(w).astype(np.int64)
    acc = np.matmul(xs, ws if k_outer else np.swapaxes(ws, -1, -2))
    got = raw(defn.compile(product, x, w)(x, w))
    assert np.array_equal(got, acc.astype(np.int32)), what
