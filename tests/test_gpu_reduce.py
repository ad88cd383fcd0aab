"""Device reductions (sum / product / reduce_max / reduce_min / argmax / argmin) against the CPU
oracle.  Integer and index results bit-exact; float sums within K * 2^-24 * sum|x| + 1 ulp (the
device folds in f64 in tree order, the reference in f64 sequentially); max/min exact bits."""
import numpy as np
import pytest

from nx_amd import nx as Nx
from nx_amd import types as T
from support import assert_bits_equal, from_numpy, seed_of, values
from test_gpu_elementwise import both, rand_raw

pytestmark = pytest.mark.gpu

SHAPES_AXES = [((1024, 1024), [1]), ((1024, 1024), [0]), ((1024, 1024), None), ((32, 512, 64), [2]),
               ((32, 512, 64), [1]), ((32, 512, 64), [0]), ((32, 512, 64), [0, 2]), ((32, 512, 64), [1, 2]),
               ((7, 13), [1]), ((7, 13), [0]), ((5, 3, 9, 2), [1, 3]), ((3, 70001), [1]), ((2, 4097, 3), [1]),
               ((1, 1), [0]), ((9,), None), ((2, 300000), [1]), ((1500000,), None), ((6, 1, 5), [1])]


def sum_bound(x64, axes, out_bits):
    """K * 2^-24 * sum|x| (+ an ulp of the output type) for the given reduction."""
    ax = tuple(range(x64.ndim)) if axes is None else tuple(axes)
    k = int(np.prod([x64.shape[a] for a in ax]))
    s = np.abs(x64).sum(axis=ax)
    eps = {64: 2.0 ** -52, 32: 2.0 ** -23, 16: 2.0 ** -7}[out_bits]
    return k * 2.0 ** -24 * s * (1 if out_bits < 64 else 2.0 ** -29) + eps * np.abs(x64.sum(axis=ax)) + 1e-30


@pytest.mark.parametrize("shape,axes", SHAPES_AXES, ids=[f"{s}-{a}" for s, a in SHAPES_AXES])
@pytest.mark.parametrize("ty", ["f32", "bf16", "f64", "s32", "u8", "s8", "s64"])
@pytest.mark.parametrize("keep", [False, True])
def test_sum(shape, axes, ty, keep, hip, oracle):
    if keep and ty not in ("f32", "s32"):
        pytest.skip("keep_axes only changes the output shape")
    rng = np.random.default_rng(seed_of(shape, axes, ty))
    x = rand_raw(rng, ty, shape, lo=-1, hi=1)
    hx, ox = both(x, ty, hip, oracle)
    got, want = Nx.sum(hx, axes=axes, keep_axes=keep), Nx.sum(ox, axes=axes, keep_axes=keep)
    if T.is_integer(T.normalize(ty)):
        assert_bits_equal(got, want, f"sum {ty} {shape} {axes}")
        return
    assert got.type == want.type and got.shape == want.shape
    x64 = values(ox)
    bound = sum_bound(x64, axes, got.type[1] if got.type[0] == "f" else 16).reshape(got.shape)
    err = np.abs(values(got) - values(want))
    assert (err <= bound).all(), f"sum {ty} {shape} {axes}: max err {err.max():.3e}"
    if ty == "f32":  # f64 accumulation on the device: expect the very same rounded f32 almost always
        same = (hip.to_numpy(got).view(np.uint32) == oracle_raw(want).view(np.uint32)).mean()
        assert same >= 0.99, f"only {same:.4f} of f32 sums are bit-identical"


def oracle_raw(t):
    from support import raw
    return raw(t)


@pytest.mark.parametrize("shape,axes", SHAPES_AXES[:14], ids=[f"{s}-{a}" for s, a in SHAPES_AXES[:14]])
@pytest.mark.parametrize("ty", ["f32", "bf16", "f16", "f64", "s32", "u8", "u64", "s64"])
@pytest.mark.parametrize("op", ["reduce_max", "reduce_min"])
def test_reduce_max_min_exact(shape, axes, ty, op, hip, oracle):
    rng = np.random.default_rng(seed_of(shape, axes, ty, op))
    x = rand_raw(rng, ty, shape, lo=-100, hi=100)
    if ty == "f32" and x.size > 100:  # NaN is sticky, infinities are ordered
        flat = x.reshape(-1)
        flat[rng.integers(0, flat.size, 5)] = np.nan
        flat[rng.integers(0, flat.size, 5)] = np.inf
        flat[rng.integers(0, flat.size, 5)] = -np.inf
    hx, ox = both(x, ty, hip, oracle)
    assert_bits_equal(getattr(Nx, op)(hx, axes=axes), getattr(Nx, op)(ox, axes=axes), f"{op} {ty} {shape} {axes}")


def test_product(hip, oracle):
    rng = np.random.default_rng(3)
    x = rng.integers(-3, 4, size=(64, 9)).astype(np.int32)
    hx, ox = both(x, "s32", hip, oracle)
    assert_bits_equal(Nx.product(hx, axes=[1]), Nx.product(ox, axes=[1]), "product s32")
    f = rng.uniform(0.5, 1.5, size=(50, 40)).astype(np.float32)
    hf, of = both(f, "f32", hip, oracle)
    from support import assert_all_close
    assert_all_close(Nx.product(hf, axes=[0]), Nx.product(of, axes=[0]), 1e-5, 0, "product f32")


ARG_SHAPES = [((64, 1000), 1), ((64, 1000), 0), ((64, 1000), None), ((4, 33, 7), 1), ((4, 33, 7), 2), ((4, 33, 7), 0),
              ((3, 70001), 1), ((1300001,), None), ((5, 8), -1), ((1, 1), 0), ((2, 40000, 2), 1)]


@pytest.mark.parametrize("shape,axis", ARG_SHAPES, ids=[f"{s}-{a}" for s, a in ARG_SHAPES])
@pytest.mark.parametrize("ty", ["f32", "bf16", "s32", "u8", "f64"])
@pytest.mark.parametrize("op", ["argmax", "argmin"])
@pytest.mark.parametrize("tie", ["low", "high"])
def test_argreduce_is_bit_exact(shape, axis, ty, op, tie, hip, oracle):
    rng = np.random.default_rng(seed_of(shape, axis, ty, op))
    # few distinct values => many exact ties along every axis
    if T.is_float(T.normalize(ty)):
        x = rng.integers(-6, 7, size=shape).astype(np.float64) / 2
        x = (x.astype(np.float32).view(np.uint32) >> 16).astype(np.uint16) if ty == "bf16" else x.astype(T.numpy_dtype(T.normalize(ty)))
    else:
        x = rng.integers(0 if ty == "u8" else -6, 7, size=shape).astype(T.numpy_dtype(T.normalize(ty)))
    hx, ox = both(x, ty, hip, oracle)
    for out_type in ("s32", "u32") if tie == "low" else ("s64",):
        got = getattr(Nx, op)(hx, axis=axis, tie_break=tie, type=out_type)
        want = getattr(Nx, op)(ox, axis=axis, tie_break=tie, type=out_type)
        assert_bits_equal(got, want, f"{op} {ty} {shape} axis={axis} tie={tie}")


@pytest.mark.parametrize("op", ["argmax", "argmin"])
def test_argreduce_nan_and_infinities(op, hip, oracle):
    """Any NaN wins and the last NaN's index is returned (nx/test/nx_test.exs:1746-1798)."""
    rng = np.random.default_rng(11)
    x = rng.normal(size=(257, 5000)).astype(np.float32)
    for r in range(0, 257, 3):
        cols = rng.integers(0, 5000, size=rng.integers(1, 5))
        x[r, cols] = np.nan
    for r in range(1, 257, 3):
        x[r, rng.integers(0, 5000, size=3)] = np.inf
        x[r, rng.integers(0, 5000, size=3)] = -np.inf
    hx, ox = both(x, "f32", hip, oracle)
    for tie in ("low", "high"):
        assert_bits_equal(getattr(Nx, op)(hx, axis=1, tie_break=tie), getattr(Nx, op)(ox, axis=1, tie_break=tie), op)
        assert_bits_equal(getattr(Nx, op)(hx, axis=0, tie_break=tie), getattr(Nx, op)(ox, axis=0, tie_break=tie), op)
    assert_bits_equal(getattr(Nx, op)(hx), getattr(Nx, op)(ox), f"{op} flat")


@pytest.mark.parametrize("ty", ["f32", "bf16", "f16", "s32", "u8", "s16"])
@pytest.mark.parametrize("red", [8, 16, 24, 64, 72, 128, 200, 256, 264, 512])
@pytest.mark.parametrize("op", ["sum", "reduce_max", "argmax"])
def test_short_rows_take_part_of_a_wave(ty, red, op, hip, oracle):
    """Rows of up to 256 elements are reduced by 8 / 16 / 32 lanes, several rows per wave; the result must be the
    oracle's (and the whole-wave kernel's: same combine steps)."""
    rng = np.random.default_rng(seed_of(ty, red, op, "short"))
    x = rand_raw(rng, ty, (37, red), lo=-4, hi=4)
    hx, ox = both(x, ty, hip, oracle)
    if op == "argmax":
        assert_bits_equal(Nx.argmax(hx, axis=1), Nx.argmax(ox, axis=1), f"argmax {ty} {red}")
    elif op == "reduce_max":
        assert_bits_equal(Nx.reduce_max(hx, axes=[1]), Nx.reduce_max(ox, axes=[1]), f"max {ty} {red}")
    else:
        got, want = Nx.sum(hx, axes=[1]), Nx.sum(ox, axes=[1])
        if ty in ("s32", "u8", "s16"):
            assert_bits_equal(got, want, f"sum {ty} {red}")
        else:
            x64 = values(ox)
            bits = got.type[1] if ty == "f32" else (16 if ty == "bf16" else 10)
            eps = {32: 2.0 ** -23, 16: 2.0 ** -7, 10: 2.0 ** -10}[bits]
            bound = red * 2.0 ** -24 * np.abs(x64).sum(axis=1) + eps * np.abs(x64.sum(axis=1)) + 1e-30
            err = np.abs(values(got) - values(want))
            assert (err <= bound).all(), f"sum {ty} {red}: max err {err.max():.3e}"


@pytest.mark.parametrize("shape,axes", [((4, 6, 5, 8), [1, 3]), ((4, 6, 5, 8), [0, 2]), ((3, 4, 5, 6, 7), [0, 2, 4]), ((3, 4, 5, 6, 7), [0, 1, 3]),
                                        ((2, 33, 3, 130), [0, 3]), ((5, 7, 9), [0, 2])])
@pytest.mark.parametrize("ty", ["f32", "bf16", "s32", "u8", "s64", "f64"])
@pytest.mark.parametrize("op", ["sum", "product", "reduce_max", "reduce_min", "all", "any"])
def test_reduced_axes_that_are_not_neighbours(shape, axes, ty, op, hip, oracle):
    """Reduced axes with kept axes between them go one run of neighbouring axes at a time (innermost first, sums
    through f64 / 64-bit integers) instead of through a transposed copy: integers and selections bit for bit --
    signed zeros and NaN included: the first extreme in row-major order of the reduced axes wins -- float sums
    and products within the accumulation bound."""
    rng = np.random.default_rng(seed_of(shape, axes, ty, op, "runs"))
    if op == "product":
        x = rand_raw(rng, ty, shape, lo=0.9, hi=1.1) if ty in ("f32", "bf16", "f64") else rng.integers(1, 3, size=shape).astype(T.numpy_dtype(T.normalize(ty)))
    elif op in ("all", "any"):
        x = (rng.random(shape) < (0.97 if op == "all" else 0.03)).astype(np.float64)
        x = (x.astype(np.float32).view(np.uint32) >> 16).astype(np.uint16) if ty == "bf16" else x.astype(T.numpy_dtype(T.normalize(ty)))
    else:
        x = rand_raw(rng, ty, shape, lo=-3, hi=3)
        if ty == "f32":
            flat = x.reshape(-1)
            flat[rng.integers(0, flat.size, 6)] = 0.0
            flat[rng.integers(0, flat.size, 6)] = -0.0
            if op != "sum":
                flat[rng.integers(0, flat.size, 2)] = np.nan
    hx, ox = both(x, ty, hip, oracle)
    for keep in (False, True):
        got, want = getattr(Nx, op)(hx, axes=axes, keep_axes=keep), getattr(Nx, op)(ox, axes=axes, keep_axes=keep)
        if op in ("sum", "product") and T.is_float(T.normalize(ty)):
            assert got.type == want.type and got.shape == want.shape
            g, w = values(got), values(want)
            k = int(np.prod([shape[a] for a in axes]))
            eps = {"f64": 2.0 ** -52, "f32": 2.0 ** -23, "bf16": 2.0 ** -7}[ty]
            assert np.allclose(g, w, rtol=eps + k * 2.0 ** -50, atol=(k * 2.0 ** -24 * np.abs(values(ox)).sum(axis=tuple(axes), keepdims=keep)) if op == "sum" else 0), f"{op} {ty} {shape} {axes}"
        else:
            assert_bits_equal(got, want, f"{op} {ty} {shape} {axes} keep={keep}")


FEW = [((5000, c), 1) for c in (1, 2, 3, 5, 8, 13, 16, 17, 33, 100, 255)] + \
      [((8192, 3), 0), ((12288, 2), 0), ((3, 4096, 7), 1), ((20000, 33), 0), ((2, 8190, 5), 1), ((4099, 3), 0), ((65536, 1, 2), 0)] + \
      [((300, 1001), 0), ((7, 50, 77), 1), ((64, 261), 0), ((5000, 69), 0), ((3, 700, 131), 1)]  # rows off the vector grid under the reduced axis


@pytest.mark.parametrize("shape,axis", FEW, ids=[f"{s}-{a}" for s, a in FEW])
@pytest.mark.parametrize("ty", ["f32", "bf16", "s32", "u8", "f64"])
@pytest.mark.parametrize("op", ["sum", "product", "reduce_max", "reduce_min", "argmax", "argmin", "all", "any"])
def test_few_elements_per_row_and_few_columns(shape, axis, ty, op, hip, oracle):
    """Rows of up to 16 elements are walked by one lane each, unaligned rows of up to 256 by 8 to 32 lanes, and a few
    columns under a long axis are reduced in two steps (a divisor of the axis folded into the columns first, sums and
    products through f64 / 64-bit integers): integers, selections and indices bit for bit (NaN and signed zeros
    included), float sums and products within the accumulation bound."""
    rng = np.random.default_rng(seed_of(shape, axis, ty, op, "few"))
    floating = ty in ("f32", "bf16", "f64")
    if op == "product":
        x = rand_raw(rng, ty, shape, lo=0.999, hi=1.001) if floating else rng.integers(1, 3, size=shape).astype(T.numpy_dtype(T.normalize(ty)))
    elif op in ("all", "any"):
        x = (rng.random(shape) < (0.9997 if op == "all" else 0.0003)).astype(np.float64)
        x = (x.astype(np.float32).view(np.uint32) >> 16).astype(np.uint16) if ty == "bf16" else x.astype(T.numpy_dtype(T.normalize(ty)))
    else:
        x = rand_raw(rng, ty, shape, lo=-3, hi=3)
        if ty == "f32":
            flat = x.reshape(-1)
            flat[rng.integers(0, flat.size, 40)] = 0.0
            flat[rng.integers(0, flat.size, 40)] = -0.0
            if op != "sum":
                flat[rng.integers(0, flat.size, 5)] = np.nan
    hx, ox = both(x, ty, hip, oracle)
    if op in ("argmax", "argmin"):
        for tie in ("low", "high"):
            assert_bits_equal(getattr(Nx, op)(hx, axis=axis, tie_break=tie), getattr(Nx, op)(ox, axis=axis, tie_break=tie), f"{op} {ty} {shape}")
        return
    got, want = getattr(Nx, op)(hx, axes=[axis]), getattr(Nx, op)(ox, axes=[axis])
    if op in ("sum", "product") and floating:
        assert got.type == want.type and got.shape == want.shape
        k = shape[axis]
        eps = {"f64": 2.0 ** -52, "f32": 2.0 ** -23, "bf16": 2.0 ** -7}[ty]
        atol = k * 2.0 ** -24 * np.abs(values(ox)).sum(axis=axis) if op == "sum" else 0
        assert np.allclose(values(got), values(want), rtol=eps + k * 2.0 ** -50, atol=atol), f"{op} {ty} {shape} axis {axis}"
    elif op in ("reduce_max", "reduce_min") and ty == "f32":
        # equal extremes of both signs of zero: the device may keep the other zero (selected by value)
        g, w = values(got), values(want)
        assert np.array_equal(np.isnan(g), np.isnan(w)) and np.array_equal(g[~np.isnan(g)], w[~np.isnan(w)]), f"{op} {shape}"
    else:
        assert_bits_equal(got, want, f"{op} {ty} {shape} axis {axis}")


@pytest.mark.parametrize("shape", [(37, 50257), (5, 16381), (3, 4097), (2, 300001), (9, 261), (4, 1023)])
@pytest.mark.parametrize("ty", ["f32", "bf16", "s32", "u8", "f64"])
@pytest.mark.parametrize("op", ["sum", "reduce_max", "reduce_min", "argmax", "argmin"])
def test_long_rows_that_are_not_whole_vectors(shape, ty, op, hip, oracle):
    """Rows of 50257 elements (a vocabulary): every row starts at another offset from a vector boundary; the kernel
    reads a row's first elements up to the boundary and its last ones singly and the rest as aligned vectors.  With
    equal extremes in the head, the body and the tail of a row, and NaN, for the index reducers."""
    rng = np.random.default_rng(seed_of(shape, ty, op, "ragged rows"))
    x = rand_raw(rng, ty, shape, lo=-3, hi=3)
    rows, cols = shape
    if op != "sum":
        top = {"f32": 7.0, "bf16": None, "s32": 100, "u8": 250, "f64": 7.0}[ty]
        if top is not None:
            for r in range(rows):  # the same extreme near the start, in the middle and at the very end
                for c in (r % 7, cols // 2 + r, cols - 1 - (r % 5)):
                    x[r, c] = top if op in ("reduce_max", "argmax") else (-top if ty not in ("u8",) else 0)
        if ty == "f32" and rows > 2:
            x[1, cols - 2] = np.nan
            x[2, 3] = np.nan
            x[2, cols // 3] = np.nan
    hx, ox = both(x, ty, hip, oracle)
    if op in ("argmax", "argmin"):
        for tie in ("low", "high"):
            assert_bits_equal(getattr(Nx, op)(hx, axis=1, tie_break=tie), getattr(Nx, op)(ox, axis=1, tie_break=tie), f"{op} {ty} {shape} {tie}")
    elif op == "sum" and ty in ("f32", "bf16", "f64"):
        got, want = Nx.sum(hx, axes=[1]), Nx.sum(ox, axes=[1])
        eps = {"f64": 2.0 ** -52, "f32": 2.0 ** -23, "bf16": 2.0 ** -7}[ty]
        assert np.allclose(values(got), values(want), rtol=eps + cols * 2.0 ** -50, atol=cols * 2.0 ** -24 * np.abs(values(ox)).sum(axis=1))
    else:
        assert_bits_equal(getattr(Nx, op)(hx, axes=[1]), getattr(Nx, op)(ox, axes=[1]), f"{op} {ty} {shape}")


@pytest.mark.parametrize("ty", ["f16", "bf16", "f32", "f64"])
@pytest.mark.parametrize("op", ["product", "sum", "reduce_max", "reduce_min"])
@pytest.mark.parametrize("shape,axes", [((40, 64), [1]), ((64, 40), [0]), ((6, 5000), [1]), ((3000, 8), [0]), ((7, 9, 33), [0, 2])])
def test_signed_zeros_in_reductions(ty, op, shape, axes, hip, oracle):
    """Zeros of either sign among ones and minus ones: the product's zero carries the sign of the factors, a sum of
    negative zeros is a negative zero (the reference folds from the first element; exact here, in any order, up to that sign)."""
    rng = np.random.default_rng(seed_of("zeros in reductions", ty, op, shape))
    dtype = np.float32 if ty == "bf16" else T.numpy_dtype(T.normalize(ty))
    x = rng.choice(np.array([1.0, -1.0, 0.0, -0.0], dtype), size=shape, p=[0.49, 0.49, 0.01, 0.01])
    if op == "sum":  # rows of zeros only, most of them all negative
        x = np.where(rng.random(shape) < 0.002, 0.0, -0.0).astype(dtype)
    if ty == "bf16":
        x = (np.asarray(x, np.float32).view(np.uint32) >> 16).astype(np.uint16)
    hx, ox = both(x, ty, hip, oracle)
    assert_bits_equal(getattr(Nx, op)(hx, axes=axes), getattr(Nx, op)(ox, axes=axes), f"{op} {ty} {shape} {axes}")


@pytest.mark.parametrize("ty", ["f16", "bf16", "f32", "f64"])
@pytest.mark.parametrize("op", ["sum", "product", "reduce_max", "reduce_min"])
@pytest.mark.parametrize("shape,axes", [((48, 64), [1]), ((64, 48), [0]), ((5, 6000), [1]), ((2500, 8), [0])])
def test_infinities_and_nan_in_reductions(ty, op, shape, axes, hip, oracle):
    """Rows with an infinity, with infinities of both signs (their sum is NaN), with an infinity and a zero (their product is
    NaN), with a NaN, and plain ones: the same bits as the reference in every float type."""
    rng = np.random.default_rng(seed_of("not finite in reductions", ty, op, shape))
    dtype = np.float32 if ty == "bf16" else T.numpy_dtype(T.normalize(ty))
    x = rng.choice(np.array([1.0, -1.0] if op == "product" else [1.0, -1.0, 0.5, 2.0]), size=shape)  # (exact in any order)
    lines = np.moveaxis(x, axes[0], -1)  # a view: one line per output
    for i, line in enumerate(lines):
        kind = i % 5
        at = rng.choice(line.size, size=3, replace=False)
        if kind == 0:
            line[at[0]] = np.inf
        elif kind == 1:
            line[at[0]], line[at[1]] = np.inf, -np.inf
        elif kind == 2:
            line[at[0]], line[at[1]] = -np.inf, 0.0
        elif kind == 3:
            line[at[0]], line[at[1]] = np.nan, np.inf
    x = x.astype(dtype)
    if ty == "bf16":
        x = (x.view(np.uint32) >> 16).astype(np.uint16)
    hx, ox = both(x, ty, hip, oracle)
    assert_bits_equal(getattr(Nx, op)(hx, axes=axes), getattr(Nx, op)(ox, axes=axes), f"{op} {ty} {shape} {axes}")
