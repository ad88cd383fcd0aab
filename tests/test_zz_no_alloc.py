"""hipnx_reduce_static -- the reduction that allocates nothing -- against hipnx_reduce, through the
C ABI: same bits on two calls in a row (the second smaller, so that it runs over what the first
left in the static scratch), for the split-row and the split-column paths; the pool's counters do
not move during the calls; a shape whose partial results do not fit is refused."""
import ctypes as C

import numpy as np
import pytest

from nx_amd import _lib as L
from nx_amd import types as T

pytestmark = pytest.mark.gpu

RED_SUM, RED_MAX, RED_MIN = 0, 1, 2  # HIPNX_RED_* of include/hipnx.h
STATIC_BYTES = 1 << 20               # HIPNX_REDUCE_STATIC_SCRATCH_BYTES


def _put(ctx, arr):
    h = C.c_void_p()
    L.check(L.lib.hipnx_buf_alloc(ctx, arr.nbytes, C.byref(h)))
    L.check(L.lib.hipnx_h2d(ctx, h, 0, arr.ctypes.data_as(C.c_void_p), arr.nbytes))
    return h


def _out(ctx, nbytes):
    h = C.c_void_p()
    L.check(L.lib.hipnx_buf_alloc(ctx, nbytes, C.byref(h)))
    return h


def _get(ctx, h, dtype, n):
    res = np.empty(n, dtype=dtype)
    L.check(L.lib.hipnx_d2h(ctx, h, 0, res.ctypes.data_as(C.c_void_p), res.nbytes))
    return res


def _stats(ctx):
    live, peak, pooled = C.c_uint64(), C.c_uint64(), C.c_uint64()
    L.check(L.lib.hipnx_mem_stats(ctx, C.byref(live), C.byref(peak), C.byref(pooled)))
    return live.value, peak.value, pooled.value


def _both(ctx, op, ty, x, outer, red, inner):
    """Runs the pooled and the static entry point on the same input; returns both results' bits."""
    code = T.code(T.normalize(ty))
    size = x.dtype.itemsize
    hx = _put(ctx, x)
    h_pool, h_static = _out(ctx, outer * inner * size), _out(ctx, outer * inner * size)
    L.check(L.lib.hipnx_reduce(ctx, op, code, code, outer, red, inner, hx, h_pool))
    before = _stats(ctx)
    L.check(L.lib.hipnx_reduce_static(ctx, op, code, code, outer, red, inner, hx, h_static))
    assert _stats(ctx) == before, "the static entry point touched the pool"
    bits = np.dtype(f"u{size}")
    want, got = _get(ctx, h_pool, bits, outer * inner), _get(ctx, h_static, bits, outer * inner)
    for h in (hx, h_pool, h_static):
        L.check(L.lib.hipnx_buf_destroy(h))
    return got, want


@pytest.fixture(scope="module")
def ctx():
    from nx_amd.backend import HipNxBackend
    return HipNxBackend._ctx(0)


# (outer, red, inner): the first of each pair splits into many segments, the second into fewer
PAIRS = [((4, 1 << 20, 1), (2, 1 << 16, 1)),          # few rows x a long contiguous axis
         ((1, 8192, 64), (1, 512, 24)),               # few columns under a long axis
         ((3, 300000, 1), (1, 40000, 1))]             # ragged lengths (scalar tail, last segment short)


@pytest.mark.parametrize("first,second", PAIRS, ids=[f"{a}-{b}" for a, b in PAIRS])
@pytest.mark.parametrize("op,ty", [(RED_SUM, "f32"), (RED_MAX, "f32"), (RED_SUM, "s32"), (RED_MIN, "f64")])
def test_static_matches_pooled_twice(ctx, first, second, op, ty):
    rng = np.random.default_rng(7)
    for outer, red, inner in (first, second):
        n = outer * red * inner
        if ty == "s32":
            x = rng.integers(-1000, 1000, size=n, dtype=np.int32)
        else:
            x = rng.uniform(-1, 1, size=n).astype(np.float32 if ty == "f32" else np.float64)
        got, want = _both(ctx, op, ty, x, outer, red, inner)
        assert np.array_equal(got, want), f"op {op} {ty} [{outer}, {red}, {inner}]: static result differs from hipnx_reduce"


def test_float_sums_over_folded_shapes_agree_within_the_accumulation_bound(ctx):
    """A few columns under a long axis: hipnx_reduce folds rows into the columns (two steps through a pool
    block), the static entry point reduces the columns directly -- another order of the same f64 additions.
    Twice in a row, the second smaller; f64 so that no final rounding hides the difference."""
    rng = np.random.default_rng(9)
    for outer, red, inner in ((1, 8192, 64), (1, 4096, 24)):
        x = rng.uniform(-1, 1, size=outer * red * inner)
        got, want = _both(ctx, RED_SUM, "f64", x, outer, red, inner)
        got, want = got.view(np.float64), want.view(np.float64)
        bound = red * 2.0 ** -53 * np.abs(x.reshape(outer, red, inner)).sum(axis=1).ravel()
        assert (np.abs(got - want) <= bound).all(), f"[{outer}, {red}, {inner}]: beyond the accumulation bound"
        exact = np.array([float(np.sum(x.reshape(outer, red, inner)[:, :, j].astype(np.longdouble))) for j in range(inner)])
        assert (np.abs(got - exact) <= bound).all()


def test_unsplit_shapes_need_no_scratch(ctx):
    rng = np.random.default_rng(8)
    x = rng.uniform(-1, 1, size=1024 * 1024).astype(np.float32)
    got, want = _both(ctx, RED_SUM, "f32", x, 1024, 1024, 1)
    assert np.array_equal(got, want)


def test_refuses_what_does_not_fit(ctx):
    # [1, 1024, 16384] f64: 16384 columns of 1024 split into segments; partials exceed 1 MiB
    outer, red, inner = 1, 1024, 16384
    x = np.zeros(outer * red * inner, dtype=np.float64)
    code = T.code(T.normalize("f64"))
    hx, ho = _put(ctx, x), _out(ctx, outer * inner * 8)
    st = L.lib.hipnx_reduce_static(ctx, RED_SUM, code, code, outer, red, inner, hx, ho)
    msg = L.last_error()
    L.check(L.lib.hipnx_reduce(ctx, RED_SUM, code, code, outer, red, inner, hx, ho))  # the pooled form takes it
    for h in (hx, ho):
        L.check(L.lib.hipnx_buf_destroy(h))
    assert st == L.EUNSUPPORTED and "static scratch" in msg, (st, msg)
