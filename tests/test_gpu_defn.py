"""Traced functions evaluated on the device: the callers one step above the callbacks
(nx/lib/nx/defn/evaluator.ex:363-388).  The device runs the traced function, the oracle runs the
same function eagerly and traced; exact ops are compared bit for bit, transcendental chains within
the tolerances of the per-op tests."""
import gc

import numpy as np
import pytest

from nx_amd.tensor import template

from nx_amd import defn
from nx_amd import nx as Nx
from nx_amd import random as Random
from nx_amd import _lib as L
from nx_amd.backend import _Context, mem_stats
from random_support import CASES, check_random_case
from support import assert_all_close, assert_bits_equal, from_numpy, raw, seed_of
from test_defn import CHAINS, build_args, f32

pytestmark = pytest.mark.gpu

EXACT = {"linear_int8", "argmax_take"}  # integer dot, conversion, one float multiply; selection and copy


@pytest.mark.parametrize("name", sorted(CHAINS))
def test_jitted_chain_on_the_device(name, hip, oracle):
    got = defn.jit(CHAINS[name])(*build_args(hip)[name])
    assert type(got.data) is hip
    want = CHAINS[name](*build_args(oracle)[name])
    if name in EXACT:
        assert_bits_equal(got, want, name)
    else:
        assert_all_close(got, want, 1e-5, 1e-7, name)
    compiled = defn.compile(CHAINS[name], *build_args(hip)[name])
    again = compiled(*build_args(hip)[name])
    assert_bits_equal(again, got, f"{name}: compiled once, same result")


def test_constants_and_created_tensors_follow_the_arguments(hip):
    # the default backend only stores data here: iota and constants of the trace go to the device
    def fun(t):
        return Nx.add(Nx.multiply(t, Nx.iota((4,), type="f32")), 2.5)
    got = defn.jit(fun)(f32([1, 2, 3, 4], hip))
    assert type(got.data) is hip and hip.to_numpy(got).tolist() == [2.5, 4.5, 8.5, 14.5]


def test_control_flow_on_the_device(hip, oracle):
    def newton_sqrt(a):
        def body(state):
            i, x = state
            return Nx.add(i, 1), Nx.multiply(0.5, Nx.add(x, Nx.divide(a, x)))
        _, x = defn.while_loop((Nx.tensor(0), a), lambda s: Nx.less(s[0], 8), body)
        return defn.cond(Nx.greater(Nx.reduce_max(a), 100.0), lambda: Nx.negate(x), lambda: x)
    values = np.asarray([1.0, 2.0, 9.0, 50.0], dtype=np.float32)
    got = defn.jit(newton_sqrt)(f32(values, hip))
    want = defn.jit(newton_sqrt)(f32(values, oracle))
    assert_bits_equal(got, want, "newton sqrt")  # add, multiply, divide: exactly rounded
    flipped = defn.jit(newton_sqrt)(f32(values * 10, hip))
    assert (hip.to_numpy(flipped) < 0).all()


def test_intermediates_go_back_to_the_pool_during_the_walk(hip):
    n = 1 << 22  # 16 MiB per f32 intermediate
    x = from_numpy(np.linspace(0, 1, n, dtype=np.float32), "f32", hip)

    def chain(t):
        for _ in range(12):
            t = Nx.exp(Nx.negate(t))
        return t
    gc.collect()  # tensors earlier tests left behind must not be freed in the middle of the walk,
    L.check(L.lib.hipnx_trim(_Context.get(0)))  # nor their larger pooled blocks be handed out for these 16 MiB
    defn.jit(chain)(x)  # warm the pool
    before = mem_stats()["live"]
    seen = []
    original = defn._Run.apply

    def sampling(self, e, node, scope):
        seen.append(mem_stats()["live"] - before)
        return original(self, e, node, scope)
    defn._Run.apply = sampling
    try:
        out = defn.jit(chain)(x)
    finally:
        defn._Run.apply = original
    assert type(out.data) is hip
    # 24 intermediates of 16 MiB: with every result dropped after its last use at most the operand in
    # flight (and the result being written) is alive at any step, never the whole chain
    assert max(seen) <= 2 * 4 * n + 4096, seen
    assert mem_stats()["live"] - before <= 4 * n + 4096  # only the output stays


@pytest.mark.parametrize("case", [c for c in CASES if c["fn"] != "key"], ids=[c["name"] for c in CASES if c["fn"] != "key"])
def test_random_known_answers_through_a_trace_on_the_device(case, hip):
    check_random_case(case, hip, through=defn.jit)


def test_traced_random_uses_the_one_kernel_cipher(hip):
    key = Random.key(99, backend=hip)
    traced = defn.jit(lambda k: Random.random_bits(k, shape=(1001,)))(key)
    previous = Random.compose_only(True)
    try:
        composed = Random.random_bits(key, shape=(1001,))
    finally:
        Random.compose_only(previous)
    assert_bits_equal(traced, composed, "random_bits traced vs composed")


# ---- captured graphs: one submission replays every kernel of a compiled function ------------------

# (argmax_take too: indices written by argmax are known to be in range of an axis of that length, so take's raising
# bounds policy has nothing to wait for)
GRAPHABLE = ["softmax", "elementwise_reduce", "linear_int8", "argmax_take"]


@pytest.mark.parametrize("name", GRAPHABLE)
def test_captured_chain_replays_with_new_inputs(name, hip):
    from nx_amd.backend import sync
    args = build_args(hip)[name]
    compiled = defn.compile(CHAINS[name], *args)
    eager = hip.to_numpy(compiled(*args)).copy()
    captured = compiled.capture(*args)
    try:
        # replays between eager work and synchronisations, every one checked against the eager result
        for _ in range(3):
            out = captured(*args)
            np.testing.assert_array_equal(hip.to_numpy(out), eager, f"{name}: replay with the captured tensors")
            compiled(*args)
            sync()
        # new values in fresh tensors of the same shapes: copied in, same kernels
        rng = np.random.default_rng(11)
        fresh = []
        for a in args:
            raw = hip.to_numpy(a)
            perm = rng.permutation(raw.size)
            fresh.append(from_numpy(raw.reshape(-1)[perm].reshape(raw.shape), a.type, hip))
        want = hip.to_numpy(compiled(*fresh)).copy()
        np.testing.assert_array_equal(hip.to_numpy(captured(*fresh)), want, f"{name}: replay with new inputs")
        np.testing.assert_array_equal(hip.to_numpy(captured(*args)), eager, f"{name}: and back")
    finally:
        captured.destroy()


def test_captured_constants_survive_the_scalar_cache(hip):
    """A constant met while capturing is the graph's own block, filled inside the capture -- also when the
    eager warm-up has left the same number in the backend's scalar cache.  After more than 1024 other
    scalars have passed through that cache (it is cleared, its blocks go back to the pool and are
    overwritten), a replay still multiplies by 0.5."""
    x_np = np.linspace(-3, 3, 4096, dtype=np.float32)
    x = from_numpy(x_np, "f32", hip)
    compiled = defn.compile(lambda t: Nx.add(Nx.multiply(t, 0.5), 0.25), x)
    want = hip.to_numpy(compiled(x)).copy()  # the warm-up: 0.5 and 0.25 are now cached scalars
    captured = compiled.capture(x)
    try:
        np.testing.assert_array_equal(hip.to_numpy(captured(x)), want)
        keep = []
        for i in range(1100):  # distinct scalars: the cache overflows and is cleared
            keep.append(Nx.multiply(x, 1.0 + i / 4096.0))
        del keep
        junk = [hip.constant(template("f32", ()), 1000.0 + i, {}) for i in range(64)]  # take the freed small blocks
        np.testing.assert_array_equal(hip.to_numpy(captured(x)), want, "replay after the cache was cleared")
        del junk
    finally:
        captured.destroy()


def test_capture_refuses_what_needs_the_host(hip):
    """`take` with indices from outside (an argument: nothing is known about them) under the raising bounds policy has
    to wait for its kernel, which a capture cannot."""
    from nx_amd._lib import HipNxError
    rng = np.random.default_rng(3)
    table = from_numpy((rng.standard_normal((100, 24)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16), "bf16", hip)
    idx = from_numpy(rng.integers(0, 100, size=16, dtype=np.uint32), "u32", hip)
    compiled = defn.compile(lambda t, i: Nx.take(t, i), table, idx)
    with pytest.raises(HipNxError, match="not possible while capturing"):
        compiled.capture(table, idx)
    # the failed capture leaves the context usable
    assert_bits_equal(compiled(table, idx), Nx.take(table, idx), "eager after a refused capture")


def test_graph_blocks_do_not_leak_into_the_pool(hip):
    n = 1 << 20
    x = from_numpy(np.linspace(-1, 1, n, dtype=np.float32), "f32", hip)

    def chain(t):
        for _ in range(6):
            t = Nx.exp(Nx.negate(t))
        return t
    compiled = defn.compile(chain, x)
    want = hip.to_numpy(compiled(x)).copy()
    captured = compiled.capture(x)
    out = captured(x)
    # eager work of the same sizes in between must not be handed the graph's blocks
    others = [Nx.exp(x) for _ in range(8)]
    np.testing.assert_array_equal(hip.to_numpy(captured(x)), want)
    np.testing.assert_array_equal(hip.to_numpy(others[0]), hip.to_numpy(Nx.exp(x)))
    del others, out
    before = mem_stats()
    captured.destroy()
    after = mem_stats()
    assert after["pooled"] >= before["pooled"]  # the graph's blocks return to the pool only now
    np.testing.assert_array_equal(hip.to_numpy(compiled(x)), want)


# ---- fused element-wise groups: one kernel per group, the same bits as node by node -----------------

def gelu_like(x, bias):
    h = Nx.add(x, bias)
    return Nx.multiply(Nx.multiply(h, 0.5), Nx.add(1.0, Nx.tanh(Nx.multiply(0.7978845608, Nx.add(h, Nx.multiply(0.044715, Nx.pow(h, 3.0)))))))


def relu_mask(x, y):
    keep = Nx.logical_and(Nx.greater(x, 0.0), Nx.less_equal(y, 0.5))
    return Nx.select(keep, Nx.sqrt(Nx.abs(x)), Nx.negate(y))


def mixed_precision(a, b):
    # every intermediate rounds to its own type: bf16 by truncation, f16 to nearest
    h = Nx.multiply(a, b)                       # bf16 * f16 -> f16? no: merged float type
    return Nx.as_type(Nx.exp(Nx.as_type(Nx.add(h, 0.25), "bf16")), "f16")


def row_and_column_operands(x, row, col):
    return Nx.divide(Nx.subtract(x, col), Nx.add(row, 1.5))


def rand_float(rng, ty, shape, backend):
    v = rng.standard_normal(shape).astype(np.float32)
    if ty == "bf16":
        return from_numpy((v.view(np.uint32) >> 16).astype(np.uint16), "bf16", backend)
    return from_numpy(v.astype(np.float16 if ty == "f16" else np.float32), ty, backend)


def reuse_and_square(x, y):
    s = Nx.add(x, y)
    return Nx.multiply(Nx.multiply(s, s), Nx.subtract(s, x))   # op(s, s) and three reads of one value


FUSED_CASES = {
    "reuse_and_square": (reuse_and_square, lambda rng, b: (rand_float(rng, "f32", (40, 64), b), rand_float(rng, "f32", (40, 64), b))),
    "long_rows_tail": (gelu_like, lambda rng, b: (rand_float(rng, "f32", (3, 4104), b), rand_float(rng, "f32", (4104,), b))),
    "gelu_like": (gelu_like, lambda rng, b: (rand_float(rng, "f32", (64, 256), b), rand_float(rng, "f32", (256,), b))),
    "gelu_like_bf16": (gelu_like, lambda rng, b: (rand_float(rng, "bf16", (8, 16, 128), b), rand_float(rng, "bf16", (128,), b))),
    "relu_mask": (relu_mask, lambda rng, b: (rand_float(rng, "f32", (1000, 24), b), rand_float(rng, "f32", (1000, 24), b))),
    "relu_mask_ragged": (relu_mask, lambda rng, b: (rand_float(rng, "f32", (37, 11), b), rand_float(rng, "f32", (37, 11), b))),
    "mixed_precision": (mixed_precision, lambda rng, b: (rand_float(rng, "bf16", (33, 40), b), rand_float(rng, "f16", (33, 40), b))),
    "row_and_column": (row_and_column_operands, lambda rng, b: (rand_float(rng, "f32", (48, 64), b), rand_float(rng, "f32", (64,), b),
                                                                 rand_float(rng, "f32", (48, 1), b))),
    "row_and_column_unaligned": (row_and_column_operands, lambda rng, b: (rand_float(rng, "f32", (5, 7), b), rand_float(rng, "f32", (7,), b),
                                                                           rand_float(rng, "f32", (5, 1), b))),
}


@pytest.fixture(params=["interpreted", "compiled"])
def fused_mode(request, hip):
    """Runs a test once with the interpreting kernels and once with each program compiled at run time."""
    from nx_amd.backend import fused_mode as set_mode
    set_mode(request.param)
    yield request.param
    set_mode("interpreted")


@pytest.mark.parametrize("name", sorted(FUSED_CASES))
def test_fused_group_is_bit_identical_to_node_by_node(name, hip, fused_mode):
    fun, make = FUSED_CASES[name]
    args = make(np.random.default_rng(3), hip)
    fused = defn.compile(fun, *args, fuse=True)
    assert fused.fused_groups >= 1
    assert_bits_equal(fused(*args), defn.compile(fun, *args)(*args), name)


@pytest.mark.parametrize("name", sorted(CHAINS))
def test_fused_configuration_chains(name, hip, fused_mode):
    args = build_args(hip)[name]
    assert_bits_equal(defn.compile(CHAINS[name], *args, fuse=True)(*args), defn.compile(CHAINS[name], *args)(*args), name)


def test_fused_kernel_is_the_path_taken(hip):
    calls = []
    original = hip.fused_elementwise.__func__

    def counting(cls, *a, **k):
        calls.append(1)
        return original(cls, *a, **k)
    hip.fused_elementwise = classmethod(counting)
    try:
        fun, make = FUSED_CASES["gelu_like"]
        args = make(np.random.default_rng(5), hip)
        defn.compile(fun, *args, fuse=True)(*args)
    finally:
        hip.fused_elementwise = classmethod(original)
    assert calls == [1]  # the whole function is one group


def test_fused_entry_point_validates_its_program(hip):
    from nx_amd._lib import FUSED_BINARY, FUSED_SET, FUSED_SRC_INPUT, FUSED_SRC_SAVED, FUSED_UNARY, HipNxError
    x = rand_float(np.random.default_rng(1), "f32", (16,), hip)
    out = x.with_(data=None)
    flat = (1, 16, [(0, 1)])
    load = {"kind": FUSED_SET, "src": FUSED_SRC_INPUT, "arg": 0, "dt": ("f", 32)}
    with pytest.raises(HipNxError, match="before anything set it"):
        hip.fused_elementwise(out, [{"kind": FUSED_UNARY, "op": 0, "dt": ("f", 32)}], [x], flat)
    with pytest.raises(HipNxError, match="reads an input that is not there"):
        hip.fused_elementwise(out, [dict(load, arg=3)], [x], flat)
    with pytest.raises(HipNxError, match="reads an empty slot"):
        hip.fused_elementwise(out, [load, {"kind": FUSED_BINARY, "op": 0, "src": FUSED_SRC_SAVED, "arg": 1, "dt": ("f", 32)}], [x], flat)
    with pytest.raises(HipNxError, match="binary op"):
        hip.fused_elementwise(out, [load, {"kind": FUSED_BINARY, "op": 9, "src": FUSED_SRC_INPUT, "arg": 0, "dt": ("f", 32)}], [x], flat)
    with pytest.raises(HipNxError, match="holds"):
        hip.fused_elementwise(out.with_(shape=(32,)), [load], [x], (1, 32, [(0, 1)]))
    got = hip.fused_elementwise(out, [load, {"kind": FUSED_UNARY, "op": 27, "dt": ("f", 32)}], [x], flat)  # negate
    np.testing.assert_array_equal(hip.to_numpy(got), -hip.to_numpy(x))


def test_each_distinct_program_is_compiled_once(hip):
    from nx_amd.backend import fused_compiled_count, fused_mode as set_mode
    fun, make = FUSED_CASES["relu_mask"]
    args = make(np.random.default_rng(8), hip)
    other = tuple(rand_float(np.random.default_rng(9), "f32", (16, 128), hip) for _ in range(2))
    want = defn.compile(fun, *args)(*args)
    set_mode("compiled")
    try:
        before = fused_compiled_count()
        fused = defn.compile(fun, *args, fuse=True)
        assert_bits_equal(fused(*args), want, "first call compiles")
        after = fused_compiled_count()
        assert after >= before  # `before + 1` unless an earlier test met the same program
        assert_bits_equal(fused(*args), want, "second call reuses")
        defn.compile(fun, *other, fuse=True)(*other)  # other shape, same program: the shape is not compiled in
        assert fused_compiled_count() == after
        set_mode("interpreted")
        assert_bits_equal(fused(*args), want, "and back")
    finally:
        set_mode("interpreted")


def test_compiled_programs_are_bounded_and_the_oldest_go_first(hip):
    """A constant is part of what a program is compiled for, so a number that changes per call makes a new
    program each time: the table stops at its limit, and a program unloaded meanwhile compiles again."""
    from nx_amd import backend as B
    from nx_amd._lib import HipNxError
    x = rand_float(np.random.default_rng(12), "f32", (32, 64), hip)
    xs = hip.to_numpy(x)

    def scaled(c):
        def fun(t):
            return Nx.multiply(Nx.tanh(t), c)
        return fun
    consts = [1.0 + i / 16 for i in range(1, 11)]  # (not 1.0: the tracer drops a multiplication by one, and the first call must compile)
    B.fused_mode("compiled")
    B.fused_cache_limit(8)
    pinned = 4  # programs that earlier tests recorded into graphs stay loaded
    try:
        for c in consts + consts[:2]:  # the first two have been unloaded by the time they come round again
            got = hip.to_numpy(defn.compile(scaled(c), x, fuse=True)(x))
            want = (np.tanh(xs.astype(np.float64)).astype(np.float32) * np.float32(c))
            np.testing.assert_allclose(got, want, rtol=2e-6)
            assert B.fused_compiled_count() <= 8 + pinned
        with pytest.raises(HipNxError, match="at least 4"):
            B.fused_cache_limit(1)
    finally:
        B.fused_cache_limit(512)
        B.fused_mode("interpreted")


def test_program_first_met_during_a_capture_runs_interpreted(hip):
    from nx_amd import backend as B

    def fresh(x, y):  # a program no other test builds
        return Nx.subtract(Nx.multiply(Nx.sigmoid(x), 1.25), Nx.floor(y))
    args = tuple(rand_float(np.random.default_rng(10), "f32", (64, 64), hip) for _ in range(2))
    want = defn.compile(fresh, *args)(*args)
    fused = defn.compile(fresh, *args, fuse=True)
    fused(*args)  # the run before a capture, as the capture rules ask -- interpreted, so nothing is compiled yet
    B.fused_mode("compiled")
    try:
        before = B.fused_compiled_count()
        B.capture_begin(0)
        try:
            out = fused(*args)
        finally:
            graph = B.capture_end(0)
        assert B.fused_compiled_count() == before  # compiling and loading a module is no work to record
        for _ in range(3):
            graph.launch()
            assert_bits_equal(out, want, "replay")
        del out
        graph.destroy()
        assert_bits_equal(fused(*args), want, "compiled after the capture")
        assert B.fused_compiled_count() == before + 1
    finally:
        B.fused_mode("interpreted")


# ---- a reduction over the last axis joins the group that feeds it ----------------------------------------

def sum_of_exp(a, b):
    return Nx.sum(Nx.exp(Nx.multiply(Nx.add(a, b), 0.5)), axes=[1])


def max_of_scaled(a, b):
    return Nx.reduce_max(Nx.multiply(Nx.subtract(a, b), 0.125), axes=[-1], keep_axes=True)


def min_of_bf16(a, b):
    return Nx.reduce_min(Nx.as_type(Nx.add(a, b), "bf16"), axes=[1])


def sum_of_sines(a, b):  # sin is outside the light instantiation of the interpreting kernels
    return Nx.sum(Nx.sin(Nx.add(a, b)), axes=[1])


REDUCED = {"sum_of_exp": sum_of_exp, "max_of_scaled": max_of_scaled, "min_of_bf16": min_of_bf16}


def test_compiled_reduction_takes_any_float_program(hip):
    from nx_amd.backend import fused_mode as set_mode
    rng = np.random.default_rng(21)
    args = (rand_float(rng, "f32", (96, 512), hip), rand_float(rng, "f32", (96, 512), hip))
    want = defn.compile(sum_of_sines, *args)(*args)
    fused = defn.compile(sum_of_sines, *args, fuse=True)
    calls = []
    original = hip.fused_elementwise.__func__

    def counting(cls, *a, **k):
        calls.append(a[4] if len(a) > 4 else k.get("reduce_op", -1))
        return original(cls, *a, **k)
    hip.fused_elementwise = classmethod(counting)
    try:
        assert_bits_equal(fused(*args), want, "interpreted: the group, then the separate reduction")
        assert calls == [0, -1]  # offered with the reduction, refused, run without it
        del calls[:]
        set_mode("compiled")
        assert_bits_equal(fused(*args), want, "compiled: one kernel")
        assert calls == [0]
    finally:
        set_mode("interpreted")
        hip.fused_elementwise = classmethod(original)


@pytest.mark.parametrize("name", sorted(REDUCED))
@pytest.mark.parametrize("shape", [(64, 256), (300, 4096), (16, 8192), (5, 40000), (4, 65536), (1, 1000000), (2, 131080), (2049, 8),
                                   (3, 7, 512)])
def test_group_with_its_row_reduction_is_bit_identical(name, shape, hip, fused_mode):
    rng = np.random.default_rng(seed_of(name, shape))
    if len(shape) == 3 and name == "sum_of_exp":
        pytest.skip("this function reduces axis 1, which is the last axis only for matrices")
    fun = REDUCED[name]
    if len(shape) == 3 and name == "min_of_bf16":
        fun = lambda a, b: Nx.reduce_min(Nx.as_type(Nx.add(a, b), "bf16"), axes=[2])  # noqa: E731
    args = (rand_float(rng, "f32", shape, hip), rand_float(rng, "f32", shape, hip))
    fused = defn.compile(fun, *args, fuse=True)
    assert fused.fused_groups == 1 and fused.roots[0].data.op == "fused" and fused.roots[0].data.args[0].reduce is not None
    assert_bits_equal(fused(*args), defn.compile(fun, *args)(*args), f"{name} {shape}")


def fused_groups_of(compiled):
    groups = []

    def seen(t):
        e = t.data
        if e.op == "fused":
            groups.append(e.args[0])
            for i in e.args[1]:
                seen(i)
        elif e.op not in ("parameter", "constant", "tensor"):
            for ch in defn._children(e):
                if isinstance(ch, defn.Tensor):
                    seen(ch)
    for r in compiled.roots:
        seen(r)
    return groups


def test_softmax_becomes_three_kernels(hip, fused_mode):
    """The scaled scores feed the max and the subtraction, the exponentials feed the sum and the
    division: both are cheap to compute again from the bf16 scores, so nothing but the two row
    statistics and the result is ever stored."""
    args = build_args(hip)["softmax"]
    fused = defn.compile(CHAINS["softmax"], *args, fuse=True)
    assert_bits_equal(fused(*args), defn.compile(CHAINS["softmax"], *args)(*args), "softmax")
    groups = fused_groups_of(fused)
    assert sorted(str(g.reduce and g.reduce[0]) for g in {id(g): g for g in groups}.values()) == ["None", "reduce_max", "sum"]
    calls = []
    original = hip.fused_elementwise.__func__

    def counting(cls, *a, **k):
        calls.append(1)
        return original(cls, *a, **k)
    hip.fused_elementwise = classmethod(counting)
    try:
        fused(*args)
    finally:
        hip.fused_elementwise = classmethod(original)
    assert len(calls) == 3


def test_value_with_an_outside_reader_is_still_stored_once(hip):
    x = rand_float(np.random.default_rng(2), "f32", (32, 64), hip)

    def fun(t):
        h = Nx.tanh(Nx.multiply(t, 0.5))
        return Nx.add(h, 1.0), Nx.dot(h, [1], h, [1])   # the dot is not element-wise: h must exist in memory
    fused = defn.compile(fun, x, fuse=True)
    plain = defn.compile(fun, x)
    for got, want in zip(fused(x), plain(x)):
        assert_bits_equal(got, want, "shared with a dot")


# ---- groups planned for compilation: 32-bit integer work and bit relabelling join in --------------------

def bits_to_unit_floats(bits):
    # the core of Nx.Random.uniform for f32 (random.ex:424-470): mantissa bits under the exponent of 1.0
    mantissa = Nx.bitwise_or(Nx.right_shift(bits, 9), 0x3F800000)
    return Nx.subtract(Nx.bitcast(mantissa, "f32"), 1.0)


def integer_mix(a, b):
    x = Nx.bitwise_xor(Nx.add(a, b), Nx.left_shift(a, 3))
    return Nx.multiply(Nx.subtract(x, 7), Nx.bitwise_not(b))


def signed_shift_and_convert(a, b):
    x = Nx.max(Nx.right_shift(Nx.negate(a), 2), Nx.min(b, 1000))
    return Nx.multiply(Nx.as_type(x, "f32"), 0.5)


def floats_to_bits_and_back(x):
    sign_cleared = Nx.bitwise_and(Nx.bitcast(x, "u32"), 0x7FFFFFFF)
    return Nx.sqrt(Nx.bitcast(sign_cleared, "f32"))


# Where the bits of a float can be looked at, every NaN a node computes is the one quiet NaN its kernel would have stored
# (0x7FC00000), bits that only pass through a relabelling stay as they are, and a conversion rounds however few significant
# bits the compiler can see in the integer (each of these once came out differently from the compiled group):
def bits_of_a_computed_nan(x):
    return Nx.bitcast(Nx.sqrt(x), "s32")                       # sqrt of a negative number: the hardware's NaN has the sign set


def relabelled_nan_bits(a):
    return Nx.bitcast(Nx.negate(Nx.max(a, 0x7FFFFFFF)), "f32")  # NaN patterns with payloads: the result's last node relabels


def shifted_integer_to_f16(a):
    return Nx.sqrt(Nx.as_type(Nx.left_shift(a, 24), "f16"))     # eight significant bits, far beyond f16's range: infinity


def sign_extended_byte_as_float(a):
    return Nx.subtract(Nx.bitcast(Nx.right_shift(a, 24), "f32"), 1.0)   # negative a: the bits of a NaN


def rand_words(rng, ty, shape, backend):
    info = np.iinfo(np.uint32 if ty == "u32" else np.int32)
    return from_numpy(rng.integers(info.min, info.max, size=shape, dtype=info.dtype, endpoint=True), ty, backend)


INT_CASES = {
    "bits_to_unit_floats": (bits_to_unit_floats, lambda rng, b: (rand_words(rng, "u32", (64, 256), b),)),
    "integer_mix_u32": (integer_mix, lambda rng, b: (rand_words(rng, "u32", (33, 128), b), rand_words(rng, "u32", (33, 128), b))),
    "integer_mix_s32": (integer_mix, lambda rng, b: (rand_words(rng, "s32", (8, 4096), b), rand_words(rng, "s32", (4096,), b))),
    "signed_shift_and_convert": (signed_shift_and_convert, lambda rng, b: (rand_words(rng, "s32", (40, 64), b), rand_words(rng, "s32", (40, 64), b))),
    "floats_to_bits_and_back": (floats_to_bits_and_back, lambda rng, b: (rand_float(rng, "f32", (1000, 8), b),)),
    "bits_of_a_computed_nan": (bits_of_a_computed_nan, lambda rng, b: (rand_float(rng, "f32", (4, 64), b),)),
    "relabelled_nan_bits": (relabelled_nan_bits, lambda rng, b: (rand_words(rng, "u32", (5, 8), b),)),
    "shifted_integer_to_f16": (shifted_integer_to_f16, lambda rng, b: (rand_words(rng, "u32", (2, 520), b),)),
    "sign_extended_byte_as_float": (sign_extended_byte_as_float, lambda rng, b: (rand_words(rng, "s32", (64, 8), b),)),
}


def test_what_a_compiled_group_sees_in_the_bits_of_a_nan(hip):
    """The same four against what they must give, worked out here."""
    x = from_numpy(np.array([-4.0, 4.0, -0.0, -1e-30] * 2, np.float32), "f32", hip)
    got = raw(defn.compile(bits_of_a_computed_nan, x, fuse="compiled")(x))
    assert got.view(np.uint32).tolist() == [0x7FC00000, 0x40000000, 0x80000000, 0x7FC00000] * 2
    a = from_numpy(np.array([0x80000001, 0x7FFFFFFF, 5, 0xFFFFFFFF, 0x80000000, 0x80000002, 0, 9], np.uint32), "u32", hip)
    got = raw(defn.compile(relabelled_nan_bits, a, fuse="compiled")(a))
    assert got.view(np.uint32).tolist() == [0x7FFFFFFF, 0x80000001, 0x80000001, 1, 0x80000000, 0x7FFFFFFE, 0x80000001, 0x80000001]
    a = from_numpy(np.array([0, 1, 2, 255, 256 + 4, 16, 64, 100], np.uint32), "u32", hip)
    got = raw(defn.compile(shifted_integer_to_f16, a, fuse="compiled")(a))
    assert got.view(np.uint16).tolist() == [0, 0x7C00, 0x7C00, 0x7C00, 0x7C00, 0x7C00, 0x7C00, 0x7C00]
    a = from_numpy(np.array([-1 << 24, 3 << 24, -128 << 24, 0, 127 << 24, -5 << 24, 1 << 23, -(1 << 23)], np.int32), "s32", hip)
    got = raw(defn.compile(sign_extended_byte_as_float, a, fuse="compiled")(a))
    assert got.view(np.uint32).tolist() == [0x7FC00000, 0xBF800000, 0x7FC00000, 0xBF800000, 0xBF800000, 0x7FC00000, 0xBF800000, 0x7FC00000]


@pytest.mark.parametrize("name", sorted(INT_CASES))
def test_compiled_group_with_integer_work_is_bit_identical(name, hip):
    from nx_amd.backend import fused_mode as set_mode
    fun, make = INT_CASES[name]
    args = make(np.random.default_rng(seed_of(name)), hip)
    want = defn.compile(fun, *args)(*args)
    fused = defn.compile(fun, *args, fuse="compiled")
    assert fused.fused_groups == 1 and fused.roots[0].data.op == "fused"  # the whole function is one kernel
    assert_bits_equal(fused(*args), want, name)
    # planned without the integer class, the same function still agrees (float parts fuse, the rest runs node by node)
    assert_bits_equal(defn.compile(fun, *args, fuse=True)(*args), want, name + " float-only plan")
    set_mode("compiled")
    try:
        assert_bits_equal(fused(*args), want, name + " in compiled mode")
    finally:
        set_mode("interpreted")


def test_integer_program_is_refused_by_the_interpreting_kernels(hip):
    from nx_amd._lib import FUSED_BINARY, FUSED_SET, FUSED_SRC_CONST, FUSED_SRC_INPUT, HipNxError
    x = rand_words(np.random.default_rng(4), "u32", (64,), hip)
    program = [{"kind": FUSED_SET, "src": FUSED_SRC_INPUT, "arg": 0, "flags": 2, "dt": ("u", 32)},
               {"kind": FUSED_BINARY, "op": 14, "src": FUSED_SRC_CONST, "imm_bits": 9, "flags": 2, "dt": ("u", 32)}]  # right_shift
    with pytest.raises(HipNxError, match="need the compiled mode"):
        hip.fused_elementwise(x.with_(data=None), program, [x], (1, 64, [(0, 1)]))
    got = hip.fused_elementwise(x.with_(data=None), program, [x], (1, 64, [(0, 1)]), mode="compiled")
    np.testing.assert_array_equal(hip.to_numpy(got), hip.to_numpy(x) >> 9)


@pytest.mark.parametrize("name", ["uniform", "normal"])
def test_random_floats_from_one_compiled_group(name, hip):
    from nx_amd import random as Random
    key = Random.key(99, backend=hip)
    fun = {"uniform": lambda k: Random.uniform_split(k, -2.0, 3.0, shape=(64, 1024)),
           "normal": lambda k: Random.normal_split(k, 1.0, 2.0, shape=(64, 1024))}[name]
    want = defn.compile(fun, key)(key)
    fused = defn.compile(fun, key, fuse="compiled")
    assert_bits_equal(fused(key), want, name)
    calls = []
    original = hip.fused_elementwise.__func__

    def counting(cls, *a, **k):
        calls.append(1)
        return original(cls, *a, **k)
    hip.fused_elementwise = classmethod(counting)
    try:
        fused(key)
    finally:
        hip.fused_elementwise = classmethod(original)
    assert len(calls) >= 1 and fused.fused_groups == 1  # everything after the cipher is one group


# ---- dot -> as_type -> multiply by the scales on the accumulators (the quantised linear layer) -----------

def linear_scaled(xq, wq, sc):
    return Nx.multiply(Nx.as_type(Nx.dot(xq, [1], wq, [1], out_type="s32"), "f32"), sc)


def rand_s8(rng, shape, backend):
    return from_numpy(rng.integers(-127, 128, size=shape, dtype=np.int8), "s8", backend)


@pytest.mark.parametrize("m,n,k", [(64, 11008, 4096), (64, 256, 4096), (16, 512, 8192), (300, 520, 256), (256, 256, 128), (1024, 1024, 1024), (8, 40, 128)])
@pytest.mark.parametrize("scales", ["per_column", "per_row", "one", "constant"])
def test_scaled_int8_dot_is_bit_identical_to_the_three_callbacks(m, n, k, scales, hip):
    rng = np.random.default_rng(seed_of(m, n, k, scales))
    x, w = rand_s8(rng, (m, k), hip), rand_s8(rng, (n, k), hip)
    if scales == "constant":
        fun, args = (lambda xq, wq: linear_scaled(xq, wq, 0.0078125)), (x, w)
    else:
        shape = {"per_column": (n,), "per_row": (m, 1), "one": (1, 1)}[scales]
        sc = from_numpy(rng.uniform(1e-3, 1e-2, size=shape).astype(np.float32), "f32", hip)
        if scales == "per_column":  # a NaN and an infinity among the scales travel like in the multiply kernel
            raw = hip.to_numpy(sc).copy()
            raw[0], raw[-1] = np.nan, np.inf
            sc = from_numpy(raw, "f32", hip)
        fun, args = linear_scaled, (x, w, sc)
    want = defn.compile(fun, *args)(*args)
    planned = defn.compile(fun, *args, fuse=True)
    assert planned.roots[0].data.op == "dot_scaled"
    calls = []
    original = hip.dot_scaled.__func__

    def counting(cls, *a, **kw):
        calls.append(1)
        return original(cls, *a, **kw)
    hip.dot_scaled = classmethod(counting)
    try:
        assert_bits_equal(planned(*args), want, f"{m}x{n}x{k} {scales}")
    finally:
        hip.dot_scaled = classmethod(original)
    assert calls == [1]


def test_scaled_dot_with_batches_and_with_the_weights_k_outer(hip):
    rng = np.random.default_rng(77)
    x, w = rand_s8(rng, (4, 48, 256), hip), rand_s8(rng, (4, 256, 80), hip)
    sc = from_numpy(rng.uniform(1e-3, 1e-2, size=(80,)).astype(np.float32), "f32", hip)

    def fun(xq, wq, s):  # batched, the right operand contracted on its middle axis
        return Nx.multiply(Nx.as_type(Nx.dot(xq, [2], [0], wq, [1], [0], out_type="s32"), "f32"), s)
    planned = defn.compile(fun, x, w, sc, fuse=True)
    assert planned.roots[0].data.op == "dot_scaled"
    assert_bits_equal(planned(x, w, sc), defn.compile(fun, x, w, sc)(x, w, sc), "batched")


def test_scaled_dot_entry_point_refuses_what_it_does_not_take(hip):
    from nx_amd._lib import EUNSUPPORTED, SCALE_PER_COLUMN, HipNxError
    rng = np.random.default_rng(5)
    x, w = rand_s8(rng, (8, 100), hip), rand_s8(rng, (40, 100), hip)  # K is not a multiple of 128
    sc = from_numpy(np.ones(40, dtype=np.float32), "f32", hip)
    out = sc.with_(data=None, shape=(8, 40))
    with pytest.raises(HipNxError) as err:
        hip.dot_scaled(out, x, [1], [], w, [1], [], sc, SCALE_PER_COLUMN)
    assert err.value.status == EUNSUPPORTED
    # through the evaluator the same shapes make the three calls instead
    planned = defn.compile(linear_scaled, x, w, sc, fuse=True)
    assert_bits_equal(planned(x, w, sc), defn.compile(linear_scaled, x, w, sc)(x, w, sc), "fallback")
    short = from_numpy(np.ones(8, dtype=np.float32), "f32", hip)
    x2, w2 = rand_s8(rng, (16, 128), hip), rand_s8(rng, (40, 128), hip)
    with pytest.raises(HipNxError, match="holds"):
        hip.dot_scaled(sc.with_(data=None, shape=(16, 40)), x2, [1], [], w2, [1], [], short, SCALE_PER_COLUMN)


# ---- stages over the same rows in one kernel (planned for compiled kernels) ------------------------------

def softmax_rows(x):
    z = Nx.multiply(x, 0.125)
    e = Nx.exp(Nx.subtract(z, Nx.reduce_max(z, axes=[-1], keep_axes=True)))
    return Nx.divide(e, Nx.sum(e, axes=[-1], keep_axes=True))


def centred_and_scaled(x, gain):  # layer-norm-like: mean, then mean of squares of the centred values
    n = x.shape[-1]
    mean = Nx.divide(Nx.sum(x, axes=[-1], keep_axes=True), float(n))
    c = Nx.subtract(x, mean)
    var = Nx.divide(Nx.sum(Nx.multiply(c, c), axes=[-1], keep_axes=True), float(n))
    return Nx.multiply(Nx.multiply(c, Nx.rsqrt(Nx.add(var, 1e-5))), gain)


def range_normalised(x):          # three statistics: minimum, maximum, and the sum of the result's numerator
    lo = Nx.reduce_min(x, axes=[-1], keep_axes=True)
    hi = Nx.reduce_max(x, axes=[-1], keep_axes=True)
    u = Nx.divide(Nx.subtract(x, lo), Nx.subtract(hi, lo))
    return Nx.divide(u, Nx.sum(u, axes=[-1], keep_axes=True))


def softmax_new_axis(x):          # statistics taken without keep_axes, then given their axis back
    m = Nx.new_axis(Nx.reduce_max(x, axes=[-1]), -1)
    e = Nx.exp(Nx.subtract(x, m))
    return Nx.divide(e, Nx.new_axis(Nx.sum(e, axes=[-1]), -1))


def log_softmax_rows(x):
    z = Nx.subtract(x, Nx.reduce_max(x, axes=[-1], keep_axes=True))
    return Nx.subtract(z, Nx.log(Nx.sum(Nx.exp(z), axes=[-1], keep_axes=True)))


def rms_scaled(x):                # one statistic, worked on with two constants and a square root; bf16 rounds at every node
    n = x.shape[-1]
    ms = Nx.divide(Nx.sum(Nx.multiply(x, x), axes=[-1], keep_axes=True), float(n))
    return Nx.divide(x, Nx.sqrt(Nx.add(ms, 1e-6)))


@pytest.mark.parametrize("ty", ["f32", "bf16"])
@pytest.mark.parametrize("shape", [(32, 512, 512), (100, 64), (7, 4096), (3, 5, 8), (1, 1024), (2049, 40)])
@pytest.mark.parametrize("name", ["softmax_rows", "centred_and_scaled", "range_normalised", "log_softmax_rows", "rms_scaled",
                                  "softmax_new_axis"])
def test_row_stages_are_bit_identical_to_node_by_node(name, shape, ty, hip):
    rng = np.random.default_rng(seed_of(name, shape, ty))
    x = rand_float(rng, ty, shape, hip)
    args = (x, rand_float(rng, ty, (shape[-1],), hip)) if name == "centred_and_scaled" else (x,)
    fun = {"softmax_rows": softmax_rows, "centred_and_scaled": centred_and_scaled, "range_normalised": range_normalised,
           "log_softmax_rows": log_softmax_rows, "rms_scaled": rms_scaled, "softmax_new_axis": softmax_new_axis}[name]
    want = defn.compile(fun, *args)(*args)
    planned = defn.compile(fun, *args, fuse="compiled")
    # work on a statistic before it is used (the mean and the variance of the second function are divided by n,
    # the variance goes through an rsqrt) belongs to the stage that makes it
    staged = True
    assert (type(planned.roots[0].data.args[0]).__name__ == "_RowCluster") == staged
    calls = []
    original = hip.fused_elementwise.__func__

    def counting(cls, *a, **k):
        if "mode" in k:
            calls.append(1)
        return original(cls, *a, **k)
    hip.fused_elementwise = classmethod(counting)
    try:
        assert_bits_equal(planned(*args), want, f"{name} {shape} {ty}")
    finally:
        hip.fused_elementwise = classmethod(original)
    if staged:
        assert calls == [1]  # one launch for all stages


@pytest.mark.parametrize("ty", ["f32", "bf16"])
@pytest.mark.parametrize("shape", [(8, 8192), (64, 4104), (16, 32000), (3, 16384), (5, 16392)])
@pytest.mark.parametrize("name", ["softmax_rows", "centred_and_scaled", "log_sum_exp_rows"])
def test_long_rows_take_a_block_each(name, shape, ty, hip):
    rng = np.random.default_rng(seed_of(name, shape, ty))
    x = rand_float(rng, ty, shape, hip)
    args = (x, rand_float(rng, ty, (shape[-1],), hip)) if name == "centred_and_scaled" else (x,)
    fun = {"softmax_rows": softmax_rows, "centred_and_scaled": centred_and_scaled, "log_sum_exp_rows": log_sum_exp_rows}[name]
    want = defn.compile(fun, *args)(*args)
    planned = defn.compile(fun, *args, fuse="compiled")
    assert type(planned.roots[0].data.args[0]).__name__ == "_RowCluster"
    calls = []
    original = hip.fused_elementwise.__func__

    def counting(cls, *a, **k):
        if "mode" in k:
            calls.append(1)
        return original(cls, *a, **k)
    hip.fused_elementwise = classmethod(counting)
    try:
        assert_bits_equal(planned(*args), want, f"{name} {shape} {ty}")
    finally:
        hip.fused_elementwise = classmethod(original)
    assert calls == [1]


def test_rows_too_long_for_carried_values_are_read_again(hip):
    x = rand_float(np.random.default_rng(7), "f32", (2048, 32776), hip)
    planned = defn.compile(softmax_rows, x, fuse="compiled")
    cluster = planned.roots[0].data.args[0]
    assert type(cluster).__name__ == "_RowCluster" and not any(ins.get("src") == 4 for ins in cluster.program)
    assert_bits_equal(planned(x), defn.compile(softmax_rows, x)(x), "rows of 32776")


def test_rows_that_the_reduction_would_split_run_stage_by_stage(hip):
    x = rand_float(np.random.default_rng(6), "f32", (4, 65536), hip)   # few rows, very long: the separate sum works in segments
    planned = defn.compile(softmax_rows, x, fuse="compiled")
    assert_bits_equal(planned(x), defn.compile(softmax_rows, x)(x), "split rows")


def test_a_few_very_long_rows_keep_their_reduction_in_the_group(hip):
    """exp(t) / sum(exp(t)) over a million values (exla/bench/softmax.exs:1-41): the sum is cut into segments as the
    separate reduction cuts it, so the group that feeds it still holds it -- one call, the same bits -- and the
    refusal of the stage program, which the shape alone decides, is asked for once."""
    from nx_amd.backend import fused_mode as set_mode
    t = rand_float(np.random.default_rng(1000000), "f32", (1000000,), hip)

    def softmax(n):
        return Nx.divide(Nx.exp(n), Nx.sum(Nx.exp(n)))
    want = defn.compile(softmax, t)(t)
    planned = defn.compile(softmax, t, fuse="compiled")
    calls = []
    original = hip.fused_elementwise.__func__

    def counting(cls, *a, **k):
        calls.append(a[4] if len(a) > 4 else k.get("reduce_op", -1))
        return original(cls, *a, **k)
    hip.fused_elementwise = classmethod(counting)
    try:
        set_mode("compiled")
        assert_bits_equal(planned(t), want, "first call")
        first = list(calls)
        del calls[:]
        assert_bits_equal(planned(t), want, "second call")
        assert calls == [0, -1], calls            # the sum inside its group, then the quotient
        assert first in ([-1, 0, -1], [0, -1])    # (with the stage program offered and refused once, where one was planned)
    finally:
        set_mode("interpreted")
        hip.fused_elementwise = classmethod(original)


def test_configuration_3_softmax_in_one_kernel(hip):
    args = build_args(hip)["softmax"]
    planned = defn.compile(CHAINS["softmax"], *args, fuse="compiled")
    assert type(planned.roots[0].data.args[0]).__name__ == "_RowCluster"
    assert_bits_equal(planned(*args), defn.compile(CHAINS["softmax"], *args)(*args), "softmax of the scores")


def log_sum_exp_rows(x):
    m = Nx.reduce_max(x, axes=[-1], keep_axes=True)
    return Nx.add(Nx.log(Nx.sum(Nx.exp(Nx.subtract(x, m)), axes=[-1], keep_axes=True)), m)


def mean_rows(x):
    return Nx.mean(x, axes=[-1], keep_axes=True)


def root_mean_square_rows(x):
    return Nx.sqrt(Nx.divide(Nx.sum(Nx.multiply(x, x), axes=[-1], keep_axes=True), float(x.shape[-1])))


def spread_rows(x):               # the result reads two other statistics
    lo = Nx.reduce_min(x, axes=[-1], keep_axes=True)
    hi = Nx.reduce_max(x, axes=[-1], keep_axes=True)
    return Nx.divide(Nx.sum(Nx.subtract(x, lo), axes=[-1], keep_axes=True), hi)


@pytest.mark.parametrize("ty", ["f32", "bf16"])
@pytest.mark.parametrize("shape", [(32, 512, 512), (100, 64), (7, 4096), (3, 5, 8), (1, 1024), (2049, 40)])
@pytest.mark.parametrize("name", ["log_sum_exp_rows", "mean_rows", "root_mean_square_rows", "spread_rows"])
def test_per_row_results_from_one_kernel_are_bit_identical(name, shape, ty, hip):
    rng = np.random.default_rng(seed_of(name, shape, ty))
    x = rand_float(rng, ty, shape, hip)
    fun = {"log_sum_exp_rows": log_sum_exp_rows, "mean_rows": mean_rows, "root_mean_square_rows": root_mean_square_rows,
           "spread_rows": spread_rows}[name]
    want = defn.compile(fun, x)(x)
    planned = defn.compile(fun, x, fuse="compiled")
    cluster = planned.roots[0].data.args[0]
    assert type(cluster).__name__ == "_RowCluster" and cluster.program[-1].get("flags") == 1
    calls = []
    original = hip.fused_elementwise.__func__

    def counting(cls, *a, **k):
        if "mode" in k:
            calls.append(1)
        return original(cls, *a, **k)
    hip.fused_elementwise = classmethod(counting)
    try:
        assert_bits_equal(planned(x), want, f"{name} {shape} {ty}")
    finally:
        hip.fused_elementwise = classmethod(original)
    assert calls == [1]


# ---- a flat index space that is no whole number of vectors (compiled groups take the partial last one) ----

@pytest.mark.parametrize("ty", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("shape", [(1,), (7,), (9,), (37, 11), (3, 5, 7), (1000003,), (255, 257)])
def test_ragged_sizes_in_compiled_groups(shape, ty, hip):
    rng = np.random.default_rng(seed_of(shape, ty))
    x, y = rand_float(rng, ty, shape, hip), rand_float(rng, ty, shape, hip)
    guard = rand_float(rng, ty, (64,), hip)   # a neighbour in memory that must stay as it is

    def fun(a, b):
        h = Nx.add(Nx.multiply(a, 0.5), b)
        return Nx.select(Nx.greater(h, 0.0), Nx.tanh(h), Nx.multiply(h, 0.01))

    want = defn.compile(fun, x, y)(x, y)
    before = hip.to_numpy(guard).copy()
    planned = defn.compile(fun, x, y, fuse="compiled")
    assert planned.roots[0].data.op == "fused" and planned.roots[0].data.args[0].layout is not None
    assert_bits_equal(planned(x, y), want, f"ragged {shape} {ty}")
    np.testing.assert_array_equal(hip.to_numpy(guard), before)
    # planned without the compiled kernels in mind, such a shape is left to the separate callbacks
    assert_bits_equal(defn.compile(fun, x, y, fuse=True)(x, y), want, f"ragged {shape} {ty}, mode-agnostic plan")


def test_ragged_integer_words(hip):
    x = rand_words(np.random.default_rng(12), "u32", (1001,), hip)
    planned = defn.compile(bits_to_unit_floats, x, fuse="compiled")
    assert planned.roots[0].data.op == "fused"
    assert_bits_equal(planned(x), defn.compile(bits_to_unit_floats, x)(x), "ragged u32 -> f32")


def test_ragged_rows_still_fall_back(hip):
    rng = np.random.default_rng(13)
    x, bias = rand_float(rng, "f32", (37, 11), hip), rand_float(rng, "f32", (11,), hip)   # a row operand: no flat index space

    def fun(a, b):
        return Nx.exp(Nx.add(a, b))
    planned = defn.compile(fun, x, bias, fuse="compiled")
    assert_bits_equal(planned(x, bias), defn.compile(fun, x, bias)(x, bias), "row operand, ragged rows")


@pytest.mark.parametrize("ty", ["f16", "bf16", "f32"])
def test_fused_groups_on_special_values(ty, hip):
    """Every unary and binary element-wise node a group can hold, on zeros of either sign, the smallest numbers, domain
    ends, infinities and NaN: the group's bits are those of the nodes run one by one, interpreted and compiled."""
    from nx_amd.backend import fused_mode as set_mode
    from test_gpu_elementwise import MATH, encode
    tiny = {"f16": 6e-8, "bf16": 1e-38, "f32": 1e-45}[ty]
    large = 8.0 if ty == "f16" else 30.0
    v = np.array([0.0, -0.0, tiny, -tiny, 1.0, -1.0, 0.5, -0.5, 2.0, -2.0, np.inf, -np.inf, np.nan, 1e-4, -1e-4, large, -large,
                  3.0, -3.0, 0.25, -0.25, 1.5, -1.5, 7.0])
    x = from_numpy(encode(v, ty), ty, hip)
    a, b = [g.ravel() for g in np.meshgrid(v[:16], v[:16], indexing="ij")]
    ha, hb = from_numpy(encode(a, ty), ty, hip), from_numpy(encode(b, ty), ty, hip)
    programs = [(f"{op} then negate", (lambda t, op=op: Nx.negate(getattr(Nx, op)(t))), (x,)) for op in MATH]
    programs += [(f"{op} plus its operand", (lambda t, op=op: Nx.add(getattr(Nx, op)(t), t)), (x,)) for op in MATH]
    programs += [(f"{op} then negate", (lambda p, q, op=op: Nx.negate(getattr(Nx, op)(p, q))), (ha, hb))
                 for op in ("add", "subtract", "multiply", "divide", "pow", "atan2", "min", "max")]
    programs += [(f"{op} times its operand", (lambda p, q, op=op: Nx.multiply(getattr(Nx, op)(p, q), q)), (ha, hb))
                 for op in ("add", "subtract", "multiply", "divide", "min", "max")]
    try:
        for name, fun, args in programs:
            want = defn.compile(fun, *args)(*args)
            for mode in ("interpreted", "compiled"):
                set_mode(mode)
                assert_bits_equal(defn.compile(fun, *args, fuse=True)(*args), want, f"{name}, {ty}, {mode}")
    finally:
        set_mode("interpreted")
