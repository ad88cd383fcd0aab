"""Random traced programs: chains of element-wise callbacks over broadcasting operands, some with row reductions
whose results flow back into the chain (the shape of a softmax or a normalisation), run node by node, as fused groups on
the interpreting kernels, as groups compiled at run time, and planned as stages of one program.  Grouping, recomputation,
carried values and operand layouts all differ between the four; the bits must not.  (The same calls made one by one outside
a trace are another matter: the tracer moves constants outwards, `(x + 0.5) + x` becomes `0.5 + (x + x)`, as the
reference's does -- nx/lib/nx/defn/expr.ex, `commute` -- which rounds differently.)"""
import os

import numpy as np
import pytest

from nx_amd import defn
from nx_amd import nx as Nx
from support import assert_bits_equal, from_numpy, seed_of

pytestmark = pytest.mark.gpu

# HIPNX_SWEEP_OFFSET=n shifts the sweep to cases n, n + 1, ... (the committed run is offset 0)
OFFSET = int(os.environ.get("HIPNX_SWEEP_OFFSET", "0"))

UNARY = ["exp", "negate", "abs", "tanh", "sigmoid", "sqrt", "log1p", "floor", "sign", "cos", "expm1", "rsqrt", "erf"]
BINARY = ["add", "subtract", "multiply", "max", "min", "divide", "atan2", "pow"]
COMPARE = ["less", "greater_equal", "equal"]
LAST = [1, 3, 7, 8, 33, 64, 100, 256, 513, 1024, 4100]
LEAD = [(), (1,), (5,), (64,), (3, 4), (2, 1), (300,)]


def make_program(rng, n_inputs):
    """A list of steps over a growing list of values; returns (steps, function)."""
    steps = []
    n = n_inputs
    reduced = False
    for _ in range(int(rng.integers(2, 10))):
        kind = rng.choice(["unary", "binary", "number", "reduce", "select", "as_type"], p=[0.3, 0.3, 0.15, 0.12, 0.08, 0.05])
        a, b, c = int(rng.integers(0, n)), int(rng.integers(0, n)), int(rng.integers(0, n))
        if kind == "unary":
            steps.append(("unary", UNARY[int(rng.integers(0, len(UNARY)))], a))
        elif kind == "binary":
            steps.append(("binary", BINARY[int(rng.integers(0, len(BINARY)))], a, b))
        elif kind == "number":
            number = [0.5, 2.0, -1.25, 3, 0.044715][int(rng.integers(0, 5))]
            steps.append(("number", ["add", "multiply", "subtract", "max", "divide"][int(rng.integers(0, 5))], a, number, bool(rng.integers(0, 2))))
        elif kind == "reduce":
            if reduced and rng.random() < 0.5:
                continue
            reduced = True
            steps.append(("reduce", ["sum", "reduce_max", "reduce_min"][int(rng.integers(0, 3))], a, bool(rng.random() < 0.8)))
        elif kind == "select":
            steps.append(("select", COMPARE[int(rng.integers(0, 3))], a, b, c))
        else:
            steps.append(("as_type", ["bf16", "f32", "f16"][int(rng.integers(0, 3))], a))
        n += 1

    def fn(*xs):
        vals = list(xs)
        for st in steps:
            if st[0] == "unary":
                v = getattr(Nx, st[1])(vals[st[2]])
            elif st[0] == "binary":
                v = getattr(Nx, st[1])(vals[st[2]], vals[st[3]])
            elif st[0] == "number":
                v = getattr(Nx, st[1])(st[3], vals[st[2]]) if st[4] else getattr(Nx, st[1])(vals[st[2]], st[3])
            elif st[0] == "reduce":
                t = vals[st[2]]
                v = getattr(Nx, st[1])(t, axes=[len(t.shape) - 1], keep_axes=st[3]) if len(t.shape) else t
            elif st[0] == "select":
                v = Nx.select(getattr(Nx, st[1])(vals[st[2]], vals[st[3]]), vals[st[3]], vals[st[4]])
            else:
                v = Nx.as_type(vals[st[2]], st[1])
            vals.append(v)
        # the last value, and an earlier one that something else may also have read
        return vals[-1], vals[n_inputs + (len(vals) - n_inputs) // 2]

    return steps, fn


def broadcastable(rng, shape):
    s = [d if rng.random() < 0.7 else 1 for d in shape]
    return tuple(s[int(rng.integers(0, len(s))):]) if rng.random() < 0.4 else tuple(s)


def operand(rng, ty, shape, hip):
    v = rng.standard_normal(shape).astype(np.float32)
    if ty == "bf16":
        return from_numpy((v.view(np.uint32) >> 16).astype(np.uint16), "bf16", hip)
    return from_numpy(v.astype(np.float16 if ty == "f16" else np.float32), ty, hip)


@pytest.mark.parametrize("case", range(120))
def test_random_program_has_the_same_bits_however_it_is_grouped(case, hip):
    from nx_amd.backend import fused_mode as set_mode
    rng = np.random.default_rng(seed_of("program", case + OFFSET))
    full = LEAD[int(rng.integers(0, len(LEAD)))] + (int(rng.choice(LAST)),)
    n_inputs = int(rng.integers(1, 4))
    args = []
    for i in range(n_inputs):
        ty = ["f32", "f32", "bf16", "f16"][int(rng.integers(0, 4))]
        args.append(operand(rng, ty, full if i == 0 else broadcastable(rng, full), hip))
    steps, fn = make_program(rng, n_inputs)
    what = f"case {case + OFFSET}: {[(tuple(a.shape), a.type) for a in args]} {steps}"
    try:
        want = defn.compile(fn, *args)(*args)
    except (ValueError, TypeError) as e:  # a shape the front end refuses (a reduced value against a full one of another rank)
        pytest.skip(f"the program does not type-check: {e}")
    try:
        for mode in ("interpreted", "compiled"):
            set_mode(mode)
            got = defn.compile(fn, *args, fuse=True)(*args)
            for g, w in zip(got, want):
                assert_bits_equal(g, w, f"fused, {mode}; {what}")
        got = defn.compile(fn, *args, fuse="compiled")(*args)
        for g, w in zip(got, want):
            assert_bits_equal(g, w, f"planned; {what}")
    finally:
        set_mode("interpreted")


@pytest.mark.parametrize("case", range(40))
def test_random_program_replays_from_a_captured_graph(case, hip):
    """The same programs recorded into a graph (node by node, or as compiled groups) and replayed: with the captured
    tensors, with new values, and back, eager work and synchronisations in between; every replay against the function run
    outside the graph."""
    from nx_amd.backend import fused_mode as set_mode, sync
    rng = np.random.default_rng(seed_of("program-graph", case + OFFSET))
    full = LEAD[int(rng.integers(0, len(LEAD)))] + (int(rng.choice(LAST)),)
    n_inputs = int(rng.integers(1, 4))
    shapes_types = [(full if i == 0 else broadcastable(rng, full), ["f32", "f32", "bf16", "f16"][int(rng.integers(0, 4))]) for i in range(n_inputs)]
    args = [operand(rng, ty, sh, hip) for sh, ty in shapes_types]
    fresh = [operand(rng, ty, sh, hip) for sh, ty in shapes_types]
    steps, fn = make_program(rng, n_inputs)
    fuse = [False, True, "compiled"][int(rng.integers(0, 3))]
    what = f"case {case + OFFSET}: fuse={fuse} {[(tuple(a.shape), a.type) for a in args]} {steps}"
    try:
        plain = defn.compile(fn, *args)
        want_args, want_fresh = plain(*args), plain(*fresh)
    except (ValueError, TypeError) as e:
        pytest.skip(f"the program does not type-check: {e}")
    set_mode("compiled")
    captured = None
    try:
        compiled = defn.compile(fn, *args, fuse=fuse)
        compiled(*args)  # (a program first met while capturing would run interpreted: compile it beforehand)
        captured = compiled.capture(*args)
        for given, want in ((args, want_args), (fresh, want_fresh), (args, want_args)):
            got = captured(*given)
            for g, w in zip(got, want):
                assert_bits_equal(g, w, f"replay; {what}")
            plain(*fresh)
            sync()
    finally:
        if captured is not None:
            captured.destroy()
        set_mode("interpreted")
