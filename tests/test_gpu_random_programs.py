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


def make_program(rng, n_inputs, in_memory=False):
    """A list of steps over a growing list of values; returns (steps, function).  `in_memory`: also nodes that are not
    element-wise and keep the shape (a reversal, a clip, a reduction along the first axis, a transposition there and back
    with work in between), whose operands must exist in memory: they cut the groups."""
    steps = []
    n = n_inputs
    reduced = False
    for _ in range(int(rng.integers(2, 10))):
        if in_memory and rng.random() < 0.25:
            steps.append((["reverse", "clip", "sum_first", "transposed_tanh"][int(rng.integers(0, 4))], int(rng.integers(0, n))))
            n += 1
            continue
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
            elif st[0] == "as_type":
                v = Nx.as_type(vals[st[2]], st[1])
            else:
                t = vals[st[1]]
                rank = len(t.shape)
                if rank == 0:
                    v = Nx.negate(t)
                elif st[0] == "reverse":
                    v = Nx.reverse(t, axes=[rank - 1])
                elif st[0] == "clip":
                    v = Nx.clip(t, -0.75, 1.5)
                elif st[0] == "sum_first":
                    v = Nx.subtract(t, Nx.sum(t, axes=[0], keep_axes=True))
                else:
                    back = list(range(rank - 1, -1, -1))
                    v = Nx.transpose(Nx.tanh(Nx.transpose(t, axes=back)), axes=back)
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


@pytest.mark.parametrize("case", range(80))
def test_random_program_with_nodes_that_cut_the_groups(case, hip):
    """Reversals, clips, reductions along the first axis and transpositions between the element-wise nodes: what a group
    reads from such a node, and what such a node reads from a group, has to be in memory at the right time."""
    from nx_amd.backend import fused_mode as set_mode
    rng = np.random.default_rng(seed_of("program-in-memory", case + OFFSET))
    full = LEAD[int(rng.integers(0, len(LEAD)))] + (int(rng.choice(LAST)),)
    n_inputs = int(rng.integers(1, 4))
    args = []
    for i in range(n_inputs):
        ty = ["f32", "f32", "bf16", "f16"][int(rng.integers(0, 4))]
        args.append(operand(rng, ty, full if i == 0 else broadcastable(rng, full), hip))
    steps, fn = make_program(rng, n_inputs, in_memory=True)
    what = f"case {case + OFFSET}: {[(tuple(a.shape), a.type) for a in args]} {steps}"
    try:
        want = defn.compile(fn, *args)(*args)
    except (ValueError, TypeError) as e:
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


# ---- programs over 32-bit integers (what Nx.Random's bits-to-floats chains are made of) -------------------------
INT_BINARY = ["add", "subtract", "multiply", "bitwise_and", "bitwise_or", "bitwise_xor", "min", "max"]
INT_NUMBERS = [0, 1, 3, 9, 31, 255, 0x3F800000, 0x7FFFFFFF, 0x9E3779B9, -1, -7]


def make_integer_program(rng, types):
    """Steps over words: integer arithmetic (wrapping), shifts by constants, relabelling of bits between u32 / s32 / f32,
    conversions to floats and float work after them.  `types` is the list of the inputs' types, extended as steps are added
    (a step only picks operands of a type it is defined for, so every program type-checks)."""
    steps, types = [], list(types)
    n_inputs = len(types)

    def pick(wanted):
        at = [i for i, t in enumerate(types) if t in wanted]
        return at[int(rng.integers(0, len(at)))] if at else None

    for _ in range(int(rng.integers(3, 12))):
        kind = rng.choice(["int2", "number", "shift", "unary", "bitcast", "as_type", "float", "select"],
                          p=[0.22, 0.18, 0.14, 0.08, 0.14, 0.1, 0.1, 0.04])
        a = pick(("u32", "s32"))
        if kind == "int2" and a is not None:
            b = pick((types[a],))
            steps.append(("binary", INT_BINARY[int(rng.integers(0, len(INT_BINARY)))], a, b))
            types.append(types[a])
        elif kind == "number" and a is not None:
            number = INT_NUMBERS[int(rng.integers(0, len(INT_NUMBERS)))]
            if types[a] == "u32" and number < 0:
                number = -number
            if types[a] == "s32" and number > 0x7FFFFFFF:
                number = 12345
            steps.append(("number", INT_BINARY[int(rng.integers(0, len(INT_BINARY)))], a, number, bool(rng.integers(0, 2))))
            types.append(types[a])
        elif kind == "shift" and a is not None:
            steps.append(("number", ["left_shift", "right_shift"][int(rng.integers(0, 2))], a, int(rng.integers(0, 32)), False))
            types.append(types[a])
        elif kind == "unary" and a is not None:
            steps.append(("unary", ["negate", "bitwise_not"][int(rng.integers(0, 2))], a))
            types.append(types[a])
        elif kind == "bitcast":
            a = int(rng.integers(0, len(types)))
            if types[a] not in ("u32", "s32", "f32"):
                continue
            to = [t for t in ("u32", "s32", "f32") if t != types[a]][int(rng.integers(0, 2))]
            steps.append(("bitcast", to, a))
            types.append(to)
        elif kind == "as_type":
            a = int(rng.integers(0, len(types)))
            to = ["f32", "bf16", "f16"][int(rng.integers(0, 3))]
            steps.append(("as_type", to, a))
            types.append(to)
        elif kind == "float":
            a = pick(("f32", "bf16", "f16"))
            if a is None:
                continue
            if rng.random() < 0.5:
                steps.append(("number", ["subtract", "multiply", "add"][int(rng.integers(0, 3))], a, [1.0, 0.5, 2.0][int(rng.integers(0, 3))], False))
            else:
                steps.append(("unary", ["abs", "sqrt", "negate", "floor"][int(rng.integers(0, 4))], a))
            types.append(types[a])
        elif kind == "select" and a is not None:
            f = pick(("f32",))
            if f is None:
                continue
            steps.append(("select_float", a, f))
            types.append("f32")

    if not steps:  # every draw fell on a step its operands' types do not allow
        steps.append(("unary", "bitwise_not", 0))

    def fn(*xs):
        vals = list(xs)
        for st in steps:
            if st[0] == "unary":
                v = getattr(Nx, st[1])(vals[st[2]])
            elif st[0] == "binary":
                v = getattr(Nx, st[1])(vals[st[2]], vals[st[3]])
            elif st[0] == "number":
                v = getattr(Nx, st[1])(st[3], vals[st[2]]) if st[4] else getattr(Nx, st[1])(vals[st[2]], st[3])
            elif st[0] == "bitcast":
                v = Nx.bitcast(vals[st[2]], st[1])
            elif st[0] == "as_type":
                v = Nx.as_type(vals[st[2]], st[1])
            else:  # a float chosen by a comparison of floats made from the integers
                as_float = Nx.as_type(vals[st[1]], "f32")
                v = Nx.select(Nx.less(as_float, vals[st[2]]), as_float, vals[st[2]])
            vals.append(v)
        return vals[-1], vals[n_inputs + (len(vals) - n_inputs) // 2]

    return steps, fn


def integer_operand(rng, ty, shape, hip):
    if ty == "f32":
        return operand(rng, ty, shape, hip)
    bits = rng.integers(0, 1 << 32, size=shape, dtype=np.uint64).astype(np.uint32)
    if rng.random() < 0.3:
        bits >>= np.uint32(rng.integers(8, 30))  # small numbers: conversions to narrow floats stay finite
    return from_numpy(bits.astype({"u32": np.uint32, "s32": np.int32, "u8": np.uint8, "s16": np.int16}[ty]), ty, hip)


def integer_operand_types(rng):
    full = LEAD[int(rng.integers(0, len(LEAD)))] + (int(rng.choice(LAST)),)
    types, shapes = [], []
    for i in range(int(rng.integers(1, 4))):
        types.append(["u32", "s32", "u32", "f32", "u8", "s16"][int(rng.integers(0, 6))] if i else ["u32", "s32"][int(rng.integers(0, 2))])
        shapes.append(full if i == 0 else broadcastable(rng, full))
    return types, shapes


@pytest.mark.parametrize("case", range(80))
def test_random_integer_program_has_the_same_bits_however_it_is_grouped(case, hip):
    from nx_amd.backend import fused_mode as set_mode
    rng = np.random.default_rng(seed_of("integer-program", case + OFFSET))
    types, shapes = integer_operand_types(rng)
    args = [integer_operand(rng, ty, sh, hip) for ty, sh in zip(types, shapes)]
    steps, fn = make_integer_program(rng, types)
    what = f"case {case + OFFSET}: {[(tuple(a.shape), a.type) for a in args]} {steps}"
    want = defn.compile(fn, *args)(*args)
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


@pytest.mark.parametrize("case", range(30))
def test_random_integer_program_replays_from_a_captured_graph(case, hip):
    """Planned for compilation, recorded, and replayed with the captured tensors, new ones, and the first again."""
    from nx_amd.backend import fused_mode as set_mode, sync
    rng = np.random.default_rng(seed_of("integer-program-graph", case + OFFSET))
    types, shapes = integer_operand_types(rng)
    args = [integer_operand(rng, ty, sh, hip) for ty, sh in zip(types, shapes)]
    fresh = [integer_operand(rng, ty, sh, hip) for ty, sh in zip(types, shapes)]
    steps, fn = make_integer_program(rng, types)
    what = f"case {case + OFFSET}: {[(tuple(a.shape), a.type) for a in args]} {steps}"
    plain = defn.compile(fn, *args)
    want_args, want_fresh = plain(*args), plain(*fresh)
    set_mode("compiled")
    captured = None
    try:
        compiled = defn.compile(fn, *args, fuse="compiled")
        compiled(*args)  # (compiled before the capture begins)
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
