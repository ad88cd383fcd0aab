"""The traced-function layer (nx_amd/defn.py) on the CPU, with the oracle as the compute backend:
the rewrites of the expression builder (they change float results, so they are part of parity), the
evaluator against eager execution, scopes and reference counts, and `Nx.Random` through a trace
against the reference's known answers."""
import numpy as np
import pytest

from nx_amd import defn
from nx_amd import nx as Nx
from nx_amd import random as Random
from nx_amd.defn import Expr
from random_support import CASES, check_random_case
from support import assert_bits_equal, from_numpy


@pytest.fixture()
def on_oracle(oracle):
    previous = Nx.default_backend(oracle)
    yield oracle
    Nx.default_backend(*previous)


def traced(fun, *args):
    """The root expressions of `fun` traced on `args`."""
    return defn.trace(fun, args).roots


def f32(values, backend):
    return from_numpy(np.asarray(values, dtype=np.float32), "f32", backend)


# ---- the builder's rewrites (nx/lib/nx/defn/expr.ex:889-984, 1597-1674) -------------------------

def test_constant_factors_merge_and_move_left(on_oracle):
    x = f32([1, 2, 3], on_oracle)
    (root,) = traced(lambda t: Nx.multiply(3.0, Nx.multiply(t, 5.0)), x)
    assert root.data.op == "multiply"
    const, rest = root.data.args
    assert const.data.op == "constant" and const.data.args == [15.0] and rest.data.op == "parameter"


def test_constant_of_an_inner_product_is_pulled_out(on_oracle):
    # d * (c * e) with d not a constant becomes c * (d * e): the order the reference multiplies in
    x = f32([1, 2, 3], on_oracle)
    (root,) = traced(lambda t, d: Nx.multiply(d, Nx.multiply(1.5, t)), x, f32([4, 5, 6], on_oracle))
    const, inner = root.data.args
    assert const.data.args == [1.5] and inner.data.op == "multiply"
    assert [a.data.op for a in inner.data.args] == ["parameter", "parameter"]


def test_neutral_elements_vanish(on_oracle):
    x = f32([1, 2, 3], on_oracle)
    for fun in (lambda t: Nx.add(t, 0), lambda t: Nx.multiply(1, t), lambda t: Nx.subtract(t, 0.0),
                lambda t: Nx.divide(t, 1), lambda t: Nx.pow(t, 1)):
        (root,) = traced(fun, x)
        assert root.data.op == "parameter"
    (root,) = traced(lambda t: Nx.add(t, Nx.subtract(0, t)), x)
    assert root.data.op == "subtract"
    (root,) = traced(lambda t: Nx.multiply(t, Nx.divide(1, t)), x)
    assert root.data.op == "divide"


def test_operations_on_constants_fold(on_oracle):
    x = f32([1, 2, 3], on_oracle)
    (root,) = traced(lambda t: Nx.multiply(t, Nx.sqrt(Nx.tensor(2.0, type="f32"))), x)
    const = root.data.args[0]
    assert const.data.op == "constant" and const.data.args == [float(np.sqrt(np.float32(2.0)))]  # rounded to f32
    (root,) = traced(lambda t: Nx.add(t, Nx.subtract(1.0, 0.25)), x)
    assert root.data.args[0].data.args == [0.75]
    (root,) = traced(lambda t: Nx.add(t, Nx.as_type(Nx.max(3, 4), "f32")), x)
    assert root.data.args[0].data.args == [4.0]


def test_squeezes_and_broadcasts_collapse(on_oracle):
    x = from_numpy(np.zeros((1, 3, 1, 4), dtype=np.float32), "f32", on_oracle)
    (root,) = traced(lambda t: Nx.squeeze(Nx.squeeze(t, axes=[0]), axes=[1]), x)
    assert root.data.op == "squeeze" and root.data.args[1] == [0, 2] and root.data.args[0].data.op == "parameter"
    v = f32([1, 2, 3], on_oracle)
    (root,) = traced(lambda t: Nx.broadcast(Nx.broadcast(t, (2, 3)), (4, 2, 3)), v)
    assert root.data.op == "broadcast" and root.data.args[0].data.op == "parameter" and root.shape == (4, 2, 3)
    (root,) = traced(lambda t: Nx.add(t, Nx.broadcast(2.0, (3,))), v)
    assert root.data.args[0].data.op == "constant"


def test_captured_compute_tensor_is_refused(on_oracle):
    outside = f32([1, 2, 3], on_oracle)
    with pytest.raises(ValueError, match="incompatible tensor implementations"):
        defn.jit(lambda t: Nx.add(t, outside))(f32([1, 2, 3], on_oracle))


def test_expressions_have_no_value(on_oracle):
    with pytest.raises(ValueError, match="cannot read the value"):
        defn.jit(lambda t: Nx.to_binary(t))(f32([1.0], on_oracle))


# ---- evaluation -----------------------------------------------------------------------------------

def softmax(t):
    z = Nx.multiply(Nx.as_type(t, "f32"), 0.125)
    e = Nx.exp(Nx.subtract(z, Nx.reduce_max(z, axes=[-1], keep_axes=True)))
    return Nx.divide(e, Nx.sum(e, axes=[-1], keep_axes=True))


def elementwise_reduce(x, y):
    return Nx.sum(Nx.exp(Nx.multiply(Nx.add(x, y), 0.5)), axes=[1])


def linear_int8(xq, w, scales):
    return Nx.multiply(Nx.as_type(Nx.dot(xq, [1], w, [1], out_type="s32"), "f32"), scales)


def argmax_take(logits, table):
    return Nx.take(table, Nx.argmax(logits, axis=1, type="u32"))


def build_args(backend):
    rng = np.random.default_rng(7)
    return {
        "softmax": (from_numpy((rng.standard_normal((4, 16, 16)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16), "bf16", backend),),
        "elementwise_reduce": (f32(rng.standard_normal((33, 65)), backend), f32(rng.standard_normal((33, 65)), backend)),
        "linear_int8": (from_numpy(rng.integers(-128, 128, (8, 64), dtype=np.int8), "s8", backend),
                        from_numpy(rng.integers(-128, 128, (48, 64), dtype=np.int8), "s8", backend),
                        f32(rng.uniform(0.01, 0.1, (48,)), backend)),
        "argmax_take": (f32(rng.standard_normal((16, 100)), backend),
                        from_numpy((rng.standard_normal((100, 24)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16), "bf16", backend)),
    }


CHAINS = {"softmax": softmax, "elementwise_reduce": elementwise_reduce, "linear_int8": linear_int8, "argmax_take": argmax_take}


@pytest.mark.parametrize("name", sorted(CHAINS))
def test_jitted_chain_equals_eager(name, on_oracle):
    args = build_args(on_oracle)[name]
    assert_bits_equal(defn.jit(CHAINS[name])(*args), CHAINS[name](*args), name)
    compiled = defn.compile(CHAINS[name], *args)
    assert_bits_equal(compiled(*args), CHAINS[name](*args), f"{name} compiled")
    assert_bits_equal(compiled(*args), CHAINS[name](*args), f"{name} compiled, second call")


def test_composite_arguments_and_results(on_oracle):
    a, b = f32([1, 2, 3], on_oracle), f32([10, 20, 30], on_oracle)
    out = defn.jit(lambda pair, scale: {"sum": Nx.add(pair[0], pair[1]), "scaled": (Nx.multiply(pair[0], scale),)})((a, b), 2.0)
    assert Nx.to_numpy(out["sum"]).tolist() == [11, 22, 33] and Nx.to_numpy(out["scaled"][0]).tolist() == [2, 4, 6]


def test_while_loop(on_oracle):
    def power_iteration(m, v):
        def body(state):
            i, vec = state
            w = Nx.dot(m, vec)
            return Nx.add(i, 1), Nx.divide(w, Nx.sqrt(Nx.sum(Nx.multiply(w, w))))
        _, vec = defn.while_loop((Nx.tensor(0), v), lambda s: Nx.less(s[0], 20), body)
        return vec
    m = f32([[2, 1], [1, 3]], on_oracle)
    v = f32([1, 0], on_oracle)
    assert_bits_equal(defn.jit(power_iteration)(m, v), power_iteration(m, v), "power iteration")


def test_while_reads_the_enclosing_scope_without_consuming_it(on_oracle):
    def fun(x):
        shifted = Nx.add(x, 1.0)  # used inside the loop on every trip and after it
        _, acc = defn.while_loop((Nx.tensor(0), shifted), lambda s: Nx.less(s[0], 3),
                                 lambda s: (Nx.add(s[0], 1), Nx.add(s[1], s[1])))
        return Nx.subtract(acc, shifted)
    x = f32([1, 2], on_oracle)
    assert Nx.to_numpy(defn.jit(fun)(x)).tolist() == [14.0, 21.0]


def test_cond_evaluates_one_branch(on_oracle):
    calls = []

    class Counting(on_oracle):
        @classmethod
        def exp(cls, out, t):
            calls.append("exp")
            return super().exp(out, t)

    def fun(x):
        shared = Nx.multiply(x, 2.0)
        return defn.cond(Nx.greater(Nx.sum(x), 0.0), lambda: Nx.add(shared, 1.0), lambda: Nx.exp(shared))
    x = from_numpy(np.asarray([1, 2], dtype=np.float32), "f32", Counting)
    previous = Nx.default_backend(Counting)
    try:
        assert Nx.to_numpy(defn.jit(fun)(x)).tolist() == [3.0, 5.0]
        assert calls == []
        y = from_numpy(np.asarray([-1, -2], dtype=np.float32), "f32", Counting)
        assert np.allclose(Nx.to_numpy(defn.jit(fun)(y)), np.exp([-2.0, -4.0]))
        assert calls == ["exp"]
    finally:
        Nx.default_backend(*previous)


def test_results_are_dropped_after_their_last_use(on_oracle):
    """Walks a chain and records how many intermediate results the evaluator still holds."""
    held = []
    original = defn._Run.apply

    def spying(self, e, x, scope):
        held.append(len(scope.results))
        return original(self, e, x, scope)
    defn._Run.apply = spying
    try:
        def chain(t):
            for _ in range(10):
                t = Nx.exp(Nx.negate(t))
            return t
        defn.jit(chain)(f32([0.5, 1.5], on_oracle))
    finally:
        defn._Run.apply = original
    assert max(held) <= 1, held  # a straight chain never holds more than the operand in flight


def test_shared_node_is_computed_once(on_oracle):
    calls = []

    class Counting(on_oracle):
        @classmethod
        def exp(cls, out, t):
            calls.append(1)
            return super().exp(out, t)

    def fun(x):
        e = Nx.exp(x)
        return Nx.add(Nx.multiply(e, e), e)
    x = from_numpy(np.asarray([0.0, 1.0], dtype=np.float32), "f32", Counting)
    previous = Nx.default_backend(Counting)
    try:
        defn.jit(fun)(x)
    finally:
        Nx.default_backend(*previous)
    assert len(calls) == 1


# ---- Nx.Random as a traced function -----------------------------------------------------------------

@pytest.mark.parametrize("case", [c for c in CASES if c["fn"] != "key"], ids=[c["name"] for c in CASES if c["fn"] != "key"])
def test_random_known_answers_through_a_trace(case, on_oracle):
    check_random_case(case, on_oracle, through=defn.jit)


# ---- fused groups: the planner (the kernel itself is tested on the device) ---------------------------

def test_fusion_groups_and_their_fallback_on_a_backend_without_the_kernel(on_oracle):
    for name, fun in CHAINS.items():
        args = build_args(on_oracle)[name]
        fused = defn.compile(fun, *args, fuse=True)
        assert_bits_equal(fused(*args), fun(*args), name)
    assert defn.compile(CHAINS["elementwise_reduce"], *build_args(on_oracle)["elementwise_reduce"], fuse=True).fused_groups == 1
    # softmax: max-reduction group, sum-reduction group, final division -- the scaled scores and the
    # exponentials are computed again inside each group instead of being stored
    assert defn.compile(CHAINS["softmax"], *build_args(on_oracle)["softmax"], fuse=True).fused_groups == 3
    assert defn.compile(CHAINS["argmax_take"], *build_args(on_oracle)["argmax_take"], fuse=True).fused_groups == 0


def test_fusion_leaves_shared_and_returned_nodes_alone(on_oracle):
    x = f32(np.linspace(-1, 1, 64), on_oracle)

    def fun(t):
        e = Nx.exp(t)                       # returned and consumed: must stay a node of its own
        return e, Nx.multiply(Nx.add(e, 1.0), 2.0)
    compiled = defn.compile(fun, x, fuse=True)
    e, y = compiled(x)
    assert compiled.roots[0].data.op == "exp" and compiled.roots[1].data.op == "fused"
    assert_bits_equal(e, Nx.exp(x), "returned intermediate")
    assert_bits_equal(y, Nx.multiply(Nx.add(Nx.exp(x), 1.0), 2.0), "group above it")


def test_fusion_is_skipped_when_the_function_has_control_flow(on_oracle):
    x = f32([1.0, 2.0], on_oracle)

    def fun(t):
        doubled = Nx.multiply(Nx.add(t, 1.0), 2.0)
        _, out = defn.while_loop((Nx.tensor(0), doubled), lambda s: Nx.less(s[0], 2), lambda s: (Nx.add(s[0], 1), Nx.add(s[1], doubled)))
        return out
    compiled = defn.compile(fun, x, fuse=True)
    assert compiled.fused_groups == 0
    assert Nx.to_numpy(compiled(x)).tolist() == [12.0, 18.0]


def test_layout_of_a_group(on_oracle):
    assert defn._layout((4, 16), [(4, 16), ()]) == (1, 64, [(0, 1), (0, 0)])
    assert defn._layout((4, 16), [(4, 16), (16,)]) == (4, 16, [(16, 1), (0, 1)])
    assert defn._layout((4, 16), [(4, 16), (4, 1)]) == (4, 16, [(16, 1), (1, 0)])
    assert defn._layout((2, 3, 16), [(2, 3, 16), (2, 3, 1), (16,)]) == (6, 16, [(16, 1), (1, 0), (0, 1)])
    assert defn._layout((5, 7), [(5, 7), (7,)]) is None            # rows are not whole vectors
    assert defn._layout((4, 16), [(4, 16), (4, 1), (1, 16), (2, 1, 16)]) is None


# ---- the quantised linear layer: dot -> as_type -> multiply by the scales becomes one node ---------------

def _roots_ops(compiled):
    return [r.data.op for r in compiled.roots]


def test_scales_after_an_int8_dot_are_absorbed_and_fall_back_without_the_kernel(on_oracle):
    rng = np.random.default_rng(0)
    x = from_numpy(rng.integers(-127, 128, size=(8, 256), dtype=np.int8), "s8", on_oracle)
    w = from_numpy(rng.integers(-127, 128, size=(32, 256), dtype=np.int8), "s8", on_oracle)
    per_column = f32(rng.uniform(1e-3, 1e-2, size=(32,)), on_oracle)
    per_row = f32(rng.uniform(1e-3, 1e-2, size=(8, 1)), on_oracle)

    def layer(xq, wq, sc):
        return Nx.multiply(Nx.as_type(Nx.dot(xq, [1], wq, [1], out_type="s32"), "f32"), sc)

    def layer_scale_first(xq, wq, sc):
        return Nx.multiply(sc, Nx.as_type(Nx.dot(xq, [1], wq, [1], out_type="s32"), "f32"))

    def layer_constant(xq, wq):
        return Nx.multiply(Nx.as_type(Nx.dot(xq, [1], wq, [1], out_type="s32"), "f32"), 0.0078125)

    for fun, args, mode in ((layer, (x, w, per_column), 1), (layer_scale_first, (x, w, per_column), 1),
                            (layer, (x, w, per_row), 2), (layer_constant, (x, w), 3)):
        planned = defn.compile(fun, *args, fuse=True)
        assert _roots_ops(planned) == ["dot_scaled"] and planned.roots[0].data.args[-1] == mode
        # the oracle has no such callback: the evaluator makes the three calls
        assert_bits_equal(planned(*args), fun(*args), f"{fun.__name__} mode {mode}")

    def sum_read_twice(xq, wq, sc):
        d = Nx.dot(xq, [1], wq, [1], out_type="s32")
        return Nx.multiply(Nx.as_type(d, "f32"), sc), d

    assert "dot_scaled" not in _roots_ops(defn.compile(sum_read_twice, x, w, per_column, fuse=True))
    odd = f32(rng.uniform(size=(8, 32)), on_oracle)  # a full matrix of scales is no scale vector
    assert "dot_scaled" not in _roots_ops(defn.compile(layer, x, w, odd, fuse=True))
    assert _roots_ops(defn.compile(layer, x, w, per_column)) == ["multiply"]  # only when fusing is asked for


# ---- groups over the same rows as stages of one program (planned for compiled kernels) -------------------

def test_softmax_is_one_node_with_three_stages_and_falls_back_group_by_group(on_oracle):
    args = build_args(on_oracle)["softmax"]
    planned = defn.compile(CHAINS["softmax"], *args, fuse="compiled")
    cluster = planned.roots[0].data.args[0]
    assert type(cluster).__name__ == "_RowCluster" and cluster.n_stages == 2
    kinds = [ins["kind"] for ins in cluster.program]
    assert kinds.count(6) == 2 and kinds.count(7) == 2 and kinds[-1] not in (6, 7)  # two stages, then the division
    assert [ins["op"] for ins in cluster.program if ins["kind"] == 6] == [1, 0]  # the maximum, then the sum
    assert any(ins.get("src") == 3 for ins in cluster.program)                   # later stages read the row statistics
    assert len(cluster.inputs) == 1                                              # only the scores come from memory
    assert_bits_equal(planned(*args), CHAINS["softmax"](*args), "softmax, group by group on a backend without the kernel")


def test_row_statistics_with_outside_readers_or_another_broadcast_stay_groups(on_oracle):
    x = f32(np.random.default_rng(3).standard_normal((16, 64)), on_oracle)

    def stat_is_returned(t):
        m = Nx.reduce_max(Nx.multiply(t, 2.0), axes=[1], keep_axes=True)
        return Nx.subtract(Nx.multiply(t, 2.0), m), m

    planned = defn.compile(stat_is_returned, x, fuse="compiled")
    assert all(type(r.data.args[0]).__name__ != "_RowCluster" for r in planned.roots if r.data.op == "fused")
    got, want = planned(x), stat_is_returned(x)
    assert_bits_equal(got[0], want[0], "value")
    assert_bits_equal(got[1], want[1], "statistic")

    sq = f32(np.random.default_rng(4).standard_normal((64, 64)), on_oracle)

    def stat_read_along_columns(t):     # {64} against {64, 64}: one value per column, not per row
        m = Nx.reduce_max(Nx.multiply(t, 2.0), axes=[1])
        return Nx.subtract(Nx.multiply(t, 2.0), m)

    planned = defn.compile(stat_read_along_columns, sq, fuse="compiled")
    assert type(planned.roots[0].data.args[0]).__name__ != "_RowCluster"
    assert_bits_equal(planned(sq), stat_read_along_columns(sq), "per column")


def test_statistics_that_are_worked_on_become_part_of_their_stage(on_oracle):
    rng = np.random.default_rng(5)
    x, gain = f32(rng.standard_normal((12, 64)), on_oracle), f32(rng.standard_normal((64,)), on_oracle)

    def layer_norm(t, g):
        n = t.shape[-1]
        mean = Nx.divide(Nx.sum(t, axes=[-1], keep_axes=True), float(n))
        c = Nx.subtract(t, mean)
        var = Nx.divide(Nx.sum(Nx.multiply(c, c), axes=[-1], keep_axes=True), float(n))
        return Nx.multiply(Nx.multiply(c, Nx.rsqrt(Nx.add(var, 1e-5))), g)

    planned = defn.compile(layer_norm, x, gain, fuse="compiled")
    cluster = planned.roots[0].data.args[0]
    assert type(cluster).__name__ == "_RowCluster" and cluster.n_stages == 2
    kinds = [ins["kind"] for ins in cluster.program]
    first_red, first_keep = kinds.index(6), kinds.index(7)
    assert kinds[:first_red] == [0]                       # the mean's stage reduces the tensor as it is
    assert kinds[first_red + 1:first_keep] == [2]         # ... and divides the sum by the row length before keeping it
    second_red, second_keep = kinds.index(6, first_keep), kinds.index(7, first_keep + 1)
    assert kinds[second_red + 1:second_keep] == [2, 2, 1]  # / n, + eps, rsqrt
    assert {t.data.op for t in cluster.inputs} == {"parameter"} and len(cluster.inputs) == 2
    assert_bits_equal(planned(x, gain), layer_norm(x, gain), "layer norm, step by step on a backend without the kernel")

    def log_softmax(t):    # the logarithm of the sum is work on the statistic too
        z = Nx.subtract(t, Nx.reduce_max(t, axes=[-1], keep_axes=True))
        return Nx.subtract(z, Nx.log(Nx.sum(Nx.exp(z), axes=[-1], keep_axes=True)))

    planned = defn.compile(log_softmax, x, fuse="compiled")
    cluster = planned.roots[0].data.args[0]
    assert type(cluster).__name__ == "_RowCluster" and cluster.n_stages == 2
    assert_bits_equal(planned(x), log_softmax(x), "log softmax")


def test_a_per_row_result_is_a_cluster_too(on_oracle):
    x = f32(np.random.default_rng(8).standard_normal((12, 64)), on_oracle)

    def log_sum_exp(t):
        m = Nx.reduce_max(t, axes=[-1], keep_axes=True)
        return Nx.add(Nx.log(Nx.sum(Nx.exp(Nx.subtract(t, m)), axes=[-1], keep_axes=True)), m)

    planned = defn.compile(log_sum_exp, x, fuse="compiled")
    cluster = planned.roots[0].data.args[0]
    assert type(cluster).__name__ == "_RowCluster" and cluster.n_stages == 2
    last = cluster.program[-1]
    assert last["kind"] == 7 and last.get("flags") == 1          # the program ends in the value per row
    assert [ins["kind"] for ins in cluster.program].count(7) == 2
    assert_bits_equal(planned(x), log_sum_exp(x), "log-sum-exp, step by step on a backend without the kernel")

    def mean_and_squeeze(t):  # one stage: the sum and its division; the squeeze stays outside
        return Nx.squeeze(Nx.mean(t, axes=[-1], keep_axes=True), axes=[1])

    planned = defn.compile(mean_and_squeeze, x, fuse="compiled")
    assert_bits_equal(planned(x), mean_and_squeeze(x), "mean")

    def plain_sum(t):         # a lone reduction is left as it is
        return Nx.sum(t, axes=[-1], keep_axes=True)

    assert defn.compile(plain_sum, x, fuse="compiled").roots[0].data.op == "sum"


def test_statistic_taken_without_its_axis_and_given_it_back(on_oracle):
    x = f32(np.random.default_rng(9).standard_normal((12, 64)), on_oracle)

    def softmax_new_axis(t):
        m = Nx.new_axis(Nx.reduce_max(t, axes=[-1]), -1)
        e = Nx.exp(Nx.subtract(t, m))
        return Nx.divide(e, Nx.new_axis(Nx.sum(e, axes=[-1]), -1))

    planned = defn.compile(softmax_new_axis, x, fuse="compiled")
    cluster = planned.roots[0].data.args[0]
    assert type(cluster).__name__ == "_RowCluster" and cluster.n_stages == 2
    assert_bits_equal(planned(x), softmax_new_axis(x), "softmax with new_axis")
