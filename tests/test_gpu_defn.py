"""Traced functions evaluated on the device: the callers one step above the callbacks
(nx/lib/nx/defn/evaluator.ex:363-388).  The device runs the traced function, the oracle runs the
same function eagerly and traced; exact ops are compared bit for bit, transcendental chains within
the tolerances of the per-op tests."""
import numpy as np
import pytest

from nx_amd import defn
from nx_amd import nx as Nx
from nx_amd import random as Random
from nx_amd.backend import mem_stats
from random_support import CASES, check_random_case
from support import assert_all_close, assert_bits_equal, from_numpy
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
