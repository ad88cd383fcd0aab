"""Sub-byte integer tensors on the device: the reference's literals, arithmetic against the low bits
of the exact result (every pair of values), and every callback family against the CPU oracle.
Integer and byte work: bit-exact."""
import numpy as np
import pytest

from nx_amd import nx as Nx
from nx_amd import types as T
from sub_byte_support import CASES, SUB_TYPES, check_case, low_bits, value_range
from support import assert_bits_equal, seed_of
from test_sub_byte import INT_OPS

pytestmark = pytest.mark.gpu


def on_both(values, ty, hip, oracle):
    return Nx.tensor(values, type=ty, backend=hip), Nx.tensor(values, type=ty, backend=oracle)


def random_values(ty, shape, *key):
    lo, hi = value_range(ty)
    return np.random.default_rng(seed_of(ty, shape, *key)).integers(lo, hi + 1, size=shape)


@pytest.mark.parametrize("case", CASES, ids=[f"{c['type']}-{i}" for i, c in enumerate(CASES)])
def test_reference_literals(case, hip):
    check_case(case, hip)


@pytest.mark.parametrize("ty", SUB_TYPES)
@pytest.mark.parametrize("n", [1, 3, 15, 16, 17, 1000, 4099])
def test_binary_round_trip_and_limit(ty, n, hip):
    v = random_values(ty, (n,), "round trip")
    t = Nx.tensor(v, type=ty, backend=hip)
    assert Nx.to_numpy(t).tolist() == v.tolist()
    host = Nx.tensor(v, type=ty)
    assert Nx.to_binary(t) == Nx.to_binary(host)
    k = max(n // 2, 1)
    assert Nx.to_binary(t, k) == Nx.to_binary(host, k) == Nx.to_binary(Nx.tensor(v[:k], type=ty))


@pytest.mark.parametrize("ty", SUB_TYPES)
@pytest.mark.parametrize("op", sorted(INT_OPS))
def test_arithmetic_keeps_the_low_bits(ty, op, hip):
    lo, hi = value_range(ty)
    vals = np.arange(lo, hi + 1)
    a, b = np.meshgrid(vals, vals, indexing="ij")
    got = getattr(Nx, op)(Nx.tensor(a, type=ty, backend=hip), Nx.tensor(b, type=ty, backend=hip))
    assert got.type == T.normalize(ty)
    assert np.array_equal(Nx.to_numpy(got), low_bits(INT_OPS[op](a, b), ty))


BINARY = ["add", "subtract", "multiply", "divide", "pow", "remainder", "atan2", "min", "max", "quotient", "bitwise_and",
          "bitwise_or", "bitwise_xor", "left_shift", "right_shift", "equal", "not_equal", "greater", "less",
          "greater_equal", "less_equal", "logical_and", "logical_or", "logical_xor"]


@pytest.mark.parametrize("op", BINARY)
@pytest.mark.parametrize("lt,rt", [("u2", "u2"), ("s4", "s4"), ("u4", "s2"), ("s2", "s32"), ("u4", "f32"), ("s4", "u8")])
def test_binary_against_the_oracle(op, lt, rt, hip, oracle):
    if op in ("bitwise_and", "bitwise_or", "bitwise_xor", "left_shift", "right_shift", "quotient") and "f" in (lt[0], rt[0]):
        pytest.skip("integer-only operation")
    shape = (33, 7)
    a = random_values(lt, shape, op, "l")
    b = random_values(rt, shape, op, "r") if rt in SUB_TYPES else np.random.default_rng(5).integers(1, 4, size=shape)
    if op in ("remainder", "quotient", "divide", "pow", "left_shift", "right_shift"):
        b = np.clip(np.abs(b), 1, value_range(rt)[1] if rt in SUB_TYPES else 3)  # positive in the type itself
    ha, oa = on_both(a, lt, hip, oracle)
    hb, ob = on_both(b, rt, hip, oracle)
    got, want = getattr(Nx, op)(ha, hb), getattr(Nx, op)(oa, ob)
    if op in ("pow", "atan2") and T.is_float(want.type):
        assert got.type == want.type
        np.testing.assert_allclose(Nx.to_float64(got), Nx.to_float64(want), rtol=2e-7)  # libm-class function, f32: 1 ulp
    else:
        assert_bits_equal(got, want, f"{op} {lt} {rt}")


@pytest.mark.parametrize("op", ["negate", "abs", "bitwise_not", "sign", "population_count", "exp", "sqrt", "is_nan", "floor"])
@pytest.mark.parametrize("ty", SUB_TYPES)
def test_unary_against_the_oracle(op, ty, hip, oracle):
    v = random_values(ty, (5, 13), op)
    if op == "sqrt":
        v = np.abs(v)
    h, o = on_both(v, ty, hip, oracle)
    got, want = getattr(Nx, op)(h), getattr(Nx, op)(o)
    if op in ("exp", "sqrt"):
        assert got.type == want.type
        np.testing.assert_allclose(Nx.to_float64(got), Nx.to_float64(want), rtol=2e-7)
    else:
        assert_bits_equal(got, want, f"{op} {ty}")


@pytest.mark.parametrize("ty", SUB_TYPES)
def test_count_leading_zeros_is_refused_like_the_reference(ty, hip):
    with pytest.raises(NotImplementedError):
        Nx.count_leading_zeros(Nx.tensor([1, 0], type=ty, backend=hip))


@pytest.mark.parametrize("ty", SUB_TYPES)
@pytest.mark.parametrize("other", ["u8", "s8", "s32", "u64", "bf16", "f16", "f32", "f64", "u2", "u4", "s2", "s4"])
def test_as_type_both_ways(ty, other, hip, oracle):
    v = random_values(ty, (41,), other)
    h, o = on_both(v, ty, hip, oracle)
    assert_bits_equal(Nx.as_type(h, other), Nx.as_type(o, other), f"{ty} -> {other}")
    if other in SUB_TYPES:
        return
    rng = np.random.default_rng(seed_of(ty, other, "back"))
    w = rng.integers(-300, 300, size=(67,)) if other[0] != "u" else rng.integers(0, 600, size=(67,))
    if T.is_float(T.normalize(other)):
        w = np.concatenate([w / 8.0, [np.inf, -np.inf, np.nan, -0.0, 7.9, -8.9]])
    hw, ow = on_both(w, other, hip, oracle)
    assert_bits_equal(Nx.as_type(hw, ty), Nx.as_type(ow, ty), f"{other} -> {ty}")


@pytest.mark.parametrize("ty", SUB_TYPES)
def test_bitcast_reads_the_same_bits(ty, hip, oracle):
    other = ("s" if ty[0] == "u" else "u") + ty[1:]
    lo, hi = value_range(ty)
    h, o = on_both(np.arange(lo, hi + 1), ty, hip, oracle)
    assert_bits_equal(Nx.bitcast(h, other), Nx.bitcast(o, other), f"bitcast {ty} {other}")
    assert Nx.to_binary(Nx.bitcast(h, other)) == Nx.to_binary(h)


@pytest.mark.parametrize("ty", SUB_TYPES)
def test_reductions_and_arg_reductions(ty, hip, oracle):
    v = random_values(ty, (9, 130), "reduce")
    h, o = on_both(v, ty, hip, oracle)
    for fn, kw in [(Nx.sum, {}), (Nx.sum, {"axes": [1]}), (Nx.product, {"axes": [0]}), (Nx.reduce_max, {"axes": [1]}),
                   (Nx.reduce_min, {"axes": [0], "keep_axes": True}), (Nx.all, {"axes": [1]}), (Nx.any, {})]:
        assert_bits_equal(fn(h, **kw), fn(o, **kw), f"{fn.__name__} {ty} {kw}")
    assert_bits_equal(Nx.argmax(h, axis=1), Nx.argmax(o, axis=1), f"argmax {ty}")
    assert_bits_equal(Nx.argmin(h, axis=0, tie_break="high"), Nx.argmin(o, axis=0, tie_break="high"), f"argmin {ty}")


@pytest.mark.parametrize("lt,rt", [("s4", "s4"), ("u4", "u4"), ("s2", "u2"), ("u4", "s8"), ("s4", "f32"), ("u2", "bf16")])
@pytest.mark.parametrize("m,k,n", [(3, 5, 4), (64, 256, 32), (130, 70, 66)])
def test_dot(lt, rt, m, k, n, hip, oracle):
    a = random_values(lt, (m, k), "dot l", rt)
    b = random_values(rt, (k, n), "dot r", lt) if rt in SUB_TYPES else np.random.default_rng(9).integers(-3, 4, size=(k, n))
    ha, oa = on_both(a, lt, hip, oracle)
    hb, ob = on_both(b, rt, hip, oracle)
    # every product and partial sum is a small integer: exact in every accumulator, so bit-exact for the float outputs too
    assert_bits_equal(Nx.dot(ha, hb), Nx.dot(oa, ob), f"dot {lt} {rt} {m}x{k}x{n}")


@pytest.mark.parametrize("ty", SUB_TYPES)
def test_data_movement(ty, hip, oracle):
    v = random_values(ty, (6, 10, 4), "move")
    h, o = on_both(v, ty, hip, oracle)
    idx_h, idx_o = on_both([4, 0, 5, 5], "s32", hip, oracle)
    checks = [
        (lambda t, i: Nx.transpose(t, [2, 0, 1])), (lambda t, i: Nx.reshape(t, (10, 24))),
        (lambda t, i: Nx.broadcast(Nx.slice(t, [0, 0, 0], [1, 10, 4]), (3, 10, 4))),
        (lambda t, i: Nx.slice(t, [1, 2, 0], [4, 5, 3], strides=[2, 1, 2])), (lambda t, i: Nx.reverse(t, [1])),
        (lambda t, i: Nx.take(t, i, axis=0)), (lambda t, i: Nx.concatenate([t, t], axis=1)),
        (lambda t, i: Nx.stack([t, t], axis=0)), (lambda t, i: Nx.pad(t, Nx.tensor(1, type=ty, backend=type(t.data)), [(1, 0, 0), (0, 2, 1), (0, 0, 0)])),
        (lambda t, i: Nx.select(Nx.greater(t, 0), t, Nx.negate(t))), (lambda t, i: Nx.clip(t, Nx.tensor(0, type=ty, backend=type(t.data)), Nx.tensor(1, type=ty, backend=type(t.data)))),
    ]
    for n, fn in enumerate(checks):
        assert_bits_equal(fn(h, idx_h), fn(o, idx_o), f"{ty} movement #{n}")


@pytest.mark.parametrize("ty", SUB_TYPES)
@pytest.mark.parametrize("shape,axis", [((19,), None), ((5, 9), 1), ((300, 7), 0)])
def test_iota_and_eye_wrap(ty, shape, axis, hip, oracle):
    assert_bits_equal(Nx.iota(shape, type=ty, axis=axis, backend=hip), Nx.iota(shape, type=ty, axis=axis, backend=oracle), "iota")
    if len(shape) == 2:
        assert_bits_equal(Nx.eye(shape, type=ty, backend=hip), Nx.eye(shape, type=ty, backend=oracle), "eye")


@pytest.mark.parametrize("ty", SUB_TYPES)
def test_scalar_operands_and_constants(ty, hip, oracle):
    v = random_values(ty, (23,), "scalars")
    h, o = on_both(v, ty, hip, oracle)
    for number in (1, -1, 3, 0.5):
        assert_bits_equal(Nx.add(h, number), Nx.add(o, number), f"{ty} + {number}")
        assert_bits_equal(Nx.multiply(number, h), Nx.multiply(number, o), f"{number} * {ty}")
