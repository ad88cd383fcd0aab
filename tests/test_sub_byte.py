"""Sub-byte integer tensors off the GPU: the packed binary format against the reference's own
literals, on the storage-only host backend and on the oracle; and the oracle's arithmetic at these
widths against what the mathematics fixes (the low bits of the unbounded result), by brute force
over every pair of values -- the reference holds no arithmetic test at these widths."""
import numpy as np
import pytest

from nx_amd import nx as Nx
from nx_amd import types as T
from nx_amd.host import HostBinary
from nx_amd.tensor import pack_sub_byte, unpack_sub_byte
from sub_byte_support import CASES, SUB_TYPES, check_case, low_bits, value_range


@pytest.mark.parametrize("case", CASES, ids=[f"{c['type']}-{i}" for i, c in enumerate(CASES)])
def test_reference_literals_on_the_host_backend(case):
    if "inspect_has" in case:
        pytest.skip("the storage-only backend has no inspect")
    check_case(case, HostBinary)


@pytest.mark.parametrize("case", CASES, ids=[f"{c['type']}-{i}" for i, c in enumerate(CASES)])
def test_reference_literals_on_the_oracle(case, oracle):
    if "inspect_has" in case:
        pytest.skip("the oracle has no inspect")
    check_case(case, oracle)


@pytest.mark.parametrize("ty", SUB_TYPES)
@pytest.mark.parametrize("n", [1, 2, 3, 4, 5, 7, 8, 9, 64, 1001])
def test_pack_and_unpack_are_inverse(ty, n):
    lo, hi = value_range(ty)
    v = np.random.default_rng(n).integers(lo, hi + 1, size=n)
    packed = pack_sub_byte(v, ty)
    assert len(packed) == (n * int(ty[1:]) + 7) // 8
    assert unpack_sub_byte(packed, ty, n).tolist() == v.tolist()
    # bit by bit: element i sits in bits [i*w, (i+1)*w) counted from the highest bit of the first byte
    w = int(ty[1:])
    bits = "".join(f"{b:08b}" for b in packed)
    assert [int(bits[i * w:(i + 1) * w], 2) for i in range(n)] == [int(x) & ((1 << w) - 1) for x in v]
    assert set(bits[n * w:]) <= {"0"}


def test_type_rules_at_small_widths():
    # Nx.Type.merge/2 and merge_number/2 (type.ex:463-474, 536-546, 694-705)
    assert T.merge("u2", "u4") == ("u", 4) and T.merge("s2", "s4") == ("s", 4)
    assert T.merge("u2", "s2") == ("s", 4) and T.merge("u4", "s4") == ("s", 8) and T.merge("u4", "s2") == ("s", 8)
    assert T.merge("u4", "f32") == ("f", 32) and T.merge("s2", "bf16") == ("bf", 16)
    assert T.merge_number("u2", 1) == ("u", 2) and T.merge_number("u2", 3) == ("u", 8)
    assert T.merge_number("s4", -2) == ("s", 4) and T.merge_number("s4", 5) == ("s", 8)
    assert T.merge_number("u4", -1) == ("s", 8) and T.merge_number("s2", 1.5) == ("f", 32)
    assert T.to_aggregate("u2") == ("u", 32) and T.to_aggregate("s4") == ("s", 32)


INT_OPS = {"add": lambda a, b: a + b, "subtract": lambda a, b: a - b, "multiply": lambda a, b: a * b,
           "bitwise_and": lambda a, b: a & b, "bitwise_or": lambda a, b: a | b, "bitwise_xor": lambda a, b: a ^ b,
           "min": np.minimum, "max": np.maximum}


@pytest.mark.parametrize("ty", SUB_TYPES)
@pytest.mark.parametrize("op", sorted(INT_OPS))
def test_oracle_arithmetic_keeps_the_low_bits(ty, op, oracle):
    lo, hi = value_range(ty)
    vals = np.arange(lo, hi + 1)
    a, b = np.meshgrid(vals, vals, indexing="ij")
    ta, tb = Nx.tensor(a, type=ty, backend=oracle), Nx.tensor(b, type=ty, backend=oracle)
    got = getattr(Nx, op)(ta, tb)
    assert got.type == T.normalize(ty)
    assert np.array_equal(Nx.to_numpy(got), low_bits(INT_OPS[op](a, b), ty))


@pytest.mark.parametrize("ty", SUB_TYPES)
def test_oracle_conversions_and_reductions(ty, oracle):
    lo, hi = value_range(ty)
    vals = np.arange(lo, hi + 1)
    t = Nx.tensor(vals, type=ty, backend=oracle)
    assert Nx.to_flat_list(Nx.as_type(t, "s32")) == vals.tolist()
    assert Nx.to_flat_list(Nx.as_type(t, "f32")) == [float(v) for v in vals]
    assert Nx.to_flat_list(Nx.sum(t)) == [int(vals.sum())] and Nx.sum(t).type[1] == 32
    assert Nx.to_flat_list(Nx.reduce_max(t)) == [hi] and Nx.reduce_max(t).type == T.normalize(ty)
    wide = Nx.tensor(np.arange(-40, 41), type="s32", backend=oracle)
    assert np.array_equal(Nx.to_numpy(Nx.as_type(wide, ty)), low_bits(np.arange(-40, 41), ty))
    f = Nx.tensor([np.inf, -np.inf, np.nan, 9.7, -3.2, 0.5], type="f32", backend=oracle)
    assert Nx.to_flat_list(Nx.as_type(f, ty)) == [hi, lo, 0] + low_bits([9, -3, 0], ty).tolist()
    other = ("s" if ty[0] == "u" else "u") + ty[1:]
    assert np.array_equal(Nx.to_numpy(Nx.bitcast(t, other)), low_bits(vals, other))
    counts = [bin(int(v) & ((1 << int(ty[1:])) - 1)).count("1") for v in vals]  # written at the type's own width
    assert Nx.to_flat_list(Nx.population_count(t)) == low_bits(counts, ty).tolist()
    assert np.array_equal(Nx.to_numpy(Nx.iota((11,), type=ty, backend=oracle)), low_bits(np.arange(11), ty))
    d = Nx.dot(t, t)
    assert d.type == T.normalize(ty) and Nx.to_flat_list(d) == low_bits([int((vals * vals).sum())], ty).tolist()
