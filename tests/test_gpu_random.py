"""`Nx.Random` on the device: the reference's known answers through the C ABI, and the device
against the oracle on shapes past the doctests.  Bits, integers and uniform floats are integer
and exactly-rounded float work: bit-exact.  Normal samples pass through log and sqrt in f64, where
the device's math library and the host's may differ in the last place: compared within 4 ulp of
the output type there (the known answers are still met bit for bit)."""
import numpy as np
import pytest

from nx_amd import nx as Nx
from nx_amd import random as Random
from random_support import CASES, check_random_case
from support import assert_all_close, assert_bits_equal, seed_of

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("case", CASES, ids=[c["name"] for c in CASES])
def test_device_matches_reference_random_known_answer(case, hip):
    check_random_case(case, hip)


def keys(seed, hip, oracle):
    return Random.key(seed, backend=hip), Random.key(seed, backend=oracle)


@pytest.mark.parametrize("shape", [(), (1,), (7,), (8,), (3, 5), (1001,), (64, 129), (2, 3, 4, 5)])
@pytest.mark.parametrize("bit_width", [8, 16, 32, 64])
def test_random_bits(shape, bit_width, hip, oracle):
    hk, ok = keys(seed_of(shape, bit_width), hip, oracle)
    got = Random.random_bits(hk, shape=shape, bit_width=bit_width)
    assert type(got.data) is hip
    assert_bits_equal(got, Random.random_bits(ok, shape=shape, bit_width=bit_width), f"random_bits {shape} {bit_width}")


@pytest.mark.parametrize("parts", [1, 2, 3, 16, 1000])
def test_split_and_fold_in(parts, hip, oracle):
    hk, ok = keys(parts * 7919, hip, oracle)
    assert_bits_equal(Random.split(hk, parts=parts), Random.split(ok, parts=parts), f"split {parts}")
    data = np.arange(parts * 3, dtype=np.int64).reshape(parts, 3) * 2654435761
    assert_bits_equal(Random.fold_in(hk, Nx.tensor(data, backend=hip)), Random.fold_in(ok, Nx.tensor(data, backend=oracle)),
                      f"fold_in {parts}")


@pytest.mark.parametrize("ty", ["u8", "s8", "u16", "s16", "u32", "s32", "u64", "s64"])
@pytest.mark.parametrize("lo,hi", [(0, 10), (-100, 100), (3, 4), (0, 127)])
def test_randint(ty, lo, hi, hip, oracle):
    if ty.startswith("u") and lo < 0:
        lo, hi = 0, hi - lo
    if hi > 127 and ty.endswith("8") and ty[0] == "s":
        hi = 127
    hk, ok = keys(seed_of(ty, lo, hi), hip, oracle)
    got, hk2 = Random.randint(hk, lo, hi, shape=(37, 11), type=ty)
    want, ok2 = Random.randint(ok, lo, hi, shape=(37, 11), type=ty)
    assert_bits_equal(got, want, f"randint {ty} [{lo}, {hi})")
    assert_bits_equal(hk2, ok2, "randint new key")
    vals = hip.to_numpy(got)
    assert vals.min() >= lo and vals.max() < hi


@pytest.mark.parametrize("ty", ["bf16", "f16", "f32", "f64"])
@pytest.mark.parametrize("lo,hi", [(0.0, 1.0), (-3.5, 12.25), (10, 15)])
def test_uniform(ty, lo, hi, hip, oracle):
    hk, ok = keys(seed_of(ty, lo, hi), hip, oracle)
    got, _ = Random.uniform(hk, lo, hi, shape=(1000, 7), type=ty)
    want, _ = Random.uniform(ok, lo, hi, shape=(1000, 7), type=ty)
    assert_bits_equal(got, want, f"uniform {ty} [{lo}, {hi})")


@pytest.mark.parametrize("ty,ulp", [("bf16", 2.0 ** -8), ("f16", 2.0 ** -11), ("f32", 2.0 ** -24), ("f64", 2.0 ** -53)])
def test_normal(ty, ulp, hip, oracle):
    hk, ok = keys(1337, hip, oracle)
    got, _ = Random.normal(hk, 10, 5, shape=(1000,), type=ty)
    want, _ = Random.normal(ok, 10, 5, shape=(1000,), type=ty)
    assert_all_close(got, want, 4 * ulp, 4 * ulp, f"normal {ty}")
    literal, _ = Random.normal(hk, shape=(512,), type=ty)
    assert_all_close(literal, Random.normal(ok, shape=(512,), type=ty)[0], 4 * ulp, 4 * ulp, f"normal literal {ty}")


def test_moments_of_a_large_sample_stay_on_the_device(hip):
    # nx/test/nx/random_test.exs:259-297: mean and variance of 10000 draws within 10 %
    key = Random.key(1234, backend=hip)
    u = Random.uniform_split(key, 10, 15, shape=(10000,))
    assert type(u.data) is hip
    vals = hip.to_numpy(u).astype(np.float64)
    assert abs(vals.mean() - 12.5) < 0.125 and abs(vals.var() - 25 / 12) < 0.21
    r = hip.to_numpy(Random.randint_split(key, 10, 95, shape=(10000,))).astype(np.float64)
    assert abs(r.mean() - 52.5) < 5.25 and abs(r.var() - 84 * 86 / 12) < 60.2
    n = hip.to_numpy(Random.normal_split(key, 10, 5, shape=(10000,))).astype(np.float64)
    assert abs(n.mean() - 10) < 1 and abs(n.std() - 5) < 0.5


@pytest.mark.parametrize("shape", [(), (1,), (2,), (7,), (8,), (3, 5), (1001,), (64, 129), (1 << 20,), ((1 << 20) + 1,)])
def test_fused_threefry_matches_the_composition(shape, hip):
    key = Random.key(seed_of(shape), backend=hip)
    fused = Random.threefry2x32(key, shape)
    previous = Random.compose_only(True)
    try:
        composed = Random.threefry2x32(key, shape)
    finally:
        Random.compose_only(previous)
    assert_bits_equal(fused, composed, f"threefry2x32 {shape}")


def test_known_answers_hold_through_the_composition_too(hip):
    previous = Random.compose_only(True)
    try:
        for case in CASES:
            check_random_case(case, hip)
    finally:
        Random.compose_only(previous)
