"""bf16 results of as_type and dot under the two encodings: truncation (Nx.BinaryBackend,
nx/lib/nx/shared.ex:136-152; the default and the oracle's) and round-to-nearest-even (what Torchx and
EXLA produce: torchx/test/torchx/nx_test.exs:380-394 expects 1/5 -> 0.2001953125)."""
import numpy as np
import pytest

from nx_amd import backend as B
from nx_amd import nx as Nx

pytestmark = pytest.mark.gpu


def bf16_rne_bits(x32: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even of f32 values to bf16 bit patterns, by integer arithmetic on the bits."""
    b = np.ascontiguousarray(x32, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = ((b + 0x7FFF + ((b >> 16) & 1)) >> 16).astype(np.uint16)
    return np.where(np.isnan(x32), np.uint16(0x7FC0), r)


@pytest.fixture
def nearest_even():
    previous = B.bf16_rounding("nearest_even")
    yield
    B.bf16_rounding(previous)


def bits(t):
    return np.frombuffer(Nx.to_binary(t), dtype=np.uint16)


def test_one_fifth_truncates_by_default(hip):
    t = Nx.as_type(Nx.tensor(np.array([0.2], dtype=np.float32), backend=hip), ("bf", 16))
    assert bits(t).tolist() == [0x3E4C]  # 0.19921875


def test_one_fifth_rounds_to_nearest(hip, nearest_even):
    # the value Torchx's own test expects for 1 / 5 in bf16
    t = Nx.as_type(Nx.tensor(np.array([0.2], dtype=np.float32), backend=hip), ("bf", 16))
    assert bits(t).tolist() == [0x3E4D]  # 0.2001953125
    assert Nx.to_flat_list(t) == [0.2001953125]


def test_as_type_f32_grid(hip, nearest_even):
    rng = np.random.default_rng(5)
    x = np.concatenate([
        rng.standard_normal(4099).astype(np.float32) * np.float32(10.0) ** rng.integers(-30, 30, 4099).astype(np.float32),
        # ties (low half exactly 0x8000) on even and odd kept bits, the carry into the exponent, the largest
        # finite value (rounds to infinity), subnormals, signed zeros, infinities, NaN
        np.array([0x3F808000, 0x3F818000, 0x3FFF8000, 0x3FFFFFFF, 0x7F7FFFFF, 0x7F7F7FFF, 0x00008000, 0x00018000,
                  0x00000001, 0x80000000, 0x00000000, 0x7F800000, 0xFF800000, 0x7FC00000, 0x7F800001],
                 dtype=np.uint32).view(np.float32)])
    got = bits(Nx.as_type(Nx.tensor(x, backend=hip), ("bf", 16)))
    assert np.array_equal(got, bf16_rne_bits(x))


def test_as_type_f64_rounds_once(hip, nearest_even):
    # 1 + 2^-8 + 2^-40 lies just above the tie between 1.0 and 1 + 2^-7: rounding to f32 first would land on
    # the tie and then on the even neighbour 1.0
    x = np.array([1.0 + 2.0 ** -8 + 2.0 ** -40, 1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, -0.2, 1e39, 6.0e-41])
    got = bits(Nx.as_type(Nx.tensor(x, backend=hip), ("bf", 16)))
    assert got.tolist() == [0x3F81, 0x3F80, 0x3F82, 0xBE4D, 0x7F80, 0x0001]


def test_as_type_integers(hip, nearest_even):
    x = np.array([257, 258, 259, -257, 65535, 0], dtype=np.int32)
    got = bits(Nx.as_type(Nx.tensor(x, backend=hip), ("bf", 16)))
    assert np.array_equal(got, bf16_rne_bits(x.astype(np.float32)))


@pytest.mark.parametrize("m,n,k", [(256, 256, 256), (512, 768, 128), (16, 4096, 4096), (48, 40, 64), (5, 7, 3)])
def test_dot_bf16_result_rounds_the_f32_accumulator(hip, nearest_even, m, n, k):
    # the same operands with an f32 result give the accumulator; the bf16 result must be its rounding
    rng = np.random.default_rng(m + n + k)
    a = Nx.as_type(Nx.tensor(rng.standard_normal((m, k)).astype(np.float32), backend=hip), ("bf", 16))
    b = Nx.as_type(Nx.tensor(rng.standard_normal((k, n)).astype(np.float32), backend=hip), ("bf", 16))
    wide = np.frombuffer(Nx.to_binary(Nx.dot(Nx.as_type(a, ("f", 32)), Nx.as_type(b, ("f", 32)))), dtype=np.float32)
    got = bits(Nx.dot(a, b))
    # the two kernels add the same exact products in f32 in different orders: the bf16 result lies within half a
    # bf16 step of the f32 one, plus that noise; truncation would be off by up to a whole step
    dec = (got.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    step = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(wide.astype(np.float64)), 1e-30))) - 7)
    assert np.all(np.abs(dec - wide) <= 0.5 * step + 1e-5 * np.sqrt(k))
    B.bf16_rounding("truncate")
    trunc = bits(Nx.dot(a, b))
    B.bf16_rounding("nearest_even")
    # against the truncated result of the very same kernel: never below it, at most one step above, and
    # above it for about half of the elements
    up = got.astype(np.int32) - trunc.astype(np.int32)
    assert up.min() >= 0 and up.max() <= 1
    if m * n >= 1024:
        assert 0.3 < up.mean() < 0.7


def test_element_wise_results_keep_truncation(hip, nearest_even):
    a = Nx.tensor([0.1], type=("bf", 16), backend=hip)
    previous = B.bf16_rounding("truncate")
    want = bits(Nx.add(a, a))
    B.bf16_rounding(previous)
    assert np.array_equal(bits(Nx.add(a, a)), want)
