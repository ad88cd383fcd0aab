"""Pins what the transcribed known answers leave open in the CPU oracle, through what the
mathematics fixes: closed forms, an independent library routine, brute force on small inputs and
cases built so that a plausible mistake (wrong fold order, FMA instead of two roundings, rounding
instead of truncation, saturation instead of wrap, a transposed operand) changes the answer."""
import itertools

import numpy as np
import pytest

from nx_amd import nx as Nx
from nx_amd import types as T
from support import from_numpy, raw, values


def t(arr, ty, oracle):
    return from_numpy(np.asarray(arr), ty, oracle)


def test_float_sum_is_a_sequential_f64_fold_from_index_zero(oracle):
    # in f64: (1e16 + 1) + -1e16 = 0 sequentially; any other association gives 1 or 2
    x = np.array([1e16, 1.0, -1e16, 1.0], dtype=np.float64)
    assert values(Nx.sum(t(x, "f64", oracle))).item() == 1.0
    assert values(Nx.sum(t(x[::-1].copy(), "f64", oracle))).item() == 0.0
    # f32 inputs are folded in f64 and rounded once: 2^24 + 1 + 1 = 2^24 + 2 exactly
    y = np.array([16777216.0, 1.0, 1.0], dtype=np.float32)
    assert values(Nx.sum(t(y, "f32", oracle))).item() == 16777218.0
    # along an axis of a 3-d tensor the reduced axes are walked in row-major order
    z = np.zeros((2, 2, 2), dtype=np.float64)
    z[0, :, 0] = [1e16, 1.0]
    z[1, :, 0] = [-1e16, 1.0]
    got = values(Nx.sum(t(z, "f64", oracle), axes=[0, 1]))
    assert got.tolist() == [1.0, 0.0]  # (((1e16 + 1) - 1e16) + 1) in the order [0,0],[0,1],[1,0],[1,1]


def test_dot_steps_multiply_then_add_with_two_roundings(oracle):
    # x*y + acc with an FMA keeps the low bits of the product; two roundings lose them
    a = np.array([[1.0 + 2.0 ** -30, 1.0]], dtype=np.float64)
    b = np.array([[1.0 + 2.0 ** -30], [-1.0]], dtype=np.float64)
    got = values(Nx.dot(t(a, "f64", oracle), t(b, "f64", oracle))).item()
    prod = np.float64(a[0, 0]) * np.float64(b[0, 0])  # rounded product
    assert got == float(prod - 1.0) and got == 2.0 ** -29  # fused would give 2^-29 + 2^-60
    # and the fold is sequential in k from acc = 0
    a = np.array([[1e16, 1.0, -1e16, 1.0]], dtype=np.float64)
    ones = np.ones((4, 1), dtype=np.float64)
    assert values(Nx.dot(t(a, "f64", oracle), t(ones, "f64", oracle))).item() == 1.0


def test_dot_against_exact_integer_arithmetic_and_wrap(oracle):
    rng = np.random.default_rng(0)
    a = rng.integers(-2 ** 31, 2 ** 31, size=(5, 7)).astype(np.int32)
    b = rng.integers(-2 ** 31, 2 ** 31, size=(7, 3)).astype(np.int32)
    exact = np.array([[sum(int(a[i, k]) * int(b[k, j]) for k in range(7)) for j in range(3)] for i in range(5)], dtype=object)
    got = raw(Nx.dot(t(a, "s32", oracle), t(b, "s32", oracle)))
    want = np.array([[((int(v) + 2 ** 31) % 2 ** 32) - 2 ** 31 for v in row] for row in exact], dtype=np.int64)
    assert np.array_equal(got.astype(np.int64), want)
    s8a = rng.integers(-128, 128, size=(4, 300)).astype(np.int8)
    s8b = rng.integers(-128, 128, size=(300, 4)).astype(np.int8)
    wrapped = (s8a.astype(np.int64) @ s8b.astype(np.int64)).astype(np.int8)  # public API type: s8, wraps
    assert np.array_equal(raw(Nx.dot(t(s8a, "s8", oracle), t(s8b, "s8", oracle))), wrapped)


def test_dot_against_an_independent_library_routine(oracle):
    rng = np.random.default_rng(1)
    a, b = rng.standard_normal((33, 129)), rng.standard_normal((129, 17))
    got = values(Nx.dot(t(a, "f64", oracle), t(b, "f64", oracle)))
    np.testing.assert_allclose(got, a @ b, rtol=0, atol=1e-13 * 129 * 4)
    # contraction axes are paired in the given order; a transposed operand would change this
    x, y = rng.standard_normal((3, 4, 5)), rng.standard_normal((5, 2, 4))
    got = values(Nx.dot(t(x, "f64", oracle), [2, 1], t(y, "f64", oracle), [0, 2]))
    np.testing.assert_allclose(got, np.einsum("ajk,kbj->ab", x, y), atol=1e-12)
    # batched: batch axes lead the output, then left-kept, then right-kept
    p, q = rng.standard_normal((3, 2, 4)), rng.standard_normal((3, 4, 5))
    got = values(Nx.dot(t(p, "f64", oracle), [2], [0], t(q, "f64", oracle), [1], [0]))
    np.testing.assert_allclose(got, np.einsum("bik,bkj->bij", p, q), atol=1e-12)


def test_bf16_encode_truncates_and_decode_is_exact(oracle):
    # every f32 with low bits set truncates toward zero; round-to-nearest would bump 0x3F80FFFF up
    bits = np.array([0x3F80FFFF, 0x3F808000, 0xBF80FFFF, 0x3E4CCCCD, 0x00010000, 0x7F7FFFFF], dtype=np.uint32)
    got = raw(Nx.as_type(t(bits.view(np.float32), "f32", oracle), "bf16"))
    assert got.tolist() == [0x3F80, 0x3F80, 0xBF80, 0x3E4C, 0x0001, 0x7F7F]
    back = raw(Nx.as_type(t(got, "bf16", oracle), "f32")).view(np.uint32)
    assert back.tolist() == [int(b) << 16 for b in got]
    # an f64 is first rounded to f32 (nearest even), then truncated: 1 + 2^-24 + 2^-40 rounds up in f32
    x = np.array([1.0 + 2.0 ** -24 + 2.0 ** -40], dtype=np.float64)
    assert raw(Nx.as_type(t(x, "f64", oracle), "f32")).view(np.uint32)[0] == 0x3F800001
    assert raw(Nx.as_type(t(x, "f64", oracle), "bf16"))[0] == 0x3F80


def test_f16_encode_rounds_to_nearest_even_like_the_ieee_library(oracle):
    rng = np.random.default_rng(2)
    x = np.concatenate([rng.uniform(-70000, 70000, 4000), rng.uniform(-1e-4, 1e-4, 4000), [65504.0, 65519.9, 2.0 ** -24, 2.0 ** -25, 1.0 + 2.0 ** -11]])
    x = x[np.abs(x) < 65520]  # beyond: the reference raises
    got = raw(Nx.as_type(t(x, "f64", oracle), "f16"))
    assert np.array_equal(got.view(np.uint16), x.astype(np.float16).view(np.uint16))


def test_float_to_integer_truncates_then_wraps_brute_force(oracle):
    vals = [0.0, 0.99, -0.99, 1.5, -1.5, 127.9, 128.0, 255.5, 256.0, -128.9, -129.0, 300.7, -300.7, 65535.9, 65536.0,
            2147483648.0, -2147483649.0, 4294967296.0, 1e10, -1e10, 2.0 ** 63, 2.0 ** 64, 2.0 ** 64 + 2.0 ** 12, 1e19, -1e19]
    x = np.array(vals, dtype=np.float64)
    for ty in ("u8", "s8", "u16", "s16", "u32", "s32", "u64", "s64"):
        bits = T.normalize(ty)[1]
        want = []
        for v in vals:
            i = int(v) & ((1 << bits) - 1)  # Python int(): truncation toward zero, unbounded
            if ty[0] == "s" and i >= 1 << (bits - 1):
                i -= 1 << bits
            want.append(i)
        got = raw(Nx.as_type(t(x, "f64", oracle), ty))
        assert [int(g) for g in got] == want, ty


def test_integer_ops_wrap_and_follow_erlang_division(oracle):
    a = np.array([127, -128, 100, -100, 7, -7], dtype=np.int8)
    b = np.array([1, -1, 100, 100, 2, 2], dtype=np.int8)
    A, B = t(a, "s8", oracle), t(b, "s8", oracle)
    assert raw(Nx.add(A, B)).tolist() == [-128, 127, -56, 0, 9, -5]
    assert raw(Nx.multiply(A, B)).tolist() == [127, -128, 16, -16, 14, -14]
    assert raw(Nx.quotient(A, B)).tolist() == [127, -128, 1, -1, 3, -3]      # div/2 truncates; -128/-1 wraps
    assert raw(Nx.remainder(A, B)).tolist() == [0, 0, 0, 0, 1, -1]            # rem/2: sign of the dividend
    assert raw(Nx.left_shift(A, t(np.array([1, 1, 9, 2, 70, 0], dtype=np.int8), "s8", oracle))).tolist() == [-2, 0, 0, 112, 0, -7]
    assert raw(Nx.right_shift(A, t(np.array([1, 1, 9, 2, 70, 0], dtype=np.int8), "s8", oracle))).tolist() == [63, -64, 0, -25, 0, -7]
    assert raw(Nx.pow(t(np.array([3, -2, 2], dtype=np.int8), "s8", oracle), t(np.array([5, 7, 9], dtype=np.int8), "s8", oracle))).tolist() == [-13, -128, 0]
    assert raw(Nx.abs(t(np.array([-128, -5], dtype=np.int8), "s8", oracle))).tolist() == [-128, 5]
    u = t(np.array([0, 1, 0x80, 0xFF], dtype=np.uint8), "u8", oracle)
    assert raw(Nx.count_leading_zeros(u)).tolist() == [8, 7, 0, 0] and raw(Nx.population_count(u)).tolist() == [0, 1, 1, 8]
    assert raw(Nx.bitwise_not(u)).tolist() == [255, 254, 127, 0]


def test_comparisons_and_extrema_with_non_finites(oracle):
    inf, nan = np.inf, np.nan
    x = t(np.array([nan, inf, -inf, 1.0, nan, inf], dtype=np.float32), "f32", oracle)
    y = t(np.array([1.0, inf, inf, nan, nan, 1.0], dtype=np.float32), "f32", oracle)
    assert raw(Nx.equal(x, y)).tolist() == [0, 1, 0, 0, 0, 0]
    assert raw(Nx.not_equal(x, y)).tolist() == [1, 0, 1, 1, 1, 1]
    assert raw(Nx.greater_equal(x, y)).tolist() == [0, 1, 0, 0, 0, 1]
    assert raw(Nx.less(x, y)).tolist() == [0, 0, 1, 0, 0, 0]
    mx = raw(Nx.max(x, y)).view(np.uint32).tolist()
    assert mx == [0x7FC00000, 0x7F800000, 0x7F800000, 0x7FC00000, 0x7FC00000, 0x7F800000]
    assert raw(Nx.logical_and(x, y)).tolist() == [1, 1, 1, 1, 1, 1]  # NaN is truthy: only zero is false


def test_round_is_half_away_from_zero_and_sign_keeps_signed_zero(oracle):
    x = t(np.array([0.5, -0.5, 1.5, 2.5, -2.5, 0.49999997], dtype=np.float32), "f32", oracle)
    assert values(Nx.round(x)).tolist() == [1.0, -1.0, 2.0, 3.0, -3.0, 0.0]
    s = raw(Nx.sign(t(np.array([-3.0, 0.0, -0.0, 9.0], dtype=np.float32), "f32", oracle))).view(np.uint32).tolist()
    assert s == [0xBF800000, 0x00000000, 0x80000000, 0x3F800000]


def test_formula_defined_functions_keep_the_reference_cancellation(oracle):
    # expm1 = exp(x) - 1 and log1p = log(x + 1) evaluated in f64, not the accurate libm variants
    x = np.array([1e-10, 3e-9], dtype=np.float64)
    assert values(Nx.expm1(t(x, "f64", oracle))).tolist() == (np.exp(x) - 1.0).tolist()
    assert values(Nx.log1p(t(x, "f64", oracle))).tolist() == np.log(x + 1.0).tolist()
    assert values(Nx.expm1(t(x, "f64", oracle))).tolist() != np.expm1(x).tolist()
    y = np.array([-3.0, 0.0, 2.0], dtype=np.float64)
    assert values(Nx.sigmoid(t(y, "f64", oracle))).tolist() == (1.0 / (np.exp(-y) + 1.0)).tolist()
    assert values(Nx.rsqrt(t(np.array([2.0]), "f64", oracle))).item() == 1.0 / np.sqrt(2.0)


def test_argmax_brute_force_over_all_small_inputs(oracle):
    alphabet = [-1.0, 0.0, 2.0, np.nan, np.inf, -np.inf]
    for row in itertools.product(alphabet, repeat=4):
        x = np.array(row, dtype=np.float32)
        for op, better in (("argmax", lambda a, b: a > b), ("argmin", lambda a, b: a < b)):
            for tie in ("low", "high"):
                cur, idx = None, -1
                for i, v in enumerate(row):  # the reference's scan, restated independently
                    take = cur is None or v != v or (cur == cur and (better(v, cur) or (tie == "high" and v == cur)))
                    if take:
                        cur, idx = v, i
                got = raw(getattr(Nx, op)(t(x, "f32", oracle), tie_break=tie)).item()
                assert got == idx, (row, op, tie)


def test_transpose_broadcast_gather_against_numpy(oracle):
    rng = np.random.default_rng(4)
    x = rng.integers(0, 1000, size=(3, 4, 5, 2)).astype(np.int32)
    for perm in itertools.permutations(range(4)):
        assert np.array_equal(raw(Nx.transpose(t(x, "s32", oracle), list(perm))), x.transpose(perm))
    v = rng.integers(0, 9, size=(4, 1)).astype(np.int32)
    assert np.array_equal(raw(Nx.broadcast(t(v, "s32", oracle), (3, 4, 6))), np.broadcast_to(v, (3, 4, 6)))
    assert np.array_equal(raw(Nx.broadcast(t(v[:, 0], "s32", oracle), (4, 3), axes=[0])), np.broadcast_to(v, (4, 3)))
    idx = np.stack([rng.integers(0, 3, size=11), rng.integers(0, 5, size=11)], axis=-1).astype(np.int32)
    got = raw(Nx.gather(t(x, "s32", oracle), t(idx, "s32", oracle), axes=[0, 2]))
    assert np.array_equal(got, np.stack([x[i, :, j, :] for i, j in idx]))
    ti = rng.integers(0, 5, size=(2, 3)).astype(np.int32)
    assert np.array_equal(raw(Nx.take(t(x, "s32", oracle), t(ti, "s32", oracle), axis=2)), np.take(x, ti, axis=2))


def test_mixed_integer_float_operands_promote_like_erlang(oracle):
    # int + float: the integer is converted to f64 exactly, the sum rounds to the f32 output once
    i = t(np.array([16777217, 3], dtype=np.int32), "s32", oracle)
    f = t(np.array([1.0, 0.5], dtype=np.float32), "f32", oracle)
    out = Nx.add(i, f)
    assert out.type == ("f", 32) and values(out).tolist() == [16777218.0, 3.5]
    d = Nx.divide(t(np.array([1, 2], dtype=np.int32), "s32", oracle), t(np.array([3, 3], dtype=np.int32), "s32", oracle))
    assert d.type == ("f", 32) and raw(d).tolist() == [np.float32(1 / 3), np.float32(2 / 3)]


def test_f16_codec_against_the_reference_table_of_shortest_decimals(oracle):
    """nx/test/fixtures/f16_table.txt (sampled, tests/golden/make_f16_sample.py) gives each f16 bit pattern
    the shortest decimal that reads back as it: encoding that decimal must give the pattern, and
    decoding the pattern must give the f16 nearest to the decimal -- on the oracle's own codec."""
    import os
    path = os.path.join(os.path.dirname(__file__), "golden", "f16_shortest_decimals_sample.txt")
    bits, text = zip(*(line.strip().split(":") for line in open(path) if line.strip()))
    bits = np.array([int(b, 16) for b in bits], dtype=np.uint16)
    finite = np.array([t not in ("NaN", "-NaN", "Infinity", "-Infinity") for t in text])
    decimals = np.array([float(t) if ok else 0.0 for t, ok in zip(text, finite)], dtype=np.float64)
    # encode: the decimal, held as f64, written as f16 (binary_backend.ex:2031-2076 through the write path)
    as_f64 = from_numpy(decimals[finite], "f64", oracle)
    encoded = np.frombuffer(Nx.to_binary(Nx.as_type(as_f64, "f16")), dtype=np.uint16)
    assert np.array_equal(encoded, bits[finite])
    # decode: the pattern read as a number is the f16 value (and that value is what the decimal encodes to, above)
    as_f16 = from_numpy(bits.view(np.float16), "f16", oracle)
    decoded = np.frombuffer(Nx.to_binary(Nx.as_type(as_f16, "f64")), dtype=np.float64)
    assert np.array_equal(decoded[finite], bits[finite].view(np.float16).astype(np.float64))
    for t, d in zip(np.array(text)[~finite], decoded[~finite]):
        assert (np.isnan(d) and "NaN" in t) or (np.isinf(d) and (d < 0) == t.startswith("-"))


def test_product_wraps_exact_integers_and_rounds_a_float_fold_once(oracle):
    """`product` (nx/lib/nx/binary_backend.ex:1327-1335): fold `acc = x * acc` from integer 1 over unbounded
    integers / f64 in row-major order of the reduced axes, encoded once to the aggregate type."""
    import math
    # s32 operands whose exact product exceeds 2^31: the low 32 bits of the unbounded product (no saturation,
    # no early wrap that a narrower intermediate would show differently for a later zero-crossing factor)
    x = np.array([65537, 65539, -3, 7, 11], dtype=np.int32)
    exact = math.prod(int(v) for v in x)
    want = ((exact + 2 ** 31) % 2 ** 32) - 2 ** 31
    assert abs(exact) > 2 ** 31
    assert raw(Nx.product(t(x, "s32", oracle))).item() == want
    # u8 -> u32: 255^5 wraps modulo 2^32, it does not saturate
    u = np.full(5, 255, dtype=np.uint8)
    assert raw(Nx.product(t(u, "u8", oracle))).item() == 255 ** 5 % 2 ** 32
    # per axis against exact arithmetic, brute force
    rng = np.random.default_rng(12)
    a = rng.integers(-50, 50, size=(3, 4, 5)).astype(np.int32)
    for axis in range(3):
        got = raw(Nx.product(t(a, "s32", oracle), axes=[axis])).astype(np.int64)
        ex = np.empty(got.shape, dtype=object)
        moved = np.moveaxis(a, axis, -1)
        for idx in np.ndindex(*moved.shape[:-1]):
            ex[idx] = ((math.prod(int(v) for v in moved[idx]) + 2 ** 31) % 2 ** 32) - 2 ** 31
        assert np.array_equal(got, ex.astype(np.int64)), axis
    # f32: the fold runs in f64 and is rounded to f32 ONCE: factors of 1 + 2^-12 keep bits in f64 that an f32
    # fold loses (the f32 fold of these forty factors ends one f32 ulp below the f64 one)
    f = np.full(40, 1.0 + 2.0 ** -12, dtype=np.float32)
    acc64 = 1.0
    acc32 = np.float32(1.0)
    for v in f:
        acc64 = float(v) * acc64
        acc32 = np.float32(v) * acc32
    want32 = np.float32(acc64)
    assert want32 != acc32  # the case separates the two formulations
    assert raw(Nx.product(t(f, "f32", oracle))).item() == want32
    # sequential from index zero: 1e-200 * 1e-200 underflows to 0 first and stays 0; the reverse order never
    # leaves the f64 range (1e300 * 1e-200 = 1e100, then * 1e-200)
    g = np.array([1e-200, 1e-200, 1e300], dtype=np.float64)
    assert values(Nx.product(t(g, "f64", oracle))).item() == 0.0
    assert values(Nx.product(t(g[::-1].copy(), "f64", oracle))).item() == (1e300 * 1e-200) * 1e-200
