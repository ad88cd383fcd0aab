"""Counter-based pseudo-random numbers: the host-side mirror of `Nx.Random`
(reference: nx/lib/nx/random.ex).

Every function is the reference's composition of front-end calls, in the same order and with the
same operand types, so the bits are the reference's on whichever backend the key lives: a key on
the device keeps the whole computation there (u32 add / xor / shift / or, iota, concatenate,
slice, as_type, bitcast are all native callbacks).  The one exception is an optimisation: the cipher
over a counter range is wrapped in a block (`Nx.BlockThreefry`), which the device backend answers
with the same words from one kernel instead of about 110 launches.  Keys are `u32[2]` tensors; functions are pure
and return `(sample, new_key)` like the reference, the `*_split` variants take a key that has
already been split.  Complex types and `shuffle`, `choice`, `gumbel`, `multivariate_normal` are
not mirrored.
"""
from __future__ import annotations

import struct
from math import prod

from . import nx as Nx
from . import types as T
from .tensor import Tensor, template

NBITS = 32
_COMPOSE_ONLY = [False]


def compose_only(flag: bool) -> bool:
    """Forces threefry2x32 through the reference's composition of callbacks even when the key's
    backend offers the words in one step (tests compare the two); returns the previous setting."""
    previous, _COMPOSE_ONLY[0] = _COMPOSE_ONLY[0], bool(flag)
    return previous

_MANTISSA = {("bf", 16): 7, ("f", 16): 10, ("f", 32): 23, ("f", 64): 52}
# Threefry-2x32 rotation schedule, two groups of four rounds (random.ex:216)
_ROTATIONS = ((13, 15, 26, 6), (17, 29, 16, 24))


def _u64(value: int, like=None) -> Tensor:
    """Nx.u64/1 of an integer, placed beside `like` when that is a tensor (constants of a jitted
    function live where its arguments live)."""
    backend = type(like.data) if isinstance(like, Tensor) else None
    t = Nx.from_binary(struct.pack("<Q", value & 0xFFFFFFFFFFFFFFFF), "u64", backend=backend)
    return Nx.reshape(t, ())


def _at(t: Tensor, i: int) -> Tensor:
    """t[i] (Access on the first axis): slice of length one, squeezed."""
    return Nx.squeeze(Nx.slice_along_axis(t, i, 1, axis=0), axes=[0])


def _assert_key(key: Tensor):
    # random.ex:1163-1183
    if key.shape != (2,):
        raise ValueError(f"expected key to have shape {{2}}, got tensor with shape {key.shape!r}")
    if key.type != ("u", 32):
        raise ValueError(f"expected key with 32-bit unsigned integer type, got key with type {key.type!r}")


def key(seed, backend=None) -> Tensor:
    """Nx.Random.key/1 (random.ex:92-119): the high and low words of a 64-bit seed."""
    if isinstance(seed, int):
        seed = _u64(seed)
        if backend is not None:
            seed = Nx.backend_transfer(seed, backend)
    elif isinstance(seed, Tensor) and seed.type == ("s", 64):
        seed = Nx.bitcast(seed, "u64")
    elif not (isinstance(seed, Tensor) and seed.type == ("u", 64)):
        raise ValueError(f"expected seed to be an integer, u64 tensor or s64 tensor, got: {seed!r}")
    k1 = Nx.right_shift(seed, 32)
    k2 = Nx.bitwise_and(seed, _u64(0xFFFFFFFF, seed))
    return Nx.as_type(Nx.stack([k1, k2]), "u32")


def split(key: Tensor, parts: int = 2) -> Tensor:
    """Nx.Random.split/2 (random.ex:148-152): `parts` new keys along a leading axis."""
    _assert_key(key)
    return threefry2x32(key, (parts, 2))


def fold_in(key: Tensor, data) -> Tensor:
    """Nx.Random.fold_in/2 (random.ex:190-208): a new key per element of `data`."""
    _assert_key(key)
    data = Nx.as_type(_beside(data, key), "u64")
    k1 = Nx.right_shift(data, 32)
    k2 = Nx.bitwise_and(data, _u64(0xFFFFFFFF, data))
    xs = Nx.as_type(Nx.reshape(Nx.stack([k1, k2]), (2, "auto")), "u32")
    x1, x2 = _threefry2x32_20_pair(xs, key)
    return Nx.reshape(Nx.stack([x1, x2], axis=-1), data.shape + (2,))


def threefry2x32(key: Tensor, shape) -> Tensor:
    """random.ex:214-229: the block cipher over the counters 0 .. size-1, keyed by `key`; an odd
    count is padded with one zero counter whose output is dropped.  Offered to the key's backend
    as a block; the default is the reference's composition."""
    shape = tuple(shape)
    if _COMPOSE_ONLY[0]:
        return _threefry2x32_composed(key, shape)
    return Nx.block(Nx.BlockThreefry(shape), [key], template(("u", 32), shape),
                    lambda _struct, key_: _threefry2x32_composed(key_, shape))


def _threefry2x32_composed(key: Tensor, shape) -> Tensor:
    size = prod(shape)
    backend = type(key.data)  # the expression builder while a function is traced
    if size % 2 == 0:
        xs = Nx.iota((2, size // 2), type="u32", backend=backend)
        return Nx.reshape(threefry2x32_20_concat(xs, key), shape)
    zero = Nx.from_binary(struct.pack("<I", 0), "u32", backend=backend)
    xs = Nx.reshape(Nx.concatenate([Nx.iota((size,), type="u32", backend=backend), zero]), (2, "auto"))
    bits = threefry2x32_20_concat(xs, key)
    return Nx.reshape(Nx.slice_along_axis(bits, 0, size, axis=0), shape)


def threefry2x32_20_concat(xs: Tensor, ks: Tensor) -> Tensor:
    nx1, nx2 = _threefry2x32_20_pair(xs, ks)  # random.ex:231-234
    return Nx.concatenate([nx1, nx2], axis=0)


def _rotate_left(x, rot: int):
    # random.ex:283-285
    return Nx.bitwise_or(Nx.left_shift(x, rot), Nx.right_shift(x, NBITS - rot))


def _threefry2x32_20_pair(xs: Tensor, ks: Tensor):
    """Twenty rounds in five groups of four (random.ex:236-281): after each group a key word and
    the group number are injected, key words and rotation groups rotate."""
    key1, key2 = _at(ks, 0), _at(ks, 1)
    x1, x2 = Nx.add(_at(xs, 0), key1), Nx.add(_at(xs, 1), key2)
    k1, k2, k3 = key2, Nx.bitwise_xor(Nx.bitwise_xor(key1, key2), 0x1BD11BDA), key1
    r1, r2 = _ROTATIONS
    for i in range(1, 6):
        for rot in r1:
            y1 = Nx.add(x1, x2)
            x1, x2 = y1, Nx.bitwise_xor(_rotate_left(x2, rot), y1)
        x1 = Nx.add(k1, x1)
        x2 = Nx.add(Nx.add(k2, i), x2)
        k1, k2, k3 = k2, k3, k1
        r1, r2 = r2, r1
    return x1, x2


def random_bits(key: Tensor, shape=(), bit_width: int = 32) -> Tensor:
    """random.ex:287-312: unsigned integers of `bit_width` bits."""
    _assert_key(key)
    shape = tuple(shape)
    if bit_width == 64:
        bits = Nx.as_type(threefry2x32(key, (2, prod(shape))), "u64")
        return Nx.reshape(Nx.bitwise_or(Nx.left_shift(_at(bits, 0), 32), _at(bits, 1)), shape)
    if bit_width == 32:
        return threefry2x32(key, shape)
    return Nx.as_type(threefry2x32(key, shape), ("u", bit_width))


def randint(key: Tensor, min_val, max_val, shape=(), type=None):
    """Nx.Random.randint/4 (random.ex:358-361): integers in [min_val, max_val)."""
    keys = split(key)
    return randint_split(_at(keys, 1), min_val, max_val, shape=shape, type=type), _at(keys, 0)


def randint_split(key: Tensor, min_val, max_val, shape=(), type=None) -> Tensor:
    """random.ex:366-408."""
    _assert_key(key)
    shape = tuple(shape)
    ty = T.normalize(type) if type is not None else T.merge(Nx.type_of(min_val), Nx.type_of(max_val))
    if ty[0] not in ("u", "s"):
        raise ValueError(f"expected integer type, got type {ty!r}")
    nbits = ty[1]
    min_val = Nx.broadcast(_beside(min_val, key), shape)
    max_val = Nx.broadcast(_beside(max_val, key), shape)
    bits = random_bits(key, shape=(2,) + shape, bit_width=nbits)
    higher_bits, lower_bits = _at(bits, 0), _at(bits, 1)
    span = Nx.as_type(Nx.subtract(max_val, min_val), ("u", nbits))
    multiplier = Nx.pow(_u64(2, key), _beside(nbits // 2, key))
    multiplier = Nx.remainder(Nx.pow(Nx.remainder(multiplier, span), 2), span)
    offset = Nx.remainder(higher_bits, span)
    offset = Nx.add(Nx.multiply(offset, multiplier), Nx.remainder(lower_bits, span))
    offset = Nx.remainder(offset, span)
    return Nx.reshape(Nx.as_type(Nx.add(min_val, offset), ty), shape)


def uniform(key: Tensor, min_val=0.0, max_val=1.0, shape=(), type=None):
    """Nx.Random.uniform/4 (random.ex:463-466): floats in [min_val, max_val)."""
    keys = split(key)
    return uniform_split(_at(keys, 1), min_val, max_val, shape=shape, type=type), _at(keys, 0)


def _float_type(left, right, type):
    # infer_float_type (random.ex:1152-1158)
    if type is not None:
        ty = T.normalize(type)
    else:
        ty = T.to_floating(T.merge(Nx.type_of(left), Nx.type_of(right)))
    if ty[0] not in ("f", "bf") or ty not in _MANTISSA:
        raise ValueError(f"expected float or complex type, got type {ty!r}")
    return ty


def _beside(value, key: Tensor) -> Tensor:
    """A number or tensor as a tensor on the key's backend."""
    t = Nx.to_tensor(value)
    return t if type(t.data) is type(key.data) else Nx.backend_transfer(t, type(key.data))


def _float_constant(value: float, ty, key: Tensor) -> Tensor:
    return Nx.as_type(_beside(Nx.tensor(float(value), type="f64"), key), ty)


def _as_float(value, ty, key: Tensor) -> Tensor:
    """Nx.as_type(value, ty) as it comes out of a traced function: a plain number is a constant that
    is encoded once, straight into `ty`; a tensor is converted from its own type."""
    if isinstance(value, Tensor):
        return Nx.as_type(_beside(value, key), ty)
    return _float_constant(value, ty, key)


def uniform_split(key: Tensor, min_value=0.0, max_value=1.0, shape=(), type=None) -> Tensor:
    """random.ex:471-493: random mantissa bits under the exponent of 1.0 give [1, 2); shifted and
    scaled into [min, max) and clamped from below."""
    _assert_key(key)
    shape = tuple(shape)
    ty = _float_type(min_value, max_value, type)
    nbits = ty[1]
    one = _float_constant(1.0, ty, key)
    u_one = Nx.bitcast(one, ("u", nbits))
    min_value = _as_float(min_value, ty, key)
    max_value = _as_float(max_value, ty, key)
    shift = Nx.as_type(_beside(nbits - _MANTISSA[ty], key), ("u", nbits))
    bits = random_bits(key, shape=shape, bit_width=nbits)
    floats = Nx.bitcast(Nx.bitwise_or(Nx.right_shift(bits, shift), u_one), ty)
    floats = Nx.subtract(floats, one)
    floats = Nx.add(Nx.multiply(floats, Nx.subtract(max_value, min_value)), min_value)
    return Nx.reshape(Nx.max(floats, min_value), shape)


def _next_after_minus_1(ty) -> float:
    """The float of type `ty` just above -1 (random.ex:1114-1124)."""
    bits = ty[1]
    if ty == ("bf", 16):
        return struct.unpack("<f", struct.pack("<I", (0xBF80 - 1) << 16))[0]
    fmt_f, fmt_i = {16: ("<e", "<H"), 32: ("<f", "<I"), 64: ("<d", "<Q")}[bits]
    x = struct.unpack(fmt_i, struct.pack(fmt_f, -1.0))[0]
    return struct.unpack(fmt_f, struct.pack(fmt_i, x - 1))[0]


def normal(key: Tensor, mean=None, standard_deviation=None, shape=(), type=None):
    """Nx.Random.normal/2,4 (random.ex:498-500, 558-561)."""
    keys = split(key)
    return normal_split(_at(keys, 1), mean, standard_deviation, shape=shape, type=type), _at(keys, 0)


def normal_split(key: Tensor, mean=None, standard_deviation=None, shape=(), type=None) -> Tensor:
    """random.ex:566-580: mean + standard_deviation * sqrt(2) * erf_inv(u), u uniform in (-1, 1).

    The reference is a traced function, and the expression builder reorders products with a
    constant factor (nx/lib/nx/defn/expr.ex:935-960, 1597-1621): sqrt(2) is folded to a constant of
    the output type, and `deviation * (sqrt2 * e)` becomes `sqrt2 * (deviation * e)` when the
    deviation is an argument.  Float products do not associate, so the order is followed here.
    With the defaults (mean 0.0 and deviation 1.0 are literals in the reference's two-argument
    form) the factor 1 and the term 0 are dropped by the builder altogether."""
    _assert_key(key)
    literal = mean is None and standard_deviation is None
    mean = 0.0 if mean is None else mean
    standard_deviation = 1.0 if standard_deviation is None else standard_deviation
    ty = _float_type(mean, standard_deviation, type)
    u = uniform_split(key, _next_after_minus_1(ty), 1, shape=shape, type=ty)
    sqrt2 = Nx.sqrt(_float_constant(2, ty, key))
    e = Nx.erf_inv(u)
    if literal:
        return Nx.multiply(sqrt2, e)
    scaled = Nx.multiply(sqrt2, Nx.multiply(_as_float(standard_deviation, ty, key), e))
    return Nx.add(scaled, _as_float(mean, ty, key))
