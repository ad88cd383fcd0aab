"""The tensor struct and host-side number <-> binary codecs.

`Tensor` mirrors `%Nx.Tensor{data, type, shape, names}` (reference: nx/lib/nx/tensor.ex:41-42):
`data` holds a backend struct, everything else is metadata owned by the front end.  A backend
fills `out.data` and never changes type / shape / names (nx/lib/nx/backend.ex:5-8).
"""
from __future__ import annotations

import math
import struct
from dataclasses import dataclass
from typing import Any, Optional, Tuple

import numpy as np

from . import types as T


@dataclass(frozen=True)
class Tensor:
    data: Any
    type: Tuple[str, int]
    shape: Tuple[int, ...]
    names: Tuple[Optional[str], ...] = ()

    def __post_init__(self):
        object.__setattr__(self, "type", T.normalize(self.type))
        object.__setattr__(self, "shape", tuple(int(d) for d in self.shape))
        if len(self.names) != len(self.shape):
            object.__setattr__(self, "names", (None,) * len(self.shape))

    @property
    def size(self) -> int:
        return math.prod(self.shape)

    @property
    def rank(self) -> int:
        return len(self.shape)

    def with_(self, **kw) -> "Tensor":
        """A copy with some fields replaced (the hot path of every callback: no re-validation of
        the fields that are carried over)."""
        t = object.__new__(Tensor)
        set_ = object.__setattr__
        set_(t, "data", kw["data"] if "data" in kw else self.data)
        set_(t, "type", T.normalize(kw["type"]) if "type" in kw else self.type)
        if "shape" in kw:
            shape = tuple(int(d) for d in kw["shape"])
            set_(t, "shape", shape)
            names = kw.get("names", ())
            set_(t, "names", tuple(names) if len(names) == len(shape) else (None,) * len(shape))
        else:
            set_(t, "shape", self.shape)
            set_(t, "names", tuple(kw["names"]) if "names" in kw and len(kw["names"]) == len(self.shape) else self.names)
        return t


def template(type, shape) -> Tensor:
    """An output template: a tensor without data, as passed as the first callback argument."""
    t = object.__new__(Tensor)  # (the hot path of every front-end call: no dataclass machinery)
    set_ = object.__setattr__
    shape = tuple(shape) if shape.__class__ is not tuple else shape
    set_(t, "data", None)
    set_(t, "type", T.normalize(type))
    set_(t, "shape", shape if all(d.__class__ is int for d in shape) else tuple(int(d) for d in shape))
    set_(t, "names", (None,) * len(shape))
    return t


# ---- number -> binary, following the reference's write path ---------------------------------
# nx/lib/nx/shared.ex:136-194: integers keep the low bits, floats round to nearest even,
# bf16 = the f32 encoding without its low 16 bits; type.ex:128-158 for the non-finite patterns.

_NAN = {16: 0x7E00, 32: 0x7FC00000, 64: 0x7FF8000000000000}


# ---- sub-byte integers: packed in a binary, one byte per element in memory ------------------
# The reference's binary is a bitstring with the first element in the highest bits
# (`<<x::size(4)>>` segments, nx/lib/nx/shared.ex:190-194).  Python has no bitstrings: a packed
# binary whose bit count is not a multiple of eight carries zero bits at the end of its last byte,
# and the element count comes from the tensor's shape.

def pack_sub_byte(values, type) -> bytes:
    """One-per-byte elements (any integer array; only the low bits count) -> packed binary."""
    bits = T.bit_size(type)
    v = np.asarray(values).astype(np.int64).ravel() & ((1 << bits) - 1)
    per = 8 // bits
    pad = (-v.size) % per
    if pad:
        v = np.concatenate([v, np.zeros(pad, dtype=np.int64)])
    v = v.reshape(-1, per)
    out = np.zeros(v.shape[0], dtype=np.int64)
    for k in range(per):
        out |= v[:, k] << (8 - bits * (k + 1))
    return out.astype(np.uint8).tobytes()


def unpack_sub_byte(binary, type, count=None) -> np.ndarray:
    """Packed binary -> one element per byte (int8 sign-extended, or uint8), `count` of them."""
    kind, bits = T.normalize(type)
    per = 8 // bits
    raw = np.frombuffer(binary, dtype=np.uint8).astype(np.int64)
    cols = [(raw >> (8 - bits * (k + 1))) & ((1 << bits) - 1) for k in range(per)]
    v = np.stack(cols, axis=1).ravel()
    if count is not None:
        if count > v.size:
            raise ValueError("binary size is too small for the requested shape")
        v = v[:count]
    if kind == "s":
        v = np.where(v >= (1 << (bits - 1)), v - (1 << bits), v)
        return v.astype(np.int8)
    return v.astype(np.uint8)


def binary_size(type, count: int) -> int:
    """Bytes of the binary of `count` elements (a partly used last byte counts)."""
    return (count * T.bit_size(type) + 7) // 8


def binary_prefix(binary, type, count: int) -> bytes:
    """The binary of the first `count` elements of a binary."""
    if not T.is_sub_byte(type):
        return bytes(binary[: count * T.size_bytes(type)])
    if (count * T.bit_size(type)) % 8 == 0:
        return bytes(binary[: binary_size(type, count)])
    return pack_sub_byte(unpack_sub_byte(binary[: binary_size(type, count)], type, count), type)


def wrap_to_type(values: np.ndarray, type) -> np.ndarray:
    """Low bits of integers as elements of `type`, one per storage element (sub-byte included)."""
    kind, bits = T.normalize(type)
    if not T.is_sub_byte(type):
        return values.astype(T.numpy_dtype(type))
    v = values.astype(np.int64) & ((1 << bits) - 1)
    if kind == "s":
        v = np.where(v >= (1 << (bits - 1)), v - (1 << bits), v)
    return v.astype(T.numpy_dtype(type))


def number_to_binary(number, type) -> bytes:
    kind, bits = T.normalize(type)
    if kind in ("u", "s"):
        if isinstance(number, float):
            if number != number or math.isinf(number):
                raise ValueError(f"cannot encode {number!r} as an integer")
            if number != int(number):
                raise ValueError(f"cannot encode the float {number!r} as an integer type")
            number = int(number)
        if bits < 8:  # a one-element bitstring, zero bits after it
            return bytes([((int(number) & ((1 << bits) - 1)) << (8 - bits))])
        return (int(number) & ((1 << bits) - 1)).to_bytes(bits // 8, "little")
    x = float(number)
    if kind == "bf":
        if x != x:
            return (0x7FC0).to_bytes(2, "little")
        with np.errstate(over="ignore"):
            f = np.float32(x)
        if np.isinf(f) and not math.isinf(x):
            raise OverflowError(f"{number!r} does not fit a 32-bit float")
        return (int(f.view(np.uint32)) >> 16).to_bytes(2, "little")
    if x != x:
        return _NAN[bits].to_bytes(bits // 8, "little")
    if bits == 64:
        return struct.pack("<d", x)
    with np.errstate(over="ignore"):
        v = np.float32(x) if bits == 32 else np.float16(x)
    if np.isinf(v) and not math.isinf(x):
        raise OverflowError(f"{number!r} does not fit a {bits}-bit float")
    return v.tobytes()


def list_to_binary(values, type) -> bytes:
    """Flat list of Python numbers -> binary (Nx.tensor/2's flattening, nx/lib/nx.ex:774-883)."""
    kind, bits = T.normalize(type)
    arr = np.asarray(values)
    if kind in ("u", "s"):
        if arr.dtype.kind == "f":
            raise ValueError("cannot build an integer tensor from floats")
        if bits < 8:
            return pack_sub_byte(arr.astype(np.int64), type)
        if arr.dtype == object:
            return b"".join(number_to_binary(v, type) for v in arr.ravel())
        return arr.astype(np.int64).astype(T.numpy_dtype(type)).tobytes()
    if kind == "bf":
        f = np.asarray(values, dtype=np.float64).astype(np.float32).ravel()
        out = (f.view(np.uint32) >> 16).astype(np.uint16)
        out[np.isnan(f)] = 0x7FC0
        return out.tobytes()
    f = np.asarray(values, dtype=np.float64).astype(T.numpy_dtype(type)).ravel()
    if np.isnan(f).any():
        raw = f.view({16: np.uint16, 32: np.uint32, 64: np.uint64}[bits]).copy()
        raw[np.isnan(f)] = _NAN[bits]
        return raw.tobytes()
    return f.tobytes()


def binary_to_numpy(binary: bytes, type, shape=None) -> np.ndarray:
    """Raw view of a tensor binary; bf16 comes back as uint16 bit patterns, sub-byte integers
    unpacked to one per byte (as many as the shape holds, or as the binary's bytes hold)."""
    if T.is_sub_byte(type):
        arr = unpack_sub_byte(binary, type, math.prod(shape) if shape is not None else None)
        return arr.reshape(shape) if shape is not None else arr
    arr = np.frombuffer(binary, dtype=T.numpy_dtype(type))
    return arr.reshape(shape) if shape is not None else arr


def bf16_bits_to_float32(bits: np.ndarray) -> np.ndarray:
    return (bits.astype(np.uint32) << 16).view(np.float32)


def to_float64(binary: bytes, type, shape=None) -> np.ndarray:
    """Decoded values as float64 (exact for every type but 64-bit integers above 2^53)."""
    raw = binary_to_numpy(binary, type, shape)
    if T.normalize(type) == ("bf", 16):
        return bf16_bits_to_float32(raw).astype(np.float64)
    return raw.astype(np.float64)
