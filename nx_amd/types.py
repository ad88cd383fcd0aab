"""Element types and the type-inference rules of Nx (reference: nx/lib/nx/type.ex).

A type is a tuple ``(kind, bits)`` with kind in {"u", "s", "f", "bf"} -- the Python spelling of
the reference's ``{:u, 8}`` .. ``{:f, 64}`` / ``{:bf, 16}`` (type.ex:27-48).  Complex and f8 types
are outside the device path and are rejected by ``normalize``.

The sub-byte integers u2, u4, s2, s4 are packed only in a tensor's binary (the reference's
bitstring: first element in the highest bits).  In memory -- on the device and in the host
backends -- each element has a byte of its own, sign- or zero-extended, as the reference's device
backends keep them (exla/lib/exla/device_buffer.ex:24-34, torchx/lib/torchx/backend.ex:428-434);
kernels see them as s8 / u8 and the backend wraps results back to the narrow width.
"""
from __future__ import annotations

import numpy as np

# numeric codes shared with include/hipnx.h
U8, U16, U32, U64, S8, S16, S32, S64, F16, BF16, F32, F64 = range(12)

_CODES = {
    ("u", 8): U8, ("u", 16): U16, ("u", 32): U32, ("u", 64): U64,
    ("s", 8): S8, ("s", 16): S16, ("s", 32): S32, ("s", 64): S64,
    ("f", 16): F16, ("bf", 16): BF16, ("f", 32): F32, ("f", 64): F64,
}
_NAMES = {
    "u8": ("u", 8), "u16": ("u", 16), "u32": ("u", 32), "u64": ("u", 64),
    "s8": ("s", 8), "s16": ("s", 16), "s32": ("s", 32), "s64": ("s", 64),
    "f16": ("f", 16), "bf16": ("bf", 16), "f32": ("f", 32), "f64": ("f", 64),
}
_SUB_BYTE = {("u", 2): U8, ("u", 4): U8, ("s", 2): S8, ("s", 4): S8}  # type -> the code kernels see
_NAMES.update({"u2": ("u", 2), "u4": ("u", 4), "s2": ("s", 2), "s4": ("s", 4)})
# bf16 has no numpy dtype: it travels as raw uint16 bit patterns
_NUMPY = {
    ("u", 8): np.uint8, ("u", 16): np.uint16, ("u", 32): np.uint32, ("u", 64): np.uint64,
    ("s", 8): np.int8, ("s", 16): np.int16, ("s", 32): np.int32, ("s", 64): np.int64,
    ("f", 16): np.float16, ("bf", 16): np.uint16, ("f", 32): np.float32, ("f", 64): np.float64,
}


def normalize(t):
    """Nx.Type.normalize!/1 (type.ex:190-230): accepts ("f", 32) or the short atom name "f32"."""
    if t.__class__ is tuple and t in _CODES:  # already normal: the common case
        return t
    if isinstance(t, str):
        if t not in _NAMES:
            raise ValueError(f"invalid numerical type: {t!r}")
        return _NAMES[t]
    t = (t[0], int(t[1]))
    if t not in _CODES and t not in _SUB_BYTE:
        raise ValueError(f"invalid numerical type: {t!r}")
    return t


def is_sub_byte(t) -> bool:
    return t in _SUB_BYTE or (t.__class__ is not tuple and normalize(t) in _SUB_BYTE)


def code(t) -> int:
    """The element type a kernel is told: sub-byte integers are held one per byte."""
    c = _CODES.get(t) if t.__class__ is tuple else None
    if c is not None:
        return c
    t = normalize(t)
    return _CODES[t] if t in _CODES else _SUB_BYTE[t]


def storage(t):
    """The type of a tensor's elements in memory: itself, or s8 / u8 for a sub-byte integer."""
    t = normalize(t)
    return (t[0], 8) if t in _SUB_BYTE else t


def from_code(c: int):
    for k, v in _CODES.items():
        if v == c:
            return k
    raise ValueError(c)


def name(t) -> str:
    t = normalize(t)
    return f"{t[0]}{t[1]}"


def size_bytes(t) -> int:
    """Bytes per element in memory (one for a sub-byte integer; its binary is packed, see bit_size)."""
    return max(normalize(t)[1] // 8, 1)


def bit_size(t) -> int:
    """Bits per element of a tensor's binary (Nx.Type's size; nx.ex:4890-4915 for Nx.bit_size/1)."""
    return normalize(t)[1]


def numpy_dtype(t):
    return np.dtype(_NUMPY[storage(t)])


def is_float(t) -> bool:
    return normalize(t)[0] in ("f", "bf")


def is_integer(t) -> bool:
    return normalize(t)[0] in ("u", "s")


_ORDER = {"u": 0, "s": 1, "bf": 2, "f": 3}


def merge(left, right):
    """Nx.Type.merge/2 (type.ex:463-488)."""
    left, right = normalize(left), normalize(right)
    if left[0] == right[0]:
        return (left[0], max(left[1], right[1]))
    a, b = (left, right) if _ORDER[left[0]] < _ORDER[right[0]] else (right, left)
    if a[0] == "u" and b[0] == "s":
        return ("s", max(min(a[1] * 2, 64), b[1]))
    return b


def _unsigned_size(x: int) -> int:  # type.ex:694-698
    return 1 if x <= 1 else 8 if x <= 0xFF else 16 if x <= 0xFFFF else 32 if x <= 0xFFFFFFFF else 64


def _signed_size(x: int) -> int:  # type.ex:700-705
    if x < 0:
        x = -x - 1
    return 1 if x <= 1 else 8 if x <= 127 else 16 if x <= 32767 else 32 if x <= 2147483647 else 64


def merge_number(t, number):
    """Nx.Type.merge_number/2 (type.ex:536-560)."""
    t = normalize(t)
    if isinstance(number, bool):
        number = int(number)
    if isinstance(number, int):
        if t[0] == "u":
            if number >= 0:
                return ("u", max(_unsigned_size(number), t[1]))
            return merge_number(("s", min(t[1] * 2, 64)), number)
        if t[0] == "s":
            return ("s", max(_signed_size(number), t[1]))
        return t
    if t[0] in ("f", "bf"):
        return t
    return ("f", 32)


def infer(number):
    """Nx.Type.infer/1 for Python scalars: integers are s32, floats f32 (type.ex:160-188)."""
    if isinstance(number, (bool, int, np.integer)):
        return ("s", 32)
    return ("f", 32)


def to_floating(t):
    """Nx.Type.to_floating/1 (type.ex:253-257)."""
    t = normalize(t)
    return t if t[0] in ("f", "bf") else merge(t, ("f", 32))


def to_aggregate(t):
    """Nx.Type.to_aggregate/1 (type.ex:329-333)."""
    t = normalize(t)
    if t == ("u", 64):
        return ("s", 64)
    if t[0] == "u":
        return ("u", 32)
    if t == ("s", 64):
        return ("s", 64)
    if t[0] == "s":
        return ("s", 32)
    return t


def binary_type(a, b):
    """Nx.Shared.binary_type/2 (shared.ex:383-388); a and b are types or Python numbers."""
    a_num, b_num = isinstance(a, (int, float)), isinstance(b, (int, float))
    if a_num and b_num:
        return infer(a + b)
    if a_num:
        return merge_number(b, a)
    if b_num:
        return merge_number(a, b)
    return merge(a, b)
