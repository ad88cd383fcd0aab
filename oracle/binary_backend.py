"""BinaryBackend -- the parity oracle: `Nx.BinaryBackend`'s callbacks over the C restatement.

TEST INFRASTRUCTURE ONLY.  Tests, the smoke check and the CPU-baseline leg of the benchmark use
it as the checker; nothing in the product imports it.

It implements the same callback interface as the device backend (reference:
nx/lib/nx/backend.ex:46-144), each callback following the cited lines of
nx/lib/nx/binary_backend.ex through `libhipnx_ref.so` (oracle/hipnx_ref.c), so that the same
front-end call can be run on either backend and compared -- the pattern of the reference's own
cross-backend suite (torchx/test/torchx/nx_test.exs:25-50).

Where the reference raises, this raises: `ReferenceRaises` carries the message.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from math import prod

import numpy as np

from nx_amd import shape as S
from nx_amd import types as T
from nx_amd.tensor import Tensor, number_to_binary, pack_sub_byte, unpack_sub_byte

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libhipnx_ref.so")


def build(force: bool = False) -> str:
    """Compiles the C restatement with gcc (seconds)."""
    src = os.path.join(_HERE, "hipnx_ref.c")
    if force or not os.path.exists(LIB_PATH) or os.path.getmtime(LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libhipnx_ref.so"], stdout=subprocess.DEVNULL)
    return LIB_PATH


def _load():
    if not os.path.exists(LIB_PATH):
        build()
    lib = C.CDLL(LIB_PATH)
    i64p, intp, vp = C.POINTER(C.c_int64), C.POINTER(C.c_int), C.c_void_p
    lib.ref_last_error.restype = C.c_char_p
    lib.ref_set_threads.argtypes = [C.c_int]
    lib.ref_binary.argtypes = [C.c_int] * 5 + [i64p, i64p, i64p, vp, vp, vp]
    lib.ref_unary.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int64, vp, vp]
    lib.ref_as_type.argtypes = [C.c_int, C.c_int, C.c_int64, vp, vp]
    lib.ref_reduce.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int64, C.c_int64, C.c_int64, vp, vp]
    lib.ref_argreduce.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int64, C.c_int64, C.c_int64, vp, vp]
    lib.ref_dot.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_int64, vp, vp, vp]
    lib.ref_transpose.argtypes = [C.c_int, C.c_int, i64p, intp, vp, vp]
    lib.ref_broadcast.argtypes = [C.c_int, C.c_int, i64p, i64p, vp, vp]
    lib.ref_gather.argtypes = [C.c_int, C.c_int, i64p, C.c_int, C.c_int64, C.c_int, vp, vp, vp]
    return lib


lib = _load()


class ReferenceRaises(Exception):
    """The reference raises here (ArgumentError / ArithmeticError); `.code` is the REF_E* status."""

    def __init__(self, code, message):
        super().__init__(message)
        self.code = code


def _check(status):
    if status:
        raise ReferenceRaises(status, lib.ref_last_error().decode())


def set_threads(n: int) -> None:
    lib.ref_set_threads(n)


def _i64(v):
    v = list(v)
    return (C.c_int64 * max(len(v), 1))(*v)


def _ints(v):
    v = list(v)
    return (C.c_int * max(len(v), 1))(*v)


BINARY_OPS = ["add", "subtract", "multiply", "divide", "pow", "remainder", "atan2", "min", "max", "quotient",
              "bitwise_and", "bitwise_or", "bitwise_xor", "left_shift", "right_shift", "equal", "not_equal",
              "greater", "less", "greater_equal", "less_equal", "logical_and", "logical_or", "logical_xor"]
UNARY_OPS = ["exp", "expm1", "log", "log1p", "sigmoid", "cos", "sin", "tan", "cosh", "sinh", "tanh", "acos", "asin",
             "atan", "acosh", "asinh", "atanh", "sqrt", "rsqrt", "cbrt", "erf", "erfc", "erf_inv", "abs",
             "bitwise_not", "ceil", "floor", "negate", "round", "sign", "count_leading_zeros", "population_count",
             "is_nan", "is_infinity"]


class BinaryBackend:
    """Backend struct: `%Nx.BinaryBackend{state: binary}` (binary_backend.ex:14-15)."""

    def __init__(self, state: bytearray):
        self.state = state

    @staticmethod
    def init(opts):  # binary_backend.ex:26-33
        if opts:
            raise ValueError("Nx.BinaryBackend accepts no options")
        return {}

    # -- helpers
    @staticmethod
    def _ptr(buf):
        return (C.c_char * max(len(buf), 1)).from_buffer(buf) if len(buf) else (C.c_char * 1)()

    @classmethod
    def _bin(cls, t: Tensor) -> bytearray:
        if isinstance(t.data, BinaryBackend):
            return t.data.state
        return bytearray(type(t.data).to_binary(t, t.size))

    @classmethod
    def _new(cls, out: Tensor):
        buf = bytearray(out.size * T.size_bytes(out.type))
        return buf, out.with_(data=cls(buf))

    # -- plumbing (binary_backend.ex:42-46, 114-165)
    # Sub-byte integers (u2, u4, s2, s4): the reference's state is the packed bitstring and every
    # callback reads `size`-bit segments and writes the low `size` bits (binary_backend.ex:2415-2438,
    # shared.ex:190-194).  Here the state holds one element per byte, extended to s8 / u8, the C
    # functions run on those, and `_narrow` keeps the low bits of what they wrote; from_binary
    # and to_binary convert from and to the packed form (first element in the highest bits).
    @classmethod
    def from_binary(cls, out, binary, opts=None):
        if T.is_sub_byte(out.type):
            return out.with_(data=cls(bytearray(unpack_sub_byte(binary, out.type, out.size).tobytes())))
        need = out.size * T.size_bytes(out.type)
        if len(binary) < need:
            raise ValueError("binary size is too small for the requested shape")
        return out.with_(data=cls(bytearray(binary[:need])))

    @classmethod
    def to_binary(cls, t, limit):
        n = min(int(limit), t.size)
        if T.is_sub_byte(t.type):
            return pack_sub_byte(np.frombuffer(bytes(t.data.state[:n]), dtype=np.uint8), t.type)
        return bytes(t.data.state[: n * T.size_bytes(t.type)])

    @classmethod
    def constant(cls, out, number, opts=None):
        if T.is_sub_byte(out.type):
            one = unpack_sub_byte(number_to_binary(number, out.type), out.type, 1).tobytes()
            return out.with_(data=cls(bytearray(one * out.size)))
        return out.with_(data=cls(bytearray(number_to_binary(number, out.type) * out.size)))

    @classmethod
    def _narrow(cls, res):
        """Keeps the low bits of a sub-byte result that was computed at 8 bits."""
        if not T.is_sub_byte(res.type):
            return res
        kind, bits = res.type
        v = np.frombuffer(bytes(res.data.state), dtype=np.uint8).astype(np.int64) & ((1 << bits) - 1)
        if kind == "s":
            v = np.where(v >= (1 << (bits - 1)), v - (1 << bits), v)
        res.data.state[:] = v.astype(np.int8 if kind == "s" else np.uint8).tobytes()
        return res

    @classmethod
    def to_batched(cls, out, t, opts):  # binary_backend.ex:178-211
        batch, total = out.shape[0], t.shape[0]
        full, rest = divmod(total, batch)
        state = bytes(cls._bin(t))
        size = out.size * T.size_bytes(out.type)
        count = full + (1 if rest and opts.get("leftover", "repeat") == "repeat" else 0)

        def one(i):
            if i < full:
                return out.with_(data=cls(bytearray(state[i * size:(i + 1) * size])))
            tail = state[full * size:]
            return out.with_(data=cls(bytearray(tail + state[:size - len(tail)])))

        return (one(i) for i in range(count))

    @classmethod
    def backend_copy(cls, t, backend, opts=None):
        return backend.from_binary(t, cls.to_binary(t, t.size), opts)

    backend_transfer = backend_copy

    @classmethod
    def backend_deallocate(cls, t):
        return "ok"

    @classmethod
    def reshape(cls, out, t):
        return out.with_(data=cls(cls._bin(t)))

    @classmethod
    def squeeze(cls, out, t, axes):
        return out.with_(data=cls(cls._bin(t)))

    @classmethod
    def bitcast(cls, out, t):
        if T.is_sub_byte(out.type):  # same bits, read with the other signedness
            return cls._narrow(out.with_(data=cls(bytearray(cls._bin(t)))))
        return out.with_(data=cls(cls._bin(t)))

    @classmethod
    def block(cls, struct, out, args, fun):  # binary_backend.ex:36-38
        return fun(struct, *args)

    # -- element-wise (binary_backend.ex:649-706, 827-832, 957-960)
    @classmethod
    def _binary(cls, op, out, l, r):
        lb, rb = cls._bin(l), cls._bin(r)
        buf, res = cls._new(out)
        _check(lib.ref_binary(op, T.code(l.type), T.code(r.type), T.code(out.type), len(out.shape), _i64(out.shape),
                              _i64(S.broadcast_strides(l.shape, out.shape)),
                              _i64(S.broadcast_strides(r.shape, out.shape)), cls._ptr(lb), cls._ptr(rb), cls._ptr(buf)))
        return cls._narrow(res)

    @classmethod
    def _unary(cls, op, out, t):
        tb = cls._bin(t)
        buf, res = cls._new(out)
        if T.is_sub_byte(t.type) and UNARY_OPS[op] == "count_leading_zeros":
            raise NotImplementedError("count_leading_zeros of a sub-byte integer")  # binary_backend.ex:962-966: no clause
        if T.is_sub_byte(t.type) and UNARY_OPS[op] == "population_count":
            # binary_backend.ex:844-850 reads each element as an unsigned segment of the type's width
            bits = np.frombuffer(bytes(tb), dtype=np.uint8) & ((1 << t.type[1]) - 1)
            counts = np.array([bin(int(b)).count("1") for b in bits], dtype=np.int64).reshape(t.shape)
            return cls._from_array(out, counts, "s64")
        _check(lib.ref_unary(op, T.code(t.type), T.code(out.type), out.size, cls._ptr(tb), cls._ptr(buf)))
        return cls._narrow(res)

    @classmethod
    def as_type(cls, out, t):  # binary_backend.ex:2031-2076
        if t.type == out.type:
            return t
        if T.is_sub_byte(out.type) and T.is_float(t.type):
            # binary_backend.ex:2056-2069: NaN -> 0, infinities -> the type's extremes, the rest
            # truncated and written at the type's width
            x = cls._numbers(t).ravel()
            kind, bits = out.type
            lo, hi = (-(1 << (bits - 1)), (1 << (bits - 1)) - 1) if kind == "s" else (0, (1 << bits) - 1)
            finite = np.isfinite(x)
            v = np.zeros(x.shape, dtype=np.int64)
            v[finite] = np.trunc(x[finite]).astype(np.int64)
            v[np.isposinf(x)] = hi
            v[np.isneginf(x)] = lo
            return cls._narrow(out.with_(data=cls(bytearray(v.astype(np.uint8).tobytes()))))
        tb = cls._bin(t)
        buf, res = cls._new(out)
        _check(lib.ref_as_type(T.code(t.type), T.code(out.type), out.size, cls._ptr(tb), cls._ptr(buf)))
        return cls._narrow(res)

    # -- data movement (binary_backend.ex:215-319, 1902-1959)
    @classmethod
    def transpose(cls, out, t, axes):
        tb = cls._bin(t)
        buf, res = cls._new(out)
        _check(lib.ref_transpose(T.size_bytes(t.type), len(t.shape), _i64(t.shape), _ints(axes), cls._ptr(tb),
                                 cls._ptr(buf)))
        return res

    @classmethod
    def broadcast(cls, out, t, shape, axes):
        strides, s = [0] * len(shape), 1
        for pos in range(len(t.shape) - 1, -1, -1):
            if t.shape[pos] != 1:
                strides[axes[pos]] = s
            s *= t.shape[pos]
        tb = cls._bin(t)
        buf, res = cls._new(out)
        _check(lib.ref_broadcast(T.size_bytes(t.type), len(shape), _i64(shape), _i64(strides), cls._ptr(tb),
                                 cls._ptr(buf)))
        return res

    @classmethod
    def gather(cls, out, t, indices, opts):
        axes = list(opts["axes"])
        rank = len(t.shape)
        if list(range(rank))[: len(axes)] != axes:  # binary_backend.ex:1907-1913
            perm = axes + [a for a in range(rank) if a not in axes]
            t = cls.transpose(t.with_(data=None, shape=S.transpose(t.shape, perm)), t, perm)
        tb, ib = cls._bin(t), cls._bin(indices)
        buf, res = cls._new(out)
        _check(lib.ref_gather(T.size_bytes(t.type), rank, _i64(t.shape), T.code(indices.type),
                              prod(indices.shape[:-1]), indices.shape[-1], cls._ptr(tb), cls._ptr(ib), cls._ptr(buf)))
        return res

    # -- reductions (binary_backend.ex:1315-1431, 2342-2360, 2469-2512)
    @classmethod
    def _view(cls, t, axes):
        """[kept..., reduced...] in sorted axis order: the traversal order of aggregate_axes."""
        rank = len(t.shape)
        if axes is None:
            return t, 1, t.size, 1
        axes = sorted(axes)
        kept = [a for a in range(rank) if a not in axes]
        perm = kept + axes
        if perm != list(range(rank)):
            t = cls.transpose(t.with_(data=None, shape=S.transpose(t.shape, perm)), t, perm)
        return t, prod(t.shape[: len(kept)]), prod(t.shape[len(kept):]), 1

    @classmethod
    def _reduce(cls, op, out, t, opts):
        view, outer, red, inner = cls._view(t, opts.get("axes"))
        tb = cls._bin(view)
        buf, res = cls._new(out)
        _check(lib.ref_reduce(op, T.code(t.type), T.code(out.type), outer, red, inner, cls._ptr(tb), cls._ptr(buf)))
        return res

    @classmethod
    def sum(cls, out, t, opts):
        return cls._reduce(0, out, t, opts)

    @classmethod
    def reduce_max(cls, out, t, opts):
        return cls._reduce(1, out, t, opts)

    @classmethod
    def reduce_min(cls, out, t, opts):
        return cls._reduce(2, out, t, opts)

    @classmethod
    def product(cls, out, t, opts):
        return cls._reduce(3, out, t, opts)

    @classmethod
    def _arg(cls, op, out, t, opts):
        axis = opts.get("axis")
        view, outer, red, inner = cls._view(t, None if axis is None else [axis])
        tie = {"low": 0, "high": 1}[opts.get("tie_break", "low")]
        tb = cls._bin(view)
        buf, res = cls._new(out)
        _check(lib.ref_argreduce(op, tie, T.code(t.type), T.code(out.type), outer, red, inner, cls._ptr(tb),
                                 cls._ptr(buf)))
        return res

    @classmethod
    def argmax(cls, out, t, opts):
        return cls._arg(0, out, t, opts)

    @classmethod
    def argmin(cls, out, t, opts):
        return cls._arg(1, out, t, opts)

    # -- dot (binary_backend.ex:476-599)
    @classmethod
    def _contract_last(cls, t, contract, nbatch):
        """bin_dot_transpose_contract_axes/2: [batch, kept, contract in the given order]."""
        rank = len(t.shape)
        kept = [a for a in range(nbatch, rank) if a not in contract]
        perm = list(range(nbatch)) + kept + list(contract)
        rows = prod(t.shape[a] for a in kept)
        if perm != list(range(rank)):
            t = cls.transpose(t.with_(data=None, shape=S.transpose(t.shape, perm)), t, perm)
        return t, rows

    @classmethod
    def dot(cls, out, l, c1, b1, r, c2, b2):
        nb = len(b1)
        K = prod(l.shape[a] for a in c1)
        batch = prod(l.shape[a] for a in b1)
        lt, M = cls._contract_last(l, c1, nb)
        rt, N = cls._contract_last(r, c2, nb)
        lb, rb = cls._bin(lt), cls._bin(rt)
        buf, res = cls._new(out)
        _check(lib.ref_dot(T.code(l.type), T.code(r.type), T.code(out.type), batch, M, N, K, cls._ptr(lb),
                           cls._ptr(rb), cls._ptr(buf)))
        return cls._narrow(res)


    # -- one step off the hot path ---------------------------------------------------------------
    # numpy restatements of byte-level / integer rules; encodings go through ref_as_type so that
    # every number reaches its binary the way number_to_binary writes it.
    @classmethod
    def _typed(cls, t):
        """The tensor's elements as a numpy array of its storage type (bf16: raw uint16)."""
        return np.frombuffer(bytes(cls._bin(t)), dtype=T.numpy_dtype(t.type)).reshape(t.shape)

    @classmethod
    def _from_array(cls, out, arr, src_type):
        """Encodes `arr` (s64 / f64 numbers) into out.type as the reference's write path does."""
        src = out.with_(data=cls(bytearray(np.ascontiguousarray(arr).tobytes())), type=T.normalize(src_type))
        return cls.as_type(out, src) if src.type != out.type else src

    @classmethod
    def _numbers(cls, t):
        """Decoded values: float64 for float types (bf16 widened), uint64 for u64, int64 otherwise."""
        a = cls._typed(t)
        if t.type == ("bf", 16):
            return (a.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        if t.type == ("u", 64):
            return a
        return a.astype(np.float64) if T.is_float(t.type) else a.astype(np.int64)

    @classmethod
    def iota(cls, out, axis, opts=None):  # binary_backend.ex:49-87
        n = out.size
        if axis is None:
            idx = np.arange(n, dtype=np.int64)
        else:
            inner = prod(out.shape[axis + 1:])
            idx = (np.arange(n, dtype=np.int64) // inner) % out.shape[axis]
        return cls._from_array(out, idx, "s64")

    @classmethod
    def eye(cls, out, opts=None):  # binary_backend.ex:90-110
        m, n = out.shape[-2], out.shape[-1]
        one = np.eye(m, n, dtype=np.int64)
        return cls._from_array(out, np.broadcast_to(one, out.shape), "s64")

    @classmethod
    def select(cls, out, pred, on_true, on_false):  # binary_backend.ex:604-648
        truth = cls._numbers(pred) != 0  # as_boolean: everything but 0, NaN included
        truth = np.broadcast_to(truth, out.shape)
        sides = []
        for side in (on_true, on_false):
            full = cls.broadcast(side.with_(data=None, shape=out.shape), side, out.shape,
                                 S.broadcast_axes(side.shape, out.shape)) if side.shape != out.shape else side
            full = cls.as_type(full.with_(data=None, type=out.type), full)
            sides.append(cls._typed(full))
        buf, res = cls._new(out)
        buf[:] = np.where(truth, sides[0], sides[1]).astype(sides[0].dtype).tobytes()
        return res

    @classmethod
    def clip(cls, out, t, min_t, max_t):  # binary_backend.ex:1788-1811
        x, lo, hi = cls._numbers(t), cls._numbers(min_t).reshape(()), cls._numbers(max_t).reshape(())
        if T.is_float(out.type):
            x, lo, hi = x.astype(np.float64), np.float64(lo), np.float64(hi)
        elif np.uint64 in (x.dtype, lo.dtype, hi.dtype):  # unbounded integers, as the reference's numbers are
            x, lo, hi = x.astype(object), int(lo), int(hi)
            c = np.where(x > lo, x, lo)
            r = np.where(c < hi, c, hi)
            wrapped = np.array([int(v) & 0xFFFFFFFFFFFFFFFF for v in r.reshape(-1)], dtype=np.uint64).reshape(r.shape)
            return cls._from_array(out, wrapped, "u64")
        with np.errstate(invalid="ignore"):
            c = np.where(x > lo, x, lo)      # element_greater(x, min) == 1 ? x : min
            r = np.where(c < hi, c, hi)      # element_less(clipped, max) == 1 ? clipped : max
        return cls._from_array(out, r, "f64" if T.is_float(out.type) else "s64")

    @classmethod
    def pad(cls, out, t, pad_value, padding_config):  # binary_backend.ex:326-431
        if t.shape == ():
            return t  # the reference hands the scalar back untouched, whatever out.type says
        if t.type != out.type:
            # the reference splices pad bytes of out.type into the binary of t and labels the result
            # with t's type (binary_backend.ex:327,352,418): not a behaviour to restate
            raise NotImplementedError("pad: the reference mixes two encodings when the types differ")
        value = cls._typed(cls.as_type(pad_value.with_(data=None, type=out.type), pad_value)).reshape(())
        a = cls._typed(t)  # elements keep their bytes: the reference pads the binary of t as it is
        for axis, (low, high, interior) in enumerate(padding_config):
            a = np.moveaxis(a, axis, -1)
            rows, n = a.shape[:-1], a.shape[-1]
            # interior padding after every element, the last run dropped again
            spread = np.full(rows + (n, interior + 1), value, dtype=a.dtype)
            spread[..., 0] = a
            seq = spread.reshape(rows + (n * (interior + 1),))[..., :max(n * (interior + 1) - interior, 0)]
            # edges: positive ones add the value, negative ones cut into the interior-padded row
            if low < 0:
                seq = seq[..., -low:]
            else:
                seq = np.concatenate([np.full(rows + (low,), value, dtype=a.dtype), seq], axis=-1)
            if high < 0:
                seq = seq[..., :seq.shape[-1] + high]
            else:
                seq = np.concatenate([seq, np.full(rows + (high,), value, dtype=a.dtype)], axis=-1)
            a = np.moveaxis(seq, -1, axis)
        buf, res = cls._new(out)
        buf[:] = np.ascontiguousarray(a).tobytes()
        return res

    @classmethod
    def slice(cls, out, t, start_indices, lengths, strides):  # binary_backend.ex:1813-1863
        a = cls._typed(t)
        window = []
        for dim, idx, length, step in zip(t.shape, start_indices, lengths, strides):
            if isinstance(idx, Tensor):
                idx = int(cls._numbers(idx).reshape(()))
            start = min(max(int(idx), 0), dim - length)  # clamp_indices
            window.append(np.s_[start:start + length:step])
        buf, res = cls._new(out)
        buf[:] = np.ascontiguousarray(a[tuple(window)]).tobytes()
        return res

    @classmethod
    def reverse(cls, out, t, axes):  # binary_backend.ex:434-474
        buf, res = cls._new(out)
        buf[:] = np.ascontiguousarray(np.flip(cls._typed(t), axis=tuple(axes))).tobytes()
        return res

    @classmethod
    def put_slice(cls, out, t, start_indices, slice_t):  # binary_backend.ex:1865-1900
        base = cls._typed(cls.as_type(t.with_(data=None, type=out.type), t)).copy()
        piece = cls._typed(cls.as_type(slice_t.with_(data=None, type=out.type), slice_t))
        window = []
        for dim, idx, length in zip(t.shape, start_indices, slice_t.shape):
            if isinstance(idx, Tensor):
                idx = int(cls._numbers(idx).reshape(()))
            start = min(max(int(idx), 0), dim - length)  # clamp_indices
            window.append(np.s_[start:start + length])
        base[tuple(window)] = piece
        buf, res = cls._new(out)
        buf[:] = base.tobytes()
        return res

    @classmethod
    def concatenate(cls, out, tensors, axis):  # binary_backend.ex:1975-1986
        parts = [cls._typed(cls.as_type(t.with_(data=None, type=out.type), t)) for t in tensors]
        buf, res = cls._new(out)
        buf[:] = np.concatenate(parts, axis=axis).tobytes()
        return res

    @classmethod
    def stack(cls, out, tensors, axis):  # binary_backend.ex:1962-1972
        parts = [cls._typed(cls.as_type(t.with_(data=None, type=out.type), t)) for t in tensors]
        buf, res = cls._new(out)
        buf[:] = np.stack(parts, axis=axis).tobytes()
        return res

    @classmethod
    def _truth_reduce(cls, fn, out, t, opts):  # binary_backend.ex:1293-1314
        axes = opts.get("axes")
        truth = cls._numbers(t) != 0
        r = fn(truth, axis=tuple(axes) if axes is not None else None)
        return cls._from_array(out, np.asarray(r).astype(np.int64).reshape(out.shape), "s64")

    @classmethod
    def all(cls, out, t, opts):
        return cls._truth_reduce(np.all, out, t, opts)

    @classmethod
    def any(cls, out, t, opts):
        return cls._truth_reduce(np.any, out, t, opts)


def _install():
    for code, name in enumerate(BINARY_OPS):
        setattr(BinaryBackend, name, classmethod(lambda cls, out, l, r, _c=code: cls._binary(_c, out, l, r)))
    for code, name in enumerate(UNARY_OPS):
        setattr(BinaryBackend, name, classmethod(lambda cls, out, t, _c=code: cls._unary(_c, out, t)))


_install()
