"""The slice of the `Nx` front end that sits above the device path (reference: nx/lib/nx.ex).

Each function does what its namesake does before it reaches a backend: converts numbers to
tensors, infers the output type and shape, builds the output template and dispatches to the
backend chosen from the operands (`impl!/1,2`, nx/lib/nx/shared.ex:449-473).  It exists so that
callers -- and the parity tests, which read like the reference's own -- can switch backend and
run unchanged.  Vectorisation and axis names are not modelled.
"""
from __future__ import annotations

import builtins
import threading
from dataclasses import dataclass
from typing import Optional
from math import prod

import numpy as np

from . import shape as S
from . import types as T
from .host import HostBinary
from .tensor import Tensor, binary_to_numpy, list_to_binary, template, to_float64

_state = threading.local()
_global_default = [(HostBinary, {})]


def default_backend(backend=None, opts=None):
    """Nx.default_backend/0,1 (nx.ex:5006-5049): per-thread override, `init/1` validates opts."""
    if backend is None:
        return getattr(_state, "backend", None) or _global_default[0]
    previous = default_backend()
    _state.backend = (backend, backend.init(opts or {}))
    return previous


def global_default_backend(backend, opts=None):
    previous = _global_default[0]
    _global_default[0] = (backend, backend.init(opts or {}))
    return previous


def _impl(*tensors):
    """impl!/1,2 (shared.ex:449-473): HostBinary loses to any other backend; two different
    compute backends cannot be mixed."""
    chosen = None
    for t in tensors:
        b = type(t.data)
        if b is HostBinary:
            continue
        if chosen is None:
            chosen = b
        elif chosen is not b:
            raise ValueError(f"cannot invoke Nx function because it relies on two incompatible tensor "
                             f"implementations: {chosen.__name__} and {b.__name__}")
    return chosen or HostBinary


# ---- creation / conversion ---------------------------------------------------------------

def _infer_list_type(arr: np.ndarray):
    return ("f", 32) if arr.dtype.kind == "f" else ("u", 8) if arr.dtype.kind == "b" else ("s", 32)


def tensor(value, type=None, backend=None) -> Tensor:
    """Nx.tensor/2 (nx.ex:774-883): nested lists / numbers -> tensor on the default backend."""
    if isinstance(value, Tensor):
        return value if type is None else as_type(value, type)
    if isinstance(value, np.ndarray) and value.dtype.kind in "iuf" and type is None and value.dtype != np.float16:
        arr = value
        ty = {"i": "s", "u": "u", "f": "f"}[arr.dtype.kind], arr.dtype.itemsize * 8
        binary = np.ascontiguousarray(arr).tobytes()
    else:
        arr = np.asarray(value)
        if arr.dtype == object:
            arr = np.asarray(value, dtype=np.float64)
        ty = T.normalize(type) if type is not None else _infer_list_type(arr)
        binary = list_to_binary(arr, ty)
    mod, opts = (backend, {}) if backend is not None and not isinstance(backend, tuple) else (backend or default_backend())
    return mod.from_binary(template(ty, arr.shape), binary, opts)


def from_binary(binary, type, backend=None, count=None) -> Tensor:
    """Nx.from_binary/3 (nx.ex:2051-2066): a flat tensor over the bytes.  A packed sub-byte binary
    whose last byte is only partly used needs `count` elements said (the reference reads it off
    the bitstring's bit size)."""
    ty = T.normalize(type)
    bits = T.bit_size(ty)
    if len(binary) == 0:
        raise ValueError("cannot build an empty tensor")
    if (len(binary) * 8) % bits:
        raise ValueError("binary has incompatible number of bits, expected a multiple of the type size")
    n = len(binary) * 8 // bits
    if count is not None:
        if not T.is_sub_byte(ty) or not n - 8 // bits < count <= n:
            raise ValueError("count does not fit the binary")
        n = count
    mod, opts = (backend, {}) if backend is not None and not isinstance(backend, tuple) else (backend or default_backend())
    return mod.from_binary(template(ty, (n,)), binary, opts)


def _def_typed_constructors():
    # Nx.u2/1 .. Nx.f64/1 (nx.ex:974-984): aliases for Nx.tensor(value, type: t)
    for name in ("u2", "u4", "u8", "u16", "u32", "u64", "s2", "s4", "s8", "s16", "s32", "s64", "bf16", "f16", "f32", "f64"):
        globals()[name] = (lambda value, _t=name: tensor(value, type=_t))


_def_typed_constructors()


def bit_size(t: Tensor) -> int:
    """Nx.bit_size/1 (nx.ex:4890-4915)."""
    return t.size * T.bit_size(t.type)


def byte_size(t: Tensor) -> int:
    """Nx.byte_size/1 (nx.ex:4860-4888): whole bytes of the binary."""
    return bit_size(t) // 8


def to_tensor(value) -> Tensor:
    """Nx.to_tensor/1 (nx.ex:2149-2157): numbers become rank-0 constants on the default backend."""
    c = value.__class__
    if c is Tensor:
        return value
    if c is float or c is int:  # (the number of `multiply(t, 0.5)`: the common case, without the checks below)
        mod, opts = getattr(_state, "backend", None) or _global_default[0]
        return mod.constant(_F32_SCALAR if c is float else _S32_SCALAR, value, opts)
    if isinstance(value, Tensor):
        return value
    if isinstance(value, (bool, int, float, np.integer, np.floating)):
        mod, opts = default_backend()
        v = value.item() if isinstance(value, np.generic) else value
        return mod.constant(template(T.infer(v), ()), v, opts)
    return tensor(value)


_F32_SCALAR, _S32_SCALAR = template(("f", 32), ()), template(("s", 32), ())  # what Nx.Type.infer/1 gives a float / an integer


def to_binary(t: Tensor, limit=None) -> bytes:
    """Nx.to_binary/2 (nx.ex:2121-2133); `limit` counts elements."""
    limit = t.size if limit is None else builtins.min(limit, t.size)
    return type(t.data).to_binary(t, limit)


def to_batched(t, batch_size: int, leftover="repeat"):
    """Nx.to_batched/3 (nx.ex:2455-2666): a lazy sequence of tensors of `batch_size` leading
    entries; a last, short batch is completed from the first entries ("repeat") or dropped
    ("discard")."""
    if not isinstance(batch_size, int) or batch_size < 1:
        raise ValueError("batch_size must be a positive integer")
    if leftover not in ("repeat", "discard"):
        raise ValueError(f"expected :leftover to be :repeat or :discard, got: {leftover!r}")
    t = to_tensor(t)
    if t.shape == ():
        raise ValueError("cannot batch non-vectorized scalar tensor")
    if t.shape[0] < batch_size:
        raise ValueError("cannot batch beyond original tensor")
    out = t.with_(shape=(batch_size,) + t.shape[1:], names=t.names)
    return _impl(t).to_batched(out, t, {"leftover": leftover})


def to_numpy(t: Tensor) -> np.ndarray:
    """Raw element array (bf16 as uint16 bit patterns)."""
    return binary_to_numpy(to_binary(t), t.type, t.shape).copy()


def to_float64(t: Tensor) -> np.ndarray:
    from .tensor import to_float64 as f
    return f(to_binary(t), t.type, t.shape)


def to_flat_list(t: Tensor):
    return to_float64(t).ravel().tolist() if T.is_float(t.type) else to_numpy(t).ravel().tolist()


def backend_copy(t: Tensor, backend=None, opts=None) -> Tensor:
    mod, o = (backend, opts or {}) if backend is not None else default_backend()
    return type(t.data).backend_copy(t, mod, o)


def backend_transfer(t: Tensor, backend=None, opts=None) -> Tensor:
    mod, o = (backend, opts or {}) if backend is not None else default_backend()
    return type(t.data).backend_transfer(t, mod, o)


def backend_deallocate(t: Tensor) -> str:
    return type(t.data).backend_deallocate(t)


def shape(t) -> tuple:
    return to_tensor(t).shape


def type_of(t):
    return to_tensor(t).type


# ---- element-wise ------------------------------------------------------------------------

_ARITH = ["add", "subtract", "multiply", "pow", "remainder", "min", "max"]
_INT_ONLY = ["quotient", "bitwise_and", "bitwise_or", "bitwise_xor", "left_shift", "right_shift"]
_FLOAT_OUT = ["divide", "atan2"]
_PRED = ["equal", "not_equal", "greater", "less", "greater_equal", "less_equal", "logical_and", "logical_or",
         "logical_xor"]


def _number_or_type(x):
    return x if isinstance(x, (int, float)) and not isinstance(x, bool) else to_tensor(x).type


def _binary(name, left, right, out_type_fun):
    if left.__class__ is Tensor and right.__class__ is Tensor:  # the common case: no number to look at
        ty = left.type if left.type == right.type else T.merge(left.type, right.type)
        l, r = left, right
    else:
        ty = T.binary_type(_number_or_type(left), _number_or_type(right))
        l, r = to_tensor(left), to_tensor(right)
    ls, rs = l.shape, r.shape
    out = template(out_type_fun(ty), ls if ls == rs or rs == () else rs if ls == () else S.binary_broadcast(ls, rs))
    lb, rb = l.data.__class__, r.data.__class__
    return getattr(lb if lb is rb else _impl(l, r), name)(out, l, r)


def _def_binary():
    g = globals()
    for name in _ARITH:
        g[name] = (lambda n: lambda left, right: _binary(n, left, right, lambda ty: ty))(name)
    for name in _INT_ONLY:
        def int_only(left, right, _n=name):
            def check(ty):
                if not T.is_integer(ty):
                    raise ValueError(f"{_n} expects integer tensors as inputs and outputs an integer tensor, "
                                     f"got: {ty!r}")
                return ty
            return _binary(_n, left, right, check)
        g[name] = int_only
    for name in _FLOAT_OUT:  # element_wise_bin_op with to_floating (nx.ex:6544, 6639)
        g[name] = (lambda n: lambda left, right: _binary(n, left, right, T.to_floating))(name)
    for name in _PRED:  # element_wise_pred_op: u8 output (nx.ex:6037-6050)
        g[name] = (lambda n: lambda left, right: _binary(n, left, right, lambda ty: ("u", 8)))(name)


_def_binary()

_MATH = ["exp", "expm1", "log", "log1p", "sigmoid", "cos", "sin", "tan", "cosh", "sinh", "tanh", "acos", "asin",
         "atan", "acosh", "asinh", "atanh", "sqrt", "rsqrt", "cbrt", "erf", "erfc", "erf_inv"]


def _def_unary():
    g = globals()
    for name in _MATH:  # nx.ex:8592-8598: out type = to_floating
        def math_fun(t, _n=name):
            t = to_tensor(t)
            return getattr(_impl(t), _n)(t.with_(data=None, type=T.to_floating(t.type)), t)
        g[name] = math_fun
    for name in ["negate", "sign"]:  # nx.ex:8703-8731
        g[name] = (lambda n: lambda t: getattr(_impl(to_tensor(t)), n)(to_tensor(t).with_(data=None), to_tensor(t)))(name)
    for name in ["floor", "ceil", "round"]:  # nx.ex:9095-9133: integers are returned as they are
        def rounding(t, _n=name):
            t = to_tensor(t)
            return t if T.is_integer(t.type) else getattr(_impl(t), _n)(t.with_(data=None), t)
        g[name] = rounding
    for name in ["bitwise_not", "population_count", "count_leading_zeros"]:  # nx.ex:8979-9091
        def bit_fun(t, _n=name):
            t = to_tensor(t)
            if not T.is_integer(t.type):
                raise ValueError(f"{_n} expects integer tensors as inputs and outputs an integer tensor, "
                                 f"got: {t.type!r}")
            return getattr(_impl(t), _n)(t.with_(data=None), t)
        g[name] = bit_fun
    for name in ["is_nan", "is_infinity"]:  # nx.ex:8628-8690: u8 output
        g[name] = (lambda n: lambda t: getattr(_impl(to_tensor(t)), n)(to_tensor(t).with_(data=None, type=("u", 8)), to_tensor(t)))(name)


_def_unary()


def abs(t):  # noqa: A001 - mirrors Nx.abs/1 (nx.ex:8746-8754): unsigned tensors are returned as-is
    t = to_tensor(t)
    return t if t.type[0] == "u" else _impl(t).abs(t.with_(data=None), t)


def as_type(t, type) -> Tensor:
    """Nx.as_type/2 (nx.ex:2863-2876): a no-op when the type already matches."""
    t = to_tensor(t)
    ty = T.normalize(type)
    return t if t.type == ty else _impl(t).as_type(t.with_(data=None, type=ty), t)


# ---- reductions ----------------------------------------------------------------------------

def _aggregate(t, op, out_type, axes=None, keep_axes=False):
    """aggregate_axes_op/4 (nx.ex:10594-10649)."""
    t = to_tensor(t)
    # the axes and the result's shape depend on the shape and the options only: worked out once per signature
    try:
        key = (t.shape, axes if axes is None else tuple(axes), keep_axes)
        known = _aggregate_shapes.get(key)
    except TypeError:  # axes that are no list of integers: the checks below say so
        key = known = None
    if known is None:
        if axes is not None:
            axes = S.normalize_axes(t.shape, axes)
            shape_ = S.contract(t.shape, axes, keep_axes)
        elif keep_axes:
            shape_, axes = (1,) * len(t.shape), list(range(len(t.shape)))
        else:
            shape_ = ()
        known = (axes, shape_)
        if key is not None:
            if len(_aggregate_shapes) > 4096:
                _aggregate_shapes.clear()
            _aggregate_shapes[key] = known
    axes, shape_ = known
    if axes == []:
        return as_type(t, out_type)
    return getattr(t.data.__class__, op)(template(out_type, shape_), t, {"axes": None if axes is None else list(axes), "keep_axes": keep_axes})


_aggregate_shapes = {}  # (shape, axes, keep_axes) -> (normalised axes, shape of the result)


def sum(t, axes=None, keep_axes=False):  # noqa: A001 - Nx.sum/2 (nx.ex:9622-9626)
    t = to_tensor(t)
    return _aggregate(t, "sum", T.to_aggregate(t.type), axes, keep_axes)


def mean(t, axes=None, keep_axes=False):
    """Nx.mean/2 (nx.ex:9745-9761): the sum divided by the number of reduced entries."""
    t = to_tensor(t)
    count = t.size if axes is None else prod(t.shape[a] for a in S.normalize_axes(t.shape, axes))
    return divide(sum(t, axes=axes, keep_axes=keep_axes), count)


def product(t, axes=None, keep_axes=False):
    t = to_tensor(t)
    return _aggregate(t, "product", T.to_aggregate(t.type), axes, keep_axes)


def reduce_max(t, axes=None, keep_axes=False):
    """Nx.reduce_max/2 (nx.ex:10496-10500): output type = input type."""
    t = to_tensor(t)
    return _aggregate(t, "reduce_max", t.type, axes, keep_axes)


def reduce_min(t, axes=None, keep_axes=False):
    t = to_tensor(t)
    return _aggregate(t, "reduce_min", t.type, axes, keep_axes)


def _argmin_or_max(t, op, axis=None, tie_break="low", keep_axis=False, type=("s", 32)):
    """argmin_or_max/3 (nx.ex:10948-11005)."""
    if tie_break not in ("low", "high"):
        raise ValueError(f"unknown value for :tie_break, expected :high or :low, got: {tie_break!r}")
    t = to_tensor(t)
    if axis is not None:
        axis = S.normalize_axis(t.shape, axis)
        shape_ = S.contract(t.shape, [axis], keep_axis)
    else:
        shape_ = ()
    out = template(T.normalize(type), shape_)
    return getattr(_impl(t), op)(out, t, {"tie_break": tie_break, "axis": axis, "keep_axis": keep_axis})


def argmax(t, **opts):
    return _argmin_or_max(t, "argmax", **opts)


def argmin(t, **opts):
    return _argmin_or_max(t, "argmin", **opts)


# ---- contraction ---------------------------------------------------------------------------

def dot(t1, *args, out_type=None):
    """Nx.dot/2, /4 and /6 (nx.ex:12836-12847, 12918-12920, 13123-13161).

    `out_type` is not part of the reference's front end: it sets the template type handed to the
    `dot` callback (both reference backends honour `out.type` whatever the operand types,
    binary_backend.ex:549-559) and is how a s8 x s8 -> s32 contraction is requested."""
    if len(args) == 1:
        t1, t2 = to_tensor(t1), to_tensor(args[0])
        n, m = len(t1.shape), len(t2.shape)
        if n == 0 or m == 0:
            return globals()["multiply"](t1, t2)
        if m == 1:
            return dot(t1, [n - 1], [], t2, [0], [], out_type=out_type)
        if n == 1:
            return dot(t1, [0], [], t2, [m - 2], [], out_type=out_type)
        return dot(t1, [n - 1], [], t2, [m - 2], [], out_type=out_type)
    if len(args) == 3:
        c1, t2, c2 = args
        return dot(t1, c1, [], t2, c2, [], out_type=out_type)
    c1, b1, t2, c2, b2 = args
    t1, t2 = to_tensor(t1), to_tensor(t2)
    ty = T.normalize(out_type) if out_type is not None else T.binary_type(t1.type, t2.type)
    # the axes and the output shape depend on the shapes and the axes given only: worked out once per signature
    key = (t1.shape, tuple(c1), tuple(b1), t2.shape, tuple(c2), tuple(b2))
    plan = _DOT_PLANS.get(key)
    if plan is None:
        n1, n2 = S.normalize_axes(t1.shape, c1), S.normalize_axes(t2.shape, c2)
        m1, m2 = S.normalize_axes(t1.shape, b1), S.normalize_axes(t2.shape, b2)
        plan = (n1, m1, n2, m2, S.dot(t1.shape, n1, m1, t2.shape, n2, m2))
        if len(_DOT_PLANS) >= 4096:
            _DOT_PLANS.clear()
        _DOT_PLANS[key] = plan
    c1, b1, c2, b2, shape = plan
    return _impl(t1, t2).dot(template(ty, shape), t1, c1, b1, t2, c2, b2)


_DOT_PLANS = {}


# ---- shape / data movement -----------------------------------------------------------------

def reshape(t, new_shape):
    """Nx.reshape/2 (nx.ex:3010-3065), with one `"auto"` dimension allowed."""
    t = to_tensor(t)
    new_shape = list(new_shape)
    if "auto" in new_shape:
        i = new_shape.index("auto")
        rest = prod(d for d in new_shape if d != "auto")
        new_shape[i] = t.size // rest if rest else 0
    if prod(new_shape) != t.size:
        raise ValueError(f"cannot reshape, current shape {S.fmt(t.shape)} is not compatible with "
                         f"new shape {S.fmt(tuple(new_shape))}")
    if tuple(new_shape) == t.shape:
        return t
    return _impl(t).reshape(t.with_(data=None, shape=tuple(new_shape)), t)


def new_axis(t, axis):
    t = to_tensor(t)
    rank = len(t.shape)
    axis = axis + rank + 1 if axis < 0 else axis
    return reshape(t, t.shape[:axis] + (1,) + t.shape[axis:])


def squeeze(t, axes=None):
    t = to_tensor(t)
    axes = [i for i, d in enumerate(t.shape) if d == 1] if axes is None else S.normalize_axes(t.shape, axes)
    if not axes:
        return t
    return _impl(t).squeeze(t.with_(data=None, shape=S.squeeze(t.shape, axes)), t, axes)


def bitcast(t, type):
    t = to_tensor(t)
    ty = T.normalize(type)
    if ty[1] != t.type[1]:
        raise ValueError("input type width must match new type width")
    return _impl(t).bitcast(t.with_(data=None, type=ty), t)


def transpose(t, axes=None):
    """Nx.transpose/2 (nx.ex:3440-3465): identity permutations return the tensor."""
    t = to_tensor(t)
    rank = len(t.shape)
    axes = list(range(rank - 1, -1, -1)) if axes is None else S.normalize_axes(t.shape, axes)
    if axes == list(range(rank)):
        return t
    return _impl(t).transpose(t.with_(data=None, shape=S.transpose(t.shape, axes)), t, axes)


def broadcast(t, new_shape, axes=None):
    """Nx.broadcast/3 (nx.ex:3180-3215)."""
    t = to_tensor(t)
    new_shape = tuple(new_shape)
    axes = S.broadcast_axes(t.shape, new_shape) if axes is None else S.normalize_axes(new_shape, axes)
    S.broadcast(t.shape, new_shape, axes)
    if t.shape == new_shape and axes == list(range(len(new_shape))):
        return t
    return _impl(t).broadcast(t.with_(data=None, shape=new_shape), t, new_shape, axes)


@dataclass(frozen=True)
class Pointer:
    """%Nx.Pointer{kind, address, data_size, handle} (nx/lib/nx/pointer.ex:8-15)."""
    kind: str
    address: Optional[int] = None
    data_size: int = 0
    handle: Optional[bytes] = None


def to_pointer(t, **opts) -> "Pointer":
    """Nx.to_pointer/2 (nx.ex:17807-17810)."""
    t = to_tensor(t)
    return _impl(t).to_pointer(t, opts)


def from_pointer(backend, pointer: "Pointer", type, shape, **opts) -> Tensor:  # noqa: A002
    """Nx.from_pointer/5 (nx.ex:17762-17775): `backend` is a module or (module, options)."""
    mod, backend_opts = backend if isinstance(backend, tuple) else (backend, {})
    return mod.from_pointer(pointer, T.normalize(type), tuple(shape), backend_opts, opts)


@dataclass(frozen=True)
class BlockTake:
    """%Nx.Block.Take{axis} (nx/lib/nx/block.ex:57-59)."""
    axis: int


@dataclass(frozen=True)
class BlockThreefry:
    """The Threefry-2x32 stream of a key over `size` counters (the body of threefry2x32/2,
    nx/lib/nx/random.ex:214-229) as a block, so a backend can produce the words in one step.  The
    reference composes it from callbacks without a block; the words are the same."""
    shape: tuple


@dataclass(frozen=True)
class BlockAllClose:
    """%Nx.Block.AllClose{equal_nan, rtol, atol} (nx/lib/nx/block.ex:37-39)."""
    equal_nan: bool = False
    rtol: float = 1.0e-5
    atol: float = 1.0e-8


def all_close(a, b, equal_nan=False, rtol=1.0e-5, atol=1.0e-8):
    """Nx.all_close/3 (nx.ex:9401-9452): |a - b| <= atol + rtol * |b| everywhere, infinities equal to
    themselves only, NaNs equal to each other on request.  Runs on the backend of its arguments,
    through block/4 like the reference."""
    a, b = to_tensor(a), to_tensor(b)

    def compose(o, x, y):
        both_int = T.is_integer(x.type) and T.is_integer(y.type)
        # abs of the lowest signed value overflows in its own width: widen first (nx.ex:9423-9427)
        abs_y = abs(as_type(y, "f64")) if both_int else abs(y)
        finite = less_equal(abs(subtract(x, y)), add(o.atol, multiply(o.rtol, abs_y)))
        if both_int:
            return all(finite)
        # inf - inf is a NaN, yet the two are equal: equal entries are checked as such
        entries = select(logical_or(is_infinity(x), is_infinity(y)), equal(x, y), finite)
        if o.equal_nan:
            entries = select(logical_and(is_nan(x), is_nan(y)), 1, entries)
        return all(entries)

    return block(BlockAllClose(equal_nan, rtol, atol), [a, b], template(("u", 8), ()), compose)


@dataclass(frozen=True)
class BlockLogicalNot:
    """%Nx.Block.LogicalNot{} (nx/lib/nx/block.ex)."""


def logical_not(t):
    """Nx.logical_not/1 (nx.ex:7345-7353): a block whose default body is `equal(t, 0)`; u8 output."""
    t = to_tensor(t)
    return block(BlockLogicalNot(), [t], template(("u", 8), t.shape), lambda _struct, x: equal(x, 0))


def block(struct, args, out, fun):
    """Nx.block/4 (nx.ex:7370-7380): lets the backend replace a composite op."""
    return _impl(*args).block(struct, out, list(args), fun)


def gather(t, indices, axes=None, **backend_opts):
    """Nx.gather/3 (nx.ex:15160-15203)."""
    t, indices = to_tensor(t), to_tensor(indices)
    if len(indices.shape) == 0:
        raise ValueError("expected indices rank to be at least 1, got: 0")
    if not T.is_integer(indices.type):
        raise ValueError(f"indices must be an integer tensor, got {indices.type!r}")
    depth = indices.shape[-1]
    axes = list(range(depth)) if axes is None else S.normalize_axes(t.shape, axes)
    if len(axes) != depth:
        raise ValueError(f"expected the last indices dimension size ({depth}) to match the number of axes")
    out = t.with_(data=None, shape=S.gather(t.shape, indices.shape, axes))
    return _impl(t, indices).gather(out, t, indices, dict(axes=axes, **backend_opts))


def take(t, indices, axis=0):
    """Nx.take/3 (nx.ex:14732-14821), non-vectorised path: wraps the default gather-based
    implementation in a `Nx.Block.Take` so a backend can do it natively."""
    t, indices = to_tensor(t), to_tensor(indices)
    if not T.is_integer(indices.type):
        raise ValueError(f"indices must be an integer tensor, got {indices.type!r}")
    axis = S.normalize_axis(t.shape, axis)
    inner_shape = S.take(t.shape, indices.shape, axis)
    out = t.with_(data=None, shape=inner_shape)

    def default(_struct, tensor_, indices_):
        gather_indices = new_axis(indices_, len(indices_.shape))
        n_idx = len(indices_.shape)
        all_axes = list(range(len(inner_shape)))
        indices_axes, tensor_axes = all_axes[:n_idx], all_axes[n_idx:]
        leading, trailing = tensor_axes[:axis], tensor_axes[axis:]
        return transpose(gather(tensor_, gather_indices, axes=[axis]), leading + indices_axes + trailing)

    return block(BlockTake(axis), [t, indices], out, default)


# ---- one step off the hot path: creation, selection, windows -------------------------------------

def all(t, axes=None, keep_axes=False):  # noqa: A001 - Nx.all/2 (nx.ex:9207-9209): u8 output
    return _aggregate(to_tensor(t), "all", ("u", 8), axes, keep_axes)


def any(t, axes=None, keep_axes=False):  # noqa: A001 - Nx.any/2 (nx.ex:9272-9274)
    return _aggregate(to_tensor(t), "any", ("u", 8), axes, keep_axes)


def iota(shape, type="s32", axis=None, backend=None):
    """Nx.iota/2 (nx.ex:1213-1260): counts along `axis`, or over the flattened tensor."""
    shape = tuple(shape)
    mod, opts = (backend, {}) if backend is not None and not isinstance(backend, tuple) else (backend or default_backend())
    if axis is not None:
        axis = S.normalize_axis(shape, axis)
    return mod.iota(template(type, shape), axis, opts)


def eye(n_or_shape, type="s32", backend=None):
    """Nx.eye/2 (nx.ex:1363-1420): identity matrices in the last two axes."""
    shape = (n_or_shape, n_or_shape) if isinstance(n_or_shape, int) else tuple(n_or_shape)
    if len(shape) < 2:
        raise ValueError(f"eye/2 expects a shape with at least 2 dimensions or an integer, got: {shape!r}")
    mod, opts = (backend, {}) if backend is not None and not isinstance(backend, tuple) else (backend or default_backend())
    return mod.eye(template(type, shape), opts)


def select(pred, on_true, on_false):
    """Nx.select/3 (nx.ex:7782-7830): the output takes the predicate's shape unless the predicate
    is a scalar, and the merged type of the two value operands."""
    pred, on_true, on_false = to_tensor(pred), to_tensor(on_true), to_tensor(on_false)
    out_type = T.binary_type(on_true.type, on_false.type)
    out_shape = S.binary_broadcast(on_true.shape, on_false.shape) if pred.shape == () else pred.shape
    for operand in (on_true, on_false):
        S.broadcast(operand.shape, out_shape, S.broadcast_axes(operand.shape, out_shape))
    return _impl(pred, on_true, on_false).select(template(out_type, out_shape), pred, on_true, on_false)


def clip(t, min, max):  # noqa: A002 - Nx.clip/3 (nx.ex:13973-14000)
    t, min, max = to_tensor(t), to_tensor(min), to_tensor(max)
    if min.shape != ():
        raise ValueError(f"min value must be a non-vectorized scalar shape, got shape {min.shape!r}")
    if max.shape != ():
        raise ValueError(f"max value must be a non-vectorized scalar shape, got shape {max.shape!r}")
    out_type = T.merge(t.type, T.merge(min.type, max.type))
    return _impl(t, min, max).clip(t.with_(data=None, type=out_type), t, min, max)


def pad(t, pad_value, padding_config):
    """Nx.pad/3 (nx.ex:4233-4250; shape rule shape.ex:1038-1071): (low, high, interior) per axis;
    negative edges crop, interior padding must be non-negative."""
    t = to_tensor(t)
    # the type is merged before the number becomes a tensor (nx.ex:4237-4238): a bf16 tensor padded with 0.0 stays bf16
    out_type = T.binary_type(t.type, pad_value if isinstance(pad_value, (int, float)) and not isinstance(pad_value, bool) else to_tensor(pad_value).type)
    pad_value = to_tensor(pad_value)
    if pad_value.shape != ():
        raise ValueError("padding value must be a scalar and non-vectorized")
    padding_config = [tuple(c) for c in padding_config]
    if len(padding_config) != len(t.shape):
        raise ValueError("invalid padding configuration, rank of padding configuration and shape must match")
    dims = []
    for dim, (low, high, interior) in zip(t.shape, padding_config):
        if interior < 0:
            raise ValueError("invalid padding configuration, interior padding must be non-negative")
        dims.append(dim + (dim - 1) * interior + low + high)
    return _impl(t, pad_value).pad(template(out_type, tuple(dims)), t, pad_value, padding_config)


def slice(t, start_indices, lengths, strides=1):  # noqa: A001 - Nx.slice/4 (nx.ex:14203-14290)
    t = to_tensor(t)
    start_indices, lengths = list(start_indices), list(lengths)
    if t.shape == () and not start_indices and not lengths:
        return t
    rank = len(t.shape)
    strides = [strides] * rank if isinstance(strides, int) else list(strides)
    if len(strides) != rank:
        raise ValueError(f"invalid strides rank for shape of rank {rank}")
    if len(start_indices) != rank:
        raise ValueError(f"invalid start indices rank for shape of rank {rank}")
    if len(lengths) != rank:
        raise ValueError(f"invalid limit indices rank for shape of rank {rank}")
    out_shape, starts = [], []
    for pos, (i, length, s) in enumerate(zip(start_indices, lengths, strides)):  # Nx.Shape.slice (shape.ex:1110-1164)
        dim = t.shape[pos]
        if not isinstance(length, int) or length < 1:
            raise ValueError(f"length at axis {pos} must be greater than or equal to 1, got: {length!r}")
        if not isinstance(s, int) or s < 1:
            raise ValueError(f"stride at axis {pos} must be greater than or equal to 1, got: {s!r}")
        if length > dim:
            raise ValueError(f"length at axis {pos} must be less than axis size of {dim}, got: {length}")
        out_shape.append(-(-length // s))
        starts.append(builtins.min(i, dim - length) if isinstance(i, int) else i)
    return _impl(t).slice(t.with_(data=None, shape=tuple(out_shape)), t, starts, lengths, strides)


def reverse(t, axes=None):
    """Nx.reverse/2 (nx.ex:13527-13543): all axes by default; no axes, no work."""
    t = to_tensor(t)
    axes = list(range(len(t.shape))) if axes is None else S.normalize_axes(t.shape, axes)
    if not axes:
        return t
    return _impl(t).reverse(t.with_(data=None), t, sorted(axes))


def put_slice(t, start_indices, slice_t):
    """Nx.put_slice/3 (nx.ex:14491-14530; shape rule shape.ex:1304-1345): the slice has the rank of
    the tensor and fits inside it; start indices are numbers or rank-0 integer tensors."""
    t, slice_t = to_tensor(t), to_tensor(slice_t)
    start_indices = list(start_indices)
    rank = len(t.shape)
    if len(start_indices) != rank:
        raise ValueError(f"invalid start indices rank for shape of rank {rank}")
    if len(slice_t.shape) != rank:
        raise ValueError(f"invalid slice for put_slice, rank of slice must match {rank}, got: {len(slice_t.shape)}")
    if builtins.any(s > d for s, d in zip(slice_t.shape, t.shape)):
        raise ValueError(f"slice shape {S.fmt(slice_t.shape)} must be less than or equal to tensor shape {S.fmt(t.shape)}")
    for i in start_indices:
        if isinstance(i, Tensor) and (i.shape != () or not T.is_integer(i.type)):
            raise ValueError("index must be an integer or a scalar integer tensor")
    out = t.with_(data=None, type=T.binary_type(t.type, slice_t.type))
    operands = [t, slice_t] + [i for i in start_indices if isinstance(i, Tensor)]
    return _impl(*operands).put_slice(out, t, start_indices, slice_t)


def slice_along_axis(t, start_index, length, axis=0, strides=1):
    """Nx.slice_along_axis/4 (nx.ex:14391-14420)."""
    t = to_tensor(t)
    axis = S.normalize_axis(t.shape, axis)
    rank = len(t.shape)
    starts = [0] * rank
    lengths = list(t.shape)
    steps = [1] * rank
    starts[axis], lengths[axis], steps[axis] = start_index, length, strides
    return slice(t, starts, lengths, steps)


def _concat_type_and_operands(tensors):
    tensors = [to_tensor(t) for t in tensors]
    if not tensors:
        raise ValueError("no tensors were given to concatenate")
    out_type = tensors[0].type
    for t in tensors[1:]:
        out_type = T.merge(out_type, t.type)
    return out_type, tensors


def concatenate(tensors, axis=0):
    """Nx.concatenate/2 (nx.ex:15343-15362; Nx.Shape.concatenate shape.ex:1713-1760)."""
    out_type, tensors = _concat_type_and_operands(tensors)
    if len(tensors) == 1:
        return tensors[0]
    first = tensors[0].shape
    axis = S.normalize_axis(first, axis)
    total = 0
    for t in tensors:
        if len(t.shape) != len(first) or builtins.any(a != b for pos, (a, b) in enumerate(zip(t.shape, first)) if pos != axis):
            raise ValueError("expected all shapes to match " + repr(first) + ", except for the axis of concatenation, got "
                             "unmatching shape: " + repr(t.shape))
        total += t.shape[axis]
    out_shape = first[:axis] + (total,) + first[axis + 1:]
    return _impl(*tensors).concatenate(template(out_type, out_shape), tensors, axis)


def stack(tensors, axis=0):
    """Nx.stack/2 (nx.ex:15502-15520; Nx.Shape.stack shape.ex:1689-1711): a new axis of the
    operands' count at `axis`."""
    out_type, tensors = _concat_type_and_operands(tensors)
    first = tensors[0].shape
    for t in tensors:
        if t.shape != first:
            raise ValueError(f"can only stack tensors of the same shape, got shapes {first!r} and {t.shape!r}")
    axis = S.normalize_axis(first + (1,), axis)
    out_shape = first[:axis] + (len(tensors),) + first[axis:]
    return _impl(*tensors).stack(template(out_type, out_shape), tensors, axis)
