"""Traced functions and their evaluator: the caller one step above the backend callbacks.

Host-side mirror of `Nx.Defn.jit` with the default compiler (reference:
nx/lib/nx/defn/compiler.ex:159-205, nx/lib/nx/defn/expr.ex, nx/lib/nx/defn/evaluator.ex).
`jit(fun)` runs `fun` once on *expressions* -- tensors whose data is an `Expr` node, built by the
`Expr` backend while the front end does its usual shape and type work -- and then walks the graph,
calling the callbacks of the backend the arguments live on (`eval_apply`, evaluator.ex:363-388).

Two things of the reference are kept because they change results or memory:
  * the expression builder rewrites sums and products with constant operands and folds
    operations on constants (expr.ex:889-984, 1597-1674).  Float arithmetic does not associate, so a
    traced `c * (k * x)` really is `(c*k) * x` in the reference, and here.
  * every node is evaluated once and dropped after its last use (reference counts per scope,
    evaluator.ex:86-210, 213-262), so device buffers of intermediates return to the pool as the
    walk proceeds.
Control flow: `while_loop` and `cond` build `:while` / `:cond` nodes whose bodies are scopes of
their own; outside a trace they run eagerly.
"""
from __future__ import annotations

import math
import itertools
import operator
import threading
from math import prod
from typing import Any, Callable, Dict, List, Optional, Tuple

import numpy as np

from . import nx as Nx
from . import types as T
from .backend_names import BINARY_OPS, UNARY_OPS
from .host import HostBinary
from .tensor import Tensor, binary_to_numpy, template

_ids = itertools.count(1)
_trace = threading.local()  # .scopes: stack of scope tags of the trace in progress


class _ExprMeta(type):
    """Any callback name not written out below builds a plain node `op(out, *args)`."""

    def __getattr__(cls, op):
        if op.startswith("_"):
            raise AttributeError(op)

        def build(out, *args):
            return cls._expr(out, op, [_to_expr_arg(a) for a in args])
        build.__name__ = op
        return build


class Expr(metaclass=_ExprMeta):
    """%Nx.Defn.Expr{id, op, args} (expr.ex:1-60) and, as a class, the backend that builds them."""

    __slots__ = ("id", "op", "args", "scope")

    def __init__(self, id, op, args, scope):  # noqa: A002
        self.id, self.op, self.args, self.scope = id, op, args, scope

    def __repr__(self):
        return f"Expr<{self.op} #{self.id}>"

    # ---- construction ------------------------------------------------------------------------
    @classmethod
    def init(cls, opts=None):
        return {}

    @classmethod
    def _expr(cls, out: Tensor, op: str, args: list) -> Tensor:
        scopes = getattr(_trace, "scopes", None)
        if not scopes:
            raise RuntimeError("expressions can only be built while a function is being traced")
        return out.with_(data=Expr(next(_ids), op, args, scopes[-1]))

    @classmethod
    def _constant(cls, out: Tensor, number) -> Tensor:
        # expr.ex:1553-1576: integers become floats in a float type; a non-integer has no integer form
        if T.is_float(out.type):
            number = float(number)
        elif not isinstance(number, (int, np.integer)) or isinstance(number, bool):
            raise ValueError(f"value {number!r} is not valid for constant of type {out.type!r}")
        else:
            number = int(number)
        return out.with_(data=Expr(("c", repr(number), out.type, out.shape), "constant", [number], None))

    # creation callbacks (expr.ex:851-871)
    @classmethod
    def constant(cls, out, number, opts=None):
        return cls._constant(out, number)

    @classmethod
    def from_binary(cls, out, binary, opts=None):
        return to_expr(HostBinary.from_binary(out, binary, {}))

    @classmethod
    def iota(cls, out, axis, opts=None):
        return cls._expr(out, "iota", [axis])

    @classmethod
    def eye(cls, out, opts=None):
        return cls._expr(out, "eye", [])

    @classmethod
    def to_binary(cls, t, limit):
        raise ValueError("cannot read the value of a tensor expression: it has no data while the function is being traced")

    @classmethod
    def backend_transfer(cls, t, backend, opts=None):
        raise ValueError("cannot transfer a tensor expression between backends")

    backend_copy = backend_transfer

    @classmethod
    def backend_deallocate(cls, t):
        return "already_deallocated"

    # ---- rewrites of the arithmetic with constants (expr.ex:889-984) ---------------------------
    @classmethod
    def add(cls, out, t1, t2):
        t1, t2 = to_expr(t1), to_expr(t2)
        c1, c2 = _const(t1), _const(t2)
        if c1 is not None and c1 == 0:
            return _ensure_compatible(t2, out)
        if c2 is not None and c2 == 0:
            return _ensure_compatible(t1, out)
        if c2 is not None:
            return cls._commute(out, "add", operator.add, c2, t2, t1)
        inner = _node(t2, "subtract")
        if inner is not None and _const(inner[0]) is not None and _const(inner[0]) == 0:
            return cls._binary_expr(out, "subtract", t1, inner[1])  # a + (0 - b) = a - b
        return cls._commute(out, "add", operator.add, c1, t1, t2)

    @classmethod
    def subtract(cls, out, t1, t2):
        t1, t2 = to_expr(t1), to_expr(t2)
        c1, c2 = _const(t1), _const(t2)
        if c2 is not None and c2 == 0:
            return _ensure_compatible(t1, out)
        if c1 is not None and c2 is not None:
            return cls._constant(out, c1 - c2)
        return cls._binary_expr(out, "subtract", t1, t2)

    @classmethod
    def multiply(cls, out, t1, t2):
        t1, t2 = to_expr(t1), to_expr(t2)
        c1, c2 = _const(t1), _const(t2)
        if c1 is not None and c1 == 1:
            return _ensure_compatible(t2, out)
        if c2 is not None and c2 == 1:
            return _ensure_compatible(t1, out)
        if c2 is not None:
            return cls._commute(out, "multiply", operator.mul, c2, t2, t1)
        inner = _node(t2, "divide")
        if inner is not None and _const(inner[0]) is not None and _const(inner[0]) == 1:
            return cls._binary_expr(out, "divide", t1, inner[1])  # a * (1 / b) = a / b
        return cls._commute(out, "multiply", operator.mul, c1, t1, t2)

    @classmethod
    def divide(cls, out, t1, t2):
        t1, t2 = to_expr(t1), to_expr(t2)
        c2 = _const(t2)
        if c2 is not None and c2 == 1:
            return _ensure_compatible(t1, out)
        return cls._binary_expr(out, "divide", t1, t2)

    @classmethod
    def pow(cls, out, t1, t2):  # noqa: A003
        t1, t2 = to_expr(t1), to_expr(t2)
        c2 = _const(t2)
        if c2 is not None and c2 == 1:
            return _ensure_compatible(t1, out)
        return cls._binary_expr(out, "pow", t1, t2)

    @classmethod
    def _commute(cls, out, op, fun, s1, t1, t2):
        """expr.ex:1597-1621: the constant of a commutative chain moves to the left, two constants
        merge (in host arithmetic, not rounded to the tensor type until the constant is used)."""
        scalar = out.with_(data=None, shape=())
        a1, a2 = t1, t2
        inner2, inner1 = _node(t2, op), _node(t1, op)
        if inner2 is not None and _const(inner2[0]) is not None:
            s2, t3 = _const(inner2[0]), inner2[1]
            if s1 is not None:
                a1, a2 = cls._constant(scalar, fun(s1, s2)), Nx.broadcast(t3, out.shape)
            else:
                a1, a2 = cls._constant(scalar, s2), Nx.broadcast(getattr(Nx, op)(t1, t3), out.shape)
        elif inner1 is not None and _const(inner1[0]) is not None:
            a1, a2 = cls._constant(scalar, _const(inner1[0])), Nx.broadcast(getattr(Nx, op)(t2, inner1[1]), out.shape)
        return cls._binary_expr(out, op, a1, a2)

    @classmethod
    def _binary_expr(cls, out, op, a1, a2):
        c1, c2 = _const(a1), _const(a2)
        if c1 is not None and c2 is not None:  # expr.ex:1628-1635: folded by a compute backend
            backend, opts = _fold_backend()
            scalar = out.with_(data=None, shape=())
            left = backend.constant(template(a1.type, ()), c1, opts)
            right = backend.constant(template(a2.type, ()), c2, opts)
            return cls._constant(out, _to_number(getattr(backend, op)(scalar, left, right)))
        if c1 is not None:
            a1 = _upcast_float_constant(a1, out.type)
        elif c2 is not None:
            a2 = _upcast_float_constant(a2, out.type)
        return cls._expr(out, op, [a1, a2])

    @classmethod
    def _unary_expr(cls, out, op, t):
        t = to_expr(t)
        c = _const(t)
        if c is None:
            return cls._expr(out, op, [t])
        backend, opts = _fold_backend()  # expr.ex:1666-1674
        value = backend.constant(template(t.type, ()), c, opts)
        return cls._constant(out, _to_number(getattr(backend, op)(out.with_(data=None, shape=()), value)))

    # ---- shape callbacks with their collapses (expr.ex:1088-1145) -------------------------------
    @classmethod
    def squeeze(cls, out, t, axes):
        t = to_expr(t)
        inner = _node(t, "squeeze")
        if inner is not None:  # a squeeze of a squeeze is one squeeze (keeps `t[i][j]` one node)
            return cls._expr(out, "squeeze", [inner[0], _merge_squeeze(sorted(inner[1]), sorted(axes), 0)])
        return cls._expr(out, "squeeze", [t, list(axes)])

    @classmethod
    def broadcast(cls, out, t, shape, axes):
        t = to_expr(t)
        inner = _node(t, "broadcast")
        if inner is not None:
            inner_t, inner_shape, inner_axes = inner
            first = _contiguous(inner_axes, 0) and _contiguous(axes, 0)
            last = (_contiguous(inner_axes, len(inner_shape) - len(inner_t.shape))
                    and _contiguous(axes, len(shape) - len(t.shape)))
            if first or last:
                return cls._expr(out, "broadcast", [inner_t, tuple(shape), list(inner_axes)])
        c = _const(t)
        if c is not None:
            return cls._constant(out, c)
        return cls._expr(out, "broadcast", [t, tuple(shape), list(axes)])

    @classmethod
    def block(cls, struct, out, args, fun):
        # expr.ex:824-842, without re-tracing the default implementation: the evaluator hands the
        # node to the backend's block/4, which runs `fun` on its own callbacks when it has no kernel
        return cls._expr(out, "block", [struct, [to_expr(a) for a in args], fun])


def _install():
    for op in BINARY_OPS:
        if op not in ("add", "subtract", "multiply", "divide", "pow"):
            def binary(out, t1, t2, _op=op):
                return Expr._binary_expr(out, _op, to_expr(t1), to_expr(t2))
            binary.__name__ = op
            setattr(Expr, op, staticmethod(binary))
    for op in list(UNARY_OPS) + ["as_type", "bitcast"]:
        def unary(out, t, _op=op):
            return Expr._unary_expr(out, _op, t)
        unary.__name__ = op
        setattr(Expr, op, staticmethod(unary))


_install()


# ---- helpers of the builder ---------------------------------------------------------------------

def _const(t) -> Optional[Any]:
    return t.data.args[0] if isinstance(t, Tensor) and isinstance(t.data, Expr) and t.data.op == "constant" else None


def _node(t, op) -> Optional[list]:
    return t.data.args if isinstance(t, Tensor) and isinstance(t.data, Expr) and t.data.op == op else None


def _contiguous(axes, start) -> bool:
    return list(axes) == list(range(start, start + len(axes)))


def _merge_squeeze(inner, axes, extra):  # expr.ex:1112-1121
    if inner and axes and inner[0] <= axes[0] + extra:
        return [inner[0]] + _merge_squeeze(inner[1:], axes, extra + 1)
    if axes:
        return [axes[0] + extra] + _merge_squeeze(inner, axes[1:], extra)
    return []


def _ensure_compatible(t, out):  # expr.ex:1589-1594
    return Nx.broadcast(Nx.as_type(t, out.type), out.shape)


def _upcast_float_constant(t, out_type):  # expr.ex:1648-1664
    if T.is_float(t.type) and T.is_float(out_type):
        return Expr._constant(t.with_(data=None, type=out_type), _const(t))
    return t


def _to_number(t: Tensor):
    value = binary_to_numpy(Nx.to_binary(t), t.type, ())
    if t.type == ("bf", 16):
        value = (np.asarray(value, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)
    return np.asarray(value).reshape(()).item()


def _fold_backend():
    """Where operations on constants are computed while tracing.  The reference folds on its host
    backend; here the backend that was the default when the trace began does it, or the device when
    that default only stores data."""
    mod, opts = getattr(_trace, "fold", None) or (None, None)
    if mod is None or mod is HostBinary or mod is Expr:
        from .backend import HipNxBackend
        return HipNxBackend, HipNxBackend.init({})
    return mod, opts


def to_expr(value) -> Tensor:
    """expr.ex:1349-1376: expressions pass, host tensors become constants (rank 0) or literals,
    numbers become constants; a tensor of a compute backend cannot be captured."""
    if isinstance(value, Tensor):
        if isinstance(value.data, Expr):
            return value
        if isinstance(value.data, HostBinary):
            if value.shape == ():
                return Expr._constant(value.with_(data=None), _to_number(value))
            return Expr._expr(value.with_(data=None), "tensor", [value])
        raise ValueError(
            f"cannot convert tensor allocated on {type(value.data).__name__} to an expression. This may mean you "
            "are passing a tensor to a traced function as a closure; pass it as an argument instead")
    if isinstance(value, (bool, int, float, np.integer, np.floating)):
        v = value.item() if isinstance(value, np.generic) else value
        return Expr._constant(template(T.infer(v), ()), v)
    raise ValueError(f"unable to build tensor expression, expected a tensor or a number, got: {value!r}")


def _to_expr_arg(a):
    if isinstance(a, Tensor):
        return to_expr(a)
    if isinstance(a, (list, tuple)) and any(isinstance(x, Tensor) for x in a):
        return [to_expr(x) if isinstance(x, Tensor) else x for x in a]
    return a


# ---- composites -----------------------------------------------------------------------------------

def _flatten(value, leaves: list):
    """Nested tuples / lists / dicts of tensors -> a structure of leaf positions."""
    if isinstance(value, (tuple, list)):
        return type(value)(_flatten(v, leaves) for v in value)
    if isinstance(value, dict):
        return {k: _flatten(v, leaves) for k, v in value.items()}
    leaves.append(value)
    return _Leaf(len(leaves) - 1)


class _Leaf:
    __slots__ = ("index",)

    def __init__(self, index):
        self.index = index


def _unflatten(structure, leaves):
    if isinstance(structure, (tuple, list)):
        return type(structure)(_unflatten(v, leaves) for v in structure)
    if isinstance(structure, dict):
        return {k: _unflatten(v, leaves) for k, v in structure.items()}
    return leaves[structure.index]


# ---- control flow ---------------------------------------------------------------------------------

def _tracing() -> bool:
    return bool(getattr(_trace, "scopes", None))


def _push_scope():
    tag = next(_ids)
    _trace.scopes.append(tag)
    return tag


def while_loop(initial, condition: Callable, body: Callable):
    """`while` of Nx.Defn.Kernel (expr.ex:306-420): `condition(state)` is a rank-0 tensor,
    `body(state)` returns a state of the same structure, shapes and types.  Everything the two use
    must come in through `state`."""
    if not _tracing():
        state = initial
        while _to_number(Nx.to_tensor(condition(state))) != 0:
            state = body(state)
        return state
    leaves: list = []
    structure = _flatten(initial, leaves)
    initial_exprs = [to_expr(Nx.to_tensor(v)) for v in leaves]
    tag = _push_scope()
    try:
        params = [Expr._expr(t.with_(data=None), "parameter", [i]) for i, t in enumerate(initial_exprs)]
        state = _unflatten(structure, params)
        pred = to_expr(Nx.to_tensor(condition(state)))
        if pred.shape != ():
            raise ValueError(f"condition must be a scalar tensor, got shape {pred.shape!r}")
        out_leaves: list = []
        out_structure = _flatten(body(state), out_leaves)
        out_exprs = [to_expr(Nx.to_tensor(v)) for v in out_leaves]
    finally:
        _trace.scopes.pop()
    if len(out_exprs) != len(initial_exprs) or any(
            (a.type, a.shape) != (b.type, b.shape) for a, b in zip(initial_exprs, out_exprs)):
        raise ValueError("the body of while must return tensors with the same shape and type as the initial arguments")
    del out_structure
    node = Expr(next(_ids), "while", [initial_exprs, pred, out_exprs, tag], _trace.scopes[-1])
    results = [Expr._expr(t.with_(data=None), "elem", [node, i]) for i, t in enumerate(initial_exprs)]
    return _unflatten(structure, results)


def cond(pred, on_true: Callable, on_false: Callable):
    """`cond` / `if` of Nx.Defn.Kernel (expr.ex:139-300): only the chosen branch is evaluated.
    The branches are thunks returning composites of the same structure, shapes and types."""
    if not _tracing():
        return on_true() if _to_number(Nx.to_tensor(pred)) != 0 else on_false()
    pred = to_expr(Nx.to_tensor(pred))
    if pred.shape != ():
        raise ValueError(f"condition must be a scalar tensor, got shape {pred.shape!r}")
    branches = []
    for thunk in (on_true, on_false):
        tag = _push_scope()
        try:
            leaves: list = []
            structure = _flatten(thunk(), leaves)
            branches.append((tag, structure, [to_expr(Nx.to_tensor(v)) for v in leaves]))
        finally:
            _trace.scopes.pop()
    (_, structure, first), (_, _, second) = branches
    if len(first) != len(second) or any((a.type, a.shape) != (b.type, b.shape) for a, b in zip(first, second)):
        raise ValueError("cond expects all branches to return compatible tensor types")
    node = Expr(next(_ids), "cond", [pred, [(tag, exprs) for tag, _, exprs in branches]], _trace.scopes[-1])
    results = [Expr._expr(t.with_(data=None), "elem", [node, i]) for i, t in enumerate(first)]
    return _unflatten(structure, results)


# ---- fusion of element-wise groups --------------------------------------------------------------------
# The reference's evaluator knows one granularity: a callback per node.  A backend that offers
# `fused_elementwise` is handed whole groups of element-wise nodes instead (one pass over memory,
# intermediates in registers, each still rounded to its node's type: same bits as node by node).
# Opt-in (`compile(..., fuse=True)`), root scope only; a group that does not fit the kernel's
# limits, or a backend without the entry point, is evaluated node by node as before.

_NARROW = (("bf", 16), ("f", 16), ("f", 32))
_TRUTH = ("u", 8)
_INT_ONLY_BINARY = ("quotient", "bitwise_and", "bitwise_or", "bitwise_xor", "left_shift", "right_shift")
_INT_ONLY_UNARY = ("bitwise_not", "count_leading_zeros", "population_count")
_COMPARE = ("equal", "not_equal", "greater", "less", "greater_equal", "less_equal")
_LOGICAL = ("logical_and", "logical_or", "logical_xor")
_EXACT_WITH_INT_CONSTANT = ("add", "subtract", "multiply", "divide", "min", "max") + _COMPARE
_INT32 = (("u", 32), ("s", 32))
_WORD = _INT32 + (("f", 32),)
# with `fuse="compiled"` a group may also compute on 32-bit integers (held as raw bits, wrapping like
# the integer kernels) and relabel 32-bit values: what Nx.Random's bits-to-floats chains are made of
_INT_FUSED_BINARY = ("add", "subtract", "multiply", "bitwise_and", "bitwise_or", "bitwise_xor", "left_shift",
                     "right_shift", "min", "max")
_INT_FUSED_UNARY = ("negate", "bitwise_not")
_plan = {"ints": False}
_SAVED_SLOTS, _MAX_INSTR, _MAX_INPUTS = 3, 32, 8
_REDUCE_CODES = {"sum": 0, "reduce_max": 1, "reduce_min": 2}  # HIPNX_RED_SUM / MAX / MIN
_EUNSUPPORTED = 7


def _fusable(t: Tensor) -> bool:
    """Whether the node computes in the f32 class of the element-wise kernels with operands and a
    result the fused kernel holds exactly."""
    e = t.data
    op, args = e.op, e.args
    if _plan["ints"]:
        if op in _INT_FUSED_BINARY and t.type in _INT32:
            if op in ("left_shift", "right_shift") and (_const(args[1]) is None or _const(args[1]) < 0):
                return False  # a negative count raises in the reference: only the separate kernel reports it
            def word_ok(a):
                if _const(a) is None:
                    return a.type == t.type
                c = _const(a)
                return T.is_integer(a.type) and float(c).is_integer() and (a.type == t.type or 0 <= c < 1 << 31)
            return all(word_ok(a) for a in args)
        if op in _INT_FUSED_UNARY and t.type in _INT32:
            return args[0].type == t.type and _const(args[0]) is None
        if op == "bitcast":
            return t.type in _WORD and args[0].type in _WORD and _const(args[0]) is None

    def value_ok(a, binary_op=None):
        if _const(a) is not None:
            if a.type in _NARROW:
                return True
            c = _const(a)
            return binary_op in _EXACT_WITH_INT_CONSTANT and T.is_integer(a.type) and abs(c) <= 1 << 24
        return a.type in _NARROW

    if op in UNARY_OPS and op not in _INT_ONLY_UNARY:
        out_ok = t.type == _TRUTH if op in ("is_nan", "is_infinity") else t.type in _NARROW
        return out_ok and value_ok(args[0])
    if op in BINARY_OPS and op not in _INT_ONLY_BINARY:
        if op == "remainder" and not (_const(args[1]) is not None and _const(args[1]) != 0 and math.isfinite(_const(args[1]))):
            return False  # :math.fmod raises for a zero divisor or a non-finite element: left to the separate kernel
        if op in _LOGICAL:
            return t.type == _TRUTH and all(a.type in _NARROW or a.type == _TRUTH for a in args)
        out_ok = t.type == _TRUTH if op in _COMPARE else t.type in _NARROW
        return out_ok and all(value_ok(a, op) for a in args)
    if op == "as_type":
        src = args[0].type
        if t.type == ("bf", 16):
            from .backend import _bf16
            if _bf16["rounding"] != "truncate":
                return False  # only the separate kernel rounds to nearest even (the setting when the function is compiled counts)
        return t.type in _NARROW and (src in _NARROW or (T.is_integer(src) and src[1] <= 32)) and _const(args[0]) is None
    if op == "select":
        pred, on_true, on_false = args
        return (t.type in _NARROW and (pred.type in _NARROW or pred.type == _TRUTH) and _const(pred) is None
                and value_ok(on_true) and value_ok(on_false))
    return False


def _layout(out_shape, in_shapes, split=None):
    """The index space as [rows, cols] with a (row stride, column stride) per input, or None: an
    input is the full shape, one value, one row shared by all rows, or one value per row.  `split`
    fixes the axis where the columns begin (a reduction over the last axis needs the rows it
    reduces)."""
    rank = len(out_shape)
    padded = [(1,) * (rank - len(s)) + tuple(s) for s in in_shapes]
    for p in (range(rank + 1) if split is None else [split]):
        rows, cols = prod(out_shape[:p]), prod(out_shape[p:])
        if cols % 8 and not (_plan["ints"] and split is None and p == 0):
            continue  # whole vectors of 8 along a row; a compiled kernel over a flat index space takes a partial last one
        strides = []
        for s in padded:
            outer, inner = s[:p], s[p:]
            dense_inner, one_inner = inner == tuple(out_shape[p:]), all(d == 1 for d in inner)
            dense_outer, one_outer = outer == tuple(out_shape[:p]), all(d == 1 for d in outer)
            if not (dense_inner or one_inner) or not (dense_outer or one_outer):
                break
            cs = 1 if dense_inner and cols > 1 else 0
            rs = (cols if cs else 1) if dense_outer and rows > 1 else 0
            if cs and rows > 1 and rs % 8:
                break
            strides.append((rs, cs))
        else:
            return rows, cols, strides
    return None


class _Program(list):
    """A group's instructions; a backend may keep its packed form of them here after the first launch."""
    packed = None


class _Group:
    """One fused group: the member nodes in evaluation order, its external inputs, and the program
    for the backend's accumulator machine (None when the group does not fit it)."""

    def __init__(self, root: Tensor, members: List[Tensor], inputs: List[Tensor]):
        self.root, self.members, self.inputs = root, members, inputs
        # planned for compiled execution (integer instructions allowed): ask the backend for that mode
        self.how = {"mode": "compiled"} if _plan["ints"] else {}
        self.program = self._assemble()
        self.layout = _layout(root.shape, [t.shape for t in inputs]) if self.program else None
        self.reduce = None  # (callback name, opts, rows layout) when a reduction of the result is part of the group

    def with_reduction(self, name: str, opts) -> Optional["_Group"]:
        """This group followed by `name` over the last axis of its result, or None when the
        backend kernel cannot take it (the reduction then stays a node of its own)."""
        rank = len(self.root.shape)
        if not self.program or rank == 0 or self.root.type not in _NARROW:
            return None
        rows_layout = _layout(self.root.shape, [t.shape for t in self.inputs], split=rank - 1)
        if rows_layout is None or rows_layout[1] == 0:
            return None
        both = object.__new__(_Group)
        both.__dict__.update(self.__dict__)
        both.reduce = (name, dict(opts), rows_layout)
        return both

    def _assemble(self):
        """Linear code for the accumulator machine: each member combines the value computed just
        before it (the accumulator) with one other operand; a value that is needed later than that
        is saved in one of three slots, and fetched back (SET) when the accumulator holds
        something else."""
        member_ids = {m.data.id: i for i, m in enumerate(self.members)}
        input_ids = {t.data.id: k for k, t in enumerate(self.inputs)}
        if len(self.inputs) > _MAX_INPUTS:
            return None
        # where each member's value is read: (reader index, operand position)
        readers: Dict[Any, List[int]] = {}
        for i, m in enumerate(self.members):
            for a in m.data.args:
                if isinstance(a, Tensor) and a.data.id in member_ids:
                    readers.setdefault(a.data.id, []).append(i)
        slots: Dict[Any, int] = {}       # member id -> slot while it is saved
        free = list(range(_SAVED_SLOTS))
        program: List[dict] = _Program()

        def source(a, raw=False):
            """(src, arg, imm) of an operand that is not the accumulator; `raw`: for an integer
            instruction (a constant is then the bits of the integer, marked by a str)."""
            if _const(a) is not None:
                return 0, 0, (str(int(_const(a)) & 0xFFFFFFFF) if raw else _imm(a))
            if a.data.id in input_ids:
                return 1, input_ids[a.data.id], 0.0
            return 2, slots[a.data.id], 0.0

        def with_imm(ins, imm):
            if isinstance(imm, str):
                ins["imm_bits"] = int(imm)
            else:
                ins["imm"] = imm
            return ins

        for i, m in enumerate(self.members):
            operands = [a for a in m.data.args if isinstance(a, Tensor)]
            prev = self.members[i - 1].data.id if i else None

            def is_acc(a):
                return prev is not None and _const(a) is None and a.data.id == prev

            op = m.data.op
            ints = m.type in _INT32 and (op in _INT_FUSED_BINARY or op in _INT_FUSED_UNARY)
            # an integer held as bits that a conversion reads (an integer *input* is converted as it is loaded)
            from_bits = op == "as_type" and operands[0].type in _INT32 and operands[0].data.id in member_ids
            raw = ints or op == "bitcast" or from_bits
            if op == "select":
                want_acc = [0]           # the predicate
            elif op in BINARY_OPS:
                want_acc = [0, 1]
            else:
                want_acc = [0]
            pos = next((p for p in want_acc if is_acc(operands[p])), None)
            if pos is None:  # the accumulator holds something else: fetch the operand
                pos = want_acc[0]
                first = operands[pos]
                if first.data.id in member_ids and _const(first) is None and first.data.id not in slots:
                    return None          # cannot happen: a member read later than next is saved below
                src, arg, imm = source(first, raw)
                keeps = first.type in _NARROW or first.type == _TRUTH or (raw and first.type in _INT32)
                program.append(with_imm({"kind": 0, "src": src, "arg": arg, "flags": 2 if raw else 0,
                                         "dt": first.type if keeps else ("f", 32)}, imm))
            others = [a for p, a in enumerate(operands) if p != pos]
            if any(_const(o) is None and o.data.id in member_ids and o.data.id not in slots for o in others):
                return None              # an operand that is neither the accumulator nor saved: cannot happen
            ins = {"dt": m.type}
            if op == "bitcast":
                ins.update(kind=5)
            elif op in UNARY_OPS:
                ins.update(kind=1, op=UNARY_OPS.index(op), flags=2 if ints else 0)
            elif op in BINARY_OPS:
                src, arg, imm = source(others[0], ints)
                with_imm(ins, imm).update(kind=2, op=BINARY_OPS.index(op), src=src, arg=arg,
                                          flags=(1 if pos == 1 else 0) | (2 if ints else 0))
            elif op == "select":
                (s1, a1, i1), (s2, a2, i2) = source(others[0]), source(others[1])
                ins.update(kind=3, src=s1, arg=a1, imm=i1, src2=s2, arg2=a2, imm2=i2)
            elif from_bits:
                ins.update(kind=4, op=T.code(operands[0].type), flags=2)
            else:
                ins.update(kind=4)
            # slots whose value was read for the last time here are free again
            for a in operands:
                if _const(a) is None and a.data.id in slots and max(readers[a.data.id]) == i:
                    free.insert(0, slots.pop(a.data.id))
            # does this result outlive the next instruction's accumulator read?
            later = [r for r in readers.get(m.data.id, []) if r != i + 1]
            next_reads = i + 1 < len(self.members) and (i + 1) in readers.get(m.data.id, [])
            next_op = self.members[i + 1].data if i + 1 < len(self.members) else None
            # the next member can only take it from the accumulator in an operand position it accepts
            takes_acc = False
            if next_reads:
                nxt_operands = [a for a in next_op.args if isinstance(a, Tensor)]
                accept = [0] if next_op.op == "select" or next_op.op not in BINARY_OPS else [0, 1]
                hits = [p for p, a in enumerate(nxt_operands) if _const(a) is None and a.data.id == m.data.id]
                takes_acc = len(hits) == 1 and hits[0] in accept
            if later or (next_reads and not takes_acc):
                if not free:
                    return None
                slot = free.pop(0)
                slots[m.data.id] = slot
                ins["flags"] = ins.get("flags", 0) | ((slot + 1) << 4)
            program.append(ins)
            if len(program) > _MAX_INSTR:
                return None
        return program

    def run(self, run: "_Run", out: Tensor, values: List[Tensor]):
        mod = run.pick(values)
        fused = getattr(mod, "fused_elementwise", None) if self.program and self.layout else None
        if self.reduce is not None:
            name, opts, rows_layout = self.reduce
            if fused is not None:
                try:
                    return fused(out, self.program, values, rows_layout, _REDUCE_CODES[name], **self.how)
                except Exception as e:  # a shape the kernel leaves to the separate reduction
                    if getattr(e, "status", None) != _EUNSUPPORTED:
                        raise
            plain = object.__new__(_Group)
            plain.__dict__.update(self.__dict__)
            plain.reduce = None
            value = plain.run(run, self.root.with_(data=None), values)
            return getattr(run.pick([value]), name)(out, value, opts)
        if fused is not None:
            try:
                return fused(out, self.program, values, self.layout, **self.how)
            except Exception as e:  # e.g. integer instructions met while the device is capturing
                if getattr(e, "status", None) != _EUNSUPPORTED:
                    raise
        # node by node, on the callbacks (a backend without the kernel, or a group that does not fit)
        done = {t.data.id: v for t, v in zip(self.inputs, values)}
        for m in self.members:
            args = []
            for a in m.data.args:
                if isinstance(a, Tensor):
                    args.append(done[a.data.id] if a.data.id in done else run.eval(a, None))
                else:
                    args.append(a)
            done[m.data.id] = getattr(run.pick(args), m.data.op)(m.with_(data=None), *args)
        return done[self.root.data.id]


def _imm(a: Tensor) -> float:
    """The constant as the f32 the kernels would load: encoded in its type, decoded again."""
    from .tensor import number_to_binary
    ty = a.type if a.type in _NARROW else ("f", 32)
    raw = np.frombuffer(number_to_binary(_const(a), ty), dtype=T.numpy_dtype(ty))
    if ty == ("bf", 16):
        return float((raw.astype(np.uint32) << 16).view(np.float32)[0])
    return float(raw.astype(np.float32)[0])


def _fuse(roots: List[Tensor], ints: bool = False) -> int:
    """Rewrites element-wise groups of the root scope into `fused` nodes, in place; returns how
    many groups were formed.  `ints`: plan for groups that are compiled for the device, which may
    compute on 32-bit integers and relabel bits as well."""
    _plan["ints"] = ints
    try:
        return _fuse_planned(roots)
    finally:
        _plan["ints"] = False


def _scale_mode(scale: Tensor, out_shape, n_axes: int, batch_axes: int):
    """How `scale` broadcasts over a contraction's result [batch..., rows..., columns...] (the last
    `n_axes` axes are the right operand's free axes): one value, one per column, one per row, or None."""
    if scale.size == 1:
        return 3
    rank = len(out_shape)
    padded = (1,) * (rank - len(scale.shape)) + tuple(scale.shape)
    if len(padded) != rank:
        return None
    if n_axes and padded == (1,) * (rank - n_axes) + tuple(out_shape[rank - n_axes:]):
        return 1
    if batch_axes == 0 and rank > n_axes and padded == tuple(out_shape[:rank - n_axes]) + (1,) * n_axes:
        return 2
    return None


def _absorb_scales(order: List[Tensor], uses) -> int:
    """multiply(as_type(dot(s8, s8) -> s32, f32), scales) becomes one `dot_scaled` node when nobody
    else reads the sum or its conversion: the quantised linear layer, finished on the accumulators."""
    found = 0
    for node in order:
        e = node.data
        if e.op != "multiply" or node.type != ("f", 32):
            continue
        for x, scale in (e.args, e.args[::-1]):
            if not (isinstance(x, Tensor) and isinstance(x.data, Expr) and x.data.op == "as_type" and uses.get(x.data.id) == 1):
                continue
            d = x.data.args[0]
            if not (isinstance(d.data, Expr) and d.data.op == "dot" and uses.get(d.data.id) == 1 and d.type == ("s", 32)):
                continue
            l, c1, b1, r, c2, b2 = d.data.args
            if l.type != ("s", 8) or r.type != ("s", 8) or not isinstance(scale, Tensor) or scale.type != ("f", 32):
                continue
            if x.shape != node.shape or d.shape != node.shape:
                continue
            mode = _scale_mode(scale, node.shape, len(r.shape) - len(c2) - len(b2), len(b1))
            if mode is None:
                continue
            e.op, e.args = "dot_scaled", [l, list(c1), list(b1), r, list(c2), list(b2), scale, mode]
            found += 1
            break
    return found


def _fuse_planned(roots: List[Tensor]) -> int:
    order, uses, seen, parents = [], {}, set(), {}

    def walk(t):
        e = t.data
        if e.op in ("constant", "tensor") or e.scope != 0:
            return
        uses[e.id] = uses.get(e.id, 0) + 1
        if e.id in seen:
            return
        seen.add(e.id)
        for child in _children(e):
            if isinstance(child, Tensor):
                parents.setdefault(child.data.id, []).append(t)
                walk(child)
        order.append(t)

    def feeds_a_row_reduction(t):
        """Whether the only reader of `t` reduces it over its last axis: one node and that reduction
        are worth a kernel of their own (the node's value is never stored)."""
        readers = parents.get(t.data.id, [])
        if len(readers) != 1 or uses.get(t.data.id) != 1 or len(t.shape) == 0:
            return False
        r = readers[0].data
        return (r.op in _REDUCE_CODES and isinstance(r.args[0], Tensor) and r.args[0].data.id == t.data.id and _over_last_axis(r.args[1], len(t.shape)))

    for r in roots:
        walk(r)
    if any(t.data.op in ("while", "cond", "elem") for t in order):
        return 0  # bodies of nested scopes read root-scope nodes that the counts above do not see
    if _absorb_scales(order, uses):
        uses.clear()
        seen.clear()
        parents.clear()
        del order[:]
        for r in roots:
            walk(r)
    def candidate(a, root):
        return (isinstance(a, Tensor) and isinstance(a.data, Expr) and a.data.op not in ("constant", "tensor", "fused")
                and a.data.scope == 0 and a.shape == root.shape and _fusable(a))

    def cheap_to_recompute(a, root):
        """A value read by several consumers may be computed again inside each group that reads it,
        when that is cheaper than storing it once and loading it in each: a short subtree whose own
        full-size inputs are no wider than the value."""
        nodes, leaf_bytes, stack, visited = 0, 0, [a], set()
        while stack:
            t = stack.pop()
            if t.data.id in visited:
                continue
            visited.add(t.data.id)
            nodes += 1
            for b in t.data.args:
                if not isinstance(b, Tensor) or _const(b) is not None:
                    continue
                if candidate(b, root):
                    stack.append(b)
                elif b.data.id not in visited:
                    visited.add(b.data.id)
                    leaf_bytes += T.size_bytes(b.type) if b.shape == root.shape else 0
        return nodes <= 6 and leaf_bytes <= T.size_bytes(a.type)

    def grow(root, recompute):
        """Members of the group under `root`.  A value all of whose readers are members that belong
        to this group alone moves in for good; any other value may be computed again inside the
        group (`shared`), and so may everything only reachable through it."""
        members, shared, own_reads = {root.data.id: root}, set(), {}
        changed = True
        while changed:
            changed = False
            own_reads.clear()  # reads by members that are this group's alone
            for m in members.values():
                if m.data.id in shared:
                    continue
                for a in m.data.args:
                    if isinstance(a, Tensor) and isinstance(a.data, Expr) and a.data.op != "constant":
                        own_reads[a.data.id] = own_reads.get(a.data.id, 0) + 1
            for m in list(members.values()):
                for a in m.data.args:
                    if not candidate(a, root) or a.data.id in members or a.data.id in taken:
                        continue
                    if own_reads.get(a.data.id, 0) == uses.get(a.data.id):
                        members[a.data.id] = a
                        changed = True
                    elif recompute and cheap_to_recompute(a, root):
                        members[a.data.id] = a
                        shared.add(a.data.id)
                        changed = True
        return members, shared, dict(own_reads)

    def build(root, members):
        ordered = [t for t in order if t.data.id in members]
        inputs, input_seen = [], set()
        for m in ordered:
            for a in m.data.args:
                if (isinstance(a, Tensor) and _const(a) is None and a.data.id not in members
                        and a.data.id not in input_seen):
                    input_seen.add(a.data.id)
                    inputs.append(a)
        # members are copies (same ids): the originals may become groups of their own later
        ordered = [t.with_(data=Expr(t.data.id, t.data.op, t.data.args, 0)) for t in ordered]
        ordered[-1] = root.with_(data=Expr(next(_ids), root.data.op, root.data.args, 0))
        return _Group(ordered[-1], ordered, inputs), inputs

    taken, formed = set(), 0
    for root in reversed(order):  # consumers first: a group grows from its last node upwards
        if root.data.id in taken or uses.get(root.data.id, 0) == 0 or not _fusable(root):
            continue
        if _plan["ints"] and len(root.shape) >= 2 and root.shape[-1] == 1:
            continue  # work on one value per row: left as nodes, so that it can join the stage that makes the value
        members, shared, inside = grow(root, recompute=True)
        # a single node is no group -- unless the plan may join it to the stages that make its per-row operands
        least = 1 if _plan["ints"] and any(isinstance(a, Tensor) and _const(a) is None and len(a.shape) >= 2
                                           and a.shape[-1] == 1 for a in root.data.args) else 2
        if feeds_a_row_reduction(root):
            least = 1
        group, inputs = build(root, members) if len(members) >= least else (None, None)
        if group is not None and shared and (group.program is None or group.layout is None):
            members, shared, inside = grow(root, recompute=False)  # too big with the recomputed parts: without them
            group, inputs = build(root, members) if len(members) >= least else (None, None)
        if group is None:
            continue
        taken.update(i for i in members if i not in shared)
        for i in shared:  # this group no longer reads the shared values; a value nobody reads is dead
            uses[i] -= inside.get(i, 0)
        dead = [i for i in shared if uses[i] == 0]
        while dead:  # the operands of a dead node lose a reader each
            gone = dead.pop()
            node = next(t for t in order if t.data.id == gone)
            for a in node.data.args:
                if isinstance(a, Tensor) and isinstance(a.data, Expr) and a.data.id in uses and _const(a) is None:
                    uses[a.data.id] -= 1
                    if uses[a.data.id] == 0:
                        dead.append(a.data.id)
        root.data.op, root.data.args = "fused", [group, inputs]
        formed += 1
    # recount the readers on the rewritten graph
    uses.clear()
    seen.clear()
    del order[:]
    for r in roots:
        walk(r)
    # a reduction over the last axis whose operand is a group nobody else reads joins that group
    for node in order:
        e = node.data
        if e.op not in _REDUCE_CODES or not isinstance(e.args[0], Tensor):
            continue
        operand, opts = e.args[0], e.args[1]
        inner = operand.data
        if not isinstance(inner, Expr) or inner.op != "fused" or uses.get(inner.id) != 1:
            continue
        rank = len(operand.shape)
        if not _over_last_axis(opts, rank):
            continue
        both = inner.args[0].with_reduction(e.op, opts)
        if both is None:
            continue
        e.op, e.args = "fused", [both, inner.args[1]]
    if _plan["ints"]:  # planned for compiled kernels: groups over the same rows become stages of one
        _cluster_rows(roots)
    return formed


def _over_last_axis(opts, rank: int) -> bool:
    """Whether a reduction with these options folds exactly the last axis -- of a vector, its only one, also when
    no axis is named (the softmax of a vector: exp(t) / sum(exp(t)))."""
    axes = opts.get("axes")
    return (rank == 1 and axes is None) or list(axes or []) == [rank - 1]


class _RowCluster:
    """Fused groups over the same rows as stages of one program.  Every stage but the last reduces
    its value along the row, may work on that one value per row (a sum divided by the row length),
    and keeps it as a row statistic that later stages read.  `steps` are the original nodes in
    evaluation order, the last one the element-wise group that produces the result: a backend
    that cannot run the program gets them one by one."""

    reduce = None
    how = {"mode": "compiled"}
    split_rows = False

    def __init__(self, steps, inputs, program, layout, n_stages):
        self.steps, self.inputs, self.program, self.layout, self.n_stages = steps, inputs, program, layout, n_stages
        self.root = steps[-1]

    def run(self, run: "_Run", out: Tensor, values: List[Tensor]):
        fused = getattr(run.pick(values), "fused_elementwise", None)
        if fused is not None and not self.split_rows:
            try:
                return fused(out, self.program, values, self.layout, **self.how)
            except Exception as e:
                if getattr(e, "status", None) != _EUNSUPPORTED:
                    raise
                # a refusal that the shape alone decides (a few very long rows, which the reductions cut into
                # segments) holds for every later call: the steps run at once from then on
                self.split_rows = "the reduction would split" in str(e)
        known = {t.data.id: v for t, v in zip(self.inputs, values)}
        for node in self.steps:
            e = node.data
            if e.op == "fused":
                group, inputs = e.args
                known[e.id] = group.run(run, node.with_(data=None), [known[t.data.id] for t in inputs])
                continue
            args = [(known[a.data.id] if a.data.id in known else run.eval(a, None)) if isinstance(a, Tensor) else a
                    for a in e.args]
            known[e.id] = getattr(run.pick(args), e.op)(node.with_(data=None), *args)
        return known[self.root.data.id]


def _cluster_rows(roots: List[Tensor]) -> int:
    """Rewrites a node, together with what makes the per-row values only it (and they themselves)
    read, into one node holding a _RowCluster.  A per-row value is a *stage*: a reduction over the
    last axis -- of a fused group's value or of a tensor as it is -- followed by a chain of
    element-wise nodes on the one value per row.  The node that is rewritten is an element-wise fused
    group over the full shape (a softmax, a layer normalisation), or itself such a per-row value
    (a log-sum-exp).  A row is walked by a wave, or by a block when it has more than 4096 elements: as the
    separate reduction walks it, whose order the stages keep."""
    order, readers, seen = [], {}, set()

    def walk(t):
        e = t.data
        if e.op in ("constant", "tensor") or e.scope != 0:
            return
        if e.id in seen:
            return
        seen.add(e.id)
        for child in _children(e):
            if isinstance(child, Tensor):
                readers.setdefault(child.data.id, set()).add(e.id)
                walk(child)
        order.append(t)

    for r in roots:
        readers.setdefault(r.data.id, set()).add("result")
        walk(r)
    position = {t.data.id: i for i, t in enumerate(order)}
    absorbed = set()  # nodes that have become part of a cluster

    def reduced_shape(t):
        """The full shape whose rows `t` reduces, when `t` is such a reduction."""
        d = t.data
        if d.op == "fused" and isinstance(d.args[0], _Group) and d.args[0].reduce is not None and d.args[0].program:
            return tuple(d.args[0].root.shape)
        if d.op in _REDUCE_CODES and isinstance(d.args[0], Tensor):
            x, opts = d.args[0], d.args[1]
            if x.type in _NARROW and _const(x) is None and _over_last_axis(opts, len(x.shape)):
                return tuple(x.shape)
        return None

    def attempt(final, full_shape, row_valued):
        e = final.data
        rank = len(full_shape)
        if rank == 0:
            return False
        cols, rows = full_shape[-1], prod(full_shape[:-1])
        if cols % 8:
            return False
        per_row = tuple(full_shape[:-1]) + (1,)
        carry_fits = cols <= 32768  # at most sixteen vectors per lane with a block per row (eight with a wave, <= 4096)

        def is_per_row(t, flat_too=False):
            if not (isinstance(t, Tensor) and isinstance(t.data, Expr) and _const(t) is None and t.type in _NARROW):
                return False
            padded = (1,) * (rank - len(t.shape)) + tuple(t.shape)
            return padded == per_row or (flat_too and tuple(t.shape) == tuple(full_shape[:-1]) and t.size == rows)

        def base_of(t):
            shape = reduced_shape(t)
            if shape != tuple(full_shape):
                return None
            if t.data.op == "fused":
                g = t.data.args[0]
                return "group" if g.reduce[2][0] == rows and g.reduce[2][1] == cols else None
            return "reduce"

        stages = {}  # id of the kept value -> (base node, [links from the base towards the kept value])

        def stage_ending_at(t, inside, is_final=False):
            """Registers the stage whose kept value is `t` (and the stages it reads), or returns False.
            `inside`: ids of the readers the cluster already has (the final value may have any readers)."""
            if t.data.id in stages:
                return True
            if t.data.id in absorbed or not is_per_row(t, flat_too=is_final):
                return False
            if not is_final and not readers.get(t.data.id, set()) <= inside:
                return False
            links, cur = [], t
            while base_of(cur) is None:
                d = cur.data
                if d.op in ("reshape", "squeeze") and isinstance(d.args[0], Tensor) and d.args[0].size == cur.size:
                    # the same values under another shape (a statistic taken without keep_axes, then given its axis back)
                    chain = d.args[0]
                    if (not is_per_row(chain, flat_too=True) or chain.data.id in stages or chain.data.id in absorbed
                            or readers.get(chain.data.id, set()) != {d.id}):
                        return False
                    links.append(cur)
                    cur = chain
                    continue
                if (d.op not in UNARY_OPS and d.op not in BINARY_OPS and d.op != "as_type") or not _fusable(cur):
                    return False
                operands = [a for a in d.args if isinstance(a, Tensor) and _const(a) is None]
                if not operands or not all(is_per_row(a, flat_too=True) for a in operands):
                    return False
                # the chain continues through the operand computed last; any other one is a kept value of another stage
                chain = max(operands, key=lambda a: position.get(a.data.id, -1))
                if chain.data.id in stages or chain.data.id in absorbed or readers.get(chain.data.id, set()) != {d.id}:
                    return False
                links.append(cur)
                cur = chain
                if len(links) > 12:
                    return False
            links.reverse()
            chain_ids = {cur.data.id} | {l.data.id for l in links}
            others = [a for l in links for a in l.data.args
                      if isinstance(a, Tensor) and _const(a) is None and a.data.id not in chain_ids]
            stages[t.data.id] = (cur, links)
            for a in others:  # a link's other operand must be a kept value of a stage of this cluster
                if not stage_ending_at(a, inside | chain_ids):
                    del stages[t.data.id]
                    return False
            if cur.data.op == "fused":  # per-row inputs of the base group join if they can (or stay inputs from memory)
                for a in cur.data.args[1]:
                    if is_per_row(a):
                        stage_ending_at(a, inside | chain_ids)
            return True

        if row_valued:
            if not stage_ending_at(final, set(), is_final=True):
                return False
        # grow: per-row inputs of the final group, then of the stages' groups, until nothing new is internal
        changed = True
        while changed:
            changed = False
            inside = {b.data.id for b, _ in stages.values()} | {l.data.id for _, ls in stages.values() for l in ls}
            pending = [a for b, _ in stages.values() if b.data.op == "fused" for a in b.data.args[1] if is_per_row(a)]
            if not row_valued:
                inside.add(e.id)
                pending += [a for a in e.args[1] if is_per_row(a)]
            for t in pending:
                if t.data.id not in stages and stage_ending_at(t, inside):
                    changed = True
        if not stages or len(stages) > 3 + (1 if row_valued else 0):
            return False
        if row_valued and len(stages) < 2 and not stages[e.id][1]:
            return False  # a lone reduction is what it already is
        kept = sorted((i for i in stages if not (row_valued and i == e.id)), key=lambda i: position[stages[i][0].data.id])
        if len(kept) > 3:
            return False
        slot = {i: k for k, i in enumerate(kept)}
        if row_valued:
            kept.append(e.id)  # last, and not a statistic anyone reads: the result
        union, index = [], {}

        def external(t):
            if t.data.id not in index:
                index[t.data.id] = len(union)
                union.append(t)
            return index[t.data.id]

        def remap(ins, key_src, key_arg, own_inputs):
            if ins.get(key_src, 0) != 1:
                return
            t = own_inputs[ins.get(key_arg, 0)]
            if t.data.id in slot:
                ins[key_src], ins[key_arg] = 3, slot[t.data.id]
            else:
                ins[key_arg] = external(t)

        def group_program(node):
            g, own = node.data.args
            for ins in g.program:
                ins = dict(ins)
                remap(ins, "src", "arg", own)
                if ins["kind"] == 3:
                    remap(ins, "src2", "arg2", own)
                program.append(ins)

        program, steps, fits = _Program(), [], True
        reduced = None  # the element-wise program of the stage before (what its reduction was taken over)

        def start_from_carry(at):
            """A stage whose program begins with the whole element-wise program of the stage before it
            (the softmax's division begins with the exponentials its sum was taken over) reads those
            values where they still are -- the lanes' registers -- instead of computing them again."""
            mine = program[at:]
            if (carry_fits and reduced and len(mine) >= len(reduced) and mine[:len(reduced)] == reduced
                    and not any(ins.get("flags", 0) >> 4 for ins in reduced)):
                program[at:] = [{"kind": 0, "src": 4, "dt": reduced[-1]["dt"]}] + mine[len(reduced):]

        for i in kept:
            base, links = stages[i]
            at = len(program)
            if base.data.op == "fused":
                group_program(base)
                code = _REDUCE_CODES[base.data.args[0].reduce[0]]
            else:
                x = base.data.args[0]
                program.append({"kind": 0, "src": 1, "arg": external(x), "dt": x.type})
                code = _REDUCE_CODES[base.data.op]
            mine = [dict(ins) for ins in program[at:]]
            start_from_carry(at)
            reduced = mine
            program.append({"kind": 6, "op": code, "dt": base.type})
            steps.append(base)
            chain = base
            for l in links:
                d = l.data
                ins = {"dt": l.type}
                if d.op in ("reshape", "squeeze"):  # nothing happens to the value
                    steps.append(l)
                    chain = l
                    continue
                if d.op in UNARY_OPS:
                    ins.update(kind=1, op=UNARY_OPS.index(d.op))
                elif d.op == "as_type":
                    ins.update(kind=4)
                else:
                    pos = next(p for p, a in enumerate(d.args) if isinstance(a, Tensor) and a.data.id == chain.data.id)
                    other = d.args[1 - pos]
                    ins.update(kind=2, op=BINARY_OPS.index(d.op), flags=1 if pos == 1 else 0)
                    if _const(other) is not None:
                        ins.update(src=0, imm=_imm(other))
                    elif other.data.id in slot and (i not in slot or slot[other.data.id] < slot[i]):
                        ins.update(src=3, arg=slot[other.data.id])
                    else:
                        fits = False
                program.append(ins)
                steps.append(l)
                chain = l
            if i in slot:
                program.append({"kind": 7, "arg": slot[i], "dt": chain.type})
            else:
                program.append({"kind": 7, "arg": 0, "flags": 1, "dt": chain.type})  # the value per row is the result
        if not row_valued:
            at = len(program)
            group_program(final)
            start_from_carry(at)
        layout = _layout(full_shape, [t.shape for t in union], split=rank - 1)
        if not fits or layout is None or len(program) > _MAX_INSTR or len(union) > _MAX_INPUTS:
            return False
        if row_valued:
            steps[-1] = steps[-1].with_(data=Expr(e.id, e.op, e.args, 0))  # (the final node is rewritten below)
        else:
            steps.append(final.with_(data=Expr(e.id, "fused", e.args, 0)))
        for node in steps[:-1]:
            absorbed.add(node.data.id)
        absorbed.add(e.id)
        e.op, e.args = "fused", [_RowCluster(steps, union, program, layout, len(kept)), union]
        return True

    formed = 0
    for node in reversed(order):  # consumers first: the longest chain that ends in a value takes it
        e = node.data
        if e.id in absorbed:
            continue
        if e.op == "fused" and isinstance(e.args[0], _Group) and e.args[0].reduce is None and e.args[0].program:
            formed += attempt(node, tuple(node.shape), False)
            continue
        # a per-row value: follow its chain down to the reduction it starts from
        cur, depth = node, 0
        while cur is not None and reduced_shape(cur) is None and depth < 12:
            d = cur.data
            operands = [a for a in d.args if isinstance(a, Tensor) and _const(a) is None] if d.op in UNARY_OPS or d.op in BINARY_OPS or d.op == "as_type" else []
            cur = max(operands, key=lambda a: position.get(a.data.id, -1)) if operands else None
            depth += 1
        if cur is not None and reduced_shape(cur) is not None and node.type in _NARROW:
            formed += attempt(node, reduced_shape(cur), True)
    return formed


# ---- the evaluator ----------------------------------------------------------------------------------

CREATION_OPS = ("eye", "iota")           # evaluator.ex:26-28
LIST_OPS = ("concatenate", "stack")
INDICES_OPS = ("slice", "put_slice")


def _children(node: Expr):
    """The tensor expressions a node reads in its own scope (Tree.apply_args, tree.ex)."""
    if node.op in ("constant", "tensor", "parameter"):
        return
    if node.op == "elem":
        yield node.args[0]  # the scope node itself (an Expr, not a tensor)
        return
    if node.op == "while":
        yield from node.args[0]
        return
    if node.op == "cond":
        yield node.args[0]
        return
    for a in (node.args[1] if node.op == "block" else node.args):
        if isinstance(a, Tensor):
            yield a
        elif isinstance(a, list):
            for x in a:
                if isinstance(x, Tensor):
                    yield x


def _expr_of(x) -> Expr:
    return x.data if isinstance(x, Tensor) else x


class _Plan:
    """Reference counts of one scope: id -> uses inside the scope (evaluator.ex:86-128), the nodes of
    enclosing scopes it reads, and the plans of the scopes nested in it."""

    def __init__(self, roots, tag, plans):
        self.tag = tag
        self.counts: Dict[Any, int] = {}
        self.outer: Dict[Any, Any] = {}  # id -> node (tensor or Expr) that belongs to an enclosing scope
        for r in roots:
            self._visit(r, plans)

    def _visit(self, x, plans):
        e = _expr_of(x)
        if e.op in ("constant", "tensor"):
            return
        if e.scope != self.tag:
            self.outer.setdefault(e.id, x)
            return
        if e.id in self.counts:
            self.counts[e.id] += 1
            return
        self.counts[e.id] = 1
        for child in _children(e):
            self._visit(child, plans)
        nested = []
        if e.op == "while":
            _, pred, body, tag = e.args
            nested.append(_Plan([pred] + list(body), tag, plans))
        elif e.op == "cond":
            nested.extend(_Plan(exprs, tag, plans) for tag, exprs in e.args[1])
        for plan in nested:
            plans[plan.tag] = plan
            for outer in plan.outer.values():  # one use per nested scope, released when the scope node is done
                self._visit(outer, plans)


class _Scope:
    def __init__(self, plan: _Plan, parent: Optional["_Scope"], params):
        self.plan, self.parent, self.params = plan, parent, params
        self.counts = dict(plan.counts)
        self.results: Dict[Any, Any] = {}


# nodes that `apply` does not evaluate as a callback on its evaluated operands
_EVALUATED_APART = frozenset(["parameter", "elem", "while", "cond", "fused", "dot_scaled", "block"]) | frozenset(CREATION_OPS)


class _Run:
    def __init__(self, plans, backend):
        self.plans, self.backend = plans, backend

    def eval(self, x, scope: _Scope):  # noqa: A003
        e = x.data if x.__class__ is Tensor else _expr_of(x)
        counts = scope.counts if scope is not None else ()  # (no scope: a group's constant, evaluated by the group itself)
        if e.id in counts and e.op not in ("tensor", "constant"):  # the usual node: one of this scope's own
            results = scope.results
            if e.id in results:
                res = results[e.id]
            else:
                res = results[e.id] = self.apply(e, x, scope)
            left = counts[e.id] = counts[e.id] - 1
            if left == 0:
                results.pop(e.id, None)
            return res
        if e.op == "tensor":
            t = e.args[0]
            mod, opts = self.backend
            return t if mod is HostBinary else Nx.backend_transfer(t, mod, opts)
        if e.op == "constant":
            mod, opts = self.backend  # evaluator.ex:212-215
            return mod.constant(x.with_(data=None), e.args[0], opts)
        owner = scope
        while owner is not None and e.id not in owner.counts:
            owner = owner.parent
        if owner is None:
            raise RuntimeError(f"evaluator cache has expired for {e!r}")
        if e.id in owner.results:
            res = owner.results[e.id]
        else:
            res = self.apply(e, x, owner)
            owner.results[e.id] = res
        if owner is scope:  # a read from a nested scope is released by the scope node (evaluator.ex:231-236)
            self.release(e.id, owner)
        return res

    def release(self, id_, owner: _Scope):
        owner.counts[id_] -= 1
        if owner.counts[id_] == 0:
            owner.results.pop(id_, None)

    def release_outer(self, plan: _Plan, scope: _Scope):
        for id_ in plan.outer:
            owner = scope
            while owner is not None and id_ not in owner.counts:
                owner = owner.parent
            if owner is not None:
                self.release(id_, owner)

    def apply(self, e: Expr, x, scope: _Scope):
        op = e.op
        if op == "parameter":
            return scope.params[e.args[0]]
        if op not in _EVALUATED_APART:
            # a callback on tensors and options (nearly every node): its operands, then the backend they are on
            args, mod = [], None
            for a in e.args:
                if a.__class__ is Tensor:
                    a = self.eval(a, scope)
                    b = a.data.__class__
                    if mod is None:
                        mod = b
                    elif mod is not b:
                        mod = False  # operands on different backends: the general rule decides
                elif a.__class__ is list and any(isinstance(v, Tensor) for v in a):
                    mod = False
                    a = [self.eval(v, scope) if isinstance(v, Tensor) else v for v in a]
                args.append(a)
            if not mod or mod is HostBinary:
                mod = self.pick([a for a in args if isinstance(a, Tensor)]) if op not in LIST_OPS and op not in INDICES_OPS else None
                if mod is None:
                    mod = self.pick(args[0]) if op in LIST_OPS else self.pick([args[0]] + [i for i in args[1] if isinstance(i, Tensor)])
            return getattr(mod, op)(x.with_(data=None), *args)
        if op == "elem":
            return self.eval(e.args[0], scope)[e.args[1]]
        if op == "while":
            initial, pred, body, tag = e.args
            state = [self.eval(t, scope) for t in initial]
            plan = self.plans[tag]
            while True:  # evaluator.ex:398-409: a fresh set of counts per trip
                trip = _Scope(plan, scope, state)
                if _to_number(self.eval(pred, trip)) == 0:
                    break
                state = [self.eval(t, trip) for t in body]
            self.release_outer(plan, scope)
            return state
        if op == "cond":
            pred, branches = e.args
            chosen = 0 if _to_number(self.eval(pred, scope)) != 0 else 1
            tag, exprs = branches[chosen]
            branch = _Scope(self.plans[tag], scope, scope.params)
            result = [self.eval(t, branch) for t in exprs]
            for tag, _ in branches:
                self.release_outer(self.plans[tag], scope)
            return result
        if op == "fused":
            group, inputs = e.args
            return group.run(self, x.with_(data=None), [self.eval(t, scope) for t in inputs])
        if op == "dot_scaled":
            l, c1, b1, r, c2, b2, scale, mode = e.args
            lv, rv, sv = self.eval(l, scope), self.eval(r, scope), self.eval(scale, scope)
            mod, out = self.pick([lv, rv, sv]), x.with_(data=None)
            one_call = getattr(mod, "dot_scaled", None)
            if one_call is not None:
                try:
                    return one_call(out, lv, c1, b1, rv, c2, b2, sv, mode)
                except Exception as err:  # a shape the kernel leaves to the separate callbacks
                    if getattr(err, "status", None) != _EUNSUPPORTED:
                        raise
            summed = mod.dot(out.with_(type=("s", 32)), lv, c1, b1, rv, c2, b2)
            return mod.multiply(out, mod.as_type(out, summed), sv)
        if op == "block":
            struct, in_args, fun = e.args
            args = [self.eval(a, scope) for a in in_args]
            return self.pick(args).block(struct, x.with_(data=None), args, fun)
        out = x.with_(data=None)
        if op in CREATION_OPS:  # evaluator.ex:368-371
            mod, opts = self.backend
            return getattr(mod, op)(out, *e.args, opts)
        args = []
        for a in e.args:
            if isinstance(a, Tensor):
                args.append(self.eval(a, scope))
            elif isinstance(a, list) and any(isinstance(v, Tensor) for v in a):
                args.append([self.eval(v, scope) if isinstance(v, Tensor) else v for v in a])
            else:
                args.append(a)
        if op in LIST_OPS:
            mod = self.pick(args[0])
        elif op in INDICES_OPS:
            mod = self.pick([args[0]] + [i for i in args[1] if isinstance(i, Tensor)])
        else:
            mod = self.pick([a for a in args if isinstance(a, Tensor)])
        return getattr(mod, op)(out, *args)

    def pick(self, tensors):
        """Nx.Shared.list_impl!/1 (shared.ex:459-472); operands that only store data follow the others,
        or the default backend when nothing else is there."""
        tensors = [t for t in tensors if isinstance(t, Tensor)]
        mod = Nx._impl(*tensors) if tensors else HostBinary
        return self.backend[0] if mod is HostBinary else mod


class Compiled:
    """A traced function: call it with arguments of the traced shapes and types."""

    def __init__(self, roots, structure, templates):
        self.roots, self.structure, self.templates = roots, structure, templates
        self.n_params = len(templates)
        self.plans: Dict[Any, _Plan] = {}
        self.plan = _Plan(roots, 0, self.plans)

    def _params(self, args):
        leaves: list = []
        _flatten(list(args), leaves)
        if len(leaves) != self.n_params:
            raise ValueError(f"expected {self.n_params} tensor arguments, got {len(leaves)}")
        params = [Nx.to_tensor(v) for v in leaves]
        for i, (p, t) in enumerate(zip(params, self.templates)):
            if (p.type, p.shape) != (t.type, t.shape):
                raise ValueError(f"argument {i} is {p.type!r}{p.shape!r}, the function was traced for {t.type!r}{t.shape!r}")
        return params

    def _evaluate(self, params):
        run = _Run(self.plans, _runtime_backend(params))
        root = _Scope(self.plan, None, params)
        results = []
        for r in self.roots:
            value = run.eval(r, root)
            # evaluator.ex:68-75: the output keeps the traced template, the data is the result's
            results.append(r.with_(data=value.data))
        return results

    def __call__(self, *args):
        return _unflatten(self.structure, self._evaluate(self._params(args)))

    def capture(self, *args) -> "Captured":
        """Records one evaluation on the device as a graph: later calls replay all its kernels with
        a single submission instead of one callback (and one launch) per node.  The function must
        not need the host while it runs: no `while_loop` / `cond`, no bounds-checked `take`."""
        return Captured(self, self._params(args))


class Captured:
    """A compiled function whose device work was captured once, on private copies of the arguments
    (`inputs`).  Calling it copies the arguments into those (pass `inputs` themselves to skip the
    copies), replays the graph and returns the captured result tensors: they are overwritten by the
    next call and die with this object."""

    def __init__(self, compiled: Compiled, params):
        from . import backend as B
        devices = {p.data.device for p in params if isinstance(p.data, B.HipNxBackend)}
        if len(devices) != 1 or any(not isinstance(p.data, B.HipNxBackend) for p in params):
            raise ValueError("capture needs every argument on one device")
        (self.device,) = devices
        self.compiled = compiled
        self.params = [Nx.backend_copy(p, B.HipNxBackend, {"device": self.device}) for p in params]
        compiled._evaluate(self.params)  # once for real: kernel attributes, pool block sizes, cached constants
        B.capture_begin(self.device)
        try:
            self.results = compiled._evaluate(self.params)
        except BaseException:
            B.capture_end(self.device).destroy()
            raise
        self.graph = B.capture_end(self.device)

    @property
    def inputs(self):
        return list(self.params)

    def __call__(self, *args):
        from . import backend as B
        new = self.compiled._params(args)
        for held, given in zip(self.params, new):
            if given.data is held.data or getattr(given.data, "ref", None) is held.data.ref:
                continue
            if not isinstance(given.data, B.HipNxBackend):
                given = Nx.backend_transfer(given, B.HipNxBackend, {"device": self.device})
            B.copy_into(held, given)
        self.graph.launch()
        return _unflatten(self.compiled.structure, self.results)

    def destroy(self):
        self.graph.destroy()
        self.results = []


def _runtime_backend(params):
    """evaluator.ex:36-38 (`__to_backend__`): constants and created tensors go to the default
    backend; when that one only stores data they go where the arguments live."""
    mod, opts = Nx.default_backend()
    if mod is HostBinary or mod is Expr:
        for p in params:
            b = type(p.data)
            if b is not HostBinary and b is not Expr:
                return b, b.init({})
    return mod, opts


def trace(fun: Callable, args, kwargs=None, fuse=False) -> Compiled:
    """Runs `fun` on parameter expressions shaped like `args` (compiler.ex:184-205: the default
    backend is the expression builder while the function runs)."""
    leaves: list = []
    structure = _flatten(list(args), leaves)
    templates = [v if isinstance(v, Tensor) else Nx.to_tensor(v) for v in leaves]
    if getattr(_trace, "scopes", None):
        raise RuntimeError("a traced function cannot be traced again from inside a trace")
    _trace.scopes = [0]
    _trace.fold = Nx.default_backend()
    previous = Nx.default_backend(Expr)
    try:
        params = [Expr._expr(t.with_(data=None), "parameter", [i]) for i, t in enumerate(templates)]
        result = fun(*_unflatten(structure, params), **(kwargs or {}))
        out_leaves: list = []
        out_structure = _flatten(result, out_leaves)
        roots = [to_expr(Nx.to_tensor(v)) for v in out_leaves]
    finally:
        Nx.default_backend(*previous)
        _trace.scopes = []
        _trace.fold = None
    if fuse not in (False, True, "compiled"):
        raise ValueError(f"fuse is False, True or \"compiled\", got: {fuse!r}")
    compiled_groups = _fuse(roots, ints=fuse == "compiled") if fuse else 0
    compiled = Compiled(roots, out_structure, [t.with_(data=None) for t in templates])
    compiled.fused_groups = compiled_groups
    return compiled


def jit(fun: Callable = None, fuse=False, **static):
    """Nx.Defn.jit/2 with the default compiler: traces on every call, like the reference's
    evaluator (evaluator.ex:41-43), then evaluates.  Keyword arguments are static options; `fuse`
    hands groups of element-wise nodes to the backend as one kernel each."""
    if fun is None:
        return lambda f: jit(f, fuse=fuse, **static)

    def call(*args, **kwargs):
        return trace(fun, args, {**static, **kwargs}, fuse=fuse)(*args)
    call.__name__ = getattr(fun, "__name__", "jitted")
    return call


def compile(fun: Callable, *templates, fuse=False, **static) -> Compiled:  # noqa: A001 - Nx.Defn.compile/3
    """Traces once for arguments shaped like `templates`; the result is called many times."""
    return trace(fun, templates, static, fuse=fuse)
