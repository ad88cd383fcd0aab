"""HipNx.Backend -- the `Nx.Backend` behaviour (reference: nx/lib/nx/backend.ex:46-144) over
libhipnx, for the eager tensor path on one MI355X.

This is the Python twin of `lib/hipnx/backend.ex`: the same callbacks, with the same argument
meaning (`op(out_template, args...) -> tensor`) and the same error behaviour, calling the same C
ABI the NIF shim binds.  The structural model is the reference's Torchx backend
(torchx/lib/torchx/backend.ex): one native call per callback, operands that live on another
backend are transferred on entry (`from_nx/1`, torchx/lib/torchx/backend.ex:2040-2041),
callbacks outside the device path raise (torchx/lib/torchx/backend.ex:2199-2210).

A device tensor's `data` is `HipNxBackend(ref, device)`: `ref` owns a flat untyped device buffer;
type, shape and strides always come from the `Tensor` structs passed to the callback.
"""
from __future__ import annotations

import ctypes as C
import threading
from math import prod

import numpy as np

from . import _lib as L
from . import shape as S
from . import types as T
from .tensor import Tensor, number_to_binary, pack_sub_byte, unpack_sub_byte, wrap_to_type

from .backend_names import BINARY_OPS, UNARY_OPS  # noqa: E402

_BIT_COUNTS = (UNARY_OPS.index("count_leading_zeros"), UNARY_OPS.index("population_count"))

RED_SUM, RED_MAX, RED_MIN, RED_PRODUCT, RED_ALL, RED_ANY = 0, 1, 2, 3, 4, 5
K_INNER, K_OUTER = 0, 1
OOB_RAISE, OOB_CLAMP, OOB_DEFER = 0, 1, 2
_bounds = {"policy": OOB_RAISE}
BF16_RNE = 12  # HIPNX_BF16_RNE: output-only type code of as_type and dot
_bf16 = {"rounding": "truncate"}


def _out_code(t) -> int:
    """The type code `as_type` and `dot` pass for their result."""
    c = T.code(t)
    return BF16_RNE if c == T.BF16 and _bf16["rounding"] == "nearest_even" else c

# callbacks of the behaviour that are not on the device path (nx/lib/nx/backend.ex:58-144)
UNSUPPORTED = ["conv", "window_sum", "window_product",
               "window_max", "window_min", "reduce", "window_reduce", "window_scatter_max", "window_scatter_min",
               "indexed_add", "indexed_put", "sort", "argsort", "fft", "ifft", "fft2", "ifft2", "triangular_solve",
               "conjugate", "real", "imag"]


class _Context:
    """One libhipnx context per device, created on first use and kept for the process
    (cf. the client registry of exla/lib/exla/client.ex:20-55)."""

    _lock = threading.Lock()
    _by_device = {}

    @classmethod
    def get(cls, device: int):
        ctx = cls._by_device.get(device)  # (a dict read is atomic; the lock is for the first use only)
        if ctx is not None:
            return ctx
        with cls._lock:
            ctx = cls._by_device.get(device)
            if ctx is None:
                handle = C.c_void_p()
                L.check(L.lib.hipnx_ctx_create(device, C.byref(handle)))
                ctx = cls._by_device[device] = handle
            return ctx


class _Ref:
    """Owns one device buffer.  Metadata-only callbacks (reshape / squeeze / bitcast) share it;
    it is deallocated when the last sharer is, or by the garbage collector."""

    __slots__ = ("ctx", "handle", "nbytes", "sharers", "keep")

    def __init__(self, ctx, nbytes: int, address=None, keep=None, ipc_handle=None):
        self.ctx = ctx
        self.handle = C.c_void_p()
        self.nbytes = nbytes
        self.sharers = 1
        self.keep = keep  # the owner of borrowed memory, kept alive with the handle
        if ipc_handle is not None:  # another process's device memory, opened through its IPC handle
            raw = C.create_string_buffer(bytes(ipc_handle), L.IPC_HANDLE_BYTES)
            L.check(L.lib.hipnx_buf_ipc_import(ctx, raw, nbytes, C.byref(self.handle)))
        elif address is None:
            L.check(L.lib.hipnx_buf_alloc(ctx, nbytes, C.byref(self.handle)))
        else:  # someone else's device memory: the handle never frees it
            L.check(L.lib.hipnx_buf_wrap(ctx, C.c_void_p(address), nbytes, C.byref(self.handle)))

    def __del__(self, _destroy=L.lib.hipnx_buf_destroy):
        try:
            handle = self.handle
        except AttributeError:  # the constructor raised before it had one
            return
        if handle is not None and handle.value:
            try:
                _destroy(handle)
            except Exception:  # interpreter shutdown
                pass
            self.handle = None


def _fresh_ref(ctx, nbytes: int, _new=object.__new__, _alloc=L.lib.hipnx_buf_alloc, _byref=C.byref, _handle=C.c_void_p) -> _Ref:
    """A buffer of the pool for a callback's result: `_Ref(ctx, nbytes)` without the argument handling of the
    general constructor (every callback allocates one)."""
    ref = _new(_Ref)
    ref.ctx = ctx
    ref.handle = handle = _handle()
    ref.nbytes = nbytes
    ref.sharers = 1
    ref.keep = None
    status = _alloc(ctx, nbytes, _byref(handle))
    if status:
        L.check(status)
    return ref


class HipNxBackend:
    """Backend struct: `%HipNx.Backend{ref, device}`."""

    __slots__ = ("ref", "device", "released")

    def __init__(self, ref: _Ref, device: int):
        self.ref = ref
        self.device = device
        self.released = False

    def __repr__(self):
        return f"HipNxBackend(device={self.device}, bytes={self.ref.nbytes})"

    # ---- options / plumbing -------------------------------------------------------------
    @staticmethod
    def init(opts):
        """init/1 (backend.ex:46): validates the backend options, cf. torchx backend.ex:49-52."""
        opts = dict(opts or {})
        unknown = set(opts) - {"device"}
        if unknown:
            raise ValueError(f"unknown keys {sorted(unknown)!r} in {opts!r}, the allowed keys are: ['device']")
        opts.setdefault("device", 0)
        return opts

    @staticmethod
    def _ctx(device):
        return _Context.get(device)

    @classmethod
    def _alloc(cls, out: Tensor, device: int) -> Tensor:
        nbytes = out.size * T.size_bytes(out.type)
        return out.with_(data=cls(_fresh_ref(_Context.get(device), nbytes), device))

    @classmethod
    def _narrow(cls, res: Tensor) -> Tensor:
        """A sub-byte result was computed at 8 bits: keep its low bits, as the reference's write of
        `<<x::size(bits)>>` does (shared.ex:190-194).  In place, on the callback's own fresh output."""
        kind, bits = res.type
        if bits < 8:
            L.check(L.lib.hipnx_narrow_int(res.data.ref.ctx, res.data.ref.handle, res.size, bits, int(kind == "s")))
        return res

    @classmethod
    def _handle(cls, t: Tensor):
        d = t.data
        if d.released:
            raise L.HipNxError(L.EFREED, "tensor has been deallocated")
        return d.ref.handle

    @classmethod
    def _from_nx(cls, t: Tensor, device: int) -> Tensor:
        """Operands that live on another backend are copied in on entry."""
        if isinstance(t.data, HipNxBackend):
            return t
        binary = t.data.__class__.to_binary(t, t.size)
        return cls.from_binary(t, binary, {"device": device})

    @staticmethod
    def _device_of(*tensors) -> int:
        for t in tensors:
            if isinstance(t.data, HipNxBackend):
                return t.data.device
        return 0

    # ---- creation / transfer -------------------------------------------------------------
    @classmethod
    def from_binary(cls, out: Tensor, binary, opts=None) -> Tensor:
        """from_binary/3 (backend.ex:50); rejects a binary shorter than the shape needs
        (torchx/c_src/torchx.cpp:119-123)."""
        opts = cls.init(opts)
        binary = bytes(binary) if not isinstance(binary, (bytes, bytearray, memoryview)) else binary
        if T.is_sub_byte(out.type):
            # packed in the binary, one element per byte on the device, as the reference's device
            # backends unpack them on entry (exla/lib/exla/device_buffer.ex:24-34)
            binary = unpack_sub_byte(binary, out.type, out.size).tobytes()
        need = out.size * T.size_bytes(out.type)
        if len(binary) < need:
            raise ValueError("binary size is too small for the requested shape")
        res = cls._alloc(out, opts["device"])
        if need:
            src = (C.c_char * need).from_buffer_copy(memoryview(binary)[:need])
            L.check(L.lib.hipnx_h2d(res.data.ref.ctx, res.data.ref.handle, 0, src, need))
        return res

    @classmethod
    def from_numpy(cls, out: Tensor, array: np.ndarray, opts=None) -> Tensor:
        """Zero-staging variant of from_binary for harnesses: uploads straight from the array."""
        opts = cls.init(opts)
        array = np.ascontiguousarray(array)
        need = out.size * T.size_bytes(out.type)
        if array.nbytes < need:
            raise ValueError("binary size is too small for the requested shape")
        res = cls._alloc(out, opts["device"])
        if need:
            L.check(L.lib.hipnx_h2d(res.data.ref.ctx, res.data.ref.handle, 0, array.ctypes.data_as(C.c_void_p), need))
        return res

    @classmethod
    def to_binary(cls, t: Tensor, limit: int) -> bytes:
        """to_binary/2 (backend.ex:57): `limit` counts elements."""
        n = min(int(limit), t.size) * T.size_bytes(t.type)
        # the device writes straight into the bytes object that is returned (allocated unfilled, as the C API
        # provides for a buffer that is filled before anyone sees it): a zeroed staging buffer and the copy out
        # of it cost four times the transfer itself (256 MiB: 124 ms against 26 ms)
        raw = _new_bytes(None, n)
        address = _bytes_address(raw)
        _advise_huge_pages(address, n)
        L.check(L.lib.hipnx_d2h(t.data.ref.ctx, cls._handle(t), 0, address, n))
        if T.is_sub_byte(t.type):  # packed again on the way out (exla/lib/exla/device_buffer.ex:65-75)
            return pack_sub_byte(np.frombuffer(raw, dtype=np.uint8), t.type)
        return raw

    @classmethod
    def to_numpy(cls, t: Tensor) -> np.ndarray:
        arr = np.empty(t.shape, dtype=T.numpy_dtype(t.type))
        L.check(L.lib.hipnx_d2h(t.data.ref.ctx, cls._handle(t), 0, arr.ctypes.data_as(C.c_void_p), arr.nbytes))
        return arr

    _scalar_cache = {}  # (device, type, encoded element) -> _Ref of a rank-0 constant
    _scalar_refs = {}   # (device, type, number, its class) -> the same _Ref, found without encoding the number

    @classmethod
    def constant(cls, out: Tensor, number, opts=None) -> Tensor:
        """constant/3 (backend.ex:49; oracle binary_backend.ex:42-46).  Rank-0 constants -- what
        `Nx.multiply(t, 0.5)` turns its number into -- are kept per device and shared: tensors are
        immutable, and the cache holds its own share of the buffer, so deallocating one user
        never frees it."""
        if out.shape == () and number.__class__ in (int, float) and (not opts or (len(opts) == 1 and "device" in opts)):
            # the number met before, on this device, in this type: its buffer at once
            device = opts["device"] if opts else 0
            memo = (device, out.type, number.hex() if number.__class__ is float else number, number.__class__)
            ref = cls._scalar_refs.get(memo)
            if ref is not None and device not in _capturing:
                ref.sharers += 1
                return out.with_(data=HipNxBackend(ref, device))
        else:
            memo = None
        opts = cls.init(opts)
        if T.is_sub_byte(out.type):
            number_to_binary(number, out.type)  # the reference's argument checks
            elem = wrap_to_type(np.array([int(number)]), out.type).tobytes()
        else:
            # the same few numbers come back all the time (the 0.5 of `multiply(t, 0.5)`): their encodings are kept
            # (a float by its sign and hex digits: 0.0 and -0.0 are equal as dictionary keys, and so are 1 and 1.0)
            if number.__class__ in (int, float, bool):
                memo = (out.type, number.hex() if number.__class__ is float else number, number.__class__)
                elem = _encoded.get(memo)
                if elem is None:
                    elem = number_to_binary(number, out.type)
                    if len(_encoded) > 4096:
                        _encoded.clear()
                    _encoded[memo] = elem
            else:
                elem = number_to_binary(number, out.type)
        if out.shape == ():
            key = (opts["device"], out.type, elem)
            ref = cls._scalar_cache.get(key)
            if opts["device"] in _capturing:
                # While capturing, a constant is always the graph's own: allocated and filled inside the
                # capture (the block belongs to the graph, the fill is replayed with it).  A cached block
                # would be referenced by address only -- once the cache lets go of it (it is cleared after
                # 1024 distinct numbers) the pool hands it to someone else and every later replay reads
                # what they wrote.
                res = cls._alloc(out, opts["device"])
                L.check(L.lib.hipnx_fill(res.data.ref.ctx, res.data.ref.handle, len(elem), elem, 1))
                return res
            if ref is None:
                if len(cls._scalar_cache) >= 1024:
                    cls._scalar_cache.clear()
                    cls._scalar_refs.clear()
                res = cls._alloc(out, opts["device"])
                L.check(L.lib.hipnx_fill(res.data.ref.ctx, res.data.ref.handle, len(elem), elem, 1))
                ref = cls._scalar_cache[key] = res.data.ref
            if memo is not None:
                if len(cls._scalar_refs) >= 4096:
                    cls._scalar_refs.clear()
                cls._scalar_refs[memo] = ref
            ref.sharers += 1
            return out.with_(data=cls(ref, opts["device"]))
        res = cls._alloc(out, opts["device"])
        L.check(L.lib.hipnx_fill(res.data.ref.ctx, res.data.ref.handle, len(elem), elem, out.size))
        return res

    @classmethod
    def backend_copy(cls, t: Tensor, backend, opts=None) -> Tensor:
        """backend_copy/3 (backend.ex:52)."""
        if backend is HipNxBackend:
            opts = cls.init(opts)
            if opts["device"] == t.data.device:
                res = cls._alloc(t, opts["device"])
                L.check(L.lib.hipnx_d2d(res.data.ref.ctx, res.data.ref.handle, 0, cls._handle(t), 0, res.data.ref.nbytes))
                return res
        return backend.from_binary(t, cls.to_binary(t, t.size), opts)

    @classmethod
    def backend_transfer(cls, t: Tensor, backend, opts=None) -> Tensor:
        """backend_transfer/3 (backend.ex:51): copy, then deallocate the source."""
        if backend is HipNxBackend and cls.init(opts)["device"] == t.data.device:
            return t
        res = cls.backend_copy(t, backend, opts)
        cls.backend_deallocate(t)
        return res

    @classmethod
    def backend_deallocate(cls, t: Tensor) -> str:
        """backend_deallocate/1 (backend.ex:53): "ok" the first time, "already_deallocated" after
        (torchx/test/torchx/device_test.exs:30-37)."""
        d = t.data
        if d.released:
            return "already_deallocated"
        d.released = True
        d.ref.sharers -= 1
        if d.ref.sharers > 0:
            return "ok"
        st = L.check(L.lib.hipnx_buf_free(d.ref.handle))
        return "ok" if st == L.OK else "already_deallocated"

    @classmethod
    def inspect(cls, t: Tensor, limit: int = 50) -> str:
        """inspect/2 (backend.ex:56): reads limit+1 elements like torchx backend.ex:2013-2035."""
        from .tensor import to_float64, binary_to_numpy
        n = min(t.size, limit + 1)
        binary = cls.to_binary(t, n)
        vals = to_float64(binary, t.type) if T.is_float(t.type) else binary_to_numpy(binary, t.type, (n,))
        body = ", ".join(str(v) for v in vals[:limit]) + (", ..." if n > limit else "")
        dims = "".join(f"[{d}]" for d in t.shape)
        return f"#Nx.Tensor<\n  {T.name(t.type)}{dims}\n  HipNx.Backend({t.data.device})\n  [{body}]\n>"

    # ---- metadata-only: the buffer is immutable, so these share it ------------------------
    @classmethod
    def _alias(cls, out: Tensor, t: Tensor) -> Tensor:
        cls._handle(t)
        t.data.ref.sharers += 1
        return out.with_(data=cls(t.data.ref, t.data.device))

    @classmethod
    def reshape(cls, out, t):
        return cls._alias(out, cls._from_nx(t, 0))

    @classmethod
    def squeeze(cls, out, t, axes):
        return cls._alias(out, cls._from_nx(t, 0))

    @classmethod
    def bitcast(cls, out, t):
        t = cls._from_nx(t, 0)
        if T.is_sub_byte(out.type) and t.type != out.type:
            # same bits, the other signedness: the byte an element lives in is extended differently
            res = cls._alloc(out, t.data.device)
            L.check(L.lib.hipnx_as_type(res.data.ref.ctx, T.code(t.type), T.code(out.type), out.size, cls._handle(t),
                                        res.data.ref.handle))
            return cls._narrow(res)
        return cls._alias(out, t)

    # ---- element-wise ----------------------------------------------------------------------
    @classmethod
    def _binary(cls, op: int, out: Tensor, l: Tensor, r: Tensor) -> Tensor:
        ld, rd = l.data, r.data
        if ld.__class__ is HipNxBackend and rd.__class__ is HipNxBackend:
            dev = ld.device
        else:
            dev = cls._device_of(l, r)
            l, r = cls._from_nx(l, dev), cls._from_nx(r, dev)
            ld, rd = l.data, r.data
        if ld.released or rd.released:
            raise L.HipNxError(L.EFREED, "tensor has been deallocated")
        # what the call needs of types and shapes repeats from call to call: worked out once per signature
        key = (l.type, l.shape, r.type, r.shape, out.type, out.shape)
        plan = _binary_plans.get(key)
        if plan is None:
            if len(_binary_plans) > 4096:
                _binary_plans.clear()
            shape = out.shape
            plan = _binary_plans[key] = (T.code(l.type), T.code(r.type), T.code(out.type), len(shape), L.i64_array(shape),
                                         L.broadcast_stride_array(l.shape, shape), L.broadcast_stride_array(r.shape, shape),
                                         out.size * T.size_bytes(out.type), out.type[1] < 8)
        lc, rc, oc, rank, dims, ls, rs, nbytes, narrow = plan
        ctx = _Context.get(dev)
        ref = _fresh_ref(ctx, nbytes)
        res = out.with_(data=HipNxBackend(ref, dev))
        status = L.lib.hipnx_binary(ctx, op, lc, rc, oc, rank, dims, ls, rs, ld.ref.handle, rd.ref.handle, ref.handle)
        if status:
            L.check(status)
        return cls._narrow(res) if narrow else res

    @classmethod
    def _unary(cls, op: int, out: Tensor, t: Tensor) -> Tensor:
        td = t.data
        if td.__class__ is HipNxBackend and t.type[1] >= 8 and out.type[1] >= 8:  # the usual call, without the detours below
            if td.released:
                raise L.HipNxError(L.EFREED, "tensor has been deallocated")
            dev = td.device
            ctx = _Context.get(dev)
            n = out.size
            ref = _fresh_ref(ctx, n * T.size_bytes(out.type))
            status = L.lib.hipnx_unary(ctx, op, T.code(t.type), T.code(out.type), n, td.ref.handle, ref.handle)
            if status:
                L.check(status)
            return out.with_(data=HipNxBackend(ref, dev))
        dev = cls._device_of(t)
        t = cls._from_nx(t, dev)
        if t.type[1] < 8 and op in _BIT_COUNTS:
            if UNARY_OPS[op] == "count_leading_zeros":  # no clause in the reference either (binary_backend.ex:962-966)
                raise NotImplementedError("count_leading_zeros of a sub-byte integer")
            # population_count reads the element as an unsigned segment of its width (binary_backend.ex:844-850)
            t = cls.bitcast(t.with_(type=("u", t.type[1])), t)
        res = cls._alloc(out, dev)
        L.check(L.lib.hipnx_unary(res.data.ref.ctx, op, T.code(t.type), T.code(out.type), out.size, cls._handle(t),
                                  res.data.ref.handle))
        return cls._narrow(res) if out.type[1] < 8 else res

    @classmethod
    def as_type(cls, out: Tensor, t: Tensor) -> Tensor:
        """as_type/2 (backend.ex:68; oracle binary_backend.ex:2031-2076)."""
        dev = cls._device_of(t)
        t = cls._from_nx(t, dev)
        if t.type == out.type:
            return t
        res = cls._alloc(out, dev)
        L.check(L.lib.hipnx_as_type(res.data.ref.ctx, T.code(t.type), _out_code(out.type), out.size, cls._handle(t),
                                    res.data.ref.handle))
        if out.type[1] < 8:
            res = cls._narrow(res)
            if T.is_float(t.type):
                # an infinity becomes the narrow type's own extreme, not the low bits of the 8-bit one
                # (binary_backend.ex:2062-2069)
                kind, bits = out.type
                lo, hi = (-(1 << (bits - 1)), (1 << (bits - 1)) - 1) if kind == "s" else (0, (1 << bits) - 1)
                u8 = out.with_(type=("u", 8))
                zero = cls.constant(t.with_(shape=()), 0.0, {"device": dev})
                extreme = cls.select(out, cls.greater(u8, t, zero), cls.constant(out.with_(shape=()), hi, {"device": dev}),
                                     cls.constant(out.with_(shape=()), lo, {"device": dev}))
                res = cls.select(out, cls.is_infinity(u8, t), extreme, res)
        return res

    # ---- reductions ------------------------------------------------------------------------
    @classmethod
    def _view_for_axes(cls, t: Tensor, axes):
        """Collapses `t` to [outer, red, inner] for a reduction over `axes` (all axes if None).
        Non-adjacent axes are brought together by a device transpose to kept ++ reduced, which
        keeps the row-major order of the reduced axes (binary_backend.ex:2469-2512)."""
        rank = len(t.shape)
        if axes is None:
            return t, 1, t.size, 1
        axes = sorted(axes)
        if not axes:
            return t, t.size, 1, 1
        if axes == list(range(axes[0], axes[-1] + 1)):
            return t, prod(t.shape[:axes[0]]), prod(t.shape[axes[0]:axes[-1] + 1]), prod(t.shape[axes[-1] + 1:])
        kept = [a for a in range(rank) if a not in axes]
        perm = kept + axes
        tt = cls.transpose(t.with_(shape=S.transpose(t.shape, perm)), t, perm)
        return tt, prod(t.shape[a] for a in kept), prod(t.shape[a] for a in axes), 1

    @classmethod
    def _reduce(cls, op: int, out: Tensor, t: Tensor, opts) -> Tensor:
        axes = opts.get("axes")
        td = t.data
        if td.__class__ is HipNxBackend:
            # the usual call -- one run of neighbouring axes (or all of them) of a tensor that is here -- by its
            # signature: the view [outer, red, inner], the type codes and the result's size are worked out once
            key = (t.type, t.shape, out.type, None if axes is None else tuple(axes))
            plan = _reduce_plans.get(key)
            if plan is None and t.type[1] >= 8 and out.type[1] >= 8:
                run = None if axes is None else sorted(a % len(t.shape) for a in axes)
                if run is None or (run and run == list(range(run[0], run[-1] + 1))):
                    _, outer, red, inner = cls._view_for_axes(t, run)
                    if len(_reduce_plans) > 4096:
                        _reduce_plans.clear()
                    plan = _reduce_plans[key] = (T.code(t.type), T.code(out.type), outer, red, inner, out.size * T.size_bytes(out.type))
            if plan is not None:
                if td.released:
                    raise L.HipNxError(L.EFREED, "tensor has been deallocated")
                ic, oc, outer, red, inner, nbytes = plan
                dev = td.device
                ctx = _Context.get(dev)
                ref = _fresh_ref(ctx, nbytes)
                status = L.lib.hipnx_reduce(ctx, op, ic, oc, outer, red, inner, td.ref.handle, ref.handle)
                if status:
                    L.check(status)
                return out.with_(data=HipNxBackend(ref, dev))
        dev = cls._device_of(t)
        t = cls._from_nx(t, dev)
        if axes is not None and len(axes) > 1 and t.type[1] >= 8:
            axes = sorted(a % len(t.shape) for a in axes)
            runs = [[a] for a in axes[:1]]
            for a in axes[1:]:
                if a == runs[-1][-1] + 1:
                    runs[-1].append(a)
                else:
                    runs.append([a])
            if len(runs) > 1:
                # Reduced axes that are not neighbours: one pass per run of neighbouring axes, innermost run
                # first, instead of a transposed copy of the whole tensor.  Sums and products pass through
                # f64 / 64-bit integers (the accumulators' own types), so the result is still rounded or
                # wrapped once; among equal extremes the first in row-major order of the reduced axes still wins.
                if op in (RED_SUM, RED_PRODUCT):
                    mid = ("f", 64) if T.is_float(out.type) else (out.type[0] if out.type[0] in ("s", "u") else "s", 64)
                else:
                    mid = out.type
                cur, shape = t, list(t.shape)
                for i, run in enumerate(reversed(runs)):
                    last = i == len(runs) - 1
                    outer, red, inner = prod(shape[:run[0]]), prod(shape[run[0]:run[-1] + 1]), prod(shape[run[-1] + 1:])
                    shape = shape[:run[0]] + shape[run[-1] + 1:]
                    step = out if last else out.with_(data=None, type=mid, shape=tuple(shape))
                    res = cls._alloc(step, dev)
                    L.check(L.lib.hipnx_reduce(res.data.ref.ctx, op, T.code(cur.type), T.code(step.type), outer, red, inner,
                                               cls._handle(cur), res.data.ref.handle))
                    cur = res
                return cur
        view, outer, red, inner = cls._view_for_axes(t, axes)
        res = cls._alloc(out, dev)
        L.check(L.lib.hipnx_reduce(res.data.ref.ctx, op, T.code(t.type), T.code(out.type), outer, red, inner,
                                   cls._handle(view), res.data.ref.handle))
        return res

    @classmethod
    def sum(cls, out, t, opts):
        return cls._reduce(RED_SUM, out, t, opts)

    @classmethod
    def product(cls, out, t, opts):
        return cls._reduce(RED_PRODUCT, out, t, opts)

    @classmethod
    def reduce_max(cls, out, t, opts):
        return cls._reduce(RED_MAX, out, t, opts)

    @classmethod
    def reduce_min(cls, out, t, opts):
        return cls._reduce(RED_MIN, out, t, opts)

    @classmethod
    def all(cls, out, t, opts):
        """all/3 (backend.ex:87; oracle binary_backend.ex:1293-1302): 1 unless an element is 0."""
        return cls._reduce(RED_ALL, out, t, opts)

    @classmethod
    def any(cls, out, t, opts):
        """any/3 (backend.ex:88; oracle binary_backend.ex:1305-1314): 1 if an element is not 0."""
        return cls._reduce(RED_ANY, out, t, opts)

    @classmethod
    def _argreduce(cls, op: int, out: Tensor, t: Tensor, opts) -> Tensor:
        dev = cls._device_of(t)
        t = cls._from_nx(t, dev)
        axis = opts.get("axis")
        tie = {"low": 0, "high": 1}[opts.get("tie_break", "low")]
        view, outer, red, inner = cls._view_for_axes(t, None if axis is None else [axis])
        res = cls._alloc(out, dev)
        L.check(L.lib.hipnx_argreduce(res.data.ref.ctx, op, tie, T.code(t.type), T.code(out.type), outer, red, inner,
                                      cls._handle(view), res.data.ref.handle))
        return res

    @classmethod
    def argmax(cls, out, t, opts):
        return cls._argreduce(0, out, t, opts)

    @classmethod
    def argmin(cls, out, t, opts):
        return cls._argreduce(1, out, t, opts)

    # ---- contraction -----------------------------------------------------------------------
    @classmethod
    def _dot_operand(cls, t: Tensor, contract, nbatch: int):
        """Returns (tensor, layout, kept_size): the operand as [batch, rows, K] (K_INNER) or
        [batch, K, rows] (K_OUTER) without a copy when the axes already sit that way, else
        transposed on the device to [batch, kept, contract] as binary_backend.ex:561-599 does."""
        rank = len(t.shape)
        batch = list(range(nbatch))
        kept = [a for a in range(nbatch, rank) if a not in contract]
        rows = prod(t.shape[a] for a in kept)
        if batch + kept + list(contract) == list(range(rank)):
            return t, K_INNER, rows
        if batch + list(contract) + kept == list(range(rank)):
            return t, K_OUTER, rows
        perm = batch + kept + list(contract)
        return cls.transpose(t.with_(shape=S.transpose(t.shape, perm)), t, perm), K_INNER, rows

    @classmethod
    def dot(cls, out: Tensor, l: Tensor, c1, b1, r: Tensor, c2, b2) -> Tensor:
        """dot/7 (backend.ex:77; oracle binary_backend.ex:476-599).  Contraction axes are paired
        in the given order; the pairs are walked in increasing left-axis order so that the left
        operand needs no copy whenever its contracted axes are adjacent."""
        dev = cls._device_of(l, r)
        l, r = cls._from_nx(l, dev), cls._from_nx(r, dev)
        # operands that already sit as [batch, rows, K] or [batch, K, rows] need no copy: that, and the
        # extents, follow from the shapes and axes alone and are worked out once per signature
        key = (l.shape, tuple(c1), len(b1), r.shape, tuple(c2))
        plan = cls._dot_plans.get(key)
        if plan is None:
            pairs = sorted(zip(c1, c2))
            c1s, c2s = [p[0] for p in pairs], [p[1] for p in pairs]
            nb = len(b1)
            direct = []
            for t, cs in ((l, c1s), (r, c2s)):
                rank = len(t.shape)
                kept = [a for a in range(nb, rank) if a not in cs]
                head = list(range(nb))
                layout = K_INNER if head + kept + cs == list(range(rank)) else K_OUTER if head + cs + kept == list(range(rank)) else None
                direct.append((layout, prod(t.shape[a] for a in kept)))
            plan = (c1s, c2s, nb, prod(l.shape[a] for a in c1s), prod(l.shape[a] for a in b1), direct)
            if len(cls._dot_plans) >= 4096:
                cls._dot_plans.clear()
            cls._dot_plans[key] = plan
        c1s, c2s, nb, K, batch, ((l_layout, M), (r_layout, N)) = plan
        lt, rt = l, r
        if l_layout is None:
            lt, l_layout, M = cls._dot_operand(l, c1s, nb)
        if r_layout is None:
            rt, r_layout, N = cls._dot_operand(r, c2s, nb)
        res = cls._alloc(out, dev)
        status = L.lib.hipnx_dot(res.data.ref.ctx, T.code(l.type), T.code(r.type), _out_code(out.type), batch, M, N, K,
                                 l_layout, r_layout, cls._handle(lt), cls._handle(rt), res.data.ref.handle)
        if status:
            L.check(status)
        return cls._narrow(res) if out.type[1] < 8 else res

    _dot_plans = {}

    # ---- data movement ---------------------------------------------------------------------
    @classmethod
    def dot_scaled(cls, out: Tensor, l: Tensor, c1, b1, r: Tensor, c2, b2, scale: Tensor, mode: int) -> Tensor:
        """`multiply(as_type(dot(l, r) with an s32 result, f32), scale)` in one kernel: the quantised
        linear layer (the evaluator offers it when it finds that chain; backend.ex:77, 68, 115).
        `mode`: SCALE_PER_COLUMN (one scale per entry of the right operand's free axes), SCALE_PER_ROW
        or SCALE_ONE.  Raises HipNxError with status EUNSUPPORTED for what the kernel does not take:
        the caller then makes the three calls."""
        if l.type != ("s", 8) or r.type != ("s", 8) or scale.type != ("f", 32) or out.type != ("f", 32):
            raise L.HipNxError(L.EUNSUPPORTED, "dot_scaled: s8 operands, f32 scales and result")
        dev = cls._device_of(l, r, scale)
        l, r, scale = cls._from_nx(l, dev), cls._from_nx(r, dev), cls._from_nx(scale, dev)
        pairs = sorted(zip(c1, c2))
        c1s, c2s = [p[0] for p in pairs], [p[1] for p in pairs]
        nb = len(b1)
        K = prod(l.shape[a] for a in c1s)
        batch = prod(l.shape[a] for a in b1)
        lt, l_layout, M = cls._dot_operand(l, c1s, nb)
        rt, r_layout, N = cls._dot_operand(r, c2s, nb)
        res = cls._alloc(out, dev)
        L.check(L.lib.hipnx_dot_scaled(res.data.ref.ctx, T.code(l.type), T.code(r.type), batch, M, N, K, l_layout, r_layout,
                                       cls._handle(lt), cls._handle(rt), mode, cls._handle(scale), res.data.ref.handle))
        return res

    @classmethod
    def transpose(cls, out: Tensor, t: Tensor, axes) -> Tensor:
        """transpose/3 (backend.ex:73; oracle binary_backend.ex:280-306)."""
        dev = cls._device_of(t)
        t = cls._from_nx(t, dev)
        res = cls._alloc(out, dev)
        L.check(L.lib.hipnx_transpose(res.data.ref.ctx, T.size_bytes(t.type), len(t.shape), L.i64_array(t.shape),
                                      L.int_array(axes), cls._handle(t), res.data.ref.handle))
        return res

    @classmethod
    def broadcast(cls, out: Tensor, t: Tensor, shape, axes) -> Tensor:
        """broadcast/4 (backend.ex:72; oracle binary_backend.ex:215-276): input axis i maps to
        output axis axes[i]; size-1 input axes and unmapped output axes repeat."""
        dev = cls._device_of(t)
        t = cls._from_nx(t, dev)
        strides = [0] * len(shape)
        s = 1
        for pos in range(len(t.shape) - 1, -1, -1):
            if t.shape[pos] != 1:
                strides[axes[pos]] = s
            s *= t.shape[pos]
        res = cls._alloc(out, dev)
        L.check(L.lib.hipnx_broadcast(res.data.ref.ctx, T.size_bytes(t.type), len(shape), L.i64_array(shape),
                                      L.i64_array(strides), cls._handle(t), res.data.ref.handle))
        return res

    @classmethod
    def _take_along(cls, out: Tensor, t: Tensor, indices: Tensor, axis: int) -> Tensor:
        """block(%Nx.Block.Take{axis}) along an axis that is not the first (backend.ex:144; nx.ex:14807-14819): one
        kernel over the tensor viewed as [outer, axis_len, inner] instead of the default's transpose, gather and
        transpose back.  An out-of-range index is reported as the default reports it: against the shape with the
        taken axis moved to the front (binary_backend.ex:1906-1912, 1949-1952)."""
        dev = cls._device_of(t, indices)
        t, indices = cls._from_nx(t, dev), cls._from_nx(indices, dev)
        shape = t.shape
        outer, axis_len, inner = prod(shape[:axis]), shape[axis], prod(shape[axis + 1:])
        moved = (axis_len,) + shape[:axis] + shape[axis + 1:]
        res = cls._alloc(out, dev)
        L.check(L.lib.hipnx_take(res.data.ref.ctx, T.size_bytes(t.type), outer, axis_len, inner, T.code(indices.type),
                                 indices.size, _bounds["policy"], len(moved), L.i64_array(moved), cls._handle(t),
                                 cls._handle(indices), res.data.ref.handle))
        return res

    @classmethod
    def gather(cls, out: Tensor, t: Tensor, indices: Tensor, opts) -> Tensor:
        """gather/4 (backend.ex:81; oracle binary_backend.ex:1902-1959): out-of-bounds indices
        raise, with the reference's message."""
        dev = cls._device_of(t, indices)
        t, indices = cls._from_nx(t, dev), cls._from_nx(indices, dev)
        axes = list(opts["axes"])
        rank = len(t.shape)
        if list(range(rank))[:len(axes)] != axes:
            perm = axes + [a for a in range(rank) if a not in axes]
            t = cls.transpose(t.with_(shape=S.transpose(t.shape, perm)), t, perm)
        depth = indices.shape[-1]
        n_tuples = prod(indices.shape[:-1])
        res = cls._alloc(out, dev)
        L.check(L.lib.hipnx_gather(res.data.ref.ctx, T.size_bytes(t.type), rank, L.i64_array(t.shape),
                                   T.code(indices.type), n_tuples, depth, opts.get("oob_policy", _bounds["policy"]),
                                   cls._handle(t), cls._handle(indices), res.data.ref.handle))
        return res

    # ---- one step off the hot path: creation, selection, windows of memory -----------------------
    @classmethod
    def iota(cls, out: Tensor, axis, opts=None) -> Tensor:
        """iota/3 (backend.ex:51; oracle binary_backend.ex:49-87): the index along `axis`, or the flat
        index when `axis` is None."""
        opts = cls.init(opts)
        res = cls._alloc(out, opts["device"])
        if axis is None:
            dim, inner = max(out.size, 1), 1
        else:
            dim, inner = out.shape[axis], prod(out.shape[axis + 1:])
        L.check(L.lib.hipnx_iota(res.data.ref.ctx, T.code(out.type), out.size, dim, inner, res.data.ref.handle))
        return cls._narrow(res) if out.type[1] < 8 else res

    @classmethod
    def eye(cls, out: Tensor, opts=None) -> Tensor:
        """eye/2 (backend.ex:50; oracle binary_backend.ex:90-110): identity in the last two axes."""
        opts = cls.init(opts)
        res = cls._alloc(out, opts["device"])
        L.check(L.lib.hipnx_eye(res.data.ref.ctx, T.code(out.type), out.size, out.shape[-2], out.shape[-1],
                                res.data.ref.handle))
        return res

    @classmethod
    def select(cls, out: Tensor, pred: Tensor, on_true: Tensor, on_false: Tensor) -> Tensor:
        """select/4 (backend.ex:84; oracle binary_backend.ex:604-648)."""
        dev = cls._device_of(pred, on_true, on_false)
        pred, on_true, on_false = (cls._from_nx(x, dev) for x in (pred, on_true, on_false))
        res = cls._alloc(out, dev)
        L.check(L.lib.hipnx_select(
            res.data.ref.ctx, T.code(pred.type), T.code(on_true.type), T.code(on_false.type), T.code(out.type),
            len(out.shape), L.i64_array(out.shape), L.i64_array(S.broadcast_strides(pred.shape, out.shape)),
            L.i64_array(S.broadcast_strides(on_true.shape, out.shape)),
            L.i64_array(S.broadcast_strides(on_false.shape, out.shape)),
            cls._handle(pred), cls._handle(on_true), cls._handle(on_false), res.data.ref.handle))
        return res

    @classmethod
    def clip(cls, out: Tensor, t: Tensor, min_t: Tensor, max_t: Tensor) -> Tensor:
        """clip/4 (backend.ex:78; oracle binary_backend.ex:1788-1811)."""
        dev = cls._device_of(t, min_t, max_t)
        t, min_t, max_t = (cls._from_nx(x, dev) for x in (t, min_t, max_t))
        res = cls._alloc(out, dev)
        L.check(L.lib.hipnx_clip(res.data.ref.ctx, T.code(t.type), T.code(min_t.type), T.code(max_t.type),
                                 T.code(out.type), out.size, cls._handle(t), cls._handle(min_t), cls._handle(max_t),
                                 res.data.ref.handle))
        return res

    @staticmethod
    def _dense_strides(shape):
        strides, s = [0] * len(shape), 1
        for a in range(len(shape) - 1, -1, -1):
            strides[a] = s
            s *= shape[a]
        return strides

    @classmethod
    def slice(cls, out: Tensor, t: Tensor, start_indices, lengths, strides) -> Tensor:
        """slice/5 (backend.ex:79; oracle binary_backend.ex:1813-1863): start indices are numbers or
        rank-0 tensors (read back when on the device) and are clamped so the window fits."""
        dev = cls._device_of(t)
        t = cls._from_nx(t, dev)
        starts = []
        for dim, idx, length in zip(t.shape, start_indices, lengths):
            if isinstance(idx, Tensor):
                idx = int(np.frombuffer(type(idx.data).to_binary(idx, 1), dtype=T.numpy_dtype(idx.type))[0])
            starts.append(min(max(int(idx), 0), dim - length))
        dense = cls._dense_strides(t.shape)
        res = cls._alloc(out, dev)
        L.check(L.lib.hipnx_strided_copy(
            res.data.ref.ctx, T.size_bytes(t.type), len(out.shape), L.i64_array(out.shape),
            L.i64_array([d * s for d, s in zip(dense, strides)]), sum(d * s for d, s in zip(dense, starts)),
            L.i64_array(cls._dense_strides(out.shape)), 0, cls._handle(t), res.data.ref.handle))
        return res

    @classmethod
    def to_batched(cls, out: Tensor, t: Tensor, opts):
        """to_batched/3 (backend.ex:58; oracle binary_backend.ex:178-211): a lazy sequence of
        batches of out.shape[0] leading entries -- each one contiguous copy; with leftover "repeat"
        a last, short batch is completed from the tensor's first entries (two copies into one
        buffer)."""
        dev = cls._device_of(t)
        t = cls._from_nx(t, dev)
        batch, total = out.shape[0], t.shape[0]
        full, rest = divmod(total, batch)
        row = prod(t.shape[1:]) * T.size_bytes(t.type)

        def window(res, first, count, at):
            # `count` leading entries starting at entry `first`, written from entry `at` of the batch
            if count and row:
                L.check(L.lib.hipnx_strided_copy(
                    res.data.ref.ctx, 1, 1, L.i64_array([count * row]), L.i64_array([1]), first * row, L.i64_array([1]),
                    at * row, cls._handle(t), res.data.ref.handle))

        def batches():
            for i in range(full + (1 if rest and opts.get("leftover", "repeat") == "repeat" else 0)):
                res = cls._alloc(out, dev)
                if i < full:
                    window(res, i * batch, batch, 0)
                else:
                    window(res, full * batch, rest, 0)
                    window(res, 0, batch - rest, rest)
                yield res

        return batches()

    @classmethod
    def pad(cls, out: Tensor, t: Tensor, pad_value: Tensor, padding_config) -> Tensor:
        """pad/4 (backend.ex:74; oracle binary_backend.ex:326-431): interior padding first, then the
        edges, where a negative edge cuts into the interior-padded axis.  Element i of an axis lands
        at low + i * (interior + 1); the ones that land inside the output are one strided copy into
        a buffer filled with the pad value.  Operands are converted to out.type first (the oracle
        splices the two encodings when they differ; EXLA and Torchx convert)."""
        if t.shape == ():
            return t  # as the oracle does, whatever out.type says
        dev = cls._device_of(t, pad_value)
        t, pad_value = cls._from_nx(t, dev), cls._from_nx(pad_value, dev)
        if any(d < 0 for d in out.shape):
            raise ValueError(f"padding configuration crops more than the tensor holds: output shape {out.shape!r}")
        if t.type != out.type:
            t = cls.as_type(t.with_(data=None, type=out.type), t)
        if pad_value.type != out.type:
            pad_value = cls.as_type(pad_value.with_(data=None, type=out.type), pad_value)
        res = cls._alloc(out, dev)
        rank = len(out.shape)
        ctx, esz = res.data.ref.ctx, T.size_bytes(out.type)
        L.check(L.lib.hipnx_broadcast(ctx, esz, rank, L.i64_array(out.shape), L.i64_array([0] * rank),
                                      cls._handle(pad_value), res.data.ref.handle))
        counts, first = [], []
        for dim, odim, (low, _high, interior) in zip(t.shape, out.shape, padding_config):
            step = interior + 1
            lo = -(min(low, 0) // step)                      # first i with low + i * step >= 0
            hi = min(dim - 1, (odim - 1 - low) // step) if odim > 0 else -1
            counts.append(max(hi - lo + 1, 0))
            first.append(lo)
        if all(counts):
            dense_in, dense_out = cls._dense_strides(t.shape), cls._dense_strides(out.shape)
            steps = [c[2] + 1 for c in padding_config]
            L.check(L.lib.hipnx_strided_copy(
                ctx, esz, rank, L.i64_array(counts), L.i64_array(dense_in), sum(f * d for f, d in zip(first, dense_in)),
                L.i64_array([s * d for s, d in zip(steps, dense_out)]),
                sum((c[0] + f * s) * d for c, f, s, d in zip(padding_config, first, steps, dense_out)),
                cls._handle(t), res.data.ref.handle))
        return res

    @classmethod
    def reverse(cls, out: Tensor, t: Tensor, axes) -> Tensor:
        """reverse/3 (backend.ex:75; oracle binary_backend.ex:434-474): one copy that reads the given
        axes backwards."""
        dev = cls._device_of(t)
        t = cls._from_nx(t, dev)
        dense = cls._dense_strides(t.shape)
        strides = [-s if a in axes else s for a, s in enumerate(dense)]
        offset = sum((t.shape[a] - 1) * dense[a] for a in axes)
        res = cls._alloc(out, dev)
        L.check(L.lib.hipnx_strided_copy(res.data.ref.ctx, T.size_bytes(t.type), len(t.shape), L.i64_array(t.shape),
                                         L.i64_array(strides), offset, L.i64_array(dense), 0, cls._handle(t), res.data.ref.handle))
        return res

    @classmethod
    def put_slice(cls, out: Tensor, t: Tensor, start_indices, slice_t: Tensor) -> Tensor:
        """put_slice/4 (backend.ex:80; oracle binary_backend.ex:1865-1900): both operands in
        out.type, start indices clamped so the slice fits, the slice written into a copy of `t`."""
        dev = cls._device_of(t, slice_t)
        t, slice_t = cls._from_nx(t, dev), cls._from_nx(slice_t, dev)
        if t.type != out.type:
            t = cls.as_type(t.with_(data=None, type=out.type), t)
        if slice_t.type != out.type:
            slice_t = cls.as_type(slice_t.with_(data=None, type=out.type), slice_t)
        starts = []
        for dim, idx, length in zip(t.shape, start_indices, slice_t.shape):
            if isinstance(idx, Tensor):
                idx = int(np.frombuffer(type(idx.data).to_binary(idx, 1), dtype=T.numpy_dtype(idx.type))[0])
            starts.append(min(max(int(idx), 0), dim - length))
        res = cls._alloc(out, dev)
        ctx = res.data.ref.ctx
        L.check(L.lib.hipnx_d2d(ctx, res.data.ref.handle, 0, cls._handle(t), 0, res.data.ref.nbytes))
        if slice_t.size:
            dense = cls._dense_strides(out.shape)
            L.check(L.lib.hipnx_strided_copy(
                ctx, T.size_bytes(out.type), len(slice_t.shape), L.i64_array(slice_t.shape),
                L.i64_array(cls._dense_strides(slice_t.shape)), 0, L.i64_array(dense),
                sum(s * d for s, d in zip(starts, dense)), cls._handle(slice_t), res.data.ref.handle))
        return res

    @classmethod
    def concatenate(cls, out: Tensor, tensors, axis: int) -> Tensor:
        """concatenate/3 (backend.ex:82; oracle binary_backend.ex:1975-1986): every operand is
        converted to the output type and copied into its window along `axis`."""
        dev = cls._device_of(*tensors)
        res = cls._alloc(out, dev)
        if not T.is_sub_byte(out.type) and len(tensors) >= 4:
            # one launch per 64 operands: the tensors viewed as [outer, their extent along the axis, inner] (two or three
            # large operands are a little faster as a copy each: 16384^2 f32 twice 0.70 ms against 0.76 ms)
            parts = []
            for t in tensors:
                t = cls._from_nx(t, dev)
                parts.append(t if t.type == out.type else cls.as_type(t.with_(data=None, type=out.type), t))
            handles = (L._buf_p * len(parts))(*[cls._handle(t) for t in parts])
            L.check(L.lib.hipnx_concat(res.data.ref.ctx, T.size_bytes(out.type), len(parts), handles,
                                       L.i64_array([t.shape[axis] for t in parts]), prod(out.shape[:axis]), prod(out.shape[axis + 1:]),
                                       res.data.ref.handle))
            return res
        out_strides = cls._dense_strides(out.shape)
        offset = 0
        for t in tensors:
            t = cls._from_nx(t, dev)
            if t.type != out.type:
                t = cls.as_type(t.with_(data=None, type=out.type), t)
            L.check(L.lib.hipnx_strided_copy(
                res.data.ref.ctx, T.size_bytes(out.type), len(t.shape), L.i64_array(t.shape),
                L.i64_array(cls._dense_strides(t.shape)), 0, L.i64_array(out_strides), offset * out_strides[axis],
                cls._handle(t), res.data.ref.handle))
            offset += t.shape[axis]
        return res

    @classmethod
    def stack(cls, out: Tensor, tensors, axis: int) -> Tensor:
        """stack/3 (backend.ex:83; oracle binary_backend.ex:1962-1972): concatenation of the operands
        with a unit axis inserted at `axis`."""
        widened = [t.with_(shape=t.shape[:axis] + (1,) + t.shape[axis:]) for t in tensors]
        return cls.concatenate(out, widened, axis)

    @classmethod
    def to_pointer(cls, t: Tensor, opts=None):
        """to_pointer/2 (backend.ex:66; semantics of exla/lib/exla/backend.ex:86-131): the device
        address of the tensor's buffer as a `Pointer` of kind "local", or with `mode: :ipc` a handle
        another process on the machine opens with `from_pointer` (kind "ipc": `handle` = the 64 bytes of
        the HIP IPC handle, `address` = the device index, as EXLA's cuda client fills them)."""
        opts = dict(opts or {})
        mode = opts.pop("mode", "local")
        opts.pop("permissions", None)  # host shared-memory permissions of EXLA's host client: nothing to set here
        if opts:
            raise ValueError(f"unknown options {sorted(opts)!r}")
        if mode not in ("local", "ipc"):
            raise ValueError(f"expected one of :local, :ipc, got: {mode!r}")
        from .nx import Pointer
        if mode == "ipc":
            raw = C.create_string_buffer(L.IPC_HANDLE_BYTES)
            L.check(L.lib.hipnx_buf_ipc_export(t.data.ref.ctx, cls._handle(t), raw))
            return Pointer(kind="ipc", address=t.data.device, data_size=t.size * T.size_bytes(t.type), handle=raw.raw)
        address = L.lib.hipnx_buf_device_ptr(cls._handle(t))
        return Pointer(kind="local", address=int(address), data_size=t.size * T.size_bytes(t.type))

    @classmethod
    def from_pointer(cls, pointer, type, shape, backend_opts=None, opts=None) -> Tensor:  # noqa: A002
        """from_pointer/5 (backend.ex:59-65; exla/lib/exla/backend.ex:133-181): a tensor over device
        memory that someone else owns.  `opts["keep"]`, if given, is held for the tensor's lifetime
        (the object that owns the memory)."""
        backend_opts, opts = cls.init(backend_opts), dict(opts or {})
        ty = T.normalize(type)
        size = prod(shape) * T.size_bytes(ty)
        if pointer.data_size != size:
            raise ValueError(f"invalid pointer data_size for shape, expected: {size}, got: {pointer.data_size}")
        if pointer.kind == "ipc":
            if pointer.handle is None or len(pointer.handle) != L.IPC_HANDLE_BYTES:
                raise ValueError(f"an :ipc pointer carries a handle of {L.IPC_HANDLE_BYTES} bytes")
            ref = _Ref(_Context.get(backend_opts["device"]), size, ipc_handle=pointer.handle)
            return Tensor(cls(ref, backend_opts["device"]), ty, tuple(shape), tuple(opts.get("names") or ()))
        if pointer.kind != "local":
            raise ValueError(f"expected a pointer of kind :local or :ipc, got: {pointer.kind!r}")
        ref = _Ref(_Context.get(backend_opts["device"]), size, address=pointer.address, keep=opts.get("keep"))
        return Tensor(cls(ref, backend_opts["device"]), ty, tuple(shape), tuple(opts.get("names") or ()))

    @classmethod
    def fused_elementwise(cls, out: Tensor, program, inputs, layout, reduce_op: int = -1, mode=None) -> Tensor:
        """A group of element-wise nodes in one kernel (the evaluator offers it groups it has found
        in a traced function).  `program` is a list of dicts with the fields of `hipnx_fused_instr`
        (`dt` as a type tuple); `layout` is (rows, cols, [(row_stride, col_stride) per input]).
        `reduce_op` (RED_SUM / RED_MAX / RED_MIN) reduces the group's value along its rows without
        storing it; `out` is then the reduction's template.  Raises HipNxError with status
        EUNSUPPORTED when the shapes do not fit the kernel: the caller then runs the nodes one by one.
        `mode` ("interpreted" / "compiled") runs this call in that mode whatever the device is set to."""
        dev = cls._device_of(*inputs) if inputs else 0
        # the library is switched when a call wants another mode than the last call had, not around every call:
        # the groups of a traced function all want the same one
        wanted = mode if mode is not None else _fused_modes.get(dev, "interpreted")
        if _fused_set.get(dev, "interpreted") != wanted:
            _set_fused_mode(wanted, dev)
        if not all(t.data.__class__ is HipNxBackend for t in inputs):
            inputs = [cls._from_nx(t, dev) for t in inputs]
        rows, cols, strides = layout
        prog = getattr(program, "packed", None)
        if prog is None:
            prog = (L.FusedInstr * len(program))()
            for q, ins in zip(prog, program):
                q.kind, q.op, q.src, q.arg = ins["kind"], ins.get("op", 0), ins.get("src", 0), ins.get("arg", 0)
                q.src2, q.arg2, q.flags, q.dt = ins.get("src2", 0), ins.get("arg2", 0), ins.get("flags", 0), T.code(ins["dt"])
                q.imm.f, q.imm2.f = ins.get("imm", 0.0), ins.get("imm2", 0.0)
                if "imm_bits" in ins:  # the constant of an integer instruction, as the bits it is
                    q.imm.bits = ins["imm_bits"]
            try:
                program.packed = prog  # a caller's list type with room for the packed form keeps it
            except AttributeError:
                pass
        n = max(len(inputs), 1)
        # types and strides repeat from call to call of a traced function: kept with the layout they belong to
        if getattr(program, "packed", None) is not prog:  # a plain list: its packed form lives for this call only
            return cls._fused_call(out, prog, len(program), inputs, layout, reduce_op, dev)
        key = (id(layout), id(prog), out.type, out.shape, *[t.type for t in inputs])
        cached = _fused_arrays.get(key)
        if cached is None or cached[0] is not layout or cached[1] is not prog:
            if len(_fused_arrays) > 4096:
                _fused_arrays.clear()
            cached = _fused_arrays[key] = (layout, prog, (C.c_int * n)(*[T.code(t.type) for t in inputs]),
                                           (C.c_int64 * n)(*[s[0] for s in strides]), (C.c_int * n)(*[s[1] for s in strides]),
                                           C.cast(prog, C.c_void_p), (C.c_void_p * n), T.code(out.type),
                                           out.size * T.size_bytes(out.type))
        _, _, dts, rs, cs, prog_ptr, handle_array, out_code, nbytes = cached
        for t in inputs:
            if t.data.released:
                raise L.HipNxError(L.EFREED, "tensor has been deallocated")
        handles = handle_array(*[t.data.ref.handle.value for t in inputs])
        ctx = _Context.get(dev)
        ref = _fresh_ref(ctx, nbytes)
        status = L.lib.hipnx_fused_elementwise(ctx, len(program), prog_ptr, len(inputs), handles, dts, rs, cs, rows, cols,
                                               reduce_op, out_code, ref.handle)
        if status:
            L.check(status)
        return out.with_(data=HipNxBackend(ref, dev))

    @classmethod
    def _fused_call(cls, out, prog, n_instr, inputs, layout, reduce_op, dev) -> Tensor:
        """fused_elementwise for a program whose packed form nobody keeps: every argument array made for this call."""
        rows, cols, strides = layout
        n = max(len(inputs), 1)
        res = cls._alloc(out, dev)
        handles = (C.c_void_p * n)(*[cls._handle(t) for t in inputs])
        L.check(L.lib.hipnx_fused_elementwise(res.data.ref.ctx, n_instr, C.cast(prog, C.c_void_p), len(inputs), handles,
                                              (C.c_int * n)(*[T.code(t.type) for t in inputs]), (C.c_int64 * n)(*[s[0] for s in strides]),
                                              (C.c_int * n)(*[s[1] for s in strides]), rows, cols, reduce_op, T.code(out.type),
                                              res.data.ref.handle))
        return res

    @classmethod
    def threefry2x32(cls, out: Tensor, key: Tensor) -> Tensor:
        """The random words of Nx.Random's threefry2x32/2 (random.ex:214-285) for `out.size`
        counters in one kernel; `out` is a u32 template.  Reached through block/4 with a
        `BlockThreefry`."""
        dev = cls._device_of(key)
        key = cls._from_nx(key, dev)
        res = cls._alloc(out, dev)
        L.check(L.lib.hipnx_threefry2x32(res.data.ref.ctx, cls._handle(key), out.size, res.data.ref.handle))
        return res

    @classmethod
    def block(cls, struct, out: Tensor, args, fun):
        """block/4 (backend.ex:144): `Nx.Block.Take` along axis 0 is one row-copy kernel; other
        blocks run their default implementation on this backend's callbacks."""
        from .nx import BlockTake, BlockThreefry
        if isinstance(struct, BlockTake) and struct.axis == 0:
            t, indices = args
            idx = indices.with_(shape=(indices.size, 1))
            return cls.gather(out, t, idx, {"axes": [0]})
        if isinstance(struct, BlockTake) and T.storage(args[0].type) == args[0].type:
            return cls._take_along(out, args[0], args[1], struct.axis)
        if isinstance(struct, BlockThreefry):
            return cls.threefry2x32(out, args[0])
        return fun(struct, *args)


def _install():
    for code, name in enumerate(BINARY_OPS):
        def binary(cls, out, l, r, _code=code):
            return cls._binary(_code, out, l, r)
        binary.__name__ = name
        binary.__doc__ = f"{name}/3 (backend.ex:115-123; oracle binary_backend.ex:649-823)."
        setattr(HipNxBackend, name, classmethod(binary))
    for code, name in enumerate(UNARY_OPS):
        def unary(cls, out, t, _code=code):
            return cls._unary(_code, out, t)
        unary.__name__ = name
        unary.__doc__ = f"{name}/2 (backend.ex:125-132; oracle binary_backend.ex:827-1005)."
        setattr(HipNxBackend, name, classmethod(unary))
    for name in UNSUPPORTED:
        def unsupported(cls, *args, _name=name, **kw):
            raise NotImplementedError(f"HipNx.Backend.{_name} is not on the device path")
        unsupported.__name__ = name
        setattr(HipNxBackend, name, classmethod(unsupported))


_install()


def sync(device: int = 0) -> None:
    L.check(L.lib.hipnx_sync(_Context.get(device)))


def timer_start(device: int = 0) -> None:
    L.check(L.lib.hipnx_timer_start(_Context.get(device)))


def timer_stop(device: int = 0) -> float:
    ms = C.c_float()
    L.check(L.lib.hipnx_timer_stop(_Context.get(device), C.byref(ms)))
    return ms.value


def timer_mark(index: int, device: int = 0) -> None:
    """Records lap mark `index` of the stopwatch on the stream (returns at once)."""
    L.check(L.lib.hipnx_timer_mark(_Context.get(device), index))


def timer_between(start: int, stop: int, device: int = 0) -> float:
    """Device milliseconds from lap mark `start` to lap mark `stop` (waits for `stop`)."""
    ms = C.c_float()
    L.check(L.lib.hipnx_timer_between(_Context.get(device), start, stop, C.byref(ms)))
    return ms.value


_capturing = set()  # devices whose context is recording instead of running


class DeviceGraph:
    """A captured sequence of device work (`hipnx_capture_begin` .. `hipnx_capture_end`): `launch`
    replays it with one submission.  Buffers allocated while capturing belong to the graph; tensors
    produced then are overwritten by every replay and die with the graph."""

    def __init__(self, handle, device):
        self.handle, self.device = handle, device

    def launch(self):
        if self.handle is None:
            raise L.HipNxError(L.EINVAL, "the graph has been destroyed")
        L.check(L.lib.hipnx_graph_launch(self.handle))

    def destroy(self):
        if self.handle is not None:
            handle, self.handle = self.handle, None
            L.check(L.lib.hipnx_graph_destroy(handle))

    def __del__(self):
        try:
            self.destroy()
        except Exception:  # interpreter shutdown: the context may be gone already
            pass


def copy_into(dst: Tensor, src: Tensor) -> None:
    """Overwrites the device memory of `dst` with `src` (same type and shape, same device)."""
    if (dst.type, dst.shape) != (src.type, src.shape) or dst.data.device != src.data.device:
        raise ValueError("copy_into needs two device tensors of one type, shape and device")
    L.check(L.lib.hipnx_d2d(dst.data.ref.ctx, HipNxBackend._handle(dst), 0, HipNxBackend._handle(src), 0, dst.data.ref.nbytes))


def capture_begin(device: int = 0) -> None:
    L.check(L.lib.hipnx_capture_begin(_Context.get(device)))
    _capturing.add(device)


def capture_end(device: int = 0) -> DeviceGraph:
    _capturing.discard(device)
    handle = C.c_void_p()
    L.check(L.lib.hipnx_capture_end(_Context.get(device), C.byref(handle)))
    return DeviceGraph(handle, device)


def mem_stats(device: int = 0):
    live, peak, pooled = C.c_uint64(), C.c_uint64(), C.c_uint64()
    L.check(L.lib.hipnx_mem_stats(_Context.get(device), C.byref(live), C.byref(peak), C.byref(pooled)))
    return {"live": live.value, "peak": peak.value, "pooled": pooled.value}


def bounds_policy(policy: str) -> str:
    """What `gather` / `take` do with an out-of-range index from now on; returns the previous setting.
    "raise" (the default, `Nx.BinaryBackend`'s behaviour: the call waits for its kernel and raises with
    the reference's message), "clamp" (EXLA's and Torchx's behaviour, asynchronous) or "defer" (raises,
    but late: the kernel records the bad index and the next call that waits for the device -- `to_binary`,
    `sync` -- raises; asynchronous, so a take costs a launch instead of a launch and a wait)."""
    names = {"raise": OOB_RAISE, "clamp": OOB_CLAMP, "defer": OOB_DEFER}
    if policy not in names:
        raise ValueError(f"expected one of {sorted(names)!r}, got: {policy!r}")
    previous = next(k for k, v in names.items() if v == _bounds["policy"])
    _bounds["policy"] = names[policy]
    return previous


def bf16_rounding(mode: str) -> str:
    """How `as_type` and `dot` encode a bf16 result from now on; returns the previous setting.
    "truncate" (the default) drops the low 16 bits of the f32 value as `Nx.BinaryBackend` does
    (nx/lib/nx/shared.ex:136-152); "nearest_even" rounds as Torchx and EXLA do
    (torchx/test/torchx/nx_test.exs:380-394 expects 1/5 -> 0.2001953125).  Element-wise results keep the
    reference backend's truncation under either setting."""
    if mode not in ("truncate", "nearest_even"):
        raise ValueError(f'expected "truncate" or "nearest_even", got: {mode!r}')
    previous = _bf16["rounding"]
    _bf16["rounding"] = mode
    return previous


def fused_mode(mode: str, device: int = 0) -> None:
    """How fused groups run on the device from now on: "interpreted" (one pair of kernels decodes any
    program; the default) or "compiled" (each distinct program is compiled for the device once, on
    first use, and kept).  Results are bit-identical."""
    _set_fused_mode(mode, device)
    _fused_modes[device] = mode


def _set_fused_mode(mode: str, device: int) -> None:
    codes = {"interpreted": L.FUSED_INTERPRETED, "compiled": L.FUSED_COMPILED}
    if mode not in codes:
        raise ValueError(f"expected one of {sorted(codes)!r}, got: {mode!r}")
    L.check(L.lib.hipnx_fused_set_mode(_Context.get(device), codes[mode]))
    _fused_set[device] = mode


_encoded = {}  # (type, class of the number, number) -> its encoding (constant/3)

_new_bytes = C.pythonapi.PyBytes_FromStringAndSize  # (NULL, n): a bytes object of n bytes whose content is the caller's to fill
_new_bytes.restype, _new_bytes.argtypes = C.py_object, [C.c_char_p, C.c_ssize_t]
_bytes_address = C.pythonapi.PyBytes_AsString
_bytes_address.restype, _bytes_address.argtypes = C.c_void_p, [C.py_object]
_libc = C.CDLL(None)
_libc.madvise.restype, _libc.madvise.argtypes = C.c_int, [C.c_void_p, C.c_size_t, C.c_int]


def _advise_huge_pages(address: int, n: int) -> None:
    """A large, fresh destination is first touched by the copy: with 4 KiB pages the page faults cost more than the
    transfer (256 MiB: 70 ms against 16 ms).  Asks for 2 MiB pages on the aligned interior, as numpy does for its
    arrays; advice only, a kernel without transparent huge pages ignores it."""
    if n >= 8 << 20:
        huge = 2 << 20
        lo, hi = (address + huge - 1) & ~(huge - 1), (address + n) & ~(huge - 1)
        if hi > lo:
            _libc.madvise(C.c_void_p(lo), hi - lo, 14)  # MADV_HUGEPAGE
_reduce_plans = {}  # (types, shape and axes of a reduction callback) -> its type codes, [outer, red, inner] view, result bytes
_binary_plans = {}  # (types and shapes of a binary callback) -> its type codes, shape and stride arrays, result bytes
_fused_modes = {}  # device -> the mode chosen with fused_mode/2: what a call that names none runs in
_fused_set = {}    # device -> the mode the library is in at this moment (a call that names one leaves it there)
_fused_arrays = {}  # (id of a layout, input types) -> (the layout itself, so the id stays its own; C arrays of types and strides)


def fused_cache_limit(programs: int, device: int = 0) -> None:
    """How many compiled programs the device's context keeps (512 unless set; at least 4).  A new program
    that finds the table full first unloads the least recently launched quarter."""
    L.check(L.lib.hipnx_fused_set_cache_limit(_Context.get(device), programs))


def fused_compiled_count(device: int = 0) -> int:
    count = C.c_int()
    L.check(L.lib.hipnx_fused_compiled_count(_Context.get(device), C.byref(count)))
    return count.value
