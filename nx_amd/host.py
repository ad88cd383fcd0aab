"""HostBinary -- a tensor that is just bytes in host memory.

It plays the part `Nx.BinaryBackend` plays for the *plumbing* of the reference (it is the backend
`Nx.tensor/2` builds literals and scalar constants on when no other default is set,
nx/lib/nx.ex:849-883, 2152-2157) and nothing more: it stores, returns and transfers a binary.
Every compute callback raises, like the reference's own storage-only test backend
(nx/test/support/backends.ex).  When a HostBinary tensor meets a device tensor in an operation
the device backend wins the dispatch and copies it in (nx/lib/nx/shared.ex:449-473).
"""
from __future__ import annotations

from . import types as T
from .tensor import Tensor, binary_prefix, binary_size, list_to_binary, number_to_binary


class HostBinary:
    def __init__(self, state: bytes):
        self.state = state
        self.released = False

    @staticmethod
    def init(opts):
        if opts:
            raise ValueError("HostBinary accepts no options")
        return {}

    @classmethod
    def from_binary(cls, out: Tensor, binary, opts=None) -> Tensor:
        if len(binary) < binary_size(out.type, out.size):
            raise ValueError("binary size is too small for the requested shape")
        return out.with_(data=cls(binary_prefix(binary, out.type, out.size)))

    @classmethod
    def constant(cls, out: Tensor, number, opts=None) -> Tensor:
        if T.is_sub_byte(out.type):
            return out.with_(data=cls(list_to_binary([int(number)] * out.size, out.type)))
        return out.with_(data=cls(number_to_binary(number, out.type) * out.size))

    @classmethod
    def to_binary(cls, t: Tensor, limit: int) -> bytes:
        if t.data.released:
            raise RuntimeError("tensor has been deallocated")
        return binary_prefix(t.data.state, t.type, min(int(limit), t.size))

    @classmethod
    def to_batched(cls, out: Tensor, t: Tensor, opts):
        """to_batched/3 (binary_backend.ex:178-211): byte ranges of the binary."""
        if T.is_sub_byte(t.type):
            raise NotImplementedError("HostBinary.to_batched of a sub-byte tensor needs a compute backend")
        state = cls.to_binary(t, t.size)
        size = out.size * T.size_bytes(out.type)
        full, rest = divmod(t.shape[0], out.shape[0])
        count = full + (1 if rest and opts.get("leftover", "repeat") == "repeat" else 0)

        def one(i):
            if i < full:
                return out.with_(data=cls(state[i * size:(i + 1) * size]))
            tail = state[full * size:]
            return out.with_(data=cls(tail + state[:size - len(tail)]))

        return (one(i) for i in range(count))

    @classmethod
    def backend_copy(cls, t: Tensor, backend, opts=None) -> Tensor:
        return backend.from_binary(t, cls.to_binary(t, t.size), opts)

    @classmethod
    def backend_transfer(cls, t: Tensor, backend, opts=None) -> Tensor:
        if backend is HostBinary:
            return t
        res = cls.backend_copy(t, backend, opts)
        cls.backend_deallocate(t)
        return res

    @classmethod
    def backend_deallocate(cls, t: Tensor) -> str:
        if t.data.released:
            return "already_deallocated"
        t.data.released = True
        t.data.state = b""
        return "ok"

    @classmethod
    def reshape(cls, out, t):
        return out.with_(data=t.data)

    squeeze = classmethod(lambda cls, out, t, axes: out.with_(data=t.data))
    bitcast = classmethod(lambda cls, out, t: out.with_(data=t.data))

    def __getattr__(self, name):
        raise AttributeError(name)


def _raise(name):
    def fn(cls, *a, **k):
        raise NotImplementedError(f"HostBinary only stores data; {name} needs a compute backend")
    return classmethod(fn)


def _install():
    from .backend_names import BINARY_OPS, UNARY_OPS
    for _n in BINARY_OPS + UNARY_OPS + ["sum", "product", "reduce_max", "reduce_min", "argmax", "argmin", "dot",
                                        "gather", "transpose", "broadcast", "as_type", "block"]:
        setattr(HostBinary, _n, _raise(_n))


_install()
