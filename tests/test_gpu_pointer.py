"""Local pointers (`Nx.to_pointer/2`, `Nx.from_pointer/5`; semantics of exla/lib/exla/backend.ex:86-181):
two tensors over one device buffer, one owner.  The :ipc kind is not built.  (Exchange with a torch
tensor needs both libraries on one HIP runtime; the torch wheel of this image carries its own, and
a second runtime in the process sees no device, so that is not tested here.)"""
import numpy as np
import pytest

from nx_amd import nx as Nx
from support import assert_bits_equal, from_numpy

pytestmark = pytest.mark.gpu


def test_pointer_round_trip_shares_the_buffer(hip):
    x = from_numpy(np.arange(24, dtype=np.float32).reshape(4, 6), "f32", hip)
    p = Nx.to_pointer(x)
    assert p.kind == "local" and p.address > 0 and p.data_size == 96 and p.handle is None
    alias = Nx.from_pointer(hip, p, "f32", (4, 6), keep=x)
    assert_bits_equal(alias, x, "alias of the same memory")
    # another view of the same bytes: 24 f32 as 48 u16
    words = Nx.from_pointer((hip, {"device": 0}), p, "u16", (48,), keep=x)
    np.testing.assert_array_equal(hip.to_numpy(words), hip.to_numpy(x).view(np.uint16).ravel())
    # deallocating the alias leaves the owner intact
    assert Nx.backend_deallocate(alias) == "ok"
    np.testing.assert_array_equal(hip.to_numpy(x), np.arange(24, dtype=np.float32).reshape(4, 6))


def test_pointer_checks(hip):
    x = from_numpy(np.zeros(8, dtype=np.float32), "f32", hip)
    p = Nx.to_pointer(x)
    with pytest.raises(ValueError, match="invalid pointer data_size for shape, expected: 64, got: 32"):
        Nx.from_pointer(hip, p, "f32", (16,))
    with pytest.raises(NotImplementedError, match=":ipc"):
        Nx.to_pointer(x, mode="ipc")
    with pytest.raises(ValueError, match="expected one of :local, :ipc"):
        Nx.to_pointer(x, mode="shared")
    from nx_amd._lib import HipNxArgumentError
    host = np.zeros(8, dtype=np.float32)
    with pytest.raises(HipNxArgumentError, match="buf_wrap"):
        Nx.from_pointer(hip, Nx.Pointer(kind="local", address=host.ctypes.data, data_size=32), "f32", (8,))
