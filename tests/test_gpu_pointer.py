"""Local pointers (`Nx.to_pointer/2`, `Nx.from_pointer/5`; semantics of exla/lib/exla/backend.ex:86-181):
two tensors over one device buffer, one owner; and the :ipc kind: a handle a second process opens
(exla/lib/exla/backend.ex:85-181, exla/c_src/exla/exla_cuda.cc:11-52).  (Exchange with a torch
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
    with pytest.raises(ValueError, match="expected one of :local, :ipc"):
        Nx.to_pointer(x, mode="shared")
    from nx_amd._lib import HipNxArgumentError
    host = np.zeros(8, dtype=np.float32)
    with pytest.raises(HipNxArgumentError, match="buf_wrap"):
        Nx.from_pointer(hip, Nx.Pointer(kind="local", address=host.ctypes.data, data_size=32), "f32", (8,))


def test_ipc_pointer_between_processes(hip):
    """to_pointer(mode: :ipc) in this process, from_pointer in a fresh child process (which opens the handle
    before anything else of it touches the GPU): the child reads the parent's values, computes on them and
    writes a reply into the shared memory; the parent reads the reply from its own tensor."""
    import os
    import subprocess
    import sys
    rows, cols = 96, 128  # 48 KiB: far below the 2 GiB limit of shared allocations
    x = from_numpy(np.arange(rows * cols, dtype=np.float32).reshape(rows, cols), "f32", hip)
    p = Nx.to_pointer(x, mode="ipc")
    assert p.kind == "ipc" and len(p.handle) == 64 and p.address == 0 and p.data_size == rows * cols * 4
    child = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ipc_child.py")
    done = subprocess.run([sys.executable, child, p.handle.hex(), str(rows), str(cols)], capture_output=True, text=True, timeout=100)
    assert done.returncode == 0, f"child failed ({done.returncode}): {done.stdout[-500:]} {done.stderr[-1500:]}"
    np.testing.assert_array_equal(hip.to_numpy(x), -np.arange(rows * cols, dtype=np.float32).reshape(rows, cols))


def test_ipc_pointer_checks(hip):
    x = from_numpy(np.zeros(8, dtype=np.float32), "f32", hip)
    p = Nx.to_pointer(x, mode="ipc")
    with pytest.raises(ValueError, match="invalid pointer data_size for shape"):
        Nx.from_pointer(hip, p, "f32", (16,))
    with pytest.raises(ValueError, match="handle of 64 bytes"):
        Nx.from_pointer(hip, Nx.Pointer(kind="ipc", address=0, data_size=32, handle=b"short"), "f32", (8,))
    alias = Nx.from_pointer(hip, Nx.to_pointer(x), "f32", (8,), keep=x)  # a wrapped buffer owns nothing to share
    from nx_amd._lib import HipNxError
    with pytest.raises(HipNxError, match="does not own"):
        Nx.to_pointer(alias, mode="ipc")
