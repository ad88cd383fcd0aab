"""Child process of tests/test_gpu_pointer.py::test_ipc_pointer_between_processes: opens the parent's
IPC pointer (nothing has touched the GPU in this process before), checks what it reads and writes a
reply into the shared memory.  argv: hex of the 64-byte handle, rows, cols."""
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

import numpy as np  # noqa: E402

from nx_amd import _lib as L  # noqa: E402
from nx_amd import nx as Nx  # noqa: E402
from nx_amd.backend import HipNxBackend as H  # noqa: E402
from nx_amd.nx import Pointer  # noqa: E402
import ctypes as C  # noqa: E402


def main():
    handle, rows, cols = bytes.fromhex(sys.argv[1]), int(sys.argv[2]), int(sys.argv[3])
    pointer = Pointer(kind="ipc", address=0, data_size=rows * cols * 4, handle=handle)
    t = Nx.from_pointer(H, pointer, "f32", (rows, cols))
    seen = H.to_numpy(t)
    want = np.arange(rows * cols, dtype=np.float32).reshape(rows, cols)
    if not np.array_equal(seen, want):
        print("child: the shared tensor does not hold what the parent wrote")
        return 3
    # a device computation on the shared tensor, and the reply written back into the parent's memory
    doubled = H.to_numpy(Nx.multiply(t, 2.0))
    if not np.array_equal(doubled, want * 2):
        print("child: multiply on the shared tensor is wrong")
        return 4
    reply = np.ascontiguousarray(-want)
    L.check(L.lib.hipnx_h2d(t.data.ref.ctx, t.data.ref.handle, 0, reply.ctypes.data_as(C.c_void_p), reply.nbytes))
    # the upload is left in flight on this process's stream: wait for it before telling the parent to look
    L.check(L.lib.hipnx_sync(t.data.ref.ctx))
    print("child: ok")
    return 0


if __name__ == "__main__":
    sys.exit(main())
