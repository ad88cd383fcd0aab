"""nx_amd -- HipNx: an MI355X-native backend for the eager tensor path of Nx.

    from nx_amd import nx as Nx, HipNxBackend
    Nx.default_backend(HipNxBackend, {"device": 0})

`nx` is the front-end slice (output templates + dispatch), `HipNxBackend` implements the
`Nx.Backend` callbacks over libhipnx.so (hand-written gfx950 kernels behind a C ABI).
Importing the backend fails loudly when the shared library has not been built.
"""
from . import nx, shape, types  # noqa: F401
from .host import HostBinary  # noqa: F401
from .tensor import Tensor  # noqa: F401


def __getattr__(name):
    # the device backend (and with it libhipnx.so) is loaded on first use
    if name == "HipNxBackend":
        from .backend import HipNxBackend
        return HipNxBackend
    if name == "backend":
        import importlib
        return importlib.import_module(".backend", __name__)
    raise AttributeError(name)
