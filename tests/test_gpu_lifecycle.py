"""Buffer life-cycle and error behaviour of the device backend through the C ABI: what the
reference's device backends guarantee to Elixir callers."""
import ctypes as C
import threading

import numpy as np
import pytest

from nx_amd import nx as Nx
from nx_amd import HostBinary
from support import from_numpy

pytestmark = pytest.mark.gpu


def test_deallocate_is_idempotent(hip):
    """torchx/test/torchx/device_test.exs:30-37: :ok, then :already_deallocated twice."""
    t = Nx.tensor([1, 2, 3], backend=hip)
    assert Nx.backend_deallocate(t) == "ok"
    assert Nx.backend_deallocate(t) == "already_deallocated"
    assert Nx.backend_deallocate(t) == "already_deallocated"


def test_use_after_deallocate_raises(hip):
    """exla/test/exla/backend_test.exs:48-50: an error, never a crash."""
    from nx_amd._lib import HipNxError
    t = Nx.tensor([1.0, 2.0], backend=hip)
    Nx.backend_deallocate(t)
    with pytest.raises(HipNxError):
        Nx.add(t, 1.0)
    with pytest.raises(HipNxError):
        Nx.to_binary(t)


def test_short_binary_is_rejected(hip):
    """torchx/c_src/torchx.cpp:119-123."""
    from nx_amd.tensor import template
    with pytest.raises(ValueError, match="too small"):
        hip.from_binary(template("f32", (4,)), b"\x00" * 15, {})


def test_init_validates_options(hip):
    assert hip.init({}) == {"device": 0}
    with pytest.raises(ValueError):
        hip.init({"devise": 0})


def test_reshape_shares_the_buffer_and_survives_source_deallocation(hip):
    t = Nx.tensor([[1, 2, 3], [4, 5, 6]], backend=hip)
    r = Nx.reshape(t, (3, 2))
    assert Nx.backend_deallocate(t) == "ok"
    assert Nx.to_flat_list(r) == [1, 2, 3, 4, 5, 6]
    assert Nx.backend_deallocate(r) == "ok"


def test_transfer_round_trip_and_mixed_operands(hip):
    host = Nx.tensor([[1.5, -2.0], [0.25, 8.0]])
    assert isinstance(host.data, HostBinary)
    dev = Nx.backend_transfer(host, hip, {"device": 0})
    assert Nx.backend_deallocate(host) == "already_deallocated"
    other = Nx.tensor([1.0, 2.0])  # stays on the host: the device backend copies it in on entry
    out = Nx.add(dev, other)
    assert type(out.data) is hip
    back = Nx.backend_copy(out, HostBinary)
    assert Nx.to_flat_list(back) == [2.5, 0.0, 1.25, 10.0]
    assert Nx.to_binary(out, limit=3) == Nx.to_binary(back)[:12]


def test_bad_arguments_are_errors_not_faults(hip):
    from nx_amd import _lib as L
    ctx = hip._ctx(0)
    buf = C.c_void_p()
    L.check(L.lib.hipnx_buf_alloc(ctx, 64, C.byref(buf)))
    dims = L.i64_array([1000])
    st = L.lib.hipnx_binary(ctx, 0, 10, 10, 10, 1, dims, L.i64_array([1]), L.i64_array([1]), buf, buf, buf)
    assert st == L.EINVAL and "holds 64 bytes" in L.last_error()
    assert L.lib.hipnx_unary(ctx, 999, 10, 10, 4, buf, buf) == L.EINVAL
    assert L.lib.hipnx_dot(ctx, 10, 10, 10, 1, 64, 64, 64, 0, 0, buf, buf, buf) == L.EINVAL
    assert L.lib.hipnx_buf_free(buf) == L.OK
    assert L.lib.hipnx_buf_free(buf) == L.ALREADY_FREED
    assert L.lib.hipnx_unary(ctx, 0, 10, 10, 4, buf, buf) == L.EFREED
    assert L.lib.hipnx_buf_destroy(buf) == L.OK


def test_concurrent_callers_share_one_context(hip, oracle):
    """NIFs arrive on arbitrary dirty-scheduler threads: eight threads issue chains at once."""
    rng = np.random.default_rng(0)
    xs = [rng.uniform(-1, 1, size=(257, 129)).astype(np.float32) for _ in range(8)]
    results, errors = [None] * 8, []

    def work(i):
        try:
            t = from_numpy(xs[i], "f32", hip)
            for _ in range(20):
                t = Nx.add(Nx.multiply(t, 0.5), 1.0)
            results[i] = Nx.to_numpy(Nx.sum(t, axes=[1]))
        except Exception as e:  # pragma: no cover
            errors.append(e)

    threads = [threading.Thread(target=work, args=(i,)) for i in range(8)]
    [th.start() for th in threads]
    [th.join() for th in threads]
    assert not errors
    for i in range(8):
        t = from_numpy(xs[i], "f32", oracle)
        for _ in range(20):
            t = Nx.add(Nx.multiply(t, 0.5), 1.0)
        want = Nx.to_numpy(Nx.sum(t, axes=[1]))
        np.testing.assert_allclose(results[i], want, rtol=1e-6)


def test_memory_statistics_track_allocations(hip):
    from nx_amd.backend import mem_stats
    before = mem_stats()["live"]
    t = Nx.tensor(np.zeros((1024, 1024), dtype=np.float32), backend=hip)
    assert mem_stats()["live"] >= before + 4 * 1024 * 1024
    Nx.backend_deallocate(t)
    assert mem_stats()["live"] == before


@pytest.mark.parametrize("nbytes", [1, 4095, 256 << 10, (256 << 10) + 1, (512 << 10) + 7, 1 << 20, (1 << 20) + 1, (2 << 20) - 3,
                                    (2 << 20) + 5, (4 << 20) + 1, (16 << 20) + 12289, (33 << 20) + 3])
def test_host_transfers_of_every_staging_shape(nbytes, hip):
    """Uploads and downloads go through the context's two pinned staging buffers in pieces (uploads up to 2 MiB, in flight
    when the call returns; downloads of any size): sizes on and beside every piece boundary come back as they went,
    through to_binary, into an array, at an offset through the C ABI, and after the source array has been overwritten."""
    import ctypes as C
    from nx_amd import _lib as L
    rng = np.random.default_rng(nbytes)
    a = rng.integers(0, 256, size=nbytes, dtype=np.uint8)
    want = a.copy()
    t = from_numpy(a, "u8", hip)
    a[:] = 0  # the upload has consumed its source
    assert Nx.to_binary(t) == want.tobytes()
    assert np.array_equal(hip.to_numpy(t), want)
    off = min(nbytes - 1, 4097)
    part = np.empty(nbytes - off, dtype=np.uint8)
    L.check(L.lib.hipnx_d2h(t.data.ref.ctx, hip._handle(t), off, part.ctypes.data_as(C.c_void_p), part.nbytes))
    assert np.array_equal(part, want[off:])
    # several small uploads in a row reuse the two buffers while earlier ones are still in flight
    if nbytes <= 1 << 20:
        parts = [rng.integers(0, 256, size=nbytes, dtype=np.uint8) for _ in range(5)]
        tensors = [from_numpy(p, "u8", hip) for p in parts]
        for p, x in zip(parts, tensors):
            assert np.array_equal(hip.to_numpy(x), p)


def test_out_of_memory_is_an_error_and_the_pool_gives_way(hip):
    """A request the device cannot meet fails with ENOMEM and leaves the context usable; blocks that the pool still
    holds are handed back to the device before a large request is refused."""
    import gc
    from nx_amd import backend as B
    from nx_amd._lib import ENOMEM, HipNxError

    def device_memory():
        free, total = C.c_size_t(), C.c_size_t()
        assert C.CDLL("libamdhip64.so").hipMemGetInfo(C.byref(free), C.byref(total)) == 0
        return free.value, total.value

    Nx.tensor([0], backend=hip)  # (the context exists)
    _, total = device_memory()
    with pytest.raises(HipNxError) as err:
        Nx.iota((total + 100 * 2 ** 30,), type="u8", backend=hip)  # more than the part has
    assert err.value.status == ENOMEM
    assert Nx.to_flat_list(Nx.add(Nx.tensor([1, 2, 3], backend=hip), 1)) == [2, 3, 4]
    # the pool keeps up to 32 GiB of freed blocks (HIPNX_POOL_MAX_MB): park 30 GiB there, then ask for 10 GiB more than
    # the device has free beside them
    held = [Nx.iota((10 * 2 ** 30,), type="u8", backend=hip) for _ in range(3)]
    del held
    gc.collect()
    assert B.mem_stats()["pooled"] >= 30 * 2 ** 30
    free, _ = device_memory()
    n = free + 10 * 2 ** 30
    c = Nx.iota((n,), type="u8", backend=hip)  # fits only once the pool has let go of its blocks
    assert B.mem_stats()["pooled"] < 30 * 2 ** 30
    assert int(hip.to_numpy(Nx.slice(c, [n - 1], [1]))[0]) == (n - 1) % 256
    del c
    gc.collect()
