"""Tensors past 2^32 elements (and, where the device has the room, past 2^32 sixteen-byte vectors): a part with 288 GB
of HBM holds them, so every index in a kernel has to be 64 bits wide.  The CPU oracle would need minutes per callback at
these sizes; the values are `iota` wrapped to u8, whose sums, extremes and positions have closed forms, and windows of
the results are compared element by element with what the formula gives."""
import numpy as np
import pytest

from nx_amd import nx as Nx

pytestmark = pytest.mark.gpu


def _release():
    """Hands the pool's blocks back between cases: these tensors are gigabytes each."""
    import gc
    gc.collect()


def window(t, start, length):
    from nx_amd.backend import HipNxBackend as H
    return H.to_numpy(Nx.slice(t, [start], [length]))


@pytest.mark.parametrize("n", [2 ** 32 + 4099, 2 ** 36 + 4099 + 16 * 5])
def test_flat_callbacks_past_32_bit_indices(n, hip):
    from nx_amd._lib import ENOMEM, HipNxError
    try:
        x = Nx.iota((n,), type="u8", backend=hip)  # x[i] = i mod 256
        y = Nx.add(x, x)                           # (2 i) mod 256
    except HipNxError as e:
        if e.status == ENOMEM:
            pytest.skip(f"the device has no room for two tensors of {n} bytes")
        raise
    tail = np.arange(n - 1000, n, dtype=np.int64)
    for start in (0, 2 ** 32 - 500, n - 1000):
        idx = np.arange(start, start + 1000, dtype=np.int64)
        np.testing.assert_array_equal(window(x, start, 1000), (idx % 256).astype(np.uint8), f"iota at {start}")
        np.testing.assert_array_equal(window(y, start, 1000), ((2 * idx) % 256).astype(np.uint8), f"add at {start}")
    del y
    _release()
    # sum: u8 -> u32, wrapping; whole periods of 0..255 and a rest
    periods, rest = divmod(n, 256)
    want = (periods * (255 * 256 // 2) + rest * (rest - 1) // 2) % 2 ** 32
    assert int(hip.to_numpy(Nx.sum(x))) == want
    assert int(hip.to_numpy(Nx.reduce_max(x))) == 255 and int(hip.to_numpy(Nx.reduce_min(x))) == 0
    # positions need 64 bits: the last 255 lies past 2^32
    last_255 = n // 256 * 256 + 255
    if last_255 >= n:
        last_255 -= 256
    assert last_255 % 256 == 255 and last_255 < n <= last_255 + 256
    assert int(hip.to_numpy(Nx.argmax(x, tie_break="high", type="s64"))) == last_255
    assert int(hip.to_numpy(Nx.argmax(x, type="s64"))) == 255
    assert int(hip.to_numpy(Nx.argmin(x, tie_break="high", type="s64"))) == (n - 1) // 256 * 256
    assert int(hip.to_numpy(Nx.argmin(x, type="s64"))) == 0
    # conversion, comparison, selection by position
    if n < 2 ** 34:  # (twice the bytes: only where three such tensors fit)
        z = Nx.as_type(x, "u16")
        np.testing.assert_array_equal(window(z, n - 1000, 1000), (tail % 256).astype(np.uint16))
        del z
        _release()
    e = Nx.equal(x, 7)
    np.testing.assert_array_equal(window(e, n - 1000, 1000), (tail % 256 == 7).astype(np.uint8))
    assert int(hip.to_numpy(Nx.sum(e))) == (n - 8) // 256 + 1
    del e
    _release()
    where = np.array([0, 2 ** 32 - 1, 2 ** 32, 2 ** 32 + 1, n - 1, n - 4099], dtype=np.int64)
    from support import from_numpy
    picked = hip.to_numpy(Nx.take(x, from_numpy(where, "s64", hip)))
    np.testing.assert_array_equal(picked, (where % 256).astype(np.uint8))
    picked = hip.to_numpy(Nx.gather(x, from_numpy(where.reshape(-1, 1), "s64", hip)))
    np.testing.assert_array_equal(picked, (where % 256).astype(np.uint8))
    # a reversed window and a strided one from the far end
    r = hip.to_numpy(Nx.reverse(Nx.slice(x, [n - 2000], [2000])))
    np.testing.assert_array_equal(r, (np.arange(n - 1, n - 2001, -1, dtype=np.int64) % 256).astype(np.uint8))
    s = hip.to_numpy(Nx.slice(x, [2 ** 32 - 10], [3000], strides=[3]))
    np.testing.assert_array_equal(s, (np.arange(2 ** 32 - 10, 2 ** 32 - 10 + 3000, 3, dtype=np.int64) % 256).astype(np.uint8))
    del x
    _release()


def test_rows_and_columns_past_32_bit_indices(hip):
    """A {65537, 65600} u8 matrix (4.3 G elements): reductions along either axis, a row broadcast, a transpose."""
    rows, cols = 65537, 65600
    x = Nx.iota((rows, cols), type="u8", backend=hip)  # x[r, c] = (r * cols + c) mod 256
    r_idx = np.arange(rows, dtype=np.int64)
    c_idx = np.arange(cols, dtype=np.int64)
    # sums along the rows: cols = 256 * 256 + 64 elements starting at (r * cols) mod 256
    start = (r_idx * cols) % 256
    per_row = np.array([(np.arange(s, s + cols, dtype=np.int64) % 256).sum() for s in start[:300]], dtype=np.int64)
    got = hip.to_numpy(Nx.sum(x, axes=[1]))
    np.testing.assert_array_equal(got[:300].astype(np.int64), per_row % 2 ** 32)
    last = (np.arange(start[-1], start[-1] + cols, dtype=np.int64) % 256).sum() % 2 ** 32
    assert int(got[-1]) == last
    # sums down the columns: x[r, c] = (c + 64 r) mod 256 since cols mod 256 = 64
    col_sums = np.array([((c + 64 * r_idx) % 256).sum() for c in c_idx[:300]], dtype=np.int64) % 2 ** 32
    got = hip.to_numpy(Nx.sum(x, axes=[0]))
    np.testing.assert_array_equal(got[:300].astype(np.int64), col_sums)
    assert int(got[-1]) == int(((c_idx[-1] + 64 * r_idx) % 256).sum() % 2 ** 32)
    # positions of the row maxima (first 255 in each row)
    am = hip.to_numpy(Nx.argmax(x, axis=1))
    np.testing.assert_array_equal(am[-300:].astype(np.int64), (255 - start[-300:]) % 256)
    # a row vector against every row, checked in the last rows
    from support import from_numpy
    v = from_numpy((c_idx % 251).astype(np.uint8), "u8", hip)
    y = Nx.add(x, v)
    got = hip.to_numpy(Nx.slice(y, [rows - 2, cols - 500], [2, 500]))
    want = ((np.arange(rows - 2, rows)[:, None] * cols + c_idx[None, -500:]) % 256 + (c_idx[None, -500:] % 251)) % 256
    np.testing.assert_array_equal(got, want.astype(np.uint8))
    del y
    _release()
    t = Nx.transpose(x)
    got = hip.to_numpy(Nx.slice(t, [cols - 3, rows - 400], [3, 400]))
    want = ((np.arange(rows - 400, rows)[None, :] * cols + np.arange(cols - 3, cols)[:, None]) % 256).astype(np.uint8)
    np.testing.assert_array_equal(got, want)
    del t, x
    _release()


def test_argmax_down_an_axis_of_more_than_2_to_the_31(hip):
    """Positions along an axis of 2^31 + 5 under two columns: the axis is searched in chunks whose winners meet by the
    reducer's own rules (ties by tie_break; a NaN beats every number and the last NaN wins)."""
    from support import from_numpy
    rows = 2 ** 31 + 5
    x = Nx.iota((rows, 2), type="u8", backend=hip)  # x[r, c] = (2 r + c) mod 256: the extremes sit at r = 127 (mod 128) and r = 0 (mod 128)
    last_127 = (rows - 1) - ((rows - 1 - 127) % 128)
    last_0 = (rows - 1) // 128 * 128
    np.testing.assert_array_equal(hip.to_numpy(Nx.argmax(x, axis=0, type="s64")), [127, 127])
    np.testing.assert_array_equal(hip.to_numpy(Nx.argmax(x, axis=0, tie_break="high", type="s64")), [last_127, last_127])
    np.testing.assert_array_equal(hip.to_numpy(Nx.argmin(x, axis=0, tie_break="high", type="s64")), [last_0, last_0])
    np.testing.assert_array_equal(hip.to_numpy(Nx.argmin(x, axis=0, type="u32")), [0, 0])
    del x
    _release()
    # floats: a NaN in the first chunk and one in the third; the later one is the answer whatever the tie_break
    n = 2 ** 31 + 2 ** 30 + 77
    f = Nx.as_type(Nx.iota((n,), type="u8", backend=hip), "bf16")
    nan = from_numpy(np.array([0x7FC0], dtype=np.uint16), "bf16", hip)
    f = Nx.put_slice(Nx.put_slice(f, [1000], nan), [2 ** 31 + 12345], nan)
    for tie in ("low", "high"):
        assert int(hip.to_numpy(Nx.argmax(f, tie_break=tie, type="s64"))) == 2 ** 31 + 12345
        assert int(hip.to_numpy(Nx.argmin(f, tie_break=tie, type="s64"))) == 2 ** 31 + 12345
    del f
    _release()


@pytest.mark.parametrize("layout", ["k-inner", "k-outer"])
def test_dot_with_an_operand_past_32_bit_offsets(layout, hip):
    """A bf16 operand of 4.3 GB (its last rows start past byte 2^32) against 256 columns: operands of small integers,
    so every sum is exact; sampled rows of the result against the same rows computed on the host."""
    from support import from_numpy
    M, K, N = 2 ** 16 + 16, 2 ** 15 + 128, 256
    shape = (M, K) if layout == "k-inner" else (K, M)
    m_axis, k_axis = (0, 1) if layout == "k-inner" else (1, 0)
    mk = Nx.add(Nx.iota(shape, type="s32", axis=m_axis, backend=hip), Nx.iota(shape, type="s32", axis=k_axis, backend=hip))
    a = Nx.as_type(Nx.subtract(Nx.remainder(mk, 5), 2), "bf16")  # a[m, k] = (m + k) mod 5 - 2
    del mk
    _release()
    k = np.arange(K, dtype=np.int64)
    b_host = ((3 * k[:, None] + np.arange(N)[None, :]) % 7 - 3).astype(np.float32)  # b[k, n]
    b = from_numpy((b_host.view(np.uint32) >> 16).astype(np.uint16), "bf16", hip)
    got = Nx.dot(a, [k_axis], b, [0], out_type="f32")
    assert got.shape == (M, N)
    rows = [0, 1, 32767, 32768, 65535, 65536, M - 1]
    for m in rows:
        want = (((m + k) % 5 - 2).astype(np.float64) @ b_host.astype(np.float64)).astype(np.float32)
        np.testing.assert_array_equal(hip.to_numpy(Nx.slice(got, [m, 0], [1, N]))[0], want, f"row {m}")
    del a, b, got
    _release()


@pytest.mark.parametrize("mode", ["interpreted", "compiled"])
def test_fused_group_past_32_bit_indices(mode, hip):
    """A fused element-wise group over 2^32 + 4099 bf16 elements, and one with its row reduction over {65537, 65600}."""
    from nx_amd import defn
    from nx_amd.backend import fused_mode as set_mode
    n = 2 ** 32 + 4099
    x = Nx.as_type(Nx.iota((n,), type="u8", backend=hip), "bf16")  # i mod 256, exact in bf16
    set_mode(mode)
    try:
        f = defn.compile(lambda t: Nx.multiply(Nx.add(t, 1.0), 0.5), x, fuse=True)
        assert f.fused_groups == 1
        y = f(x)
        for start in (0, 2 ** 32 - 500, n - 1000):
            idx = np.arange(start, start + 1000, dtype=np.int64)
            want = (((idx % 256).astype(np.float32) + 1.0) * 0.5)
            want = (want.view(np.uint32) >> 16).astype(np.uint16)  # bf16 by truncation (every value here is exact anyway)
            np.testing.assert_array_equal(hip.to_numpy(Nx.slice(y, [start], [1000])), want, f"window at {start}")
        del y, x
        _release()
        rows, cols = 65537, 65600
        m = Nx.as_type(Nx.iota((rows, cols), type="u8", backend=hip), "f32")
        g = defn.compile(lambda t: Nx.sum(Nx.multiply(t, 2.0), axes=[1]), m, fuse=True)
        got = hip.to_numpy(g(m))
        start = (np.arange(rows, dtype=np.int64) * cols) % 256
        for r in (0, 1, 300, rows - 2, rows - 1):
            want = 2.0 * (np.arange(start[r], start[r] + cols, dtype=np.int64) % 256).sum()
            assert got[r] == np.float32(want), f"row {r}"
        del m
        _release()
    finally:
        set_mode("interpreted")
