"""Device take / gather / transpose / broadcast against the CPU oracle: pure copies, bit-exact."""
import numpy as np
import pytest

from nx_amd import nx as Nx
from support import assert_bits_equal, from_numpy, seed_of
from test_gpu_elementwise import both, rand_raw

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape,perm", [((64, 48), [1, 0]), ((5, 64, 48), [0, 2, 1]), ((3, 4, 5, 6), [3, 1, 0, 2]),
                                         ((2, 3, 4), [1, 0, 2]), ((1, 7, 1, 9), [3, 2, 1, 0]), ((130, 70), [1, 0]),
                                         ((2, 2, 2, 2, 2, 2, 3), [6, 0, 5, 1, 4, 2, 3]), ((4096, 33), [1, 0])])
@pytest.mark.parametrize("ty", ["u8", "bf16", "f32", "s64"])
def test_transpose(shape, perm, ty, hip, oracle):
    rng = np.random.default_rng(seed_of(shape, perm, ty))
    x = rand_raw(rng, ty, shape)
    hx, ox = both(x, ty, hip, oracle)
    assert_bits_equal(Nx.transpose(hx, perm), Nx.transpose(ox, perm), f"transpose {shape} {perm}")


@pytest.mark.parametrize("shape,new,axes", [((3,), (4, 3), None), ((3, 1), (3, 5), None), ((2,), (2, 6), [0]),
                                             ((), (7, 3), None), ((1, 4, 1), (5, 4, 9), None), ((4, 2), (4, 3, 2), [0, 2])])
def test_broadcast(shape, new, axes, hip, oracle):
    rng = np.random.default_rng(seed_of(shape, new))
    x = rand_raw(rng, "f32", shape)
    hx, ox = both(x, "f32", hip, oracle)
    assert_bits_equal(Nx.broadcast(hx, new, axes), Nx.broadcast(ox, new, axes), f"broadcast {shape}->{new}")


@pytest.mark.parametrize("rows,cols,ty", [(1000, 64, "bf16"), (1000, 4096, "bf16"), (77, 3, "f32"), (500, 1, "u8"),
                                           (300, 17, "s64"), (32000, 128, "bf16"), (50, 1000, "f32")])
@pytest.mark.parametrize("idx_ty", ["u32", "s32", "s64", "u8"])
def test_take_rows(rows, cols, ty, idx_ty, hip, oracle):
    rng = np.random.default_rng(seed_of(rows, cols, ty, idx_ty))
    table = rand_raw(rng, ty, (rows, cols))
    hi = min(rows, 256 if idx_ty == "u8" else rows)
    idx = rng.integers(0, hi, size=(4, 333)).astype(np.dtype({"u32": np.uint32, "s32": np.int32, "s64": np.int64, "u8": np.uint8}[idx_ty]))
    ht, ot = both(table, ty, hip, oracle)
    hi_, oi = both(idx, idx_ty, hip, oracle)
    got, want = Nx.take(ht, hi_), Nx.take(ot, oi)
    assert_bits_equal(got, want, f"take {rows}x{cols} {ty} idx {idx_ty}")
    assert np.array_equal(hip.to_numpy(got), table[idx.astype(np.int64)])  # closed form


@pytest.mark.parametrize("axis", [0, 1, 2, -1])
def test_take_other_axes(axis, hip, oracle):
    rng = np.random.default_rng(axis + 10)
    t = rand_raw(rng, "f32", (6, 7, 8))
    idx = rng.integers(0, 6, size=(3, 2)).astype(np.int32)
    ht, ot = both(t, "f32", hip, oracle)
    hi_, oi = both(idx, "s32", hip, oracle)
    got = Nx.take(ht, hi_, axis=axis)
    assert_bits_equal(got, Nx.take(ot, oi, axis=axis), f"take axis {axis}")
    assert np.array_equal(hip.to_numpy(got), np.take(t, idx, axis=axis))


@pytest.mark.parametrize("axes", [None, [0], [1], [0, 2], [2, 0], [1, 2]])
def test_gather(axes, hip, oracle):
    rng = np.random.default_rng(7)
    t = rand_raw(rng, "s32", (5, 6, 7))
    depth = 3 if axes is None else len(axes)
    dims = [5, 6, 7] if axes is None else [[5, 6, 7][a] for a in axes]
    idx = np.stack([rng.integers(0, d, size=(4, 9)) for d in dims], axis=-1).astype(np.int64)
    ht, ot = both(t, "s32", hip, oracle)
    hi_, oi = both(idx, "s64", hip, oracle)
    assert_bits_equal(Nx.gather(ht, hi_, axes=axes), Nx.gather(ot, oi, axes=axes), f"gather axes={axes}")


def test_gather_out_of_bounds_raises_like_the_reference(hip, oracle):
    from nx_amd._lib import HipNxArgumentError
    from oracle.binary_backend import ReferenceRaises
    t = np.arange(12, dtype=np.int32).reshape(3, 4)
    for bad in ([[0, 0], [3, 1], [9, 9]], [[2, -1]], [[0, 4]], [[-7, 0]]):
        idx = np.array(bad, dtype=np.int32)
        ht, ot = both(t, "s32", hip, oracle)
        hi_, oi = both(idx, "s32", hip, oracle)
        with pytest.raises(ReferenceRaises) as want:
            Nx.gather(ot, oi)
        with pytest.raises(HipNxArgumentError) as got:
            Nx.gather(ht, hi_)
        assert str(want.value) in str(got.value)
    # and the first offender in index order is the one reported
    idx = np.zeros((5000, 1), dtype=np.int32)
    idx[4000], idx[1234], idx[4999] = 77, -5, 99
    ht = from_numpy(t, "s32", hip)
    with pytest.raises(HipNxArgumentError, match="index -5 is out of bounds for axis 0 in shape \\{3, 4\\}"):
        Nx.gather(ht, from_numpy(idx, "s32", hip))


def test_gather_clamp_policy_matches_the_compiled_backends(hip):
    """EXLA clamps out-of-range indices (exla/test/exla/defn/expr_test.exs:3478-3481):
    gather([[1,2],[3,4]], [[-1,-1],[10,11],[-1,10]]) -> [1, 4, 2]."""
    t = from_numpy(np.array([[1, 2], [3, 4]], dtype=np.int32), "s32", hip)
    idx = from_numpy(np.array([[-1, -1], [10, 11], [-1, 10]], dtype=np.int32), "s32", hip)
    from nx_amd.backend import OOB_CLAMP
    assert hip.to_numpy(Nx.gather(t, idx, oob_policy=OOB_CLAMP)).tolist() == [1, 4, 2]


def test_to_batched_known_answers_and_cyclic_rows(hip):
    from to_batched_support import check_counts, check_known_answers
    check_known_answers(hip)
    check_counts(hip)


@pytest.mark.parametrize("ty", ["u8", "bf16", "f32", "s64", "u4"])
@pytest.mark.parametrize("shape,batch", [((1000, 33), 64), ((7, 3, 5), 2), ((4096,), 1000)])
def test_to_batched_against_the_oracle(ty, shape, batch, hip, oracle):
    from nx_amd import nx as Nx
    n = int(np.prod(shape))
    values = (np.arange(n) % 7).reshape(shape)
    h, o = Nx.tensor(values, type=ty, backend=hip), Nx.tensor(values, type=ty, backend=oracle)
    for leftover in ("repeat", "discard"):
        got, want = list(Nx.to_batched(h, batch, leftover=leftover)), list(Nx.to_batched(o, batch, leftover=leftover))
        assert len(got) == len(want)
        for g, w in zip(got, want):
            assert g.type == w.type and g.shape == w.shape and Nx.to_binary(g) == Nx.to_binary(w)


# ---- the vectorised forms: 16-byte lanes on shapes that sit on, next to and across their boundaries ---------

@pytest.mark.parametrize("ty", ["u8", "s16", "bf16", "f32", "s64"])
@pytest.mark.parametrize("shape,new,axes", [((1,), (1031, 64), None), ((64,), (1031, 64), None), ((1031, 1), (1031, 64), None),
                                             ((), (257, 48), None), ((48,), (9, 48), None), ((9, 1), (9, 48), None),
                                             ((5, 1, 16), (5, 7, 16), None), ((1, 7, 1), (3, 7, 32), None), ((33,), (130, 33), None),
                                             ((130, 1), (130, 33), None), ((16,), (16, 40), [0])])
def test_broadcast_vector_lanes(ty, shape, new, axes, hip, oracle):
    """Rows, columns and single values repeated into outputs whose innermost axis is a whole number of 16-byte
    vectors (the vector kernel: one load, one repeated element, or gathered elements per vector) and into ones
    where it is not (one element per lane)."""
    rng = np.random.default_rng(seed_of(ty, shape, new, "vec"))
    x = rand_raw(rng, ty, shape)
    hx, ox = both(x, ty, hip, oracle)
    assert_bits_equal(Nx.broadcast(hx, new, axes), Nx.broadcast(ox, new, axes), f"broadcast {ty} {shape}->{new}")


@pytest.mark.parametrize("ty", ["u8", "bf16", "f32", "s64"])
@pytest.mark.parametrize("n", [1, 7, 15, 16, 17, 64, 1000, 4097, 65536 + 3])
def test_constant_fill_counts(ty, n, hip, oracle):
    """A constant is written as 16-byte vectors of the repeated element plus a tail of fewer than 16 bytes."""
    value = 3 if ty != "f32" else 2.5
    got = Nx.broadcast(Nx.tensor(value, type=ty, backend=hip), (n,))
    want = Nx.broadcast(Nx.tensor(value, type=ty, backend=oracle), (n,))
    assert_bits_equal(got, want, f"fill {ty} {n}")


@pytest.mark.parametrize("ty", ["u8", "bf16", "f32", "s64"])
@pytest.mark.parametrize("shape", [(64, 64), (128, 128), (256, 64), (64, 256), (8, 8), (16, 48), (2, 192, 320), (3, 64, 72),
                                   (130, 66), (136, 72), (1000, 24)])
def test_transpose_tiles(ty, shape, hip, oracle):
    """Swaps of the last two axes on whole tiles, ragged tiles, row counts that are and are not a multiple of a
    16-byte vector (the vector kernel and the element kernel)."""
    rng = np.random.default_rng(seed_of(ty, shape, "tiles"))
    x = rand_raw(rng, ty, shape)
    hx, ox = both(x, ty, hip, oracle)
    perm = list(range(len(shape) - 2)) + [len(shape) - 1, len(shape) - 2]
    assert_bits_equal(Nx.transpose(hx, perm), Nx.transpose(ox, perm), f"transpose {ty} {shape}")


@pytest.mark.parametrize("ty", ["u8", "s16", "bf16", "f32"])
@pytest.mark.parametrize("shape,starts,lengths", [((40, 100), [1, 1], [39, 99]), ((40, 100), [0, 3], [40, 64]), ((40, 100), [5, 7], [30, 33]),
                                                   ((9, 257), [0, 1], [9, 256]), ((3, 4, 50), [1, 1, 5], [2, 3, 41]), ((300,), [13], [270]),
                                                   ((64, 31), [0, 0], [64, 31]), ((64, 32), [1, 0], [63, 32])])
def test_slices_off_the_vector_grid(ty, shape, starts, lengths, hip, oracle):
    """Dense rows that start or end off a 16-byte boundary: whole vectors at element alignment, the last,
    partial vector of a row by element."""
    rng = np.random.default_rng(seed_of(ty, shape, starts, "runs"))
    x = rand_raw(rng, ty, shape)
    hx, ox = both(x, ty, hip, oracle)
    assert_bits_equal(Nx.slice(hx, starts, lengths), Nx.slice(ox, starts, lengths), f"slice {ty} {shape} {starts}")
    axes = [len(shape) - 1]
    assert_bits_equal(Nx.reverse(hx, axes=axes), Nx.reverse(ox, axes=axes), f"reverse {ty} {shape}")
    sl_h, sl_o = Nx.slice(hx, starts, lengths), Nx.slice(ox, starts, lengths)
    assert_bits_equal(Nx.reverse(sl_h, axes=axes), Nx.reverse(sl_o, axes=axes), f"reverse of a slice {ty} {shape}")
    cfg = [(1, 2, 0)] * len(shape)
    pad_h, pad_o = Nx.tensor(0, type=ty, backend=hip), Nx.tensor(0, type=ty, backend=oracle)
    assert_bits_equal(Nx.pad(hx, pad_h, cfg), Nx.pad(ox, pad_o, cfg), f"pad {ty} {shape}")


TAKE_ALONG = [((40, 300, 16), 1, "bf16"), ((40, 300, 16), 2, "bf16"), ((7, 129, 5), 1, "f32"), ((7, 129, 5), 2, "f32"), ((513, 1000), 1, "u8"),
              ((513, 1000), 1, "f32"), ((3, 4, 50, 6), 2, "s64"), ((3, 4, 50, 6), 3, "s16"), ((2, 3, 64, 24), 2, "bf16"), ((1, 9, 4096), 2, "f32")]


@pytest.mark.parametrize("shape,axis,ty", TAKE_ALONG, ids=[f"{s}-{a}-{t}" for s, a, t in TAKE_ALONG])
@pytest.mark.parametrize("idx_ty", ["s32", "u8", "s64"])
def test_take_along_an_inner_axis_is_one_kernel(shape, axis, ty, idx_ty, hip, oracle):
    """take along an axis that is not the first: the tensor viewed as [outer, axis, inner], slices of every width
    (a single element along the last axis, 2 to 16 bytes, whole vectors) -- against the oracle's gather +
    transpose and against numpy."""
    rng = np.random.default_rng(seed_of(shape, axis, ty, idx_ty, "along"))
    t = rand_raw(rng, ty, shape)
    hi = min(shape[axis], 256 if idx_ty == "u8" else shape[axis])
    idx = rng.integers(0, hi, size=(5, 21)).astype(np.dtype({"s32": np.int32, "u8": np.uint8, "s64": np.int64}[idx_ty]))
    ht, ot = both(t, ty, hip, oracle)
    hi_, oi = both(idx, idx_ty, hip, oracle)
    got = Nx.take(ht, hi_, axis=axis)
    assert_bits_equal(got, Nx.take(ot, oi, axis=axis), f"take {shape} axis {axis} {ty}")
    assert np.array_equal(hip.to_numpy(got), np.take(t, idx.astype(np.int64), axis=axis))


def test_take_along_an_inner_axis_reports_a_bad_index_like_the_reference(hip, oracle):
    """The reference's take is gather on the tensor with the taken axis moved to the front, and its message names
    that shape and axis 0 (binary_backend.ex:1906-1912, 1949-1952)."""
    from nx_amd._lib import HipNxArgumentError
    from oracle.binary_backend import ReferenceRaises
    t = np.arange(3 * 4 * 5, dtype=np.float32).reshape(3, 4, 5)
    idx = np.array([1, 9, 0, -2], dtype=np.int32)
    ht, ot = both(t, "f32", hip, oracle)
    hi_, oi = both(idx, "s32", hip, oracle)
    with pytest.raises((ReferenceRaises, ValueError)) as ref:
        Nx.take(ot, oi, axis=2)
    assert "index 9 is out of bounds for axis 0 in shape {5, 3, 4}" in str(ref.value)
    with pytest.raises(HipNxArgumentError, match="index 9 is out of bounds for axis 0 in shape \\{5, 3, 4\\}"):
        Nx.take(ht, hi_, axis=2)
    with pytest.raises(HipNxArgumentError, match="index 9 is out of bounds for axis 0 in shape \\{4, 3, 5\\}"):
        Nx.take(ht, hi_, axis=1)
    # and the device is usable afterwards
    assert np.array_equal(hip.to_numpy(Nx.take(ht, from_numpy(np.array([4, 0], dtype=np.int32), "s32", hip), axis=2)), t[:, :, [4, 0]])


@pytest.mark.parametrize("rows,cols,ty", [(300, 1024, "f32"), (260, 4096, "bf16"), (512, 2048, "u8"), (256, 512, "s64"),
                                           (700, 16384, "f64"), (300, 2056, "bf16")])
@pytest.mark.parametrize("idx_ty,picks", [("s32", 1024), ("s64", 2048), ("u32", 4104), ("u8", 8192)])
def test_take_along_the_last_axis_of_long_rows(rows, cols, ty, idx_ty, picks, hip, oracle):
    """Rows of 2 KB and more with at least half as many picks as the row has elements are staged in local memory;
    fewer picks, rows of other sizes and index types of other widths take the kernel that reads through the
    caches.  Both against numpy (the oracle's loop takes minutes at these sizes) and, on a corner, the oracle."""
    rng = np.random.default_rng(seed_of(rows, cols, ty, idx_ty, picks, "long rows"))
    t = rand_raw(rng, ty, (rows, cols))
    hi = min(cols, 256 if idx_ty == "u8" else cols)
    np_idx = {"s32": np.int32, "u32": np.uint32, "s64": np.int64, "u8": np.uint8}[idx_ty]
    idx = rng.integers(0, hi, size=(picks,)).astype(np_idx)
    got = Nx.take(from_numpy(t, ty, hip), from_numpy(idx, idx_ty, hip), axis=1)
    assert np.array_equal(hip.to_numpy(got).view(np.uint8), np.take(t, idx.astype(np.int64), axis=1).view(np.uint8))
    ot, oi = from_numpy(t[:3, :], ty, oracle), from_numpy(idx[:64], idx_ty, oracle)
    assert_bits_equal(Nx.slice(got, [0, 0], [3, 64]), Nx.take(ot, oi, axis=1), f"take last axis {ty} {idx_ty}")


def test_take_along_the_last_axis_of_long_rows_reports_and_clamps(hip):
    """The three bounds policies on the kernel that stages rows: the raising one names the first bad index in index
    order, the clamping one pins it to the ends of the axis, the deferring one reports at the next wait."""
    from nx_amd import backend as B
    from nx_amd._lib import HipNxArgumentError
    rng = np.random.default_rng(5)
    t = rng.standard_normal((300, 1024)).astype(np.float32)
    idx = rng.integers(0, 1024, size=(1024,)).astype(np.int32)
    idx[700], idx[333], idx[1000] = 1024, -7, 5000
    ht, hi_ = from_numpy(t, "f32", hip), from_numpy(idx, "s32", hip)
    with pytest.raises(HipNxArgumentError, match="index -7 is out of bounds for axis 0 in shape \\{1024, 300\\}"):
        Nx.take(ht, hi_, axis=1)
    good = np.clip(idx, 0, 1023)
    assert np.array_equal(hip.to_numpy(Nx.take(ht, from_numpy(good, "s32", hip), axis=1)), t[:, good])
    previous = B.bounds_policy("clamp")
    try:
        assert np.array_equal(hip.to_numpy(Nx.take(ht, hi_, axis=1)), t[:, good])
        B.bounds_policy("defer")
        late = Nx.take(ht, hi_, axis=1)
        with pytest.raises(HipNxArgumentError, match="is out of bounds"):
            Nx.to_binary(late)
        B.sync()
    finally:
        B.bounds_policy(previous)


@pytest.mark.parametrize("shape,new,axes", [((300,), (300, 1001), [0]), ((1001,), (300, 1001), None), ((), (7, 33), None), ((5, 1, 3), (5, 77, 3), None),
                                             ((9, 1), (4, 9, 13), None), ((2, 3), (2, 50257, 3), [0, 2])])
@pytest.mark.parametrize("ty", ["u8", "bf16", "f32", "s64"])
def test_broadcast_to_rows_that_are_not_whole_vectors(shape, new, axes, ty, hip, oracle):
    """An innermost output axis that is not a multiple of 16 bytes: vectors of the flat output that run across row ends,
    the last one partial."""
    rng = np.random.default_rng(seed_of(shape, new, ty, "flat"))
    x = rand_raw(rng, ty, shape)
    got = Nx.broadcast(from_numpy(x, ty, hip), new, axes)
    if int(np.prod(new)) <= 50000:
        assert_bits_equal(got, Nx.broadcast(from_numpy(x, ty, oracle), new, axes), f"broadcast {shape}->{new}")
    ax = axes if axes is not None else list(range(len(new) - len(shape), len(new)))
    lifted = x.reshape([new[a] if a in ax and x.shape[ax.index(a)] != 1 else 1 for a in range(len(new))]) if x.ndim else x
    assert np.array_equal(hip.to_numpy(got).view(np.uint8), np.broadcast_to(lifted, new).copy().view(np.uint8))


@pytest.mark.parametrize("shape,perm", [((5, 7, 9), [2, 0, 1]), ((5, 7, 9), [1, 2, 0]), ((3, 11, 2, 13), [3, 1, 0, 2]), ((6, 50257), [1, 0]),
                                         ((4, 3, 1001), [1, 0, 2])])
@pytest.mark.parametrize("ty", ["u8", "bf16", "f32", "s64"])
def test_transposes_with_odd_extents(shape, perm, ty, hip):
    rng = np.random.default_rng(seed_of(shape, perm, ty, "odd"))
    x = rand_raw(rng, ty, shape)
    got = hip.to_numpy(Nx.transpose(from_numpy(x, ty, hip), perm))
    assert np.array_equal(got.view(np.uint8), np.ascontiguousarray(np.transpose(x, perm)).view(np.uint8))


def _index_bound(t):
    import ctypes as C
    from nx_amd import _lib as L
    bound = C.c_int64(-1)
    L.check(L.lib.hipnx_buf_index_bound(t.data.ref.handle, C.byref(bound)))
    return bound.value


def test_indices_written_by_argmax_need_no_bounds_wait(hip, oracle):
    """`argmax` writes positions along an axis; `take` along an axis at least as long cannot meet a bad one, so
    the raising policy has nothing to wait for (the reference checks every index, binary_backend.ex:1949-1952:
    same results, same error for indices that CAN be out of range)."""
    import ctypes as C
    from nx_amd import _lib as L
    from nx_amd import backend as B
    from nx_amd._lib import HipNxArgumentError
    rng = np.random.default_rng(11)
    logits = rng.standard_normal((300, 1000)).astype(np.float32)
    logits[7, 999] = 50.0  # one row points at the last entry
    table = rand_raw(rng, "bf16", (1000, 64))
    hl, ol = both(logits, "f32", hip, oracle)
    ht, ot = both(table, "bf16", hip, oracle)
    hidx, oidx = Nx.argmax(hl, axis=1, type="u32"), Nx.argmax(ol, axis=1, type="u32")
    assert _index_bound(hidx) == 1000
    assert_bits_equal(Nx.take(ht, hidx), Nx.take(ot, oidx), "take of argmax indices")
    assert _index_bound(hidx) == 1000  # reading does not change what is known
    # the same indices into a shorter axis CAN be out of range: checked at once, the reference's message
    short = from_numpy(table[:500].copy(), "bf16", hip)
    picks = np.argmax(logits, axis=1)
    first_bad = int(picks[picks >= 500][0])  # the first offender in index order is the one reported
    with pytest.raises(HipNxArgumentError, match=f"index {first_bad} is out of bounds for axis 0 in shape \\{{500, 64\\}}"):
        Nx.take(short, hidx)
    # with the bound known, the raising policy runs inside a captured graph (it would have to wait otherwise)
    B.capture_begin(0)
    try:
        inside = Nx.take(ht, hidx)
    finally:
        graph = B.capture_end(0)
    graph.launch()
    assert_bits_equal(inside, Nx.take(ot, oidx), "take of argmax indices in a captured graph")
    del inside
    graph.destroy()
    assert _index_bound(Nx.argmax(hl, axis=1, type="s64")) == 1000
    # an output type too narrow for the axis wraps the index: no claim
    assert _index_bound(Nx.argmax(hl, axis=1, type="u8")) == 0
    assert _index_bound(Nx.argmax(hl, axis=1, type="s8")) == 0
    assert _index_bound(Nx.argmax(from_numpy(logits[:, :128].copy(), "f32", hip), axis=1, type="s8")) == 128
    # written again, the buffer holds whatever was written
    zero = np.zeros(1, dtype=np.uint32)
    L.check(L.lib.hipnx_fill(hidx.data.ref.ctx, hidx.data.ref.handle, 4, zero.ctypes.data_as(C.c_void_p), 300))
    assert _index_bound(hidx) == 0
    # and indices from anywhere else are checked as ever
    foreign = from_numpy(np.array([3, 1000, 2], dtype=np.uint32), "u32", hip)
    assert _index_bound(foreign) == 0
    with pytest.raises(HipNxArgumentError, match="index 1000 is out of bounds for axis 0 in shape \\{1000, 64\\}"):
        Nx.take(ht, foreign)
    assert B.bounds_policy("raise") == "raise"
