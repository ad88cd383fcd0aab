"""Device select / clip / slice / concatenate / stack / iota / eye / all / any against the CPU oracle
on seeded inputs.  Everything here is selection, copying or counting: the bar is bit-exact."""
import numpy as np
import pytest

from nx_amd import nx as Nx
from support import assert_bits_equal, from_numpy, seed_of
from test_gpu_elementwise import both, rand_raw

pytestmark = pytest.mark.gpu

TYPES = ["u8", "s8", "u16", "s16", "u32", "s32", "u64", "s64", "bf16", "f16", "f32", "f64"]


def pair(rng, ty, shape, hip, oracle, special=False, small=False):
    a = rand_raw(rng, ty, shape, lo=-100, hi=100)
    if small and ty[0] in "us":  # keep integers where every float type can hold them (as_type raises otherwise)
        a = (a % 100).astype(a.dtype)
    if special and ty in ("bf16", "f16", "f32", "f64") and a.size >= 4:
        flat = a.reshape(-1)
        bits = {"bf16": (0x7FC0, 0x7F80, 0xFF80, 0x8000), "f16": (0x7E00, 0x7C00, 0xFC00, 0x8000)}
        if ty in bits:
            flat[:4] = bits[ty]
        else:
            flat[:4] = [np.nan, np.inf, -np.inf, -0.0]
    return both(a, ty, hip, oracle)


@pytest.mark.parametrize("ty", TYPES)
@pytest.mark.parametrize("shape,axis", [((7,), None), ((3, 5), 0), ((3, 5), 1), ((2, 3, 4), 1), ((1000, 37), None), ((4, 1, 6), 2)])
def test_iota(ty, shape, axis, hip, oracle):
    assert_bits_equal(Nx.iota(shape, type=ty, axis=axis, backend=hip), Nx.iota(shape, type=ty, axis=axis, backend=oracle),
                      f"iota {ty} {shape} axis {axis}")


@pytest.mark.parametrize("ty", TYPES)
@pytest.mark.parametrize("shape", [(3, 3), (2, 5), (5, 2), (3, 4, 2), (2, 2, 7, 9), (257, 300)])
def test_eye(ty, shape, hip, oracle):
    assert_bits_equal(Nx.eye(shape, type=ty, backend=hip), Nx.eye(shape, type=ty, backend=oracle), f"eye {ty} {shape}")


SELECT_SHAPES = [((64, 33), (64, 33), (64, 33)), ((), (5, 7), (5, 7)), ((5, 7), (), (7,)), ((4, 3, 6), (1, 3, 6), (4, 3, 1)),
                 ((1000, 129), (129,), ()), ((3, 5), (3, 1), (1, 5)), ((), (), ())]


@pytest.mark.parametrize("pt,tt,ft", [("u8", "f32", "f32"), ("s32", "s32", "f32"), ("f32", "bf16", "bf16"), ("bf16", "s8", "s64"),
                                      ("u8", "u64", "u64"), ("f64", "f16", "f32"), ("s64", "u8", "s16"), ("f16", "f64", "s32")])
@pytest.mark.parametrize("ps,ts,fs", SELECT_SHAPES)
def test_select(pt, tt, ft, ps, ts, fs, hip, oracle):
    rng = np.random.default_rng(seed_of(pt, tt, ft, ps, ts, fs))
    praw = rand_raw(rng, pt, ps, lo=-2, hi=2)
    if praw.size:
        praw.reshape(-1)[:: 3] = 0  # plenty of false entries
    hp, op = both(praw, pt, hip, oracle)
    ht, ot = pair(rng, tt, ts, hip, oracle, special=True)
    hf, of = pair(rng, ft, fs, hip, oracle, special=True)
    assert_bits_equal(Nx.select(hp, ht, hf), Nx.select(op, ot, of), f"select {pt} {tt} {ft} {ps} {ts} {fs}")


def test_select_treats_nan_and_negative_zero_as_the_reference_does(hip, oracle):
    pred = np.array([np.nan, -0.0, 0.0, 1e-30, -np.inf], dtype=np.float32)
    a, b = np.arange(5, dtype=np.int32), -np.arange(5, dtype=np.int32) - 1
    got = Nx.select(from_numpy(pred, "f32", hip), from_numpy(a, "s32", hip), from_numpy(b, "s32", hip))
    want = Nx.select(from_numpy(pred, "f32", oracle), from_numpy(a, "s32", oracle), from_numpy(b, "s32", oracle))
    assert_bits_equal(got, want, "select truthiness")
    assert hip.to_numpy(got).tolist() == [0, -2, -3, 3, 4]


def bound(number, backend):
    """A clip bound as the front end would make it from a plain number: s32 or f32, rank 0."""
    ty = "f32" if isinstance(number, float) else "s32"
    return from_numpy(np.array(number, dtype=np.float32 if ty == "f32" else np.int32), ty, backend)


@pytest.mark.parametrize("ty", TYPES)
@pytest.mark.parametrize("lo,hi", [(-10, 10), (2.5, 7), (-3, 4.25), (5, -5)])
@pytest.mark.parametrize("shape", [(1001,), (16, 64)])
def test_clip(ty, lo, hi, shape, hip, oracle):
    if ty.startswith("u") and (lo < 0 or hi < 0):
        lo, hi = abs(lo), abs(hi)
    rng = np.random.default_rng(seed_of(ty, lo, hi, shape))
    ht, ot = pair(rng, ty, shape, hip, oracle, special=True)
    got = Nx.clip(ht, bound(lo, hip), bound(hi, hip))
    want = Nx.clip(ot, bound(lo, oracle), bound(hi, oracle))
    assert_bits_equal(got, want, f"clip {ty} [{lo}, {hi}] {shape}")


SLICES = [((100,), [10], [50], [1]), ((100,), [3], [90], [7]), ((20, 30), [2, 3], [10, 20], [1, 1]), ((20, 30), [0, 1], [20, 29], [3, 4]),
          ((6, 8, 64), [1, 2, 0], [4, 5, 64], [1, 1, 1]), ((6, 8, 64), [0, 0, 16], [6, 8, 32], [1, 2, 1]),
          ((4, 5, 6, 7), [3, 4, 5, 6], [1, 1, 1, 1], [1, 1, 1, 1]), ((512, 512), [100, 64], [300, 256], [1, 1]), ((9, 9), [50, -3], [4, 4], [1, 1])]


@pytest.mark.parametrize("ty", ["u8", "bf16", "f32", "s64"])
@pytest.mark.parametrize("shape,starts,lengths,strides", SLICES)
def test_slice(ty, shape, starts, lengths, strides, hip, oracle):
    rng = np.random.default_rng(seed_of(ty, shape, starts))
    ht, ot = pair(rng, ty, shape, hip, oracle)
    assert_bits_equal(Nx.slice(ht, starts, lengths, strides), Nx.slice(ot, starts, lengths, strides),
                      f"slice {ty} {shape} {starts} {lengths} {strides}")


def test_slice_with_tensor_start_indices(hip, oracle):
    rng = np.random.default_rng(5)
    ht, ot = pair(rng, "f32", (12, 40), hip, oracle)
    hs = [from_numpy(np.array(7, dtype=np.int32), "s32", hip), from_numpy(np.array(100, dtype=np.int64), "s64", hip)]
    os_ = [from_numpy(np.array(7, dtype=np.int32), "s32", oracle), from_numpy(np.array(100, dtype=np.int64), "s64", oracle)]
    assert_bits_equal(Nx.slice(ht, hs, [3, 8]), Nx.slice(ot, os_, [3, 8]), "slice with tensor starts")


CONCATS = [([(3,), (4,), (1,)], 0), ([(2, 3), (5, 3)], 0), ([(2, 3), (2, 64), (2, 1)], 1), ([(4, 2, 8), (4, 3, 8), (4, 7, 8)], 1),
           ([(2, 3, 4), (2, 3, 12)], -1), ([(256, 128), (256, 128)], 0), ([(256, 128), (256, 256)], 1)]


@pytest.mark.parametrize("types", [("f32",), ("bf16",), ("s8", "s32"), ("u8", "f16", "s64"), ("f32", "f64"), ("s64",)])
@pytest.mark.parametrize("shapes,axis", CONCATS)
def test_concatenate(types, shapes, axis, hip, oracle):
    rng = np.random.default_rng(seed_of(types, shapes, axis))
    hs, os_ = [], []
    for i, shape in enumerate(shapes):
        h, o = pair(rng, types[i % len(types)], shape, hip, oracle, small=True)
        hs.append(h)
        os_.append(o)
    assert_bits_equal(Nx.concatenate(hs, axis=axis), Nx.concatenate(os_, axis=axis), f"concatenate {types} {shapes} axis {axis}")


@pytest.mark.parametrize("types", [("f32",), ("s8", "f32"), ("bf16",)])
@pytest.mark.parametrize("shape,count,axis", [((5,), 3, 0), ((5,), 3, 1), ((4, 6), 2, 1), ((4, 6), 5, -1), ((), 4, 0), ((64, 64), 3, 0)])
def test_stack(types, shape, count, axis, hip, oracle):
    rng = np.random.default_rng(seed_of(types, shape, count, axis))
    hs, os_ = [], []
    for i in range(count):
        h, o = pair(rng, types[i % len(types)], shape, hip, oracle, small=True)
        hs.append(h)
        os_.append(o)
    assert_bits_equal(Nx.stack(hs, axis=axis), Nx.stack(os_, axis=axis), f"stack {types} {shape} x{count} axis {axis}")


@pytest.mark.parametrize("ty", TYPES)
@pytest.mark.parametrize("shape,axes", [((50,), None), ((8, 9), [0]), ((8, 9), [1]), ((4, 5, 6), [0, 2]), ((3, 1000), [1]), ((1000, 3), [0]),
                                        ((70000,), None)])
@pytest.mark.parametrize("op", ["all", "any"])
def test_all_any(ty, shape, axes, op, hip, oracle):
    rng = np.random.default_rng(seed_of(ty, shape, axes, op))
    a = rand_raw(rng, ty, shape, lo=-3, hi=3)
    flat = a.reshape(-1)
    if op == "all":
        flat[flat == 0] = 1
        flat[rng.integers(0, flat.size, size=max(1, flat.size // 40))] = 0  # a few zeros: some slices fail
    else:
        flat[:] = 0
        flat[rng.integers(0, flat.size, size=max(1, flat.size // 40))] = 1
    ha, oa = both(a, ty, hip, oracle)
    fn = getattr(Nx, op)
    assert_bits_equal(fn(ha, axes=axes), fn(oa, axes=axes), f"{op} {ty} {shape} {axes}")
    assert_bits_equal(fn(ha, axes=axes, keep_axes=True), fn(oa, axes=axes, keep_axes=True), f"{op} keep {ty} {shape} {axes}")


def test_all_any_count_nan_as_true(hip, oracle):
    a = np.array([[np.nan, 1.0], [0.0, -0.0]], dtype=np.float32)
    for op in ("all", "any"):
        got = getattr(Nx, op)(from_numpy(a, "f32", hip), axes=[1])
        want = getattr(Nx, op)(from_numpy(a, "f32", oracle), axes=[1])
        assert_bits_equal(got, want, op)
    assert hip.to_numpy(Nx.all(from_numpy(a, "f32", hip), axes=[1])).tolist() == [1, 0]


def test_clip_compares_u64_as_unbounded_numbers(hip, oracle):
    # u64 against s32 bounds gives s64: 2^63 and above must land on the upper bound, not wrap below the lower one
    x = np.array([0, 5, 2**63 - 1, 2**63, 2**64 - 1, 999, 1001], dtype=np.uint64)
    want = Nx.clip(from_numpy(x, "u64", oracle), bound(3, oracle), bound(1000, oracle))
    got = Nx.clip(from_numpy(x, "u64", hip), bound(3, hip), bound(1000, hip))
    assert_bits_equal(got, want, "clip u64 with signed bounds")
    assert hip.to_numpy(got).tolist() == [3, 5, 1000, 1000, 1000, 999, 1000]


PADS = [((10,), [(2, 1, 3)]), ((10,), [(-3, -2, 0)]), ((10,), [(-5, 2, 2)]), ((7, 9), [(1, 2, 0), (3, 0, 1)]), ((7, 9), [(-2, -1, 2), (-4, 5, 3)]),
        ((4, 5, 6), [(0, 0, 0), (1, 1, 1), (-1, -1, 0)]), ((4, 5, 6), [(-1, 1, 1), (-2, 1, 1), (-2, 1, 1)]), ((3, 1, 8), [(0, 0, 2), (4, 4, 7), (0, 0, 0)]),
        ((512, 384), [(16, 16, 0), (64, 64, 0)]), ((512, 384), [(0, 0, 1), (-8, -8, 0)]), ((6,), [(-3, -3, 0)]), ((6,), [(-20, 4, 3)]),
        ((5, 4), [(0, 0, 0), (0, 0, 0)])]


@pytest.mark.parametrize("ty", ["u8", "s16", "bf16", "f32", "s64", "f64"])
@pytest.mark.parametrize("shape,config", PADS)
def test_pad(ty, shape, config, hip, oracle):
    rng = np.random.default_rng(seed_of(ty, shape, config))
    ht, ot = pair(rng, ty, shape, hip, oracle, special=True)
    hv, ov = pair(rng, ty, (), hip, oracle)
    assert_bits_equal(Nx.pad(ht, hv, config), Nx.pad(ot, ov, config), f"pad {ty} {shape} {config}")


@pytest.mark.parametrize("ty,vty", [("s32", "f32"), ("u8", "s16"), ("bf16", "f32"), ("f32", "s64"), ("s8", "u8")])
def test_pad_converts_both_operands_to_the_merged_type(ty, vty, hip, oracle):
    # the oracle follows the reference, which splices the two encodings when the types differ; the device
    # converts first, as the compiled backends do: compare with the oracle applied after its own as_type
    rng = np.random.default_rng(seed_of(ty, vty))
    ht, ot = pair(rng, ty, (6, 11), hip, oracle, small=True)
    hv, ov = pair(rng, vty, (), hip, oracle, small=True)
    config = [(1, -1, 1), (-2, 3, 2)]
    got = Nx.pad(ht, hv, config)
    want = Nx.pad(Nx.as_type(ot, got.type), Nx.as_type(ov, got.type), config)
    assert_bits_equal(got, want, f"pad {ty} with {vty}")


@pytest.mark.parametrize("ty", ["u8", "bf16", "f32", "s64"])
@pytest.mark.parametrize("shape,axes", [((10,), None), ((7, 9), [0]), ((7, 9), [1]), ((7, 9), None), ((4, 5, 6), [0, 2]), ((4, 5, 6), [1]),
                                        ((3, 1, 8), [1]), ((256, 384), [1]), ((256, 384), [0]), ((1,), None)])
def test_reverse(ty, shape, axes, hip, oracle):
    rng = np.random.default_rng(seed_of(ty, shape, axes))
    ht, ot = pair(rng, ty, shape, hip, oracle)
    assert_bits_equal(Nx.reverse(ht, axes=axes), Nx.reverse(ot, axes=axes), f"reverse {ty} {shape} {axes}")


PUTS = [((10,), (3,), [4]), ((10,), (10,), [0]), ((10,), (4,), [9]), ((6, 8), (2, 3), [1, 2]), ((6, 8), (6, 1), [0, -5]), ((4, 5, 6), (1, 5, 2), [3, 0, 100]),
        ((256, 256), (64, 128), [32, 64]), ((5, 5), (0, 3), [1, 1])]


@pytest.mark.parametrize("types", [("f32", "f32"), ("s32", "f32"), ("bf16", "s8"), ("u8", "s16"), ("s64", "s64")])
@pytest.mark.parametrize("shape,piece,starts", PUTS)
def test_put_slice(types, shape, piece, starts, hip, oracle):
    rng = np.random.default_rng(seed_of(types, shape, piece, starts))
    ht, ot = pair(rng, types[0], shape, hip, oracle, small=True)
    hs, os_ = pair(rng, types[1], piece, hip, oracle, small=True)
    assert_bits_equal(Nx.put_slice(ht, starts, hs), Nx.put_slice(ot, starts, os_), f"put_slice {types} {shape} {piece} {starts}")
    # the operand is left as it was
    assert_bits_equal(ht, ot, "put_slice operand")


def test_put_slice_with_tensor_start_indices(hip, oracle):
    rng = np.random.default_rng(9)
    ht, ot = pair(rng, "f32", (12, 40), hip, oracle)
    hs, os_ = pair(rng, "f32", (3, 8), hip, oracle)
    hi = [from_numpy(np.array(7, dtype=np.int32), "s32", hip), from_numpy(np.array(100, dtype=np.int64), "s64", hip)]
    oi = [from_numpy(np.array(7, dtype=np.int32), "s32", oracle), from_numpy(np.array(100, dtype=np.int64), "s64", oracle)]
    assert_bits_equal(Nx.put_slice(ht, hi, hs), Nx.put_slice(ot, oi, os_), "put_slice with tensor starts")


@pytest.mark.parametrize("ty", ["f32", "bf16"])  # f16 overflows here: the reference raises, the device writes infinities
def test_iota_beyond_the_exact_integers_of_f32(ty, hip, oracle):
    # above 2^24 the integer -> float conversion rounds: to nearest even, once (binary_backend.ex:49-75 writes the
    # integer as a float of the type)
    n = (1 << 25) + 24
    got = Nx.iota((n,), type=ty, backend=hip)
    if ty == "f32":
        np.testing.assert_array_equal(hip.to_numpy(got), np.arange(n, dtype=np.int64).astype(np.float32))
    tail = Nx.slice(got, [n - 4096], [4096])
    want = Nx.slice(Nx.iota((n,), type=ty, backend=oracle), [n - 4096], [4096])
    assert_bits_equal(tail, want, f"iota {ty} tail")


@pytest.mark.parametrize("ty", ["u8", "bf16", "f32", "s64"])
@pytest.mark.parametrize("axis", [0, 1, 2])
def test_concatenate_of_many_operands_is_a_launch_per_64(ty, axis, hip):
    """150 operands of different (some odd, one empty) extents along the axis go in three launches, each operand found by
    where it begins within an output row; a stack of 70; an operand of another type is converted first.  Bit for bit
    against numpy."""
    import numpy as np
    from nx_amd import nx as Nx
    from nx_amd import types as T
    from support import from_numpy
    rng = np.random.default_rng(axis * 7 + len(ty))
    dt = T.numpy_dtype(T.normalize(ty))
    base = [3, 5, 4]
    parts = []
    for i in range(150):
        shape = list(base)
        shape[axis] = 0 if i == 17 else int(rng.integers(1, 9))
        parts.append(rng.integers(0, 200, size=shape).astype(dt) if ty != "bf16" else rng.integers(0, 60000, size=shape).astype(np.uint16))
    got = Nx.concatenate([from_numpy(p, ty, hip) for p in parts], axis=axis)
    assert np.array_equal(hip.to_numpy(got).view(np.uint8), np.concatenate(parts, axis=axis).view(np.uint8))
    same = [rng.integers(0, 200, size=(4, 7)).astype(dt) if ty != "bf16" else rng.integers(0, 60000, size=(4, 7)).astype(np.uint16) for _ in range(70)]
    stacked = Nx.stack([from_numpy(p, ty, hip) for p in same], axis=1)
    assert np.array_equal(hip.to_numpy(stacked).view(np.uint8), np.stack(same, axis=1).view(np.uint8))
    if ty == "f32":
        mixed = Nx.concatenate([from_numpy(np.arange(6, dtype=np.float32).reshape(2, 3), "f32", hip), from_numpy(np.arange(4, dtype=np.int32).reshape(2, 2), "s32", hip)], axis=1)
        assert hip.to_numpy(mixed).tolist() == [[0.0, 1.0, 2.0, 0.0, 1.0], [3.0, 4.0, 5.0, 2.0, 3.0]]
