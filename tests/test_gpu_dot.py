"""Device Nx.dot against the CPU oracle.

Bar: integer results bit-exact (s8 x s8 -> s32 / s8 on MFMA, everything else on the plain
kernel); float results within the K-scaled bound
    |d| <= 2K * 2^-24 * sum_k |a_k b_k|  +  1 ulp(out type) * |ref|
(the device accumulates in f32 on MFMA, the reference sequentially in f64), and for f64 operands
within 1e-13 relative to sum|a_k b_k|."""
import numpy as np
import pytest

from nx_amd import nx as Nx
from nx_amd import types as T
from support import assert_bits_equal, from_numpy, seed_of, values
from test_gpu_elementwise import both, rand_raw

pytestmark = pytest.mark.gpu

ULP = {("bf", 16): 2.0 ** -7, ("f", 16): 2.0 ** -10, ("f", 32): 2.0 ** -23, ("f", 64): 2.0 ** -52}


def check_float_dot(got, want, a64, b64, eq, K, what):
    """a64/b64: decoded operands; eq: einsum spec producing the output from |a|, |b|."""
    assert got.type == want.type and got.shape == want.shape, what
    mag = np.einsum(eq, np.abs(a64), np.abs(b64)).reshape(got.shape)
    ref = values(want)
    acc = 2.0 ** -24 if got.type != ("f", 64) and True else 2.0 ** -50
    bound = 2 * max(K, 1) * acc * mag + ULP[got.type] * np.abs(ref) + 1e-30
    err = np.abs(values(got) - ref)
    assert (err <= bound).all(), f"{what}: max err/bound {np.max(err / bound):.3f}"


MNK = [(128, 128, 64), (256, 256, 256), (130, 70, 136), (1, 1, 8), (17, 300, 1000), (512, 64, 2048), (64, 11008 // 8, 4096),
       (33, 33, 40), (200, 129, 8), (5, 7, 3), (64, 64, 7)]


@pytest.mark.parametrize("M,N,K", MNK)
@pytest.mark.parametrize("ty", ["bf16", "f16", "f32", "f64"])
@pytest.mark.parametrize("layout", ["nn", "nt", "tn", "tt"])
def test_float_matmul_layouts(M, N, K, ty, layout, hip, oracle):
    if ty == "f64" and M * N * K > 5_000_000:
        pytest.skip("plain-kernel path: covered at smaller sizes")
    rng = np.random.default_rng(seed_of(M, N, K, ty))
    a_shape = (M, K) if layout[0] == "n" else (K, M)
    b_shape = (K, N) if layout[1] == "n" else (N, K)
    a, b = rand_raw(rng, ty, a_shape, lo=-1, hi=1), rand_raw(rng, ty, b_shape, lo=-1, hi=1)
    ha, oa = both(a, ty, hip, oracle)
    hb, ob = both(b, ty, hip, oracle)
    c1 = [1] if layout[0] == "n" else [0]
    c2 = [0] if layout[1] == "n" else [1]
    got, want = Nx.dot(ha, c1, hb, c2), Nx.dot(oa, c1, ob, c2)
    eq = ("mk" if layout[0] == "n" else "km") + "," + ("kn" if layout[1] == "n" else "nk") + "->mn"
    check_float_dot(got, want, values(oa), values(ob), eq, K, f"dot {ty} {layout} {M}x{N}x{K}")


@pytest.mark.parametrize("M,N,K", [(64, 344, 4096), (128, 128, 128), (7, 9, 16), (130, 70, 1024), (64, 64, 48), (3, 5, 7)])
@pytest.mark.parametrize("out_type", ["s32", "s8", "s64"])
def test_int8_dot_is_bit_exact(M, N, K, out_type, hip, oracle):
    rng = np.random.default_rng(seed_of(M, N, K))
    x = rng.integers(-127, 128, size=(M, K)).astype(np.int8)
    w = rng.integers(-127, 128, size=(N, K)).astype(np.int8)
    hx, ox = both(x, "s8", hip, oracle)
    hw, ow = both(w, "s8", hip, oracle)
    ot = None if out_type == "s8" else out_type  # s8 is what the public API infers (wraps)
    assert_bits_equal(Nx.dot(hx, [1], hw, [1], out_type=ot), Nx.dot(ox, [1], ow, [1], out_type=ot), f"s8 dot -> {out_type}")
    # exact closed form as an independent check of both
    exact = x.astype(np.int64) @ w.astype(np.int64).T
    got = hip.to_numpy(Nx.dot(hx, [1], hw, [1], out_type="s32"))
    assert np.array_equal(got, exact.astype(np.int32))


@pytest.mark.parametrize("lt,rt", [("s32", "s32"), ("u8", "u8"), ("s16", "s64"), ("u32", "s8"), ("s64", "s64"), ("u8", "s8")])
def test_integer_dot_is_bit_exact(lt, rt, hip, oracle):
    rng = np.random.default_rng(seed_of(lt, rt))
    a, b = rand_raw(rng, lt, (19, 45)), rand_raw(rng, rt, (45, 23))
    ha, oa = both(a, lt, hip, oracle)
    hb, ob = both(b, rt, hip, oracle)
    assert_bits_equal(Nx.dot(ha, hb), Nx.dot(oa, ob), f"dot {lt} {rt}")


@pytest.mark.parametrize("lt,rt", [("f32", "bf16"), ("s8", "f32"), ("f16", "f32"), ("f64", "f32")])
def test_mixed_type_dot(lt, rt, hip, oracle):
    rng = np.random.default_rng(seed_of(lt, rt))
    a, b = rand_raw(rng, lt, (40, 64), lo=-1, hi=1), rand_raw(rng, rt, (64, 24), lo=-1, hi=1)
    ha, oa = both(a, lt, hip, oracle)
    hb, ob = both(b, rt, hip, oracle)
    check_float_dot(Nx.dot(ha, hb), Nx.dot(oa, ob), values(oa), values(ob), "mk,kn->mn", 64, f"dot {lt} {rt}")


BATCHED = [((32, 64, 64), [2], [0], (32, 48, 64), [2], [0], "bmk,bnk->bmn"),
           ((4, 16, 40), [1], [0], (4, 16, 24), [1], [0], "bkm,bkn->bmn"),
           ((3, 5, 32, 8), [3], [0, 1], (3, 5, 8, 16), [2], [0, 1], "abmk,abkn->abmn"),
           ((2, 8, 16, 4), [1, 3], [0], (2, 4, 8, 6), [2, 1], [0], "bkml,blkn->bmn"),
           ((6, 10), [0, 1], [], (10, 6), [1, 0], [], "ab,ba->"),
           ((4, 6, 5), [1], [], (3, 6, 2), [1], [], "amb,cmd->abcd"),
           ((8, 3), [], [], (2, 5), [], [], "ab,cd->abcd")]


@pytest.mark.parametrize("case", BATCHED, ids=[c[-1] for c in BATCHED])
@pytest.mark.parametrize("ty", ["bf16", "f32", "s32", "s8"])
def test_general_contraction_and_batch_axes(case, ty, hip, oracle):
    ls, c1, b1, rs, c2, b2, eq = case
    rng = np.random.default_rng(seed_of(eq, ty))
    a, b = rand_raw(rng, ty, ls, lo=-1, hi=1), rand_raw(rng, ty, rs, lo=-1, hi=1)
    ha, oa = both(a, ty, hip, oracle)
    hb, ob = both(b, ty, hip, oracle)
    got, want = Nx.dot(ha, c1, b1, hb, c2, b2), Nx.dot(oa, c1, b1, ob, c2, b2)
    if T.is_integer(T.normalize(ty)):
        assert_bits_equal(got, want, f"dot {eq} {ty}")
    else:
        K = int(np.prod([ls[x] for x in c1])) if c1 else 1
        check_float_dot(got, want, values(oa), values(ob), eq, K, f"dot {eq} {ty}")


def test_dot_matches_closed_form_on_small_integers_in_bf16(hip):
    """Small-integer operands make every partial sum exact in f32: the MFMA result must equal the
    integer matrix product exactly, whatever the accumulation order."""
    rng = np.random.default_rng(2)
    a = rng.integers(-4, 5, size=(256, 512))
    b = rng.integers(-4, 5, size=(512, 384))
    bits = lambda m: (m.astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    ha, hb = from_numpy(bits(a), "bf16", hip), from_numpy(bits(b), "bf16", hip)
    got = values(Nx.dot(Nx.as_type(ha, "f32"), Nx.as_type(hb, "f32")))
    assert np.array_equal(got, (a @ b).astype(np.float64))
    got_bf = values(Nx.dot(ha, hb, out_type="f32"))
    assert np.array_equal(got_bf, (a @ b).astype(np.float64))


@pytest.mark.parametrize("M,N,K", [(256, 256, 256), (64, 48, 128), (130, 72, 256), (512, 528, 384), (16, 4096, 128)])
@pytest.mark.parametrize("layout", ["nn", "nt", "tn", "tt"])
def test_int8_dot_every_operand_layout_is_bit_exact(M, N, K, layout, hip, oracle):
    """K-outer s8 operands are transposed inside the MFMA kernel (or by a pass when the row count
    is ragged): all four layouts must give the exact integer product."""
    rng = np.random.default_rng(seed_of(M, N, K, layout))
    a = rng.integers(-128, 128, size=(M, K) if layout[0] == "n" else (K, M)).astype(np.int8)
    b = rng.integers(-128, 128, size=(K, N) if layout[1] == "n" else (N, K)).astype(np.int8)
    c1 = [1] if layout[0] == "n" else [0]
    c2 = [0] if layout[1] == "n" else [1]
    got = hip.to_numpy(Nx.dot(from_numpy(a, "s8", hip), c1, from_numpy(b, "s8", hip), c2, out_type="s32"))
    am = a if layout[0] == "n" else a.T
    bm = b if layout[1] == "n" else b.T
    exact = (am.astype(np.float64) @ bm.astype(np.float64)).astype(np.int64)  # exact: |sum| < 2^53
    assert np.array_equal(got, exact.astype(np.int32))
    want = Nx.dot(from_numpy(a, "s8", oracle), c1, from_numpy(b, "s8", oracle), c2, out_type="s32")
    assert np.array_equal(got, np.frombuffer(Nx.to_binary(want), dtype=np.int32).reshape(M, N))


@pytest.mark.parametrize("ty,M,N,K", [("f32", 128, 128, 64), ("f32", 100, 36, 96), ("f32", 102, 38, 96), ("bf16", 136, 72, 128),
                                      ("f16", 264, 200, 192), ("bf16", 132, 76, 64), ("f32", 300, 260, 2048)])
@pytest.mark.parametrize("layout", ["nn", "nt", "tn", "tt"])
def test_float_dot_pipelined_kernel_layouts(ty, M, N, K, layout, hip, oracle):
    rng = np.random.default_rng(seed_of(ty, M, N, K, layout))
    a = rand_raw(rng, ty, (M, K) if layout[0] == "n" else (K, M), lo=-1, hi=1)
    b = rand_raw(rng, ty, (K, N) if layout[1] == "n" else (N, K), lo=-1, hi=1)
    ha, oa = both(a, ty, hip, oracle)
    hb, ob = both(b, ty, hip, oracle)
    c1 = [1] if layout[0] == "n" else [0]
    c2 = [0] if layout[1] == "n" else [1]
    eq = ("mk" if layout[0] == "n" else "km") + "," + ("kn" if layout[1] == "n" else "nk") + "->mn"
    check_float_dot(Nx.dot(ha, c1, hb, c2), Nx.dot(oa, c1, ob, c2), values(oa), values(ob), eq, K, f"{ty} {layout} {M}x{N}x{K}")


# Few rows against a long K-inner matrix (M <= 64, K a multiple of 4096 bytes, N >= 256) take
# the weight-streaming kernel: ragged row counts, a column count that is not a multiple of the
# 64 columns of a work-group, every MFMA element type, and a batch.
@pytest.mark.parametrize("M", [1, 16, 33, 64])
@pytest.mark.parametrize("ty,N,K", [("s8", 300, 4096), ("s8", 1000, 8192), ("bf16", 264, 2048), ("f16", 257, 4096),
                                    ("f32", 320, 1024), ("bf16", 1024, 4096)])
def test_few_rows_against_long_matrix(M, ty, N, K, hip, oracle):
    rng = np.random.default_rng(seed_of(M, ty, N, K))
    if ty == "s8":
        x = rng.integers(-127, 128, size=(M, K)).astype(np.int8)
        w = rng.integers(-127, 128, size=(N, K)).astype(np.int8)
        hx, ox = both(x, ty, hip, oracle)
        hw, ow = both(w, ty, hip, oracle)
        got, want = Nx.dot(hx, [1], hw, [1], out_type="s32"), Nx.dot(ox, [1], ow, [1], out_type="s32")
        assert_bits_equal(got, want, f"few rows s8 {M}x{N}x{K}")
    else:
        x, w = rand_raw(rng, ty, (M, K), lo=-1, hi=1), rand_raw(rng, ty, (N, K), lo=-1, hi=1)
        hx, ox = both(x, ty, hip, oracle)
        hw, ow = both(w, ty, hip, oracle)
        got, want = Nx.dot(hx, [1], hw, [1]), Nx.dot(ox, [1], ow, [1])
        check_float_dot(got, want, values(ox), values(ow), "mk,nk->mn", K, f"few rows {ty} {M}x{N}x{K}")


@pytest.mark.parametrize("M", [1, 24, 64])
@pytest.mark.parametrize("ty,N,K", [("bf16", 264, 2048), ("f16", 1024, 1056), ("s8", 400, 4096), ("bf16", 120, 640), ("bf16", 328, 192),
                                    ("s8", 12304, 1152), ("s8", 1040, 1024), ("s8", 48, 2048)])
def test_few_rows_against_weights_stored_k_outer(M, ty, N, K, hip, oracle):
    """x . W with W stored [K, N], the plain Nx.dot(x, w): a few rows of a 2-byte type take the 128-row kernels
    (which read a K-outer operand by transposing loads, K split over work-groups when long), int8 the 64-row tiles
    with 64 or -- for many columns -- 128 columns of the weights, read by the byte-transposing loads; a contraction
    length that is an odd number of slabs takes one slab per phase."""
    rng = np.random.default_rng(seed_of(M, ty, N, K, "k-outer weights"))
    if ty == "s8":
        x = rng.integers(-127, 128, size=(M, K)).astype(np.int8)
        w = rng.integers(-127, 128, size=(K, N)).astype(np.int8)
        hx, ox = both(x, ty, hip, oracle)
        hw, ow = both(w, ty, hip, oracle)
        assert_bits_equal(Nx.dot(hx, hw, out_type="s32"), Nx.dot(ox, ow, out_type="s32"), f"few rows s8 {M}x{N}x{K} NN")
    else:
        x, w = rand_raw(rng, ty, (M, K), lo=-1, hi=1), rand_raw(rng, ty, (K, N), lo=-1, hi=1)
        hx, ox = both(x, ty, hip, oracle)
        hw, ow = both(w, ty, hip, oracle)
        check_float_dot(Nx.dot(hx, hw), Nx.dot(ox, ow), values(ox), values(ow), "mk,kn->mn", K, f"few rows {ty} {M}x{N}x{K} NN")


@pytest.mark.parametrize("ty,M,N,K", [("bf16", 64, 1024, 1152), ("s8", 33, 520, 1152), ("f16", 7, 300, 4224), ("s8", 64, 11008, 4096)])
def test_few_rows_one_and_two_slabs_per_phase(ty, M, N, K, hip, oracle):
    """K-inner operands on 64 x 64 tiles of the two-group kernel: K of an odd number of slabs walks one slab per
    phase through eight stages, an even number two per phase through four."""
    rng = np.random.default_rng(seed_of(ty, M, N, K, "rows phases"))
    if ty == "s8":
        x = rng.integers(-127, 128, size=(M, K)).astype(np.int8)
        w = rng.integers(-127, 128, size=(N, K)).astype(np.int8)
        got = hip.to_numpy(Nx.dot(from_numpy(x, ty, hip), [1], from_numpy(w, ty, hip), [1], out_type="s32"))
        assert np.array_equal(got, x.astype(np.int32) @ w.astype(np.int32).T)
    else:
        x, w = rand_raw(rng, ty, (M, K), lo=-1, hi=1), rand_raw(rng, ty, (N, K), lo=-1, hi=1)
        hx, ox = both(x, ty, hip, oracle)
        hw, ow = both(w, ty, hip, oracle)
        check_float_dot(Nx.dot(hx, [1], hw, [1]), Nx.dot(ox, [1], ow, [1]), values(ox), values(ow), "mk,nk->mn", K, f"few rows {ty} {M}x{N}x{K}")


def test_few_rows_against_long_matrix_batched(hip, oracle):
    rng = np.random.default_rng(7)
    x = rng.integers(-127, 128, size=(3, 20, 4096)).astype(np.int8)
    w = rng.integers(-127, 128, size=(3, 272, 4096)).astype(np.int8)
    hx, ox = both(x, "s8", hip, oracle)
    hw, ow = both(w, "s8", hip, oracle)
    got = Nx.dot(hx, [2], [0], hw, [2], [0], out_type="s32")
    want = Nx.dot(ox, [2], [0], ow, [2], [0], out_type="s32")
    assert_bits_equal(got, want, "few rows s8 batched")


# Shapes large enough for the 256 x 256 tile (at least 192 of them), ragged at both edges, in every
# operand layout: covers the transposing-read staging of K-outer bf16 and s8 operands on both
# sides.  The oracle runs on a sample of output rows.
@pytest.mark.parametrize("ty", ["bf16", "s8"])
@pytest.mark.parametrize("layout", ["nn", "nt", "tn", "tt"])
def test_large_ragged_dot_on_the_big_tile(ty, layout, hip, oracle):
    M, N, K = 2064, 6160, 256
    rng = np.random.default_rng(seed_of(ty, layout, "big tile"))
    if ty == "s8":
        a = rng.integers(-127, 128, size=(M, K)).astype(np.int8)
        b = rng.integers(-127, 128, size=(K, N)).astype(np.int8)
    else:
        a, b = rand_raw(rng, ty, (M, K), lo=-1, hi=1), rand_raw(rng, ty, (K, N), lo=-1, hi=1)
    la = a if layout[0] == "n" else np.ascontiguousarray(a.T)
    lb = b if layout[1] == "n" else np.ascontiguousarray(b.T)
    c1 = [1] if layout[0] == "n" else [0]
    c2 = [0] if layout[1] == "n" else [1]
    kw = {"out_type": "s32"} if ty == "s8" else {}
    got = Nx.dot(from_numpy(la, ty, hip), c1, from_numpy(lb, ty, hip), c2, **kw)
    assert got.shape == (M, N)
    rows = np.unique(np.concatenate([[0, 255, 256, M - 1], rng.integers(0, M, size=24)]))
    oa, ob = from_numpy(np.ascontiguousarray(a[rows]), ty, oracle), from_numpy(b, ty, oracle)
    want = Nx.dot(oa, ob, **kw)
    got_rows = from_numpy(np.ascontiguousarray(hip.to_numpy(got)[rows]), "s32" if ty == "s8" else ty, oracle)
    if ty == "s8":
        assert_bits_equal(got_rows, want, f"big tile s8 {layout}")
    else:
        check_float_dot(got_rows, want, values(oa), values(ob), "mk,kn->mn", K, f"big tile {ty} {layout}")


@pytest.mark.parametrize("ty", ["bf16", "f16"])
@pytest.mark.parametrize("M,N,K", [(1024, 6144, 256), (1000, 6200, 384), (2048, 3080, 128)])
@pytest.mark.parametrize("layout", ["nn", "nt", "tn", "tt"])
def test_half_width_tiles_of_the_two_group_kernel(ty, M, N, K, layout, hip, oracle):
    """Problems whose grid of 256 x 256 tiles would leave CUs idle take 256 x 128 tiles (wave tiles 64 x 64 or
    128 x 32): whole and ragged grids, all four operand layouts."""
    rng = np.random.default_rng(seed_of(ty, M, N, K, layout, "w128"))
    a, b = rand_raw(rng, ty, (M, K), lo=-1, hi=1), rand_raw(rng, ty, (K, N), lo=-1, hi=1)
    la = a if layout[0] == "n" else np.ascontiguousarray(a.T)
    lb = b if layout[1] == "n" else np.ascontiguousarray(b.T)
    c1 = [1] if layout[0] == "n" else [0]
    c2 = [0] if layout[1] == "n" else [1]
    got = Nx.dot(from_numpy(la, ty, hip), c1, from_numpy(lb, ty, hip), c2)
    assert got.shape == (M, N)
    rows = np.unique(np.concatenate([[0, 127, 128, 255, 256, M - 1], rng.integers(0, M, size=18)]))
    oa, ob = from_numpy(np.ascontiguousarray(a[rows]), ty, oracle), from_numpy(b, ty, oracle)
    want = Nx.dot(oa, ob)
    got_rows = from_numpy(np.ascontiguousarray(hip.to_numpy(got)[rows]), ty, oracle)
    check_float_dot(got_rows, want, values(oa), values(ob), "mk,kn->mn", K, f"256x128 tiles {ty} {layout}")


@pytest.mark.parametrize("ty,M,N,K", [("bf16", 333, 777, 555), ("f16", 256, 512, 1000), ("f32", 300, 260, 250), ("s8", 384, 320, 1001),
                                      ("bf16", 2, 4100, 2050)])
@pytest.mark.parametrize("layout", ["nn", "nt", "tn", "tt"])
def test_contraction_lengths_off_the_slab_grid_are_padded(ty, M, N, K, layout, hip, oracle):
    """A K that is not a whole number of 128-byte slabs: large problems run on zero-extended copies of the
    operands (products of two zeros add nothing), so int8 stays exact and floats stay within the bound."""
    rng = np.random.default_rng(seed_of(ty, M, N, K, layout, "pad"))
    if ty == "s8":
        a = rng.integers(-127, 128, size=(M, K)).astype(np.int8)
        b = rng.integers(-127, 128, size=(K, N)).astype(np.int8)
    else:
        a, b = rand_raw(rng, ty, (M, K), lo=-1, hi=1), rand_raw(rng, ty, (K, N), lo=-1, hi=1)
    la = a if layout[0] == "n" else np.ascontiguousarray(a.T)
    lb = b if layout[1] == "n" else np.ascontiguousarray(b.T)
    c1 = [1] if layout[0] == "n" else [0]
    c2 = [0] if layout[1] == "n" else [1]
    kw = {"out_type": "s32"} if ty == "s8" else {}
    got = Nx.dot(from_numpy(la, ty, hip), c1, from_numpy(lb, ty, hip), c2, **kw)
    assert got.shape == (M, N)
    rows = np.unique(np.concatenate([[0, M - 1], rng.integers(0, M, size=10)]))
    oa, ob = from_numpy(np.ascontiguousarray(a[rows]), ty, oracle), from_numpy(b, ty, oracle)
    want = Nx.dot(oa, ob, **kw)
    got_rows = from_numpy(np.ascontiguousarray(hip.to_numpy(got)[rows]), "s32" if ty == "s8" else ty, oracle)
    if ty == "s8":
        assert_bits_equal(got_rows, want, f"padded K s8 {layout}")
    else:
        check_float_dot(got_rows, want, values(oa), values(ob), "mk,kn->mn", K, f"padded K {ty} {layout}")


@pytest.mark.parametrize("ty,M,N,K", [("bf16", 128, 1024, 4096), ("s8", 128, 1024, 4096), ("f16", 200, 520, 2048), ("f32", 132, 384, 2048),
                                      ("bf16", 768, 4096, 4096), ("f16", 1000, 4100, 4096),
                                      ("s8", 384, 512, 8192), ("bf16", 512, 1024, 2048),
                                      # f32 is cut much earlier: 64 ways, two ways with two slabs each, 64 x 32 tiles
                                      ("f32", 256, 264, 4096), ("f32", 128, 128, 128), ("f32", 520, 512, 512), ("f32", 1024, 1024, 1024)])
@pytest.mark.parametrize("layout", ["nn", "nt", "tn", "tt"])
def test_long_k_on_an_under_filled_grid_is_split(ty, M, N, K, layout, hip, oracle):
    """A few hundred rows against a long K leave most CUs without a 128 x 128 tile; K is then split over
    several work-groups per tile and the partial results are added by a second pass.  int8 must stay exact,
    floats within the bound of an f32 accumulation in any order."""
    rng = np.random.default_rng(seed_of(ty, M, N, K, layout, "split"))
    if ty == "s8":
        a = rng.integers(-127, 128, size=(M, K)).astype(np.int8)
        b = rng.integers(-127, 128, size=(K, N)).astype(np.int8)
    else:
        a, b = rand_raw(rng, ty, (M, K), lo=-1, hi=1), rand_raw(rng, ty, (K, N), lo=-1, hi=1)
    la = a if layout[0] == "n" else np.ascontiguousarray(a.T)
    lb = b if layout[1] == "n" else np.ascontiguousarray(b.T)
    c1 = [1] if layout[0] == "n" else [0]
    c2 = [0] if layout[1] == "n" else [1]
    kw = {"out_type": "s32"} if ty == "s8" else {}
    got = Nx.dot(from_numpy(la, ty, hip), c1, from_numpy(lb, ty, hip), c2, **kw)
    assert got.shape == (M, N)
    rows = np.unique(np.concatenate([[0, 127, M - 1], rng.integers(0, M, size=13)]))
    oa, ob = from_numpy(np.ascontiguousarray(a[rows]), ty, oracle), from_numpy(b, ty, oracle)
    want = Nx.dot(oa, ob, **kw)
    got_rows = from_numpy(np.ascontiguousarray(hip.to_numpy(got)[rows]), "s32" if ty == "s8" else ty, oracle)
    if ty == "s8":
        assert_bits_equal(got_rows, want, f"split K s8 {layout}")
    else:
        check_float_dot(got_rows, want, values(oa), values(ob), "mk,kn->mn", K, f"split K {ty} {layout}")


@pytest.mark.parametrize("ty,M,N,K", [("bf16", 512, 520, 256), ("bf16", 300, 528, 128), ("f16", 264, 344, 128), ("bf16", 1024, 6152, 64),
                                      ("bf16", 130, 76, 64), ("f16", 64, 40, 128)])
def test_two_byte_outputs_land_in_their_own_columns(ty, M, N, K, hip):
    """The MFMA kernel writes bf16 / f16 results two column tiles at a time, lanes trading halves
    so that each stores 16 bytes.  A selection matrix (one 1.0 per column) makes every output a
    copy of one input element, so any mix-up of lanes, tiles or columns shows as a wrong value
    -- exact, no tolerance."""
    rng = np.random.default_rng(seed_of(ty, M, N, K))
    a = rand_raw(rng, ty, (M, K), lo=-1, hi=1)
    pick = (7 * np.arange(N) + 3) % K
    b = np.zeros((K, N), dtype=a.dtype)
    b[pick, np.arange(N)] = np.uint16(0x3F80) if ty == "bf16" else np.float16(1.0)
    got = values(Nx.dot(from_numpy(a, ty, hip), from_numpy(b, ty, hip)))
    want = values(from_numpy(np.ascontiguousarray(a[:, pick]), ty, hip))
    assert got.shape == (M, N)
    assert np.array_equal(got, want)  # (-0.0 == 0.0: a lone product plus zeros may lose the sign of a zero)


@pytest.mark.parametrize("ty,M,N,K", [("bf16", 1024, 1024, 1024), ("bf16", 1000, 904, 576), ("f16", 520, 1288, 640), ("bf16", 200, 136, 512),
                                      ("s8", 1024, 1024, 1024), ("s8", 2056, 3080, 1152), ("f16", 2048, 2048, 1088)])
@pytest.mark.parametrize("layout", ["nn", "nt", "tn", "tt"])
def test_two_groups_sharing_k_on_128_tiles(ty, M, N, K, layout, hip, oracle):
    """Grids of 128 x 128 tiles that fit the CUs once (for int8: any grid, both operands K-inner) are walked by two
    groups of waves that take the even and the odd slabs of K and add their partial sums at the end: even and odd
    numbers of slabs, whole and ragged grids, all four layouts.  int8 exact, floats within the bound."""
    rng = np.random.default_rng(seed_of(ty, M, N, K, layout, "pp128"))
    if ty == "s8":
        a = rng.integers(-127, 128, size=(M, K)).astype(np.int8)
        b = rng.integers(-127, 128, size=(K, N)).astype(np.int8)
    else:
        a, b = rand_raw(rng, ty, (M, K), lo=-1, hi=1), rand_raw(rng, ty, (K, N), lo=-1, hi=1)
    la = a if layout[0] == "n" else np.ascontiguousarray(a.T)
    lb = b if layout[1] == "n" else np.ascontiguousarray(b.T)
    c1 = [1] if layout[0] == "n" else [0]
    c2 = [0] if layout[1] == "n" else [1]
    kw = {"out_type": "s32"} if ty == "s8" else {}
    got = Nx.dot(from_numpy(la, ty, hip), c1, from_numpy(lb, ty, hip), c2, **kw)
    assert got.shape == (M, N)
    rows = np.unique(np.concatenate([[0, 31, 32, 63, 64, 127, 128, M - 1], rng.integers(0, M, size=16)]))
    oa, ob = from_numpy(np.ascontiguousarray(a[rows]), ty, oracle), from_numpy(b, ty, oracle)
    want = Nx.dot(oa, ob, **kw)
    got_rows = from_numpy(np.ascontiguousarray(hip.to_numpy(got)[rows]), "s32" if ty == "s8" else ty, oracle)
    if ty == "s8":
        assert_bits_equal(got_rows, want, f"128 tiles, two groups, s8 {layout}")
    else:
        check_float_dot(got_rows, want, values(oa), values(ob), "mk,kn->mn", K, f"128 tiles, two groups, {ty} {layout}")


@pytest.mark.parametrize("ty,M,N,K,out_type", [("bf16", 1024, 1032, 1024, None), ("f16", 520, 776, 576, None), ("bf16", 768, 512, 640, "f32"),
                                               ("s8", 1024, 520, 1152, "s32"), ("s8", 264, 392, 1024, "s8")])
def test_two_groups_sharing_k_put_every_output_in_its_place(ty, M, N, K, out_type, hip):
    """A selection matrix (a single 1 per column, spread over even and odd slabs) makes every output a copy of one
    input element: a tile half, row or column that ends up with the wrong group shows as a wrong value -- exact."""
    rng = np.random.default_rng(seed_of(ty, M, N, K, "pp128 pick"))
    pick = (37 * np.arange(N) + 11) % K
    if ty == "s8":
        a = rng.integers(-127, 128, size=(M, K)).astype(np.int8)
        b = np.zeros((N, K), dtype=np.int8)
        b[np.arange(N), pick] = 1
        got = hip.to_numpy(Nx.dot(from_numpy(a, ty, hip), [1], from_numpy(b, ty, hip), [1], out_type=out_type))
        assert got.shape == (M, N)
        assert np.array_equal(got.astype(np.int64), a[:, pick].astype(np.int64))
        return
    a = rand_raw(rng, ty, (M, K), lo=-1, hi=1)
    b = np.zeros((K, N), dtype=a.dtype)
    b[pick, np.arange(N)] = np.uint16(0x3F80) if ty == "bf16" else np.float16(1.0)
    kw = {"out_type": out_type} if out_type else {}
    got = values(Nx.dot(from_numpy(a, ty, hip), from_numpy(b, ty, hip), **kw))
    want = values(from_numpy(np.ascontiguousarray(a[:, pick]), ty, hip))
    assert got.shape == (M, N)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("M,N,K", [(1, 1, 4096), (1, 1, 70003), (16, 16, 8192), (3, 5, 4100), (32, 1, 5000), (1, 32, 12288), (7, 2, 40000)])
@pytest.mark.parametrize("ty", ["f32", "bf16", "f64", "s8", "s32", "u8"])
@pytest.mark.parametrize("layout", ["nn", "nt", "tn", "tt"])
def test_few_outputs_over_a_long_contraction(M, N, K, ty, layout, hip, oracle):
    """The dot of two long vectors, a handful of outputs over K >= 4096: a work-group per output and segment of K with
    partial sums in f64 / 64-bit integers and a pass that adds the segments (one lane walking all of K took 0.26 s for 4M
    elements).  Integers bit for bit (s8 widened to s32, s32 and u8 in their own wrapping types), floats within the
    bound of an accumulation in any order; batched once."""
    rng = np.random.default_rng(seed_of(M, N, K, ty, layout, "few outputs"))
    integer = ty in ("s8", "s32", "u8")
    a_shape = (M, K) if layout[0] == "n" else (K, M)
    b_shape = (K, N) if layout[1] == "n" else (N, K)
    if integer:
        lo, hi = (-127, 128) if ty != "u8" else (0, 256)
        a = rng.integers(lo, hi, size=a_shape).astype(T.numpy_dtype(T.normalize(ty)))
        b = rng.integers(lo, hi, size=b_shape).astype(T.numpy_dtype(T.normalize(ty)))
    else:
        a, b = rand_raw(rng, ty, a_shape, lo=-1, hi=1), rand_raw(rng, ty, b_shape, lo=-1, hi=1)
    ha, oa = both(a, ty, hip, oracle)
    hb, ob = both(b, ty, hip, oracle)
    c1 = [1] if layout[0] == "n" else [0]
    c2 = [0] if layout[1] == "n" else [1]
    kw = {"out_type": "s32"} if ty == "s8" else {}
    got, want = Nx.dot(ha, c1, hb, c2, **kw), Nx.dot(oa, c1, ob, c2, **kw)
    if integer:
        assert_bits_equal(got, want, f"dot {ty} {layout} {M}x{N}x{K}")
    else:
        eq = ("mk" if layout[0] == "n" else "km") + "," + ("kn" if layout[1] == "n" else "nk") + "->mn"
        check_float_dot(got, want, values(oa), values(ob), eq, K, f"dot {ty} {layout} {M}x{N}x{K}")


def test_few_outputs_over_a_long_contraction_batched(hip, oracle):
    rng = np.random.default_rng(77)
    a, b = rand_raw(rng, "f32", (3, 2, 6000), lo=-1, hi=1), rand_raw(rng, "f32", (3, 6000, 4), lo=-1, hi=1)
    ha, oa = both(a, "f32", hip, oracle)
    hb, ob = both(b, "f32", hip, oracle)
    got, want = Nx.dot(ha, [2], [0], hb, [1], [0]), Nx.dot(oa, [2], [0], ob, [1], [0])
    check_float_dot(got, want, values(oa), values(ob), "bmk,bkn->bmn", 6000, "batched few outputs")
    v = rng.integers(-100, 100, size=(1 << 20,)).astype(np.int32)
    hv, ov = both(v, "s32", hip, oracle)
    assert_bits_equal(Nx.dot(hv, hv), Nx.dot(ov, ov), "vector . vector s32")


@pytest.mark.parametrize("M,N,K", [(300, 10, 784), (1000, 1, 512), (65, 32, 256), (2000, 17, 128), (4099, 3, 1152)])
@pytest.mark.parametrize("ty", ["f32", "bf16", "f16", "s8"])
@pytest.mark.parametrize("layout", ["nn", "nt", "tn", "tt"])
def test_many_rows_against_a_few_columns(M, N, K, ty, layout, hip, oracle):
    """A layer with a few outputs ([60000, 784] . [784, 10]): tiles of 128 x 32, and a K that is not whole slabs
    contracted in place with its last part from padded copies.  int8 exact, floats within the accumulation bound,
    and every output in its own place (rows and columns off every tile edge)."""
    rng = np.random.default_rng(seed_of(M, N, K, ty, layout, "narrow"))
    if ty == "s8":
        a = rng.integers(-127, 128, size=(M, K)).astype(np.int8)
        b = rng.integers(-127, 128, size=(K, N)).astype(np.int8)
    else:
        a, b = rand_raw(rng, ty, (M, K), lo=-1, hi=1), rand_raw(rng, ty, (K, N), lo=-1, hi=1)
    la = a if layout[0] == "n" else np.ascontiguousarray(a.T)
    lb = b if layout[1] == "n" else np.ascontiguousarray(b.T)
    c1 = [1] if layout[0] == "n" else [0]
    c2 = [0] if layout[1] == "n" else [1]
    kw = {"out_type": "s32"} if ty == "s8" else {}
    got = Nx.dot(from_numpy(la, ty, hip), c1, from_numpy(lb, ty, hip), c2, **kw)
    assert got.shape == (M, N)
    rows = np.unique(np.concatenate([[0, 63, 64, min(127, M - 1), min(128, M - 1), M - 1], rng.integers(0, M, size=20)]))
    oa, ob = from_numpy(np.ascontiguousarray(a[rows]), ty, oracle), from_numpy(b, ty, oracle)
    want = Nx.dot(oa, ob, **kw)
    got_rows = from_numpy(np.ascontiguousarray(hip.to_numpy(got)[rows]), "s32" if ty == "s8" else ty, oracle)
    if ty == "s8":
        assert_bits_equal(got_rows, want, f"narrow s8 {layout}")
        full = a.astype(np.int64) @ b.astype(np.int64)
        assert np.array_equal(hip.to_numpy(got).astype(np.int64), full)
    else:
        check_float_dot(got_rows, want, values(oa), values(ob), "mk,kn->mn", K, f"narrow {ty} {layout}")


def test_more_batch_items_than_a_grid_dimension_holds(hip, oracle):
    """100000 small matrices (a transform per point): the batch goes in runs of 65535 items.  Integer-valued f32, so
    every product and sum is exact and numpy's einsum is the answer bit for bit; a few items against the oracle."""
    rng = np.random.default_rng(31)
    a = rng.integers(-8, 9, size=(70001, 3, 3)).astype(np.float32)
    b = rng.integers(-8, 9, size=(70001, 3, 2)).astype(np.float32)
    got = Nx.dot(from_numpy(a, "f32", hip), [2], [0], from_numpy(b, "f32", hip), [1], [0])
    assert got.shape == (70001, 3, 2)
    assert np.array_equal(hip.to_numpy(got), np.einsum("bmk,bkn->bmn", a, b))
    pick = [0, 65534, 65535, 65536, 70000]
    want = Nx.dot(from_numpy(a[pick], "f32", oracle), [2], [0], from_numpy(b[pick], "f32", oracle), [1], [0])
    assert_bits_equal(from_numpy(hip.to_numpy(got)[pick], "f32", oracle), want, "batch of 70001")


@pytest.mark.parametrize("ty", ["f32", "bf16", "s32"])
def test_a_dot_product_per_batch_item(ty, hip, oracle):
    """[B, 1, K] . [B, K, 1]: one output per item, each a work-group of the reduction kernel."""
    rng = np.random.default_rng(seed_of(ty, "rowwise dot"))
    if ty == "s32":
        a, b = rng.integers(-100, 100, size=(3000, 1, 512)).astype(np.int32), rng.integers(-100, 100, size=(3000, 512, 1)).astype(np.int32)
    else:
        a, b = rand_raw(rng, ty, (3000, 1, 512), lo=-1, hi=1), rand_raw(rng, ty, (3000, 512, 1), lo=-1, hi=1)
    ha, oa = both(a, ty, hip, oracle)
    hb, ob = both(b, ty, hip, oracle)
    got, want = Nx.dot(ha, [2], [0], hb, [1], [0]), Nx.dot(oa, [2], [0], ob, [1], [0])
    if ty == "s32":
        assert_bits_equal(got, want, "row-wise dot s32")
    else:
        check_float_dot(got, want, values(oa), values(ob), "bmk,bkn->bmn", 512, f"row-wise dot {ty}")


def test_millions_of_rows_against_a_tiny_matrix(hip):
    """[2M, 3] . [3, 3] (points times a transform): K is not a multiple of 16 bytes, so the plain kernel runs, with
    131072 tiles of rows along the grid's first dimension.  Integer-valued f32: exact."""
    rng = np.random.default_rng(9)
    a = rng.integers(-8, 9, size=(2_000_003, 3)).astype(np.float32)
    b = rng.integers(-8, 9, size=(3, 3)).astype(np.float32)
    got = hip.to_numpy(Nx.dot(from_numpy(a, "f32", hip), from_numpy(b, "f32", hip)))
    assert np.array_equal(got, a @ b)


@pytest.mark.parametrize("ty", ["f64", "s32", "u8", "s64"])
@pytest.mark.parametrize("layout", ["nn", "nt", "tn", "tt"])
def test_plain_kernel_on_64_tiles(ty, layout, hip, oracle):
    """Types without a matrix-core path (f64, wide integers) on tiles of 64 x 64 with sixteen outputs per lane, from 512
    tiles on: every output is still accumulated over k in order, so integers are exact and f64 agrees with the oracle's
    sequential f64 sum bit for bit.  Shapes off the tile and K-step grids."""
    M, N, K = 1500, 1400, 37
    rng = np.random.default_rng(seed_of(ty, layout, "plain 64"))
    if ty == "f64":
        a, b = rng.standard_normal((M, K)), rng.standard_normal((K, N))
    else:
        dt = T.numpy_dtype(T.normalize(ty))
        lo, hi = (0, 200) if ty == "u8" else (-1000, 1000)
        a, b = rng.integers(lo, hi, size=(M, K)).astype(dt), rng.integers(lo, hi, size=(K, N)).astype(dt)
    la = a if layout[0] == "n" else np.ascontiguousarray(a.T)
    lb = b if layout[1] == "n" else np.ascontiguousarray(b.T)
    c1 = [1] if layout[0] == "n" else [0]
    c2 = [0] if layout[1] == "n" else [1]
    got = Nx.dot(from_numpy(la, ty, hip), c1, from_numpy(lb, ty, hip), c2)
    rows = np.unique(np.concatenate([[0, 63, 64, M - 1], rng.integers(0, M, size=8)]))
    want = Nx.dot(from_numpy(np.ascontiguousarray(a[rows]), ty, oracle), from_numpy(b, ty, oracle))
    assert_bits_equal(from_numpy(np.ascontiguousarray(hip.to_numpy(got)[rows]), ty, oracle), want, f"plain 64 {ty} {layout}")
    if ty != "f64":
        wide = (a.astype(np.int64) @ b.astype(np.int64)).astype(T.numpy_dtype(T.normalize(ty)))
        assert np.array_equal(hip.to_numpy(got), wide)


@pytest.mark.parametrize("M,K,N", [(3, 3, 1), (4, 4, 4), (1, 7, 5), (8, 2, 8), (2, 64, 2)])
@pytest.mark.parametrize("ty", ["f32", "bf16", "s32", "f64"])
def test_many_small_matrices(M, K, N, ty, hip, oracle):
    """A batch of small matrices takes one lane per output over the whole batch; k in order, so the oracle's bits."""
    rng = np.random.default_rng(seed_of(M, K, N, ty, "small batched"))
    Bn = 777
    if ty == "s32":
        a, b = rng.integers(-99, 99, size=(Bn, M, K)).astype(np.int32), rng.integers(-99, 99, size=(Bn, K, N)).astype(np.int32)
    else:
        a, b = rand_raw(rng, ty, (Bn, M, K), lo=-2, hi=2), rand_raw(rng, ty, (Bn, K, N), lo=-2, hi=2)
    ha, oa = both(a, ty, hip, oracle)
    hb, ob = both(b, ty, hip, oracle)
    assert_bits_equal(Nx.dot(ha, [2], [0], hb, [1], [0]), Nx.dot(oa, [2], [0], ob, [1], [0]), f"small batched {ty} {M}x{K}x{N}")
    # the other layouts: contract the first axis of the left operand, the last of the right
    at, bt = np.ascontiguousarray(a.transpose(0, 2, 1)), np.ascontiguousarray(b.transpose(0, 2, 1))
    hat, oat = both(at, ty, hip, oracle)
    hbt, obt = both(bt, ty, hip, oracle)
    assert_bits_equal(Nx.dot(hat, [1], [0], hbt, [2], [0]), Nx.dot(oat, [1], [0], obt, [2], [0]), f"small batched tt {ty}")


@pytest.mark.parametrize("S,R,K", [(1, 4096, 1024), (4, 1000, 300), (2, 257, 5000), (3, 70000, 256)])
@pytest.mark.parametrize("ty", ["f32", "f64", "s32"])
@pytest.mark.parametrize("side", ["vectors_left", "vectors_right"])
@pytest.mark.parametrize("small_layout", ["k_inner", "k_outer"])
def test_a_few_vectors_against_a_matrix(S, R, K, ty, side, small_layout, hip, oracle):
    """A few vectors against a matrix in f32 and wider types: with the matrix stored [N, K] (contiguous along k) the
    reduction kernel, a work-group per output; stored [K, N] the tiled kernels.  Integers exact, floats in the bound."""
    rng = np.random.default_rng(seed_of(S, R, K, ty, side, small_layout, "few vectors"))
    if ty == "s32":
        small, big = rng.integers(-99, 99, size=(S, K)).astype(np.int32), rng.integers(-99, 99, size=(K, R)).astype(np.int32)
    else:
        small, big = rand_raw(rng, ty, (S, K), lo=-1, hi=1), rand_raw(rng, ty, (K, R), lo=-1, hi=1)
    for big_layout in ("k_outer", "k_inner"):
        sm = small if small_layout == "k_inner" else np.ascontiguousarray(small.T)
        bg = big if big_layout == "k_outer" else np.ascontiguousarray(big.T)
        cs, cb = ([1] if small_layout == "k_inner" else [0]), ([0] if big_layout == "k_outer" else [1])
        hs, os_ = both(sm, ty, hip, oracle)
        hb, ob = both(bg, ty, hip, oracle)
        if side == "vectors_left":
            got, want, eq = Nx.dot(hs, cs, hb, cb), Nx.dot(os_, cs, ob, cb), "sk,kr->sr"
            a64, b64 = values(from_numpy(small, ty, oracle)), values(from_numpy(big, ty, oracle))
        else:
            got, want, eq = Nx.dot(hb, cb, hs, cs), Nx.dot(ob, cb, os_, cs), "kr,sk->rs"
            a64, b64 = values(from_numpy(big, ty, oracle)), values(from_numpy(small, ty, oracle))
        if ty == "s32":
            assert_bits_equal(got, want, f"few vectors s32 {side} {big_layout}")
        else:
            check_float_dot(got, want, a64, b64, eq, K, f"few vectors {ty} {side} {small_layout} {big_layout}")


@pytest.mark.parametrize("layout", ["nn", "nt", "tn", "tt"])
@pytest.mark.parametrize("M,N,K", [(128, 128, 64), (256, 384, 512), (130, 70, 144), (1024, 1024, 256), (64, 2048, 1024), (33, 40, 16), (2000, 16, 4096)])
def test_f64_contraction_on_the_matrix_cores(M, N, K, layout, hip, oracle):
    """f64 operands whose K is a whole number of 128-byte slabs (16 elements) and whose result has 256 elements or more
    take the MFMA f64 path (`v_mfma_f64_16x16x4_f64`, f64 accumulators): within the accumulation bound of the oracle's
    sequential f64 sum, and exact where every partial sum is (small integers).  Other f64 shapes stay on the plain
    kernels, which add over k in order and so match the oracle bit for bit (test_plain_kernel_on_64_tiles)."""
    rng = np.random.default_rng(seed_of(M, N, K, layout, "f64 mfma"))
    a_shape = (M, K) if layout[0] == "n" else (K, M)
    b_shape = (K, N) if layout[1] == "n" else (N, K)
    c1, c2 = [1] if layout[0] == "n" else [0], [0] if layout[1] == "n" else [1]
    a, b = rng.standard_normal(a_shape), rng.standard_normal(b_shape)
    ha, oa = both(a, "f64", hip, oracle)
    hb, ob = both(b, "f64", hip, oracle)
    got, want = Nx.dot(ha, c1, hb, c2), Nx.dot(oa, c1, ob, c2)
    am = a if layout[0] == "n" else a.T
    bm = b if layout[1] == "n" else b.T
    check_float_dot(got, want, am, bm, "mk,kn->mn", K, f"f64 {M}x{N}x{K} {layout}")
    ai, bi = rng.integers(-50, 51, size=a_shape).astype(np.float64), rng.integers(-50, 51, size=b_shape).astype(np.float64)
    exact = (ai if layout[0] == "n" else ai.T) @ (bi if layout[1] == "n" else bi.T)
    res = hip.to_numpy(Nx.dot(from_numpy(ai, "f64", hip), c1, from_numpy(bi, "f64", hip), c2))
    assert np.array_equal(res, exact)
    # an f32 result from f64 operands: one rounding of the f64 sum
    res32 = hip.to_numpy(Nx.dot(from_numpy(ai, "f64", hip), c1, from_numpy(bi, "f64", hip), c2, out_type="f32"))
    assert np.array_equal(res32, exact.astype(np.float32))


@pytest.mark.parametrize("ty", ["f16", "bf16", "f32", "f64"])
@pytest.mark.parametrize("m,k,n", [(1, 1, 1), (5, 1, 7), (64, 1, 64), (3, 2, 4), (16, 16, 16), (33, 64, 40), (128, 128, 128), (1, 256, 1)])
def test_zero_products_leave_a_positive_zero(ty, m, k, n, hip, oracle):
    """The reference adds every product to a sum that starts at 0, so products that are all -0 (a negative factor
    times +0) give +0, with one term (K = 1) as with many; outputs whose terms cancel are +0 as well."""
    rng = np.random.default_rng(seed_of("zero products", ty, m, k, n))
    dtype = np.float32 if ty == "bf16" else T.numpy_dtype(T.normalize(ty))
    a = rng.choice(np.array([-1.0, -2.0, 1.0, 0.0, -0.0]), size=(m, k)).astype(dtype)
    b = rng.choice(np.array([0.0, -0.0, 0.0, 1.0, -1.0]), size=(k, n), p=[0.4, 0.3, 0.1, 0.1, 0.1]).astype(dtype)
    if ty == "bf16":
        a, b = [(np.asarray(v, np.float32).view(np.uint32) >> 16).astype(np.uint16) for v in (a, b)]
    ha, oa = both(a, ty, hip, oracle)
    hb, ob = both(b, ty, hip, oracle)
    assert_bits_equal(Nx.dot(ha, hb), Nx.dot(oa, ob), f"dot {ty} {m}x{k}x{n}")
    assert_bits_equal(Nx.dot(ha, [0], hb, [1]) if m == n else Nx.dot(hb, [0], ha, [1]),
                      Nx.dot(oa, [0], ob, [1]) if m == n else Nx.dot(ob, [0], oa, [1]), f"dot {ty} other axes")
