"""The five benchmark configurations at their full shapes on the device, checked against the CPU
oracle (whole output where the oracle finishes in seconds, a row sample otherwise) and through
size-independent properties (closed forms, checksums over every output tile)."""
import numpy as np
import pytest

from nx_amd import nx as Nx
from nx_amd import workloads as W
from nx_amd.tensor import template
from support import assert_all_close, assert_bits_equal, from_numpy, values

pytestmark = pytest.mark.gpu


def test_config1_elementwise_and_row_sum(hip, oracle):
    a, b = W.elementwise_reduce()
    def chain(backend):
        x = Nx.add(from_numpy(a, "f32", backend), from_numpy(b, "f32", backend))
        y = Nx.multiply(x, 0.5)
        e = Nx.exp(y)
        return x, y, e, Nx.sum(e, axes=[1])
    hx, hy, he, hs = chain(hip)
    ox, oy, oe, os_ = chain(oracle)
    assert_bits_equal(hx, ox, "add")            # correctly rounded: bit-exact
    assert_bits_equal(hy, oy, "multiply")
    assert_all_close(he, oe, 1e-5, 0, "exp")    # 1e-5 relative: the stated f32 element-wise bar
    # sum: K * 2^-24 * sum|x| + 1 ulp, K = 1024, evaluated on the device's own exp output
    e64 = values(he)
    bound = 1024 * 2.0 ** -24 * np.abs(e64).sum(axis=1) + 2.0 ** -23 * np.abs(e64.sum(axis=1))
    ref = Nx.sum(Nx.backend_copy(he, oracle), axes=[1])
    assert (np.abs(values(hs) - values(ref)) <= bound).all()
    assert hs.shape == (1024,) and hs.type == ("f", 32)


def _sample_rows(rng, n, k):
    return np.sort(rng.choice(n, size=k, replace=False))


def test_config2_dense_gemm_bf16_4096(hip, oracle):
    a, b = W.dense_gemm_bf16()
    ha, hb = from_numpy(a, "bf16", hip), from_numpy(b, "bf16", hip)
    out = Nx.dot(ha, hb)
    assert out.type == ("bf", 16) and out.shape == (4096, 4096)
    got = W.bf16_to_f32(hip.to_numpy(out)).astype(np.float64)
    a64, b64 = W.bf16_to_f32(a).astype(np.float64), W.bf16_to_f32(b).astype(np.float64)
    # oracle on 48 sampled rows (each against all of B)
    rows = _sample_rows(np.random.default_rng(0), 4096, 48)
    want = Nx.dot(from_numpy(a[rows], "bf16", oracle), from_numpy(b, "bf16", oracle))
    ref = values(want)
    mag = np.abs(a64[rows]) @ np.abs(b64)
    bound = 2 * 4096 * 2.0 ** -24 * mag + 2.0 ** -7 * np.abs(ref)
    err = np.abs(got[rows] - ref)
    assert (err <= bound).all(), f"max err/bound {np.max(err / bound):.3f}"
    same = (hip.to_numpy(out)[rows] == np.frombuffer(Nx.to_binary(want), dtype=np.uint16).reshape(ref.shape)).mean()
    assert same > 0.95, f"only {same:.3f} of sampled outputs are bit-identical to the reference"
    # checksum over every tile: C @ 1 against A @ (B @ 1), within output-rounding noise
    chk = a64 @ b64.sum(axis=1)
    tol = 2.0 ** -8 * (np.abs(a64) @ np.abs(b64)).sum(axis=1) / 64 + 1e-6
    assert (np.abs(got.sum(axis=1) - chk) <= tol + 2.0 ** -8 * np.abs(got).sum(axis=1)).all()


def test_config2_dense_gemm_f32_2048(hip, oracle):
    a, b = W.dense_gemm_f32()
    out = Nx.dot(from_numpy(a, "f32", hip), from_numpy(b, "f32", hip))
    got = hip.to_numpy(out).astype(np.float64)
    rows = _sample_rows(np.random.default_rng(1), 2048, 64)
    ref = values(Nx.dot(from_numpy(a[rows], "f32", oracle), from_numpy(b, "f32", oracle)))
    mag = np.abs(a[rows].astype(np.float64)) @ np.abs(b.astype(np.float64))
    assert (np.abs(got[rows] - ref) <= 2048 * 2.0 ** -24 * mag + 2.0 ** -23 * np.abs(ref)).all()
    full = a.astype(np.float64) @ b.astype(np.float64)  # independent library routine
    mag_full = np.abs(a.astype(np.float64)) @ np.abs(b.astype(np.float64))
    assert (np.abs(got - full) <= 2048 * 2.0 ** -24 * mag_full + 2.0 ** -23 * np.abs(full)).all()


def test_config2c_int8_gemm_4096_is_bit_exact(hip, oracle):
    a, b = W.dense_gemm_s8()
    out = Nx.dot(from_numpy(a, "s8", hip), from_numpy(b, "s8", hip), out_type="s32")
    got = hip.to_numpy(out)
    rows = _sample_rows(np.random.default_rng(2), 4096, 32)
    want = Nx.dot(from_numpy(a[rows], "s8", oracle), from_numpy(b, "s8", oracle), out_type="s32")
    assert np.array_equal(got[rows], np.frombuffer(Nx.to_binary(want), dtype=np.int32).reshape(32, 4096))
    # exact checksums over every row and column
    a64, b64 = a.astype(np.int64), b.astype(np.int64)
    assert np.array_equal(got.astype(np.int64).sum(axis=1), a64 @ b64.sum(axis=1))
    assert np.array_equal(got.astype(np.int64).sum(axis=0), a64.sum(axis=0) @ b64)


def test_config3_attention_scores_and_softmax(hip, oracle):
    q, k = W.attention_scores()
    def scores(backend):
        return Nx.dot(from_numpy(q, "bf16", backend), [2], [0], from_numpy(k, "bf16", backend), [2], [0])
    hs, os_ = scores(hip), scores(oracle)
    assert hs.shape == (32, 512, 512) and hs.type == ("bf", 16)
    q64, k64 = W.bf16_to_f32(q).astype(np.float64), W.bf16_to_f32(k).astype(np.float64)
    mag = np.einsum("bmk,bnk->bmn", np.abs(q64), np.abs(k64))
    ref = values(os_)
    assert (np.abs(values(hs) - ref) <= 2 * 64 * 2.0 ** -24 * mag + 2.0 ** -7 * np.abs(ref)).all()
    # softmax chain on the same bf16 scores (the device's), each op one callback
    def softmax(s):
        f = Nx.as_type(s, "f32")
        z = Nx.multiply(f, 0.125)
        m = Nx.reduce_max(z, axes=[2], keep_axes=True)
        e = Nx.exp(Nx.subtract(z, m))
        d = Nx.sum(e, axes=[2], keep_axes=True)
        return f, z, m, Nx.divide(e, d)
    hf, hz, hm, hp = softmax(hs)
    of, oz, om, op = softmax(Nx.backend_copy(hs, oracle))
    assert_bits_equal(hf, of, "as_type")
    assert_bits_equal(hz, oz, "scale")
    assert_bits_equal(hm, om, "reduce_max")
    assert_all_close(hp, op, 1e-5, 1e-7, "softmax")
    assert np.allclose(values(hp).sum(axis=2), 1.0, atol=1e-5)


def test_config4_int8_weight_only_linear(hip, oracle):
    w, x, scales = W.int8_linear()
    hw, hx = from_numpy(w, "s8", hip), from_numpy(x, "s8", hip)
    acc = Nx.dot(hx, [1], hw, [1], out_type="s32")
    assert acc.shape == (64, 11008)
    exact = (x.astype(np.float64) @ w.astype(np.float64).T).astype(np.int64)  # closed form; exact: |sum| < 2^53
    assert np.array_equal(hip.to_numpy(acc), exact.astype(np.int32))
    rows = np.array([0, 17, 63])
    want = Nx.dot(from_numpy(x[rows], "s8", oracle), [1], from_numpy(w, "s8", oracle), [1], out_type="s32")
    assert np.array_equal(hip.to_numpy(acc)[rows], np.frombuffer(Nx.to_binary(want), dtype=np.int32).reshape(3, 11008))
    y = Nx.multiply(Nx.as_type(acc, "f32"), from_numpy(scales, "f32", hip))
    oy = Nx.multiply(Nx.as_type(Nx.backend_copy(acc, oracle), "f32"), from_numpy(scales, "f32", oracle))
    assert_bits_equal(y, oy, "dequantise")
    # the public API infers s8 for s8 x s8 and wraps
    wrapped = Nx.dot(hx, [1], hw, [1])
    assert wrapped.type == ("s", 8)
    assert np.array_equal(hip.to_numpy(wrapped), exact.astype(np.int8))


def test_config5_argmax_with_ties_and_embedding_take(hip, oracle):
    logits, table, tied = W.logits_and_table()
    hl = hip.from_numpy(template("f32", logits.shape), logits)
    idx = Nx.argmax(hl, axis=1, tie_break="low", type="u32")
    assert idx.type == ("u", 32) and idx.shape == (8192,)
    got = hip.to_numpy(idx)
    assert np.array_equal(got, np.argmax(logits, axis=1).astype(np.uint32))  # first occurrence
    # oracle on the tied rows plus a sample of the rest
    rows = np.unique(np.concatenate([tied, np.arange(0, 8192, 97)]))
    want = Nx.argmax(from_numpy(logits[rows], "f32", oracle), axis=1, tie_break="low", type="u32")
    assert np.array_equal(got[rows], np.frombuffer(Nx.to_binary(want), dtype=np.uint32))
    high = hip.to_numpy(Nx.argmax(hl, axis=1, tie_break="high", type="u32"))
    assert (high[tied] >= got[tied]).all() and (high[tied] > got[tied]).mean() > 0.9 and np.array_equal(np.delete(high, tied), np.delete(got, tied))
    ht = from_numpy(table, "bf16", hip)
    emb = Nx.take(ht, idx)
    assert emb.shape == (8192, 4096) and emb.type == ("bf", 16)
    assert np.array_equal(hip.to_numpy(emb), table[got])
    small = Nx.take(from_numpy(table, "bf16", oracle), from_numpy(got[:64], "u32", oracle))
    assert np.array_equal(hip.to_numpy(emb)[:64], np.frombuffer(Nx.to_binary(small), dtype=np.uint16).reshape(64, 4096))
