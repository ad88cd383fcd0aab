"""Seeded synthetic inputs of the benchmark configurations (host-side numpy; not `Nx.Random`:
parity only needs the same bytes to reach both backends).  bf16 arrays are uint16 bit patterns
obtained by truncating the f32 sample, so the stored value is exactly what both sides decode."""
from __future__ import annotations

import numpy as np


def bf16_bits(x: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(x, dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16)


def bf16_to_f32(bits: np.ndarray) -> np.ndarray:
    return (bits.astype(np.uint32) << 16).view(np.float32)


def elementwise_reduce(seed=1, n=1024):
    """config 1: a, b f32 {n, n} uniform[-1, 1)."""
    rng = np.random.default_rng(seed)
    return (rng.uniform(-1, 1, size=(n, n)).astype(np.float32), rng.uniform(-1, 1, size=(n, n)).astype(np.float32))


def dense_gemm_bf16(seed=2, n=4096):
    """config 2: A, B bf16 {n, n}, entries normal(0, 1) / 64."""
    rng = np.random.default_rng(seed)
    return (bf16_bits(rng.standard_normal((n, n), dtype=np.float32) / 64),
            bf16_bits(rng.standard_normal((n, n), dtype=np.float32) / 64))


def dense_gemm_f32(seed=3, n=2048):
    rng = np.random.default_rng(seed)
    return (rng.standard_normal((n, n), dtype=np.float32) / 64, rng.standard_normal((n, n), dtype=np.float32) / 64)


def dense_gemm_s8(seed=4, n=4096):
    rng = np.random.default_rng(seed)
    return (rng.integers(-127, 128, size=(n, n), dtype=np.int8), rng.integers(-127, 128, size=(n, n), dtype=np.int8))


def attention_scores(seed=5, batch=32, seq=512, dim=64):
    """config 3: Q, K bf16 {batch, seq, dim} normal(0, 1)."""
    rng = np.random.default_rng(seed)
    return (bf16_bits(rng.standard_normal((batch, seq, dim), dtype=np.float32)),
            bf16_bits(rng.standard_normal((batch, seq, dim), dtype=np.float32)))


def int8_linear(seed=6, out_features=11008, in_features=4096, tokens=64):
    """config 4: W s8 {out, in}, X s8 {tokens, in} uniform ints in [-127, 127]; f32 scales
    uniform[1e-3, 1e-2) per output column."""
    rng = np.random.default_rng(seed)
    return (rng.integers(-127, 128, size=(out_features, in_features), dtype=np.int8),
            rng.integers(-127, 128, size=(tokens, in_features), dtype=np.int8),
            rng.uniform(1e-3, 1e-2, size=(out_features,)).astype(np.float32))


def logits_and_table(seed=7, rows=8192, vocab=32000, width=4096):
    """config 5: logits f32 {rows, vocab} normal(0, 2) with 1 % of the rows holding injected exact
    ties of the row maximum (some before the original); table bf16 {vocab, width} normal(0, 0.02)."""
    rng = np.random.default_rng(seed)
    logits = rng.standard_normal((rows, vocab), dtype=np.float32)
    logits *= 2
    tied = rng.choice(rows, size=max(rows // 100, 1), replace=False)
    for r in tied:
        m = logits[r].max()
        cols = rng.choice(vocab, size=int(rng.integers(1, 4)), replace=False)
        logits[r, cols] = m
    table = bf16_bits(rng.standard_normal((vocab, width), dtype=np.float32) * np.float32(0.02))
    return logits, table, np.sort(tied)
