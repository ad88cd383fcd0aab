"""Shared helpers of the parity suite: build tensors from fixture specs, run one front-end call on
a chosen backend, compare results the way the reference's assertions do
(nx/lib/nx/testing.ex:22-68 assert_equal with NaN == NaN, 151-176 assert_all_close)."""
import json
import math
import os

import numpy as np

from nx_amd import nx as Nx
from nx_amd import types as T
from nx_amd.tensor import Tensor, binary_to_numpy, list_to_binary, template, to_float64

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def seed_of(*parts) -> int:
    """Deterministic seed from test parameters (Python's hash() of strings changes per process)."""
    import zlib
    return zlib.crc32(repr(parts).encode())


def load_cases(name="nx_known_answers.json"):
    with open(os.path.join(GOLDEN, name)) as f:
        return json.load(f)["cases"]


def _num(x):
    return {"inf": math.inf, "-inf": -math.inf, "nan": math.nan}[x] if isinstance(x, str) else x


def _map(v):
    return [_map(e) for e in v] if isinstance(v, list) else _num(v)


def _has_float(v):
    return any(_has_float(e) for e in v) if isinstance(v, list) else isinstance(v, float)


def spec_to_tensor(spec, backend):
    """{"v": literal, "t": type} or {"iota": shape, "t": type} -> tensor on `backend`."""
    if not isinstance(spec, dict):
        return spec  # plain number or axis list
    if "iota" in spec:
        shape = tuple(spec["iota"])
        ty = T.normalize(spec.get("t", "s32"))
        vals = np.arange(int(np.prod(shape)), dtype=np.int64).reshape(shape)
        vals = vals.astype(np.float64) if T.is_float(ty) else vals
    else:
        v = _map(spec["v"])
        ty = T.normalize(spec["t"]) if "t" in spec else (("f", 32) if _has_float(v) else ("s", 32))
        vals = np.asarray(v, dtype=np.float64 if T.is_float(ty) else np.int64)
    return backend.from_binary(template(ty, vals.shape), list_to_binary(vals, ty), {})


def from_numpy(arr, ty, backend):
    """Raw element array (bf16 as uint16 bits) -> tensor on `backend`."""
    ty = T.normalize(ty)
    shape = np.shape(arr)  # ascontiguousarray turns a rank-0 array into {1}
    arr = np.ascontiguousarray(arr, dtype=T.numpy_dtype(ty))
    return backend.from_binary(template(ty, shape), arr.tobytes(), {})


def run_case(case, backend):
    op, opts = case["op"], dict(case.get("opts", {}))
    if op in ("iota", "eye"):  # creation: the shape is a plain list, the backend is an option
        return getattr(Nx, op)(case["args"][0], backend=backend, **opts)
    if op in ("concatenate", "stack"):  # a list of operands
        return getattr(Nx, op)([spec_to_tensor(a, backend) for a in case["args"][0]], **opts)
    if op == "slice":  # start indices may be rank-0 tensors
        t, starts, lengths = case["args"]
        return Nx.slice(spec_to_tensor(t, backend), [spec_to_tensor(i, backend) for i in starts], lengths, **opts)
    if op == "put_slice":  # start indices are numbers or rank-0 tensors
        t, starts, piece = case["args"]
        return Nx.put_slice(spec_to_tensor(t, backend), [spec_to_tensor(i, backend) for i in starts], spec_to_tensor(piece, backend))
    if op == "pad":  # the padding configuration is a plain list of (low, high, interior)
        t, value, config = case["args"]
        return Nx.pad(spec_to_tensor(t, backend), spec_to_tensor(value, backend), config)
    args = [spec_to_tensor(a, backend) for a in case["args"]]
    if op not in ("iota", "eye") and args and not any(isinstance(a, Tensor) for a in args):
        # only plain numbers (`Nx.add(1, 2)`): they would land on the default backend; a rank-0 tensor
        # of the type a number infers to (`Nx.tensor(1)`) on the backend under test is the same call
        args[0] = spec_to_tensor({"v": case["args"][0]}, backend)
    if op in ("dot", "dot4", "dot6"):
        return Nx.dot(*args)
    if op == "as_type":
        return Nx.as_type(args[0], opts["type"])
    if op == "softmax":
        e = Nx.exp(args[0])
        return Nx.divide(e, Nx.sum(e))
    return getattr(Nx, op)(*args, **opts)


def raw(t: Tensor) -> np.ndarray:
    return binary_to_numpy(Nx.to_binary(t), t.type, t.shape)


def values(t: Tensor) -> np.ndarray:
    return to_float64(Nx.to_binary(t), t.type, t.shape)


def assert_bits_equal(actual: Tensor, expected: Tensor, what=""):
    """Same type, same shape, same bit pattern in every element."""
    assert actual.type == expected.type, f"{what}: type {actual.type} != {expected.type}"
    assert actual.shape == expected.shape, f"{what}: shape {actual.shape} != {expected.shape}"
    a, e = raw(actual), raw(expected)
    ab, eb = a.view(_uint(a.dtype)).ravel(), e.view(_uint(e.dtype)).ravel()
    if not np.array_equal(ab, eb):
        bad = np.flatnonzero(ab != eb)
        i = int(bad[0])
        raise AssertionError(f"{what}: {bad.size} of {ab.size} elements differ; first at flat index {i}: "
                             f"got {a.ravel()[i]!r} (0x{int(ab[i]):x}) expected {e.ravel()[i]!r} (0x{int(eb[i]):x})")


def _uint(dtype):
    return {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[np.dtype(dtype).itemsize]


def assert_all_close(actual: Tensor, expected: Tensor, rtol, atol=0.0, what=""):
    """|a - e| <= atol + rtol*|e| elementwise; NaN matches NaN, infinities must match exactly."""
    assert actual.type == expected.type, f"{what}: type {actual.type} != {expected.type}"
    assert actual.shape == expected.shape, f"{what}: shape {actual.shape} != {expected.shape}"
    a, e = values(actual).ravel(), values(expected).ravel()
    nan_a, nan_e = np.isnan(a), np.isnan(e)
    assert np.array_equal(nan_a, nan_e), f"{what}: NaN positions differ"
    inf = np.isinf(e) | np.isinf(a)
    assert np.array_equal(a[inf], e[inf]), f"{what}: infinities differ"
    ok = ~(nan_e | inf)
    err = np.abs(a[ok] - e[ok])
    bound = atol + rtol * np.abs(e[ok])
    if not (err <= bound).all():
        i = int(np.argmax(err - bound))
        raise AssertionError(f"{what}: max violation at {i}: got {a[ok][i]!r} expected {e[ok][i]!r} "
                             f"(err {err[i]:.3e} > bound {bound[i]:.3e})")


def expected_tensor(case, backend):
    exp = case["expect"]
    return spec_to_tensor({"v": exp["v"], "t": exp["t"]}, backend)


def check_case(case, backend, raises_types):
    """Runs one golden case on `backend` and checks it against the transcribed expectation."""
    if "raises" in case:
        try:
            Nx.to_binary(run_case(case, backend))  # a device reports what its kernels met when the result is read
        except raises_types as e:
            assert case["raises"] in str(e), f"{case['name']}: message {str(e)!r} lacks {case['raises']!r}"
            return
        raise AssertionError(f"{case['name']}: expected an error containing {case['raises']!r}")
    result = run_case(case, backend)
    exp = case["expect"]
    expected = expected_tensor(case, backend)
    if "rtol" in exp:
        assert_all_close(result, expected, exp["rtol"], exp.get("atol", 0.0), case["name"])
    else:
        assert_bits_equal(result, expected, case["name"])
