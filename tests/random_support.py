"""Runs the transcribed `Nx.Random` known answers (tests/golden/nx_random_known_answers.json)."""
import zlib

from nx_amd import nx as Nx
from nx_amd import random as Random
from support import assert_all_close, assert_bits_equal, load_cases, spec_to_tensor
from nx_amd.tensor import template
from support import list_to_binary, _map  # noqa: F401 - shared literal decoding
import numpy as np
from nx_amd import types as T

CASES = load_cases("nx_random_known_answers.json")
# results that pass through erf_inv: the reference's implementation lives in a package that is not
# vendored, so the last bits are not pinned; tolerances in units of the type's precision
LOOSE_RTOL = {("bf", 16): 2.0 ** -7, ("f", 16): 2.0 ** -9, ("f", 32): 2.0 ** -21, ("f", 64): 2.0 ** -40}


def run_random_case(case, backend, through=None):
    seed = zlib.adler32(case["seed_of_name"].encode()) if "seed_of_name" in case else case["seed"]
    key = Random.key(seed, backend=backend)
    fn = case["fn"]
    if fn == "key":
        return key
    args = [spec_to_tensor(a, backend) for a in case.get("args", [])]
    opts = dict(case.get("opts", {}))
    if "shape" in opts:
        opts["shape"] = tuple(opts["shape"])
    fun = getattr(Random, fn)
    if through is not None:  # e.g. defn.jit: the options are static, the key and operands are arguments
        fun = through(fun, **opts)
        opts = {}
    out = fun(key, *args, **opts)
    return out[0] if isinstance(out, tuple) else out  # (sample, new_key) for the unsplit variants


def check_random_case(case, backend, through=None):
    result = run_random_case(case, backend, through)
    assert type(result.data) is backend, f"{case['name']}: result left the backend of the key"
    exp = case["expect"]
    ty = T.normalize(exp["t"])
    vals = np.asarray(_map(exp["v"]), dtype=np.float64 if T.is_float(ty) else np.uint64 if ty == ("u", 64) else np.int64)
    expected = backend.from_binary(template(ty, vals.shape), list_to_binary(vals, ty), {})
    if case.get("exact", True) and not case.get("close"):
        assert_bits_equal(result, expected, case["name"])
    else:
        # "close": the reference's own test compares with assert_all_close
        rtol = 1e-4 if case.get("close") else LOOSE_RTOL[ty]
        assert_all_close(result, expected, rtol, 0.0, case["name"])
