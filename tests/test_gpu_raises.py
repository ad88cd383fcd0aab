"""Where the reference raises instead of returning a value -- integer quotient / remainder by zero, a
negative shift count, a negative integer exponent, float remainder by zero or of a non-finite element
(binary_backend.ex:711-750), a gather index out of range -- the oracle raises, and the device raises
late: its kernels record the case and the next call that waits for the device (reading the result)
raises the same exception.  Afterwards the context is usable again."""
import numpy as np
import pytest

from nx_amd import _lib as L
from nx_amd import nx as Nx
from nx_amd import backend as B
from support import from_numpy, raw

pytestmark = pytest.mark.gpu

# op, left, right, type, the oracle's / the device's exception text
CASES = [("quotient", [7, 8, 9], [2, 0, 3], "s32", "bad argument in arithmetic expression"),
         ("remainder", [7, 8, 9], [2, 3, 0], "s64", "bad argument in arithmetic expression"),
         ("remainder", [7, 8, 9], [0, 3, 1], "u8", "bad argument in arithmetic expression"),
         ("left_shift", [1, 2, 3], [1, -1, 2], "s32", "cannot left shift by -1"),
         ("right_shift", [16, 32, 64], [1, 2, -5], "s16", "cannot right shift by -5"),
         ("pow", [2, 3, 4], [2, -2, 1], "s32", "ArithmeticError"),
         ("remainder", [1.5, 2.5, 3.5], [1.0, 0.0, 2.0], "f32", "bad argument in arithmetic expression"),
         ("remainder", [1.5, np.inf, 3.5], [1.0, 2.0, 2.0], "f32", "not a number"),
         ("remainder", [1.5, 2.5, 3.5], [1.0, np.nan, 2.0], "f64", "not a number")]


@pytest.mark.parametrize("op,a,b,ty,text", CASES, ids=[f"{c[0]}-{c[3]}-{i}" for i, c in enumerate(CASES)])
@pytest.mark.parametrize("shape", ["vector", "broadcast"])
def test_device_raises_late_what_the_reference_raises(op, a, b, ty, text, shape, hip, oracle):
    from oracle.binary_backend import ReferenceRaises
    dt = {"s32": np.int32, "s64": np.int64, "u8": np.uint8, "s16": np.int16, "f32": np.float32, "f64": np.float64}[ty]
    a, b = np.asarray(a, dtype=dt), np.asarray(b, dtype=dt)
    if shape == "broadcast":  # the rank-N kernel: a column against a row
        a = a.reshape(3, 1)
    with pytest.raises(ReferenceRaises) as ref:
        getattr(Nx, op)(from_numpy(a, ty, oracle), from_numpy(b, ty, oracle))
    assert text in str(ref.value)
    res = getattr(Nx, op)(from_numpy(a, ty, hip), from_numpy(b, ty, hip))  # enqueued: nothing to report yet
    with pytest.raises(L.HipNxError) as dev:
        Nx.to_binary(res)
    assert dev.value.status == L.ERAISED and text in str(dev.value)
    assert isinstance(dev.value, ArithmeticError if str(ref.value).startswith("ArithmeticError") else ValueError)
    # reported once; the word is re-armed and the context works on
    ok = Nx.add(from_numpy(np.arange(4, dtype=np.int32), "s32", hip), 1)
    assert raw(ok).tolist() == [1, 2, 3, 4]
    B.sync()


def test_good_operands_report_nothing(hip, oracle):
    a, b = np.array([7, -8, 9], dtype=np.int32), np.array([2, 3, -4], dtype=np.int32)
    for op in ("quotient", "remainder"):
        got, want = getattr(Nx, op)(from_numpy(a, "s32", hip), from_numpy(b, "s32", hip)), getattr(Nx, op)(from_numpy(a, "s32", oracle), from_numpy(b, "s32", oracle))
        assert raw(got).tolist() == raw(want).tolist()
    B.sync()


def test_deferred_bounds_policy_raises_at_the_next_wait(hip):
    table = from_numpy(np.arange(40, dtype=np.float32).reshape(10, 4), "f32", hip)
    previous = B.bounds_policy("defer")
    try:
        rows = Nx.take(table, from_numpy(np.array([1, 3, 9], dtype=np.int32), "s32", hip))
        assert raw(rows)[:, 0].tolist() == [4.0, 12.0, 36.0]
        bad = Nx.take(table, from_numpy(np.array([1, 10, 2], dtype=np.int32), "s32", hip))  # returns at once
        with pytest.raises(L.HipNxArgumentError) as e:
            Nx.to_binary(bad)
        assert e.value.status == L.ERAISED and "index 10 is out of bounds" in str(e.value)
        B.sync()  # re-armed
    finally:
        B.bounds_policy(previous)
    with pytest.raises(L.HipNxArgumentError) as e:  # the default policy raises from the call itself
        Nx.take(table, from_numpy(np.array([1, 10, 2], dtype=np.int32), "s32", hip))
    assert e.value.status == L.EINDEX and "index 10 is out of bounds for axis 0 in shape {10, 4}" in str(e.value)


@pytest.mark.parametrize("ty", ["f32", "f64", "bf16"])
def test_reduce_max_min_over_signed_zeros_may_keep_the_other_zero(ty, hip, oracle):
    """Among equal extremes the reference keeps the one it met first (Kernel.max / min); the device's tree
    reduction selects by value only, so of +0.0 and -0.0 it may return the other one.  Stated here: the
    results are equal as numbers and differ at most in the sign of a zero."""
    x = np.array([[0.0, -0.0, -1.0], [-0.0, 0.0, -2.0], [-0.0, -0.0, -3.0], [0.0, 0.0, 1.0]], dtype=np.float64)
    from support import values
    from test_gpu_elementwise import both
    src = x.astype(np.float32) if ty != "f64" else x
    if ty == "bf16":
        src = (src.view(np.uint32) >> 16).astype(np.uint16)
    h, o = both(src, ty, hip, oracle)
    for op in (Nx.reduce_max, Nx.reduce_min):
        got, want = values(op(h, axes=[1])), values(op(o, axes=[1]))
        assert np.array_equal(got, want)  # -0.0 == 0.0 as numbers
        same_sign = np.signbit(got) == np.signbit(want)
        assert same_sign[~((got == 0) & (want == 0))].all()  # only a zero may differ in sign
