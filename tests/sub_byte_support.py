"""Shared checks for the sub-byte integer types (u2, u4, s2, s4) on any backend."""
import json
import os

import numpy as np

from nx_amd import nx as Nx

with open(os.path.join(os.path.dirname(__file__), "golden", "nx_sub_byte_known_answers.json")) as f:
    CASES = json.load(f)["cases"]

SUB_TYPES = ["u2", "u4", "s2", "s4"]


def value_range(ty):
    bits = int(ty[1:])
    return (0, (1 << bits) - 1) if ty[0] == "u" else (-(1 << (bits - 1)), (1 << (bits - 1)) - 1)


def low_bits(values, ty):
    """What the mathematics fixes: the low `bits` bits of an unbounded integer, read as the type."""
    bits = int(ty[1:])
    v = np.asarray(values, dtype=np.int64) & ((1 << bits) - 1)
    if ty[0] == "s":
        v = np.where(v >= (1 << (bits - 1)), v - (1 << bits), v)
    return v


def check_case(case, backend):
    t = Nx.tensor(case["values"], type=case["type"], backend=backend)
    assert t.type == (case["type"][0], int(case["type"][1:]))
    flat = case["values"] if isinstance(case["values"], list) else [case["values"]]
    assert Nx.to_flat_list(t) == flat, case["ref"]
    if "binary_hex" in case:
        assert Nx.to_binary(t).hex() == case["binary_hex"], case["ref"]
    if "byte_size" in case:
        assert Nx.byte_size(t) == case["byte_size"] and Nx.bit_size(t) == case["bit_size"], case["ref"]
    if case.get("round_trip"):
        back = Nx.from_binary(Nx.to_binary(t), case["type"], backend=backend, count=len(flat))
        assert back.type == t.type and back.shape == t.shape and Nx.to_flat_list(back) == flat, case["ref"]
    for piece in case.get("inspect_has", []):
        assert piece in type(t.data).inspect(t), case["ref"]
