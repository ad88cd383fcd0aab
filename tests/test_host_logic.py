"""Host-side front end: type inference, shape inference and dispatch, checked against the values
the reference's own doctests state (nx/lib/nx/type.ex, nx/lib/nx/shape.ex)."""
import numpy as np
import pytest

from nx_amd import HostBinary, nx as Nx
from nx_amd import shape as S
from nx_amd import types as T
from nx_amd.tensor import list_to_binary, number_to_binary


def test_merge_follows_type_ex_doctests():  # nx/lib/nx/type.ex:405-461
    assert T.merge(("s", 8), ("s", 8)) == ("s", 8)
    assert T.merge(("s", 8), ("s", 64)) == ("s", 64)
    assert T.merge(("s", 8), ("u", 8)) == ("s", 16)
    assert T.merge(("s", 16), ("u", 8)) == ("s", 16)
    assert T.merge(("s", 8), ("u", 16)) == ("s", 32)
    assert T.merge(("s", 32), ("u", 8)) == ("s", 32)
    assert T.merge(("s", 8), ("u", 32)) == ("s", 64)
    assert T.merge(("s", 8), ("u", 64)) == ("s", 64)
    assert T.merge(("s", 8), ("bf", 16)) == ("bf", 16)
    assert T.merge(("s", 64), ("bf", 16)) == ("bf", 16)
    assert T.merge(("f", 32), ("bf", 16)) == ("f", 32)
    assert T.merge(("f", 64), ("bf", 16)) == ("f", 64)
    assert T.merge(("f", 16), ("bf", 16)) == ("f", 16)
    assert T.merge(("u", 64), ("f", 16)) == ("f", 16)


def test_merge_number_follows_type_ex_doctests():  # nx/lib/nx/type.ex:496-534
    assert T.merge_number(("u", 8), 0) == ("u", 8)
    assert T.merge_number(("u", 8), 255) == ("u", 8)
    assert T.merge_number(("u", 8), 256) == ("u", 16)
    assert T.merge_number(("u", 8), -1) == ("s", 16)
    assert T.merge_number(("u", 8), -32768) == ("s", 16)
    assert T.merge_number(("u", 8), -32769) == ("s", 32)
    assert T.merge_number(("s", 8), 127) == ("s", 8)
    assert T.merge_number(("s", 8), 128) == ("s", 16)
    assert T.merge_number(("s", 8), -129) == ("s", 16)
    assert T.merge_number(("s", 8), 1.0) == ("f", 32)
    assert T.merge_number(("u", 64), -1337) == ("s", 64)
    assert T.merge_number(("f", 32), 1) == ("f", 32)
    assert T.merge_number(("f", 64), 1.0) == ("f", 64)
    assert T.merge_number(("bf", 16), 3) == ("bf", 16)


def test_to_floating_and_to_aggregate():  # nx/lib/nx/type.ex:236-257, 310-333
    assert T.to_floating(("s", 8)) == ("f", 32) and T.to_floating(("bf", 16)) == ("bf", 16)
    assert T.to_floating(("u", 64)) == ("f", 32) and T.to_floating(("f", 64)) == ("f", 64)
    assert T.to_aggregate(("s", 8)) == ("s", 32) and T.to_aggregate(("u", 16)) == ("u", 32)
    assert T.to_aggregate(("u", 64)) == ("s", 64) and T.to_aggregate(("s", 64)) == ("s", 64)
    assert T.to_aggregate(("bf", 16)) == ("bf", 16) and T.to_aggregate(("f", 32)) == ("f", 32)


def test_binary_broadcast():  # nx/lib/nx/shape.ex:286-376
    assert S.binary_broadcast((3, 1), (1, 4)) == (3, 4)
    assert S.binary_broadcast((8, 1, 6, 1), (7, 1, 5)) == (8, 7, 6, 5)
    assert S.binary_broadcast((), (2, 2)) == (2, 2)
    with pytest.raises(ValueError, match="cannot broadcast tensor of dimensions \\{2, 2\\} to \\{2, 3\\}"):
        S.binary_broadcast((2, 2), (2, 3))
    assert S.broadcast_strides((3, 1), (2, 3, 4)) == [0, 1, 0]
    assert S.broadcast_strides((4,), (3, 4)) == [0, 1]
    assert S.broadcast_strides((), (3, 4)) == [0, 0]
    assert S.broadcast_strides((2, 3), (2, 3)) == [3, 1]


def test_contract_dot_take_gather_shapes():
    assert S.contract((4, 1, 2), [1], False) == (4, 2)  # nx/lib/nx/shape.ex:399-411
    assert S.contract((2, 4, 6, 5), [1, 3], False) == (2, 6)
    assert S.contract((2, 4, 6, 5), [1, 3], True) == (2, 1, 6, 1)
    assert S.dot((2, 7, 8, 3, 1), [3, 1, 2], [], (1, 8, 3, 7, 3), [2, 3, 1], []) == (2, 1, 1, 3)
    assert S.dot((32, 512, 64), [2], [0], (32, 512, 64), [2], [0]) == (32, 512, 512)
    assert S.dot((3, 2, 1, 3, 2), [2], [0, 1], (3, 2, 1, 1, 4), [3], [0, 1]) == (3, 2, 3, 2, 1, 4)
    with pytest.raises(ValueError, match="right tensor must be batched"):
        S.dot((2, 3), [1], [0], (3, 2), [0], [])
    with pytest.raises(ValueError, match="successive dimensions starting from 0"):
        S.dot((2, 3, 4), [2], [1], (2, 4, 3), [1], [0])
    with pytest.raises(ValueError, match="does not equal"):
        S.dot((2, 3), [1], [], (4, 2), [0], [])
    assert S.take((32000, 4096), (8192,), 0) == (8192, 4096)
    assert S.take((2, 2), (3, 2), 1) == (2, 3, 2)
    assert S.gather((32000, 4096), (8192, 1), [0]) == (8192, 4096)
    assert S.gather((2, 2), (3, 2), [0, 1]) == (3,)
    assert S.normalize_axis((4, 5), -1) == 1
    with pytest.raises(ValueError):
        S.normalize_axis((4, 5), 2)
    with pytest.raises(ValueError):
        S.normalize_axes((4, 5), [0, 0])


def test_number_encoding_follows_the_reference_write_path():
    # bf16 truncates (nx/lib/nx/floating.ex:60-64): 1/5 -> 0x3E4C = 0.19921875
    assert number_to_binary(0.2, "bf16") == (0x3E4C).to_bytes(2, "little")
    # canonical non-finites (nx/lib/nx/type.ex:128-158)
    assert number_to_binary(float("nan"), "f32") == (0x7FC00000).to_bytes(4, "little")
    assert number_to_binary(float("nan"), "bf16") == (0x7FC0).to_bytes(2, "little")
    assert number_to_binary(float("inf"), "bf16") == (0x7F80).to_bytes(2, "little")
    assert number_to_binary(float("-inf"), "f16") == (0xFC00).to_bytes(2, "little")
    assert number_to_binary(-0.0, "bf16") == (0x8000).to_bytes(2, "little")
    # integers wrap (nx/lib/nx/shared.ex:190-194)
    assert number_to_binary(300, "u8") == bytes([44]) and number_to_binary(-1, "u16") == b"\xff\xff"
    assert list_to_binary([1, 2, 3], "s16") == np.array([1, 2, 3], dtype=np.int16).tobytes()
    with pytest.raises(OverflowError):
        number_to_binary(1e39, "f32")


def test_front_end_templates_and_dispatch():
    t = Nx.tensor([[1, 2], [3, 4]])
    assert t.type == ("s", 32) and t.shape == (2, 2) and isinstance(t.data, HostBinary)
    assert Nx.tensor([1.0, 2.0]).type == ("f", 32)
    assert Nx.tensor([1, 2], type="bf16").type == ("bf", 16)
    assert Nx.to_binary(Nx.tensor([1, 2, 3]), limit=2) == np.array([1, 2], dtype=np.int32).tobytes()
    assert Nx.reshape(t, (4,)).shape == (4,) and Nx.reshape(t, ("auto", 1)).shape == (4, 1)
    assert Nx.as_type(t, "s32") is t and Nx.transpose(t, [0, 1]) is t
    with pytest.raises(NotImplementedError):  # the host holder stores, a compute backend computes
        Nx.add(t, 1)
    with pytest.raises(ValueError, match="cannot broadcast"):
        Nx.add(Nx.tensor([[1, 2], [3, 4]]), Nx.tensor([[1, 2, 3], [4, 5, 6]]))
    with pytest.raises(ValueError, match="integer tensors"):
        Nx.bitwise_and(Nx.tensor([1.0]), Nx.tensor([1.0]))
    with pytest.raises(ValueError, match="tie_break"):
        Nx.argmax(t, tie_break="middle")
    assert Nx.default_backend()[0] is HostBinary


def test_front_end_runs_unchanged_on_the_oracle_backend(oracle):
    """The same calls, another backend: the drop-in property the device backend relies on."""
    t = Nx.tensor([[1, 2], [3, 4]], backend=oracle)
    assert Nx.to_flat_list(Nx.add(t, 1)) == [2, 3, 4, 5]
    assert Nx.multiply(t, 0.5).type == ("f", 32) and Nx.divide(t, 2).type == ("f", 32)
    assert Nx.sum(Nx.as_type(t, "s8")).type == ("s", 32) and Nx.equal(t, 2).type == ("u", 8)
    assert Nx.to_flat_list(Nx.take(t, Nx.tensor([1, 0, 1], backend=oracle), axis=1)) == [2, 1, 2, 4, 3, 4]
    assert Nx.dot(Nx.as_type(t, "s8"), Nx.as_type(t, "s8")).type == ("s", 8)
    assert Nx.argmax(t, axis=0, type="u32").type == ("u", 32)
    assert Nx.exp(t).type == ("f", 32) and Nx.exp(Nx.as_type(t, "bf16")).type == ("bf", 16)


def test_to_batched_known_answers_on_the_host_backend_and_the_oracle(oracle):
    from nx_amd.host import HostBinary
    from to_batched_support import check_counts, check_known_answers
    for backend in (HostBinary, oracle):
        check_known_answers(backend)
        check_counts(backend)


def test_pad_merges_its_type_before_the_number_becomes_a_tensor(oracle):
    """nx.ex:4237-4238: binary_type(tensor, pad_value) sees the number, so a bf16 tensor padded with 0.0 stays
    bf16 and an s32 tensor padded with 0 stays s32."""
    Nx.default_backend(oracle)
    bf = Nx.as_type(Nx.tensor([1.0, 2.0]), "bf16")
    assert Nx.pad(bf, 0.0, [(1, 1, 0)]).type == ("bf", 16)
    assert Nx.pad(Nx.tensor([1, 2]), 0, [(1, 1, 0)]).type == ("s", 32)
    assert Nx.to_flat_list(Nx.pad(bf, 0.0, [(1, 2, 0)])) == [0.0, 1.0, 2.0, 0.0, 0.0]
