# Cross-backend parity in the style of torchx/test/torchx/nx_test.exs:25-50: run the op on
# HipNx and on Nx.BinaryBackend, bring both to the host and compare.
defmodule HipNx.ParityTest do
  use ExUnit.Case, async: true

  defp on_both(fun, args) do
    hip = apply(fun, Enum.map(args, &Nx.backend_copy(&1, {HipNx.Backend, device: 0})))
    ref = apply(fun, Enum.map(args, &Nx.backend_copy(&1, Nx.BinaryBackend)))
    {Nx.backend_transfer(hip, Nx.BinaryBackend), ref}
  end

  test "integer ops and indexing are bit-exact" do
    a = Nx.iota({7, 9}, type: :s32)
    b = Nx.tensor([3, -2, 5, 1, 1, 1, 2, 2, 9], type: :s32)
    for fun <- [&Nx.add/2, &Nx.multiply/2, &Nx.remainder/2, &Nx.bitwise_xor/2, &Nx.greater/2] do
      {hip, ref} = on_both(fun, [a, b])
      assert Nx.to_binary(hip) == Nx.to_binary(ref)
    end
    {hip, ref} = on_both(&Nx.argmax(&1, axis: 1, type: :u32), [Nx.remainder(a, 4)])
    assert Nx.to_binary(hip) == Nx.to_binary(ref)
    {hip, ref} = on_both(&Nx.take(&1, &2), [a, Nx.tensor([6, 0, 6, 3])])
    assert Nx.to_binary(hip) == Nx.to_binary(ref)
  end

  test "float element-wise and dot stay within tolerance" do
    key = Nx.Random.key(7)
    {x, key} = Nx.Random.uniform(key, -1.0, 1.0, shape: {64, 128})
    {y, _} = Nx.Random.uniform(key, -1.0, 1.0, shape: {128, 32})
    {hip, ref} = on_both(&Nx.exp/1, [x])
    assert Nx.all_close(hip, ref, rtol: 1.0e-5) == Nx.tensor(1, type: :u8)
    {hip, ref} = on_both(&Nx.dot/2, [x, y])
    assert Nx.all_close(hip, ref, rtol: 1.0e-4, atol: 1.0e-5) == Nx.tensor(1, type: :u8)
  end

  test "deallocation is idempotent" do
    t = Nx.tensor([1, 2, 3], backend: {HipNx.Backend, device: 0})
    assert Nx.backend_deallocate(t) == :ok
    assert Nx.backend_deallocate(t) == :already_deallocated
  end
end
