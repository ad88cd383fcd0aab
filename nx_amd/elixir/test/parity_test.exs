# Cross-backend parity in the shape of torchx/test/torchx/nx_test.exs:25-118: every op over a sweep of
# type pairs on HipNx and on Nx.BinaryBackend, both brought to the host and compared; operands that
# live on different backends; broadcasting scalars and columns on either side.
defmodule HipNx.ParityTest do
  use ExUnit.Case, async: false

  @types [{:s, 8}, {:u, 8}, {:s, 16}, {:u, 16}, {:s, 32}, {:u, 32}, {:s, 64}, {:u, 64}, {:bf, 16}, {:f, 16}, {:f, 32}, {:f, 64}]
  @ints [{:s, 8}, {:u, 8}, {:s, 16}, {:u, 16}, {:s, 32}, {:u, 32}, {:s, 64}, {:u, 64}]
  @ops [:add, :subtract, :multiply, :divide, :pow, :remainder, :atan2, :max, :min]
  @compare [:equal, :not_equal, :greater, :less, :greater_equal, :less_equal]
  @logical [:logical_and, :logical_or, :logical_xor]
  @bitwise [:bitwise_and, :bitwise_or, :bitwise_xor, :left_shift, :right_shift, :quotient]
  @unary [:abs, :ceil, :floor, :negate, :round, :sign, :exp, :log1p, :sigmoid, :tanh, :sqrt, :erf]
  @hip {HipNx.Backend, device: 0}

  defp host(t), do: Nx.backend_copy(t, Nx.BinaryBackend)

  defp close?(hip, ref) do
    case Nx.type(ref) do
      {kind, _} when kind in [:s, :u] -> Nx.to_binary(host(hip)) == Nx.to_binary(ref)
      {_, 16} -> Nx.all_close(host(hip), ref, rtol: 1.0e-2, atol: 1.0e-3, equal_nan: true) == Nx.tensor(1, type: :u8)
      _ -> Nx.all_close(host(hip), ref, rtol: 1.0e-5, atol: 1.0e-6, equal_nan: true) == Nx.tensor(1, type: :u8)
    end
  end

  defp check_binary(op, data_a \\ [[5, 6], [7, 8]], data_b \\ [[1, 2], [3, 4]], type_a, type_b) do
    a = Nx.tensor(data_a, type: type_a, backend: @hip)
    b = Nx.tensor(data_b, type: type_b, backend: @hip)
    ref = apply(Nx, op, [host(a), host(b)])
    assert close?(apply(Nx, op, [a, b]), ref)
    # one operand on the host backend: it is copied in on entry
    assert close?(apply(Nx, op, [a, host(b)]), ref)
    assert close?(apply(Nx, op, [host(a), b]), ref)
  end

  describe "binary ops" do
    for op <- @ops ++ @compare ++ @logical, type_a <- @types, type_b <- @types do
      test "#{op}(#{Nx.Type.to_string(type_a)}, #{Nx.Type.to_string(type_b)})" do
        check_binary(unquote(op), unquote(Macro.escape(type_a)), unquote(Macro.escape(type_b)))
      end
    end

    for op <- @ops ++ @compare ++ @logical, type <- @types do
      test "#{op}(#{Nx.Type.to_string(type)}) broadcasts scalars and columns on either side" do
        op = unquote(op)
        type = unquote(Macro.escape(type))
        check_binary(op, 1, [1, 2, 3], type, type)
        check_binary(op, [1, 2, 3], 1, type, type)
        check_binary(op, [[1], [2]], [[1, 2, 3], [4, 5, 6]], type, type)
        check_binary(op, [[1, 2, 3], [4, 5, 6]], [[1], [2]], type, type)
      end
    end

    for op <- @bitwise, type_a <- @ints, type_b <- @ints do
      test "#{op}(#{Nx.Type.to_string(type_a)}, #{Nx.Type.to_string(type_b)})" do
        check_binary(unquote(op), unquote(Macro.escape(type_a)), unquote(Macro.escape(type_b)))
      end
    end

    test "remainder with u64 operands beyond the signed range" do
      a = Nx.tensor([9_223_372_036_854_775_808, 18_446_744_073_709_551_321], type: :u64, backend: @hip)
      assert Nx.to_flat_list(Nx.remainder(a, Nx.tensor(10, type: :u64, backend: @hip))) == [8, 1]
    end
  end

  describe "unary ops and conversions" do
    for op <- @unary, type <- @types do
      test "#{op}(#{Nx.Type.to_string(type)})" do
        t = Nx.tensor([[1, 2], [3, 4]], type: unquote(Macro.escape(type)), backend: @hip)
        assert close?(apply(Nx, unquote(op), [t]), apply(Nx, unquote(op), [host(t)]))
      end
    end

    for from <- @types, to <- @types do
      test "as_type #{Nx.Type.to_string(from)} -> #{Nx.Type.to_string(to)}" do
        t = Nx.tensor([0, 1, 2, 100, 127], type: unquote(Macro.escape(from)), backend: @hip)
        assert Nx.to_binary(host(Nx.as_type(t, unquote(Macro.escape(to))))) == Nx.to_binary(Nx.as_type(host(t), unquote(Macro.escape(to))))
      end
    end
  end

  describe "reductions, dot and indexing" do
    for type <- @types do
      test "sum / reduce_max / argmax over each axis (#{Nx.Type.to_string(type)})" do
        t = Nx.tensor([[3, 1, 4, 1], [5, 9, 2, 6], [5, 3, 5, 8]], type: unquote(Macro.escape(type)), backend: @hip)
        for axis <- [0, 1] do
          assert close?(Nx.sum(t, axes: [axis]), Nx.sum(host(t), axes: [axis]))
          assert close?(Nx.reduce_max(t, axes: [axis]), Nx.reduce_max(host(t), axes: [axis]))
          # ties: the first index for :low, the last for :high
          assert Nx.to_binary(host(Nx.argmax(t, axis: axis))) == Nx.to_binary(Nx.argmax(host(t), axis: axis))
          assert Nx.to_binary(host(Nx.argmax(t, axis: axis, tie_break: :high))) == Nx.to_binary(Nx.argmax(host(t), axis: axis, tie_break: :high))
        end
      end
    end

    test "dot with contraction and batch axes" do
      key = Nx.Random.key(7)
      {x, key} = Nx.Random.uniform(key, -1.0, 1.0, shape: {4, 64, 128})
      {y, _} = Nx.Random.uniform(key, -1.0, 1.0, shape: {4, 32, 128})
      hip = Nx.dot(Nx.backend_copy(x, @hip), [2], [0], Nx.backend_copy(y, @hip), [2], [0])
      assert Nx.all_close(host(hip), Nx.dot(x, [2], [0], y, [2], [0]), rtol: 1.0e-4, atol: 1.0e-5) == Nx.tensor(1, type: :u8)
      a = Nx.iota({64, 256}, type: :s8)
      assert Nx.to_binary(host(Nx.dot(Nx.backend_copy(a, @hip), [1], Nx.backend_copy(a, @hip), [1]))) == Nx.to_binary(Nx.dot(a, [1], a, [1]))
    end

    test "take, gather and their bounds" do
      t = Nx.iota({7, 9}, type: :s32, backend: @hip)
      assert Nx.to_binary(host(Nx.take(t, Nx.tensor([6, 0, 6, 3])))) == Nx.to_binary(Nx.take(host(t), Nx.tensor([6, 0, 6, 3])))
      assert_raise ArgumentError, ~r/index 7 is out of bounds for axis 0 in shape \{7, 9\}/, fn ->
        Nx.take(t, Nx.tensor([1, 7]))
      end
    end
  end

  describe "what the reference raises for" do
    test "integer division by zero is raised when the result is read" do
      q = Nx.quotient(Nx.tensor([1, 2], backend: @hip), Nx.tensor([1, 0], backend: @hip))
      assert_raise ArithmeticError, ~r/bad argument in arithmetic expression/, fn -> Nx.to_binary(q) end
    end

    test "a negative shift count" do
      s = Nx.left_shift(Nx.tensor([1, 2], backend: @hip), Nx.tensor([1, -1], backend: @hip))
      assert_raise ArgumentError, ~r/cannot left shift by -1/, fn -> Nx.to_binary(s) end
    end
  end

  describe "bf16 encodings" do
    # torchx/test/torchx/nx_test.exs:380-394 expects the nearest value; Nx.BinaryBackend truncates
    test "1/5 truncates by default and rounds to nearest even on request" do
      t = Nx.tensor([0.2], type: :f32, backend: @hip)
      assert Nx.to_binary(Nx.as_type(t, :bf16)) == <<0x3E4C::16-native>>
      Application.put_env(:hipnx, :bf16_rounding, :nearest_even)

      try do
        assert Nx.to_binary(Nx.as_type(t, :bf16)) == <<0x3E4D::16-native>>
      after
        Application.delete_env(:hipnx, :bf16_rounding)
      end
    end
  end

  describe "plumbing" do
    test "deallocation is idempotent" do
      t = Nx.tensor([1, 2, 3], backend: @hip)
      assert Nx.backend_deallocate(t) == :ok
      assert Nx.backend_deallocate(t) == :already_deallocated
    end

    test "local pointers share the buffer" do
      t = Nx.tensor([1.0, 2.0, 3.0], backend: @hip)
      p = Nx.to_pointer(t, mode: :local)
      assert %Nx.Pointer{kind: :local, data_size: 12} = p
      alias_t = Nx.from_pointer(@hip, p, {:f, 32}, {3})
      assert Nx.to_binary(alias_t) == Nx.to_binary(t)
    end

    test "an ipc pointer carries the 64-byte handle and the device index" do
      t = Nx.tensor([1.0, 2.0, 3.0], backend: @hip)
      assert %Nx.Pointer{kind: :ipc, address: 0, data_size: 12, handle: <<_::binary-size(64)>>} = Nx.to_pointer(t, mode: :ipc)
    end
  end
end
