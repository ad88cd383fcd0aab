defmodule HipNx.Backend do
  @moduledoc """
  An `Nx.Backend` for one AMD Instinct MI355X over `libhipnx` (hand-written gfx950 kernels).

      Nx.default_backend({HipNx.Backend, device: 0})

  Native callbacks: the element-wise binary and unary ops, `as_type`, `sum`, `product`,
  `reduce_max`, `reduce_min`, `argmax`, `argmin`, `dot`, `gather`, `take` (through
  `Nx.Block.Take`), `transpose`, `broadcast`, and the plumbing (`from_binary`, `to_binary`,
  `constant`, transfers, `reshape`/`squeeze`/`bitcast`, `inspect`).  Every other callback of the
  behaviour runs on `Nx.BinaryBackend` after a device-to-host copy and comes back with
  `from_binary` -- the same escape hatch `EXLA.Backend` uses for `concatenate`/`stack`.

  Results follow `Nx.BinaryBackend`: integers, indices and argmax bit-exact; `+ - * /`, comparisons,
  `as_type` and selections bit-exact for floats too; libm-class functions within 1 ulp of the output
  type; `dot` and `sum` over floats within the bound of an f32 accumulation of the same terms.

  This module cannot be compiled in the repository's build container (no BEAM); its Python twin
  `nx_amd/backend.py` exercises the same C ABI with the same lowering and is what the test-suite
  runs.
  """
  @behaviour Nx.Backend

  @enforce_keys [:ref, :device]
  defstruct [:ref, :device]

  alias Nx.Tensor, as: T
  alias HipNx.NIF

  @binary_ops ~w(add subtract multiply divide pow remainder atan2 min max quotient bitwise_and
                 bitwise_or bitwise_xor left_shift right_shift equal not_equal greater less
                 greater_equal less_equal logical_and logical_or logical_xor)a
  @unary_ops ~w(exp expm1 log log1p sigmoid cos sin tan cosh sinh tanh acos asin atan acosh asinh
                atanh sqrt rsqrt cbrt erf erfc erf_inv abs bitwise_not ceil floor negate round sign
                count_leading_zeros population_count is_nan is_infinity)a
  @dtypes %{{:u, 8} => 0, {:u, 16} => 1, {:u, 32} => 2, {:u, 64} => 3, {:s, 8} => 4, {:s, 16} => 5,
            {:s, 32} => 6, {:s, 64} => 7, {:f, 16} => 8, {:bf, 16} => 9, {:f, 32} => 10, {:f, 64} => 11,
            # sub-byte integers live one per byte on the device, as in EXLA.DeviceBuffer: kernels see s8 / u8
            {:u, 2} => 0, {:u, 4} => 0, {:s, 2} => 4, {:s, 4} => 4}

  ## Options and context

  @impl true
  def init(opts), do: Keyword.validate!(opts, device: 0)

  defp ctx(device) do
    key = {__MODULE__, :ctx, device}

    case :persistent_term.get(key, nil) do
      nil ->
        ctx = unwrap!(NIF.ctx_create(device))
        :persistent_term.put(key, ctx)
        ctx

      ctx ->
        ctx
    end
  end

  defp unwrap!({:ok, value}), do: value
  defp unwrap!({:error, {status, msg}}) when status in [2, 6], do: raise(ArgumentError, List.to_string(msg))

  # HIPNX_ERAISED: what a kernel issued earlier met (the reference raises for it at once; a device
  # cannot, so the next call that waits for the device -- to_binary, inspect, backend_copy -- does)
  defp unwrap!({:error, {8, msg}}) do
    case List.to_string(msg) do
      "ArithmeticError: " <> rest -> raise(ArithmeticError, rest)
      "ArgumentError: " <> rest -> raise(ArgumentError, rest)
      other -> raise(RuntimeError, "HipNx: " <> other)
    end
  end
  defp unwrap!({:error, {_status, msg}}), do: raise(RuntimeError, "HipNx: " <> List.to_string(msg))

  defp dt(type), do: Map.get(@dtypes, type) || raise(ArgumentError, "HipNx does not support type #{inspect(type)}")

  # The result type of as_type and dot.  `config :hipnx, bf16_rounding: :nearest_even` encodes bf16 results
  # as Torchx and EXLA do (HIPNX_BF16_RNE = 12); the default truncates as Nx.BinaryBackend does.
  defp out_dt({:bf, 16}) do
    if Application.get_env(:hipnx, :bf16_rounding, :truncate) == :nearest_even, do: 12, else: dt({:bf, 16})
  end

  defp out_dt(type), do: dt(type)
  defp bytes(%T{type: {_, bits}, shape: shape}), do: max(div(bits, 8), 1) * Nx.size(shape)

  # a result of a sub-byte type was computed at 8 bits: keep its low bits (Nx.Shared's `<<x::size(bits)>>`)
  defp to_nx(ref, device, %T{type: {kind, bits}} = out) when bits < 8 do
    ref = unwrap!(NIF.narrow_int(ctx(device), ref, Nx.size(out), bits, if(kind == :s, do: 1, else: 0)))
    %{out | data: %__MODULE__{ref: ref, device: device}}
  end

  defp to_nx(ref, device, %T{} = out), do: %{out | data: %__MODULE__{ref: ref, device: device}}

  # operands living on another backend are copied in on entry (cf. Torchx.Backend.from_nx/1)
  defp from_nx(%T{data: %__MODULE__{ref: ref, device: device}}, _), do: {ref, device}

  defp from_nx(%T{} = t, device) do
    %T{data: %__MODULE__{ref: ref}} = Nx.backend_transfer(t, {__MODULE__, device: device})
    {ref, device}
  end

  defp device_of(tensors) do
    Enum.find_value(tensors, 0, fn
      %T{data: %__MODULE__{device: d}} -> d
      _ -> nil
    end)
  end

  ## Creation and transfer

  @impl true
  def from_binary(%T{} = out, binary, opts) do
    device = init(opts)[:device]
    to_nx(unwrap!(NIF.from_binary(ctx(device), unpack(binary, out.type), bytes(out))), device, out)
  end

  # packed bitstring <-> one element per byte (cf. EXLA.DeviceBuffer.place_on_device/4 and read/2)
  defp unpack(data, {:u, size}) when size in [2, 4],
    do: for(<<x::native-size(size) <- data>>, into: <<>>, do: <<x::native-8>>)

  defp unpack(data, {:s, size}) when size in [2, 4],
    do: for(<<x::native-signed-size(size) <- data>>, into: <<>>, do: <<x::native-signed-8>>)

  defp unpack(data, _type), do: IO.iodata_to_binary(data)

  defp pack(data, {:u, size}) when size in [2, 4],
    do: for(<<x::native-8 <- data>>, into: <<>>, do: <<x::native-size(size)>>)

  defp pack(data, {:s, size}) when size in [2, 4],
    do: for(<<x::native-signed-8 <- data>>, into: <<>>, do: <<x::native-signed-size(size)>>)

  defp pack(data, _type), do: data

  @impl true
  def to_binary(%T{data: %__MODULE__{ref: ref, device: device}, type: {_, bits}} = t, limit) do
    n = min(limit, Nx.size(t))
    pack(unwrap!(NIF.to_binary(ctx(device), ref, n * max(div(bits, 8), 1))), t.type)
  end

  @impl true
  def constant(%T{type: type} = out, number, opts) do
    device = init(opts)[:device]
    %T{data: %Nx.BinaryBackend{state: elem}} = Nx.BinaryBackend.constant(%{out | shape: {}, names: []}, number, [])
    to_nx(unwrap!(NIF.fill(ctx(device), unpack(elem, type), Nx.size(out))), device, out)
  end

  @impl true
  def backend_copy(%T{data: %__MODULE__{ref: ref, device: device}} = t, __MODULE__, opts) do
    if init(opts)[:device] == device do
      to_nx(unwrap!(NIF.copy(ctx(device), ref, bytes(t))), device, t)
    else
      from_binary(t, to_binary(t, Nx.size(t)), opts)
    end
  end

  def backend_copy(t, backend, opts), do: backend.from_binary(t, to_binary(t, Nx.size(t)), opts)

  @impl true
  def backend_transfer(%T{data: %__MODULE__{device: device}} = t, __MODULE__, opts) do
    if init(opts)[:device] == device do
      t
    else
      copy = backend_copy(t, __MODULE__, opts)
      backend_deallocate(t)
      copy
    end
  end

  def backend_transfer(t, backend, opts) do
    copy = backend_copy(t, backend, opts)
    backend_deallocate(t)
    copy
  end

  @impl true
  def backend_deallocate(%T{data: %__MODULE__{ref: ref}}) do
    case NIF.deallocate(ref) do
      :ok -> :ok
      :already_deallocated -> :already_deallocated
      other -> unwrap!(other)
    end
  end

  @impl true
  def inspect(%T{} = t, inspect_opts) do
    limit = if inspect_opts.limit == :infinity, do: :infinity, else: inspect_opts.limit + 1
    t |> to_binary(min(limit, Nx.size(t))) |> then(&Nx.Backend.inspect(t, &1, inspect_opts))
  end

  ## Metadata-only callbacks: buffers are immutable, so the handle is shared

  @impl true
  def reshape(out, %T{} = t), do: share(out, t)
  @impl true
  def squeeze(out, %T{} = t, _axes), do: share(out, t)
  @impl true
  def bitcast(out, %T{} = t), do: share(out, t)

  defp share(out, t) do
    device = device_of([t])
    {ref, _} = from_nx(t, device)
    # a second owner of the same device memory: copy on the device keeps deallocation simple
    to_nx(unwrap!(NIF.copy(ctx(device), ref, bytes(out))), device, out)
  end

  ## Element-wise

  for {op, code} <- Enum.with_index(@binary_ops) do
    @impl true
    def unquote(op)(out, l, r), do: binary(unquote(code), out, l, r)
  end

  defp binary(code, %T{shape: shape} = out, %T{} = l, %T{} = r) do
    device = device_of([l, r])
    {lref, _} = from_nx(l, device)
    {rref, _} = from_nx(r, device)
    dims = Tuple.to_list(shape)

    ref =
      NIF.binary(ctx(device), code, dt(l.type), dt(r.type), dt(out.type), dims,
        broadcast_strides(l.shape, shape), broadcast_strides(r.shape, shape), lref, rref, bytes(out))

    to_nx(unwrap!(ref), device, out)
  end

  # element strides of `shape` viewed in `out_shape` (right-aligned), 0 on broadcast axes
  defp broadcast_strides(shape, out_shape) do
    rank = tuple_size(out_shape)
    padded = List.duplicate(1, rank - tuple_size(shape)) ++ Tuple.to_list(shape)

    {strides, _} =
      padded
      |> Enum.reverse()
      |> Enum.map_reduce(1, fn dim, acc -> {if(dim == 1, do: 0, else: acc), acc * dim} end)

    Enum.reverse(strides)
  end

  for {op, code} <- Enum.with_index(@unary_ops) do
    @impl true
    def unquote(op)(out, t), do: unary(unquote(code), out, t)
  end

  defp unary(code, out, %T{} = t) do
    device = device_of([t])
    {ref, _} = from_nx(t, device)
    to_nx(unwrap!(NIF.unary(ctx(device), code, dt(t.type), dt(out.type), Nx.size(out), ref, bytes(out))), device, out)
  end

  @impl true
  def as_type(%T{type: type}, %T{type: type} = t), do: t
  def as_type(out, %T{} = t) do
    device = device_of([t])
    {ref, _} = from_nx(t, device)
    to_nx(unwrap!(NIF.unary(ctx(device), -1, dt(t.type), out_dt(out.type), Nx.size(out), ref, bytes(out))), device, out)
  end

  ## Reductions

  @impl true
  def sum(out, t, opts), do: reduce_op(0, out, t, opts)
  @impl true
  def reduce_max(out, t, opts), do: reduce_op(1, out, t, opts)
  @impl true
  def reduce_min(out, t, opts), do: reduce_op(2, out, t, opts)
  @impl true
  def product(out, t, opts), do: reduce_op(3, out, t, opts)
  @impl true
  def all(out, t, opts), do: reduce_op(4, out, t, opts)
  @impl true
  def any(out, t, opts), do: reduce_op(5, out, t, opts)

  defp reduce_op(code, out, %T{} = t, opts) do
    device = device_of([t])

    # (sub-byte integers keep the single pass: their intermediates would have to be packed and unpacked)
    case if(elem(t.type, 1) >= 8, do: axis_runs(opts[:axes]), else: []) do
      [_, _ | _] = runs ->
        # reduced axes that are not neighbours: one pass per run of neighbouring axes, innermost run first,
        # instead of a transposed copy; sums and products pass through f64 / 64-bit integers (the
        # accumulators' own types), so the result is still rounded or wrapped once
        mid =
          cond do
            code not in [0, 3] -> out.type
            Nx.Type.float?(out.type) -> {:f, 64}
            true -> {elem(out.type, 0), 64}
          end

        last_run = hd(runs)

        runs
        |> Enum.reverse()
        |> Enum.reduce(t, fn run, cur ->
          dims = Tuple.to_list(cur.shape)
          first = hd(run)
          last = List.last(run)
          shape = List.to_tuple(Enum.take(dims, first) ++ Enum.drop(dims, last + 1))
          step = if run == last_run, do: out, else: %{out | type: mid, shape: shape, names: List.duplicate(nil, tuple_size(shape))}
          {ref, _} = from_nx(cur, device)
          outer = prod(Enum.take(dims, first))
          red = prod(Enum.slice(dims, first..last))
          inner = prod(Enum.drop(dims, last + 1))
          to_nx(unwrap!(NIF.reduce(ctx(device), code, dt(cur.type), dt(step.type), outer, red, inner, ref, bytes(step))), device, step)
        end)

      _ ->
        {view, outer, red, inner} = view_for_axes(t, opts[:axes], device)
        {ref, _} = from_nx(view, device)
        to_nx(unwrap!(NIF.reduce(ctx(device), code, dt(t.type), dt(out.type), outer, red, inner, ref, bytes(out))), device, out)
    end
  end

  # the sorted axes as runs of neighbours: [1, 3, 4] -> [[1], [3, 4]]
  defp axis_runs(nil), do: []

  defp axis_runs(axes) do
    axes
    |> Enum.sort()
    |> Enum.chunk_while(
      [],
      fn a, acc ->
        case acc do
          [prev | _] when a != prev + 1 -> {:cont, Enum.reverse(acc), [a]}
          _ -> {:cont, [a | acc]}
        end
      end,
      fn
        [] -> {:cont, []}
        acc -> {:cont, Enum.reverse(acc), []}
      end
    )
  end

  @impl true
  def argmax(out, t, opts), do: arg_op(0, out, t, opts)
  @impl true
  def argmin(out, t, opts), do: arg_op(1, out, t, opts)

  defp arg_op(code, out, %T{} = t, opts) do
    device = device_of([t])
    tie = if opts[:tie_break] == :high, do: 1, else: 0
    axes = if opts[:axis], do: [opts[:axis]], else: nil
    {view, outer, red, inner} = view_for_axes(t, axes, device)
    {ref, _} = from_nx(view, device)

    to_nx(unwrap!(NIF.argreduce(ctx(device), code, tie, dt(t.type), dt(out.type), outer, red, inner, ref, bytes(out))),
      device, out)
  end

  # collapses to [outer, red, inner]; non-adjacent axes are brought together by a device
  # transpose to kept ++ reduced, which keeps the row-major order of the reduced axes
  defp view_for_axes(t, nil, _device), do: {t, 1, Nx.size(t), 1}

  defp view_for_axes(%T{shape: shape} = t, axes, _device) do
    axes = Enum.sort(axes)
    dims = Tuple.to_list(shape)
    first = hd(axes)
    last = List.last(axes)

    if axes == Enum.to_list(first..last) do
      {t, prod(Enum.take(dims, first)), prod(Enum.slice(dims, first..last)), prod(Enum.drop(dims, last + 1))}
    else
      kept = Nx.axes(t) -- axes
      perm = kept ++ axes
      tt = transpose(%{t | shape: permute(shape, perm), names: permute_names(t.names, perm)}, t, perm)
      {tt, prod(Enum.map(kept, &elem(shape, &1))), prod(Enum.map(axes, &elem(shape, &1))), 1}
    end
  end

  defp prod(list), do: Enum.product(list)
  defp permute(shape, perm), do: perm |> Enum.map(&elem(shape, &1)) |> List.to_tuple()
  defp permute_names(names, perm), do: Enum.map(perm, &Enum.at(names, &1))

  ## Contraction

  @impl true
  def dot(out, %T{} = l, c1, b1, %T{} = r, c2, b2) do
    device = device_of([l, r])
    # walk the contraction pairs in increasing left-axis order: no copy of the left operand
    # whenever its contracted axes are adjacent (the pairing itself is kept)
    {c1, c2} = Enum.zip(c1, c2) |> Enum.sort() |> Enum.unzip()
    nb = length(b1)
    k = prod(Enum.map(c1, &elem(l.shape, &1)))
    batch = prod(Enum.map(b1, &elem(l.shape, &1)))
    {lt, l_layout, m} = dot_operand(l, c1, nb)
    {rt, r_layout, n} = dot_operand(r, c2, nb)
    {lref, _} = from_nx(lt, device)
    {rref, _} = from_nx(rt, device)

    ref =
      NIF.dot(ctx(device), dt(l.type), dt(r.type), out_dt(out.type), batch, m, n, k, l_layout, r_layout, lref, rref, bytes(out))

    to_nx(unwrap!(ref), device, out)
  end

  # [batch, rows, K] (layout 0) or [batch, K, rows] (layout 1) in place when the axes already
  # sit that way, else transposed to [batch, kept, contract] as Nx.BinaryBackend does
  defp dot_operand(%T{shape: shape} = t, contract, nb) do
    rank = tuple_size(shape)
    batch = Enum.to_list(0..(nb - 1)//1)
    kept = Enum.to_list(nb..(rank - 1)//1) -- contract
    rows = prod(Enum.map(kept, &elem(shape, &1)))
    identity = Enum.to_list(0..(rank - 1)//1)

    cond do
      batch ++ kept ++ contract == identity -> {t, 0, rows}
      batch ++ contract ++ kept == identity -> {t, 1, rows}
      true ->
        perm = batch ++ kept ++ contract
        {transpose(%{t | shape: permute(shape, perm), names: permute_names(t.names, perm)}, t, perm), 0, rows}
    end
  end

  ## Data movement

  @impl true
  def transpose(out, %T{type: {_, bits}} = t, axes) do
    device = device_of([t])
    {ref, _} = from_nx(t, device)
    to_nx(unwrap!(NIF.transpose(ctx(device), div(bits, 8), Tuple.to_list(t.shape), axes, ref, bytes(out))), device, out)
  end

  @impl true
  def broadcast(out, %T{type: {_, bits}} = t, shape, axes) do
    device = device_of([t])
    {ref, _} = from_nx(t, device)
    in_dims = Tuple.to_list(t.shape)

    {pairs, _} =
      Enum.zip(in_dims, axes)
      |> Enum.reverse()
      |> Enum.map_reduce(1, fn {dim, axis}, acc -> {{axis, if(dim == 1, do: 0, else: acc)}, acc * dim} end)

    by_axis = Map.new(pairs)
    strides = for a <- 0..(tuple_size(shape) - 1)//1, do: Map.get(by_axis, a, 0)
    to_nx(unwrap!(NIF.broadcast(ctx(device), div(bits, 8), Tuple.to_list(shape), strides, ref, bytes(out))), device, out)
  end

  @impl true
  def gather(out, %T{type: {_, bits}} = t, %T{} = indices, opts) do
    device = device_of([t, indices])
    axes = opts[:axes]
    t_axes = Nx.axes(t)

    t =
      if List.starts_with?(t_axes, axes) do
        t
      else
        perm = axes ++ (t_axes -- axes)
        transpose(%{t | shape: permute(t.shape, perm), names: permute_names(t.names, perm)}, t, perm)
      end

    {tref, _} = from_nx(t, device)
    {iref, _} = from_nx(indices, device)
    depth = elem(indices.shape, tuple_size(indices.shape) - 1)
    n_tuples = div(Nx.size(indices), depth)

    ref =
      NIF.gather(ctx(device), div(bits, 8), Tuple.to_list(t.shape), dt(indices.type), n_tuples, depth, 0, tref, iref, bytes(out))

    to_nx(unwrap!(ref), device, out)
  end

  @impl true
  def block(%Nx.Block.Take{axis: 0}, out, [t, indices], _fun) do
    gather(out, t, %{indices | shape: {Nx.size(indices), 1}, names: [nil, nil]}, axes: [0])
  end

  # along any other axis: one kernel over the tensor viewed as [outer, axis, inner] instead of the default's
  # transpose, gather and transpose back (nx.ex:14807-14819); a bad index is reported against the shape
  # with the taken axis moved to the front, as the default reports it (binary_backend.ex:1906-1912)
  def block(%Nx.Block.Take{axis: axis}, %T{type: {_, bits}} = out, [t, indices], _fun) when bits >= 8 do
    device = device_of([t, indices])
    {tref, _} = from_nx(t, device)
    {iref, _} = from_nx(indices, device)
    dims = Tuple.to_list(t.shape)
    {before, [axis_len | rest]} = Enum.split(dims, axis)

    ref =
      NIF.take(ctx(device), div(bits, 8), Enum.product(before), axis_len, Enum.product(rest), dt(indices.type),
        Nx.size(indices), 0, [axis_len | before ++ rest], tref, iref, bytes(out))

    to_nx(unwrap!(ref), device, out)
  end

  def block(struct, _out, args, fun), do: apply(fun, [struct | args])

  ## Selection, windows and creation

  @impl true
  def select(%T{shape: shape} = out, %T{} = pred, %T{} = on_true, %T{} = on_false) do
    device = device_of([pred, on_true, on_false])
    {pref, _} = from_nx(pred, device)
    {tref, _} = from_nx(on_true, device)
    {fref, _} = from_nx(on_false, device)

    ref =
      NIF.select(ctx(device), dt(pred.type), dt(on_true.type), dt(on_false.type), dt(out.type), Tuple.to_list(shape),
        broadcast_strides(pred.shape, shape), broadcast_strides(on_true.shape, shape),
        broadcast_strides(on_false.shape, shape), pref, tref, fref, bytes(out))

    to_nx(unwrap!(ref), device, out)
  end

  @impl true
  def clip(out, %T{} = t, %T{} = min, %T{} = max) do
    device = device_of([t, min, max])
    {ref, _} = from_nx(t, device)
    {mn, _} = from_nx(min, device)
    {mx, _} = from_nx(max, device)

    to_nx(unwrap!(NIF.clip(ctx(device), dt(t.type), dt(min.type), dt(max.type), dt(out.type), Nx.size(out), ref, mn, mx,
      bytes(out))), device, out)
  end

  @impl true
  def slice(%T{shape: out_shape, type: {_, bits}} = out, %T{shape: shape} = t, start_indices, lengths, strides) do
    device = device_of([t])
    {ref, _} = from_nx(t, device)
    dense = dense_strides(shape)

    # dynamic starts are read back and clamped as binary_backend.ex:1813-1863 does
    starts =
      [start_indices, Tuple.to_list(shape), lengths]
      |> Enum.zip_with(fn [idx, dim, len] ->
        idx = if is_struct(idx, T), do: Nx.to_number(idx), else: idx
        idx |> max(0) |> min(dim - len)
      end)

    offset = Enum.zip_with(starts, dense, &(&1 * &2)) |> Enum.sum()
    in_strides = Enum.zip_with(strides, dense, &(&1 * &2))

    ref =
      NIF.strided_copy(ctx(device), div(bits, 8), Tuple.to_list(out_shape), in_strides, offset, dense_strides(out_shape), 0,
        ref, bytes(out))

    to_nx(unwrap!(ref), device, out)
  end

  @impl true
  def to_batched(%T{shape: out_shape} = out, %T{shape: shape} = t, opts) do
    # byte windows of the leading axis, lazily; a short last batch wraps to the first entries
    # (binary_backend.ex:178-211)
    device = device_of([t])
    {ref, _} = from_nx(t, device)
    batch = elem(out_shape, 0)
    total = elem(shape, 0)
    row = div(bytes(t), max(total, 1))
    full = div(total, batch)
    rest = rem(total, batch)
    last = if rest != 0 and opts[:leftover] == :repeat, do: full, else: full - 1

    window = fn buf, first, count, at ->
      if count * row > 0 do
        unwrap!(NIF.strided_copy(ctx(device), 1, [count * row], [1], first * row, [1], at * row, ref, buf))
      end
    end

    Stream.map(0..last//1, fn i ->
      buf = unwrap!(NIF.alloc(ctx(device), bytes(out)))

      if i < full do
        window.(buf, i * batch, batch, 0)
      else
        window.(buf, full * batch, rest, 0)
        window.(buf, 0, batch - rest, rest)
      end

      to_nx(buf, device, out)
    end)
  end

  @impl true
  def pad(_out, %T{shape: {}} = t, _pad_value, _config), do: t

  def pad(%T{shape: out_shape, type: {_, bits} = type} = out, %T{shape: shape} = t, %T{} = pad_value, config) do
    device = device_of([t, pad_value])
    t = if t.type == type, do: t, else: as_type(%{t | type: type}, t)
    pad_value = if pad_value.type == type, do: pad_value, else: as_type(%{pad_value | type: type}, pad_value)
    {ref, _} = from_nx(t, device)
    {vref, _} = from_nx(pad_value, device)
    out_dims = Tuple.to_list(out_shape)
    filled = unwrap!(NIF.broadcast(ctx(device), div(bits, 8), out_dims, List.duplicate(0, length(out_dims)), vref, bytes(out)))

    # element i of an axis lands at low + i * (interior + 1); keep the ones that land inside
    ranges =
      [Tuple.to_list(shape), out_dims, config]
      |> Enum.zip_with(fn [dim, odim, {low, _high, interior}] ->
        step = interior + 1
        lo = -Integer.floor_div(min(low, 0), step)
        hi = if odim > 0, do: min(dim - 1, Integer.floor_div(odim - 1 - low, step)), else: -1
        {lo, max(hi - lo + 1, 0), step, low}
      end)

    if Enum.all?(ranges, fn {_, count, _, _} -> count > 0 end) do
      dense_in = dense_strides(shape)
      dense_out = dense_strides(out_shape)
      in_offset = Enum.zip_with(ranges, dense_in, fn {lo, _, _, _}, d -> lo * d end) |> Enum.sum()
      out_offset = Enum.zip_with(ranges, dense_out, fn {lo, _, step, low}, d -> (low + lo * step) * d end) |> Enum.sum()
      out_strides = Enum.zip_with(ranges, dense_out, fn {_, _, step, _}, d -> step * d end)
      counts = Enum.map(ranges, &elem(&1, 1))
      unwrap!(NIF.strided_copy(ctx(device), div(bits, 8), counts, dense_in, in_offset, out_strides, out_offset, ref, filled))
    end

    to_nx(filled, device, out)
  end

  @impl true
  def reverse(%T{type: {_, bits}} = out, %T{shape: shape} = t, axes) do
    device = device_of([t])
    {ref, _} = from_nx(t, device)
    dense = dense_strides(shape)
    strides = dense |> Enum.with_index() |> Enum.map(fn {s, a} -> if a in axes, do: -s, else: s end)
    offset = axes |> Enum.map(&((elem(shape, &1) - 1) * Enum.at(dense, &1))) |> Enum.sum()

    to_nx(unwrap!(NIF.strided_copy(ctx(device), div(bits, 8), Tuple.to_list(shape), strides, offset, dense, 0, ref, bytes(out))),
      device, out)
  end

  @impl true
  def put_slice(%T{shape: shape, type: {_, bits} = type} = out, %T{} = t, start_indices, %T{shape: slice_shape} = slice) do
    device = device_of([t, slice])
    t = if t.type == type, do: t, else: as_type(%{t | type: type}, t)
    slice = if slice.type == type, do: slice, else: as_type(%{slice | type: type}, slice)
    {ref, _} = from_nx(t, device)
    {sref, _} = from_nx(slice, device)

    starts =
      [start_indices, Tuple.to_list(shape), Tuple.to_list(slice_shape)]
      |> Enum.zip_with(fn [idx, dim, len] ->
        idx = if is_struct(idx, T), do: Nx.to_number(idx), else: idx
        idx |> max(0) |> min(dim - len)
      end)

    dense = dense_strides(shape)
    buf = unwrap!(NIF.copy(ctx(device), ref, bytes(out)))

    if Nx.size(slice_shape) > 0 do
      at = Enum.zip_with(starts, dense, &(&1 * &2)) |> Enum.sum()
      unwrap!(NIF.strided_copy(ctx(device), div(bits, 8), Tuple.to_list(slice_shape), dense_strides(slice_shape), 0, dense, at, sref, buf))
    end

    to_nx(buf, device, out)
  end

  @impl true
  def concatenate(%T{shape: out_shape, type: {_, bits} = type} = out, tensors, axis) do
    device = device_of(tensors)
    out_strides = dense_strides(out_shape)
    step = Enum.at(out_strides, axis)
    buf = unwrap!(NIF.alloc(ctx(device), bytes(out)))

    Enum.reduce(tensors, 0, fn %T{shape: shape} = t, at ->
      t = if t.type == type, do: t, else: as_type(%{t | type: type}, t)
      {ref, _} = from_nx(t, device)

      unwrap!(
        NIF.strided_copy(ctx(device), div(bits, 8), Tuple.to_list(shape), dense_strides(shape), 0, out_strides, at * step,
          ref, buf)
      )

      at + elem(shape, axis)
    end)

    to_nx(buf, device, out)
  end

  @impl true
  def stack(out, tensors, axis) do
    widened = Enum.map(tensors, fn %T{shape: shape, names: names} = t ->
      %{t | shape: Tuple.insert_at(shape, axis, 1), names: List.insert_at(names, axis, nil)}
    end)

    concatenate(out, widened, axis)
  end

  @impl true
  def iota(%T{shape: shape} = out, axis, opts) do
    device = opts[:device] || 0
    n = Nx.size(shape)

    {dim, inner} =
      if axis, do: {elem(shape, axis), shape |> Tuple.to_list() |> Enum.drop(axis + 1) |> prod()}, else: {max(n, 1), 1}

    to_nx(unwrap!(NIF.iota(ctx(device), dt(out.type), n, dim, inner, bytes(out))), device, out)
  end

  @impl true
  def eye(%T{shape: shape} = out, opts) do
    device = opts[:device] || 0
    rank = tuple_size(shape)

    to_nx(unwrap!(NIF.eye(ctx(device), dt(out.type), Nx.size(shape), elem(shape, rank - 2), elem(shape, rank - 1),
      bytes(out))), device, out)
  end

  @doc """
  The words of `Nx.Random`'s `threefry2x32/2` for `Nx.size(out)` counters in one kernel
  (`out` is a u32 template). Not a behaviour callback.
  """
  def threefry2x32(%T{} = out, %T{} = key) do
    device = device_of([key])
    {ref, _} = from_nx(key, device)
    to_nx(unwrap!(NIF.threefry2x32(ctx(device), ref, Nx.size(out), bytes(out))), device, out)
  end

  defp dense_strides(shape) do
    {strides, _} = shape |> Tuple.to_list() |> Enum.reverse() |> Enum.map_reduce(1, fn dim, acc -> {acc, acc * dim} end)
    Enum.reverse(strides)
  end

  ## Everything else: round trip through Nx.BinaryBackend

  fallbacks =
    Nx.Backend.behaviour_info(:callbacks) --
      (Module.definitions_in(__MODULE__, :def) ++ [from_pointer: 5, to_pointer: 2])

  for {name, arity} <- fallbacks do
    args = Macro.generate_arguments(arity, __MODULE__)

    @impl true
    def unquote(name)(unquote_splicing(args)) do
      device = device_of(Enum.filter(unquote(args), &is_struct(&1, T)))

      host = fn
        %T{data: %__MODULE__{}} = t -> Nx.backend_copy(t, Nx.BinaryBackend)
        list when is_list(list) -> Enum.map(list, &if(is_struct(&1, T), do: Nx.backend_copy(&1, Nx.BinaryBackend), else: &1))
        other -> other
      end

      result = apply(Nx.BinaryBackend, unquote(name), Enum.map(unquote(args), host))

      back = fn
        %T{data: %Nx.BinaryBackend{}} = t -> Nx.backend_transfer(t, {__MODULE__, device: device})
        other -> other
      end

      case result do
        list when is_list(list) -> Enum.map(list, back)
        other -> back.(other)
      end
    end
  end

  ## Pointers (cf. EXLA.Backend.to_pointer/2 and from_pointer/5, exla/lib/exla/backend.ex:85-181)

  @impl true
  def to_pointer(%T{data: %__MODULE__{ref: ref, device: device}} = t, opts) do
    opts = Keyword.validate!(opts, mode: :local, permissions: 0o400)

    case opts[:mode] do
      :local ->
        %Nx.Pointer{kind: :local, address: unwrap!(NIF.device_ptr(ref)), data_size: bytes(t)}

      :ipc ->
        # the 64 bytes of the HIP IPC handle; address carries the device index, as EXLA's cuda client does
        handle = unwrap!(NIF.ipc_export(ctx(device), ref))
        %Nx.Pointer{kind: :ipc, handle: handle, address: device, data_size: bytes(t)}

      mode ->
        raise ArgumentError, "expected one of :local, :ipc, got: #{inspect(mode)}"
    end
  end

  @impl true
  def from_pointer(%Nx.Pointer{} = pointer, type, dims, backend_opts, opts) do
    device = init(backend_opts)[:device]
    opts = Keyword.validate!(opts, [:names])
    template = Nx.template(dims, type, names: opts[:names])
    size = bytes(template)

    case pointer do
      %Nx.Pointer{data_size: other} when other != size ->
        raise ArgumentError, "invalid pointer data_size for shape, expected: #{size}, got: #{other}"

      %Nx.Pointer{kind: :local, address: address} ->
        # the memory stays with its owner: deallocating this tensor never frees it
        to_nx(unwrap!(NIF.wrap(ctx(device), address, size)), device, template)

      %Nx.Pointer{kind: :ipc, handle: handle} when is_binary(handle) and byte_size(handle) == 64 ->
        # another OS process's buffer: deallocating this tensor closes the mapping, never frees the memory
        to_nx(unwrap!(NIF.ipc_import(ctx(device), handle, size)), device, template)

      %Nx.Pointer{kind: :ipc} ->
        raise ArgumentError, "an :ipc pointer carries a handle of 64 bytes"
    end
  end
end
