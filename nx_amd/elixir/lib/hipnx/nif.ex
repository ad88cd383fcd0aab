defmodule HipNx.NIF do
  @moduledoc false
  # Stubs replaced by c_src/hipnx_nif.c at load time (same scheme as torchx/lib/torchx/nif.ex).
  @on_load :__on_load__

  def __on_load__ do
    path = :filename.join(:code.priv_dir(:hipnx), ~c"hipnx_nif")
    :erlang.load_nif(path, 0)
  end

  def device_count, do: err()
  def ctx_create(_device), do: err()
  def from_binary(_ctx, _binary, _nbytes), do: err()
  def to_binary(_ctx, _buf, _nbytes), do: err()
  def alloc(_ctx, _nbytes), do: err()
  def deallocate(_buf), do: err()
  def copy(_ctx, _buf, _nbytes), do: err()
  def fill(_ctx, _elem, _count), do: err()
  def binary(_ctx, _op, _l_dt, _r_dt, _out_dt, _dims, _l_strides, _r_strides, _l, _r, _out_bytes), do: err()
  def unary(_ctx, _op, _in_dt, _out_dt, _n, _in, _out_bytes), do: err()
  def reduce(_ctx, _op, _in_dt, _out_dt, _outer, _red, _inner, _in, _out_bytes), do: err()
  def argreduce(_ctx, _op, _tie, _in_dt, _out_dt, _outer, _red, _inner, _in, _out_bytes), do: err()
  def dot(_ctx, _l_dt, _r_dt, _out_dt, _batch, _m, _n, _k, _l_layout, _r_layout, _l, _r, _out_bytes), do: err()
  def transpose(_ctx, _elem_bytes, _dims, _perm, _in, _out_bytes), do: err()
  def broadcast(_ctx, _elem_bytes, _dims, _strides, _in, _out_bytes), do: err()
  def gather(_ctx, _elem_bytes, _dims, _idx_dt, _n_tuples, _depth, _policy, _t, _idx, _out_bytes), do: err()
  def take(_ctx, _elem_bytes, _outer, _axis_len, _inner, _idx_dt, _n_idx, _policy, _msg_dims, _t, _idx, _out_bytes), do: err()
  def select(_ctx, _p_dt, _t_dt, _f_dt, _out_dt, _dims, _p_strides, _t_strides, _f_strides, _p, _t, _f, _out_bytes), do: err()
  def clip(_ctx, _in_dt, _min_dt, _max_dt, _out_dt, _n, _in, _min, _max, _out_bytes), do: err()
  def strided_copy(_ctx, _elem_bytes, _dims, _in_strides, _in_offset, _out_strides, _out_offset, _in, _out_or_bytes), do: err()
  def iota(_ctx, _out_dt, _n, _dim, _inner, _out_bytes), do: err()
  def eye(_ctx, _out_dt, _n, _rows, _cols, _out_bytes), do: err()
  def narrow_int(_ctx, _buf, _n, _bits, _signed), do: err()
  def device_ptr(_buf), do: err()
  def wrap(_ctx, _address, _nbytes), do: err()
  def ipc_export(_ctx, _buf), do: err()
  def ipc_import(_ctx, _handle, _nbytes), do: err()
  def threefry2x32(_ctx, _key, _n, _out_bytes), do: err()
  def sync(_ctx), do: err()

  defp err, do: :erlang.nif_error(:undef)
end
