"""ctypes binding of libhipnx.so -- the same C ABI the Elixir NIF shim binds (include/hipnx.h).

There is no fallback: if the shared library is missing the import of this module fails, and if
no GPU is present every compute entry point fails with HipNxError.
"""
from __future__ import annotations

import ctypes as C
import functools
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("HIPNX_LIB", os.path.join(_HERE, "lib", "libhipnx.so"))

# status codes of include/hipnx.h
OK, ALREADY_FREED, EINVAL, EFREED, ENOMEM, EHIP, EINDEX, EUNSUPPORTED, ERAISED = range(9)


class HipNxError(RuntimeError):
    """A failed libhipnx call; `.status` is the HIPNX_E* code."""

    def __init__(self, status: int, message: str):
        super().__init__(f"HipNx: {message}")
        self.status = status


class HipNxArgumentError(HipNxError, ValueError):
    """Status codes the Elixir side maps to ArgumentError (EINVAL, EINDEX)."""


class HipNxArithmeticError(HipNxError, ArithmeticError):
    """ERAISED with the reference's ArithmeticError text (div / rem by zero, negative integer exponent)."""


if not os.path.exists(LIB_PATH):
    raise ImportError(
        f"libhipnx.so not found at {LIB_PATH}: build it first "
        "(python -c 'import __graft_entry__ as g; g.build()' or make -C nx_amd/csrc)")

lib = C.CDLL(LIB_PATH)

class _Imm(C.Union):
    _fields_ = [("f", C.c_float), ("bits", C.c_uint32)]


class FusedInstr(C.Structure):
    """hipnx_fused_instr of include/hipnx.h (imm / imm2 as a float or as raw bits)."""
    _fields_ = [("kind", C.c_uint8), ("op", C.c_uint8), ("src", C.c_uint8), ("arg", C.c_uint8), ("src2", C.c_uint8),
                ("arg2", C.c_uint8), ("flags", C.c_uint8), ("dt", C.c_uint8), ("imm", _Imm), ("imm2", _Imm)]


FUSED_SET, FUSED_UNARY, FUSED_BINARY, FUSED_SELECT, FUSED_AS_TYPE, FUSED_BITCAST = range(6)
FUSED_FLAG_SWAP, FUSED_FLAG_INT = 1, 2
FUSED_SRC_CONST, FUSED_SRC_INPUT, FUSED_SRC_SAVED = range(3)
FUSED_SAVED, FUSED_MAX_INSTR, FUSED_MAX_INPUTS = 3, 32, 8
FUSED_INTERPRETED, FUSED_COMPILED = 0, 1
IPC_HANDLE_BYTES = 64
SCALE_NONE, SCALE_PER_COLUMN, SCALE_PER_ROW, SCALE_ONE = range(4)

_ctx_p, _buf_p = C.c_void_p, C.c_void_p
_i64p, _intp = C.POINTER(C.c_int64), C.POINTER(C.c_int)

# name -> argtypes, in the order of include/hipnx.h; every function returns int except
# hipnx_buf_device_ptr
PROTOTYPES = {
    "hipnx_device_count": [_intp],
    "hipnx_ctx_create": [C.c_int, C.POINTER(_ctx_p)],
    "hipnx_ctx_destroy": [_ctx_p],
    "hipnx_sync": [_ctx_p],
    "hipnx_last_error": [C.c_char_p, C.c_size_t],
    "hipnx_mem_stats": [_ctx_p, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)],
    "hipnx_trim": [_ctx_p],
    "hipnx_timer_start": [_ctx_p],
    "hipnx_timer_stop": [_ctx_p, C.POINTER(C.c_float)],
    "hipnx_timer_mark": [_ctx_p, C.c_int],
    "hipnx_timer_between": [_ctx_p, C.c_int, C.c_int, C.POINTER(C.c_float)],
    "hipnx_buf_alloc": [_ctx_p, C.c_size_t, C.POINTER(_buf_p)],
    "hipnx_buf_free": [_buf_p],
    "hipnx_buf_destroy": [_buf_p],
    "hipnx_buf_size": [_buf_p, C.POINTER(C.c_size_t)],
    "hipnx_buf_device_ptr": [_buf_p],
    "hipnx_buf_index_bound": [_buf_p, _i64p],
    "hipnx_buf_wrap": [_ctx_p, C.c_void_p, C.c_size_t, C.POINTER(_buf_p)],
    "hipnx_buf_ipc_export": [_ctx_p, _buf_p, C.c_void_p],
    "hipnx_buf_ipc_import": [_ctx_p, C.c_void_p, C.c_size_t, C.POINTER(_buf_p)],
    "hipnx_h2d": [_ctx_p, _buf_p, C.c_size_t, C.c_void_p, C.c_size_t],
    "hipnx_d2h": [_ctx_p, _buf_p, C.c_size_t, C.c_void_p, C.c_size_t],
    "hipnx_d2d": [_ctx_p, _buf_p, C.c_size_t, _buf_p, C.c_size_t, C.c_size_t],
    "hipnx_fill": [_ctx_p, _buf_p, C.c_int, C.c_void_p, C.c_int64],
    "hipnx_binary": [_ctx_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _i64p, _i64p, _i64p, _buf_p, _buf_p, _buf_p],
    "hipnx_unary": [_ctx_p, C.c_int, C.c_int, C.c_int, C.c_int64, _buf_p, _buf_p],
    "hipnx_as_type": [_ctx_p, C.c_int, C.c_int, C.c_int64, _buf_p, _buf_p],
    "hipnx_reduce": [_ctx_p, C.c_int, C.c_int, C.c_int, C.c_int64, C.c_int64, C.c_int64, _buf_p, _buf_p],
    "hipnx_reduce_static": [_ctx_p, C.c_int, C.c_int, C.c_int, C.c_int64, C.c_int64, C.c_int64, _buf_p, _buf_p],
    "hipnx_argreduce": [_ctx_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int64, C.c_int64, C.c_int64, _buf_p, _buf_p],
    "hipnx_dot": [_ctx_p, C.c_int, C.c_int, C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_int, C.c_int,
                  _buf_p, _buf_p, _buf_p],
    "hipnx_dot_scaled": [_ctx_p, C.c_int, C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_int, C.c_int,
                         _buf_p, _buf_p, C.c_int, _buf_p, _buf_p],
    "hipnx_transpose": [_ctx_p, C.c_int, C.c_int, _i64p, _intp, _buf_p, _buf_p],
    "hipnx_broadcast": [_ctx_p, C.c_int, C.c_int, _i64p, _i64p, _buf_p, _buf_p],
    "hipnx_gather": [_ctx_p, C.c_int, C.c_int, _i64p, C.c_int, C.c_int64, C.c_int, C.c_int, _buf_p, _buf_p, _buf_p],
    "hipnx_take": [_ctx_p, C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_int, C.c_int64, C.c_int, C.c_int, _i64p, _buf_p, _buf_p,
                   _buf_p],
    "hipnx_select": [_ctx_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _i64p, _i64p, _i64p, _i64p, _buf_p, _buf_p,
                     _buf_p, _buf_p],
    "hipnx_clip": [_ctx_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int64, _buf_p, _buf_p, _buf_p, _buf_p],
    "hipnx_concat": [_ctx_p, C.c_int, C.c_int, C.POINTER(_buf_p), _i64p, C.c_int64, C.c_int64, _buf_p],
    "hipnx_strided_copy": [_ctx_p, C.c_int, C.c_int, _i64p, _i64p, C.c_int64, _i64p, C.c_int64, _buf_p, _buf_p],
    "hipnx_iota": [_ctx_p, C.c_int, C.c_int64, C.c_int64, C.c_int64, _buf_p],
    "hipnx_eye": [_ctx_p, C.c_int, C.c_int64, C.c_int64, C.c_int64, _buf_p],
    "hipnx_narrow_int": [_ctx_p, _buf_p, C.c_int64, C.c_int, C.c_int],
    "hipnx_fused_set_mode": [_ctx_p, C.c_int],
    "hipnx_fused_compiled_count": [_ctx_p, C.POINTER(C.c_int)],
    "hipnx_fused_set_cache_limit": [_ctx_p, C.c_int],
    "hipnx_threefry2x32": [_ctx_p, _buf_p, C.c_int64, _buf_p],
    "hipnx_fused_elementwise": [_ctx_p, C.c_int, C.c_void_p, C.c_int, C.POINTER(C.c_void_p), _intp, _i64p, _intp, C.c_int64,
                                C.c_int64, C.c_int, C.c_int, _buf_p],
    "hipnx_capture_begin": [_ctx_p],
    "hipnx_capture_end": [_ctx_p, C.POINTER(C.c_void_p)],
    "hipnx_graph_launch": [C.c_void_p],
    "hipnx_graph_destroy": [C.c_void_p],
}

for _name, _args in PROTOTYPES.items():
    _fn = getattr(lib, _name)  # AttributeError here = the library lacks a declared symbol
    _fn.argtypes = _args
    _fn.restype = C.c_void_p if _name == "hipnx_buf_device_ptr" else C.c_int


def last_error() -> str:
    buf = C.create_string_buffer(512)
    lib.hipnx_last_error(buf, 512)
    return buf.value.decode("utf-8", "replace")


def check(status: int) -> int:
    """Raises on every status except OK and ALREADY_FREED (which the caller interprets)."""
    if status in (OK, ALREADY_FREED):
        return status
    message = last_error()
    if status == ERAISED:  # the reference's exception, surfaced late (include/hipnx.h HIPNX_ERAISED)
        cls = HipNxArithmeticError if message.startswith("ArithmeticError") else HipNxArgumentError
    else:
        cls = HipNxArgumentError if status in (EINVAL, EINDEX) else HipNxError
    raise cls(status, message)


@functools.lru_cache(maxsize=4096)
def _i64_array_cached(values: tuple):
    return (C.c_int64 * max(len(values), 1))(*values)


def i64_array(values):
    """A C array of int64 for dims / strides (read-only on the C side, so equal tuples share one)."""
    return _i64_array_cached(tuple(values))


@functools.lru_cache(maxsize=4096)
def broadcast_stride_array(shape: tuple, out_shape: tuple):
    """The element strides of `shape` viewed in `out_shape` (0 on broadcast axes) as a C array."""
    from . import shape as S
    return _i64_array_cached(S._broadcast_strides(shape, out_shape))


def int_array(values):
    values = list(values)
    return (C.c_int * max(len(values), 1))(*values)
