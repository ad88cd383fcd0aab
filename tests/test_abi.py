"""The C-ABI shared library loads and exports every symbol include/hipnx.h declares, and the
ctypes prototype table covers exactly that set.  No compute calls: this runs without a GPU."""
import ctypes as C
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "hipnx.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hipnx_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_functions()
    for must in ("hipnx_ctx_create", "hipnx_buf_alloc", "hipnx_buf_free", "hipnx_h2d", "hipnx_d2h", "hipnx_binary",
                 "hipnx_unary", "hipnx_as_type", "hipnx_reduce", "hipnx_argreduce", "hipnx_dot", "hipnx_gather",
                 "hipnx_transpose", "hipnx_broadcast", "hipnx_fill", "hipnx_last_error"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from nx_amd import _lib
    lib = C.CDLL(_lib.LIB_PATH)
    for name in declared_functions():
        assert hasattr(lib, name), f"libhipnx.so lacks {name}"


def test_prototype_table_matches_the_header():
    from nx_amd import _lib
    assert sorted(_lib.PROTOTYPES) == declared_functions()


def test_enum_values_match_between_header_and_host_code():
    from nx_amd import backend, types
    text = open(os.path.join(ROOT, "include", "hipnx.h")).read()
    m = re.search(r"HIPNX_ADD = 0,(.*?)HIPNX_NBINARY", text, flags=re.S)
    ops = ["add"] + [x.strip().lower().replace("hipnx_", "") for x in m.group(1).split(",") if x.strip()]
    assert ops == backend.BINARY_OPS
    m = re.search(r"HIPNX_EXP = 0,(.*?)HIPNX_NUNARY", text, flags=re.S)
    ops = ["exp"] + [x.strip().lower().replace("hipnx_", "") for x in m.group(1).split(",") if x.strip()]
    ops = [{"clz": "count_leading_zeros", "popcount": "population_count"}.get(o, o) for o in ops]
    assert ops == backend.UNARY_OPS
    for name, code in (("U8", 0), ("S8", 4), ("F16", 8), ("BF16", 9), ("F32", 10), ("F64", 11)):
        assert re.search(rf"HIPNX_{name} = {code}\b", text)
        assert getattr(types, name) == code


def test_calls_fail_cleanly_without_a_device_or_with_bad_handles():
    from nx_amd import _lib as L
    n = C.c_int(-1)
    assert L.lib.hipnx_device_count(C.byref(n)) == L.OK and n.value >= 0
    if n.value == 0:
        ctx = C.c_void_p()
        assert L.lib.hipnx_ctx_create(0, C.byref(ctx)) != L.OK
        assert "no HIP device" in L.last_error()
    assert L.lib.hipnx_sync(None) == L.EINVAL
    assert L.lib.hipnx_buf_free(None) == L.EINVAL


def test_oracle_is_not_reachable_from_the_product():
    """The CPU oracle is test infrastructure: nothing under nx_amd/ may import or load it."""
    pkg = os.path.join(ROOT, "nx_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".h", ".cuh")) or f == "Makefile":
                text = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle\b", text, flags=re.M), f"{f} imports the oracle"
                assert "hipnx_ref" not in text and "oracle/" not in text, f"{f} names the oracle library"
