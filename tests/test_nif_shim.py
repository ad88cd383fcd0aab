"""The Elixir half cannot be built here (no Erlang/OTP in the image).  What can be checked on text is:
the `erl_nif` shim parses and type-checks against a declaration-only stand-in of <erl_nif.h>
(tests/erl_nif_standin/erl_nif.h: spelling and arity of every erl_nif call and of every hipnx_* call,
nothing about behaviour), and its function table agrees with the stubs of `HipNx.NIF` name by name and
arity by arity."""
import os
import re
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
NIF_C = os.path.join(ROOT, "nx_amd", "elixir", "c_src", "hipnx_nif.c")
NIF_EX = os.path.join(ROOT, "nx_amd", "elixir", "lib", "hipnx", "nif.ex")
BACKEND_EX = os.path.join(ROOT, "nx_amd", "elixir", "lib", "hipnx", "backend.ex")


def test_shim_passes_a_syntax_and_type_check_against_the_stand_in_header():
    done = subprocess.run(["gcc", "-fsyntax-only", "-Wall", "-Wextra", "-Werror", "-I", os.path.join(ROOT, "tests", "erl_nif_standin"),
                           "-I", os.path.join(ROOT, "include"), NIF_C], capture_output=True, text=True)
    assert done.returncode == 0, done.stderr[-3000:]


def _table():
    src = open(NIF_C).read()
    body = src[src.index("static ErlNifFunc funcs[]"):]
    return {name: int(arity) for name, arity in re.findall(r'\{"(\w+)",\s*(\d+),\s*nif_\w+,', body)}


def _stubs():
    out = {}
    for name, args in re.findall(r"^\s*def (\w+)(?:\(([^)]*)\))?, do: err\(\)", open(NIF_EX).read(), re.M):
        out[name] = len([a for a in args.split(",") if a.strip()]) if args else 0
    return out


def test_function_table_matches_the_elixir_stubs():
    table, stubs = _table(), _stubs()
    assert table and table == stubs, {k: (table.get(k), stubs.get(k)) for k in set(table) | set(stubs) if table.get(k) != stubs.get(k)}


def test_backend_only_calls_nifs_that_exist_with_the_right_arity():
    table = _table()
    src = open(BACKEND_EX).read()
    calls = re.findall(r"NIF\.(\w+)\(", src)
    assert calls and set(calls) <= set(table), sorted(set(calls) - set(table))
    # arity of each call site: count top-level commas up to the matching parenthesis
    for m in re.finditer(r"NIF\.(\w+)\(", src):
        depth, i, commas, empty = 1, m.end(), 0, True
        while depth:
            c = src[i]
            if c in "([{":
                depth += 1
            elif c in ")]}":
                depth -= 1
            elif c == "," and depth == 1:
                commas += 1
            if depth and not c.isspace():
                empty = False
            i += 1
        arity = 0 if empty else commas + 1
        assert arity == table[m.group(1)], f"NIF.{m.group(1)} called with {arity} arguments, the table has {table[m.group(1)]}"
