"""The TypeScript binding that a jsgrad maintainer would add (integration/jsgrad/) against the C header and the ctypes table.

No JavaScript runtime with an FFI exists in the build image, so the files cannot be executed here; what can be checked
is that the symbol table of hip_bindings.ts names every declaration of include/jsgrad_hip.h with the header's arity and
types, that it agrees with denograd_amd/ffi.py (the table the GPU tests call through), that every symbol the other
TypeScript files call exists with the number of arguments they pass, and that the packed layout of jsgrad_hip_step_t
written there is the C compiler's."""
import ctypes as C
import os
import re
import subprocess
import sys

import pytest

from denograd_amd import ffi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TS_DIR = os.path.join(ROOT, "integration", "jsgrad")
BINDINGS = os.path.join(TS_DIR, "runtime", "hip_bindings.ts")
ALIASES = {"P": "pointer", "B": "buffer", "I": "i32", "U32": "u32", "F": "f32", "D": "f64", "U": "usize", "U64": "u64"}


def ts_table():
    """{symbol: ([Deno FFI parameter types], result type)} parsed from the TypeScript text itself."""
    text = open(BINDINGS).read()
    alias_line = re.search(r"^const P = .*$", text, flags=re.M).group(0)
    aliases = dict(re.findall(r"(\w+) = '(\w+)'", alias_line))
    assert aliases == ALIASES
    out = {}
    for name, params, result in re.findall(r"^\s*(jsgrad_hip_\w+): \{ parameters: \[([^\]]*)\], result: (\w+) \}", text, flags=re.M):
        assert name not in out, f"{name} listed twice"
        out[name] = ([aliases[p.strip()] for p in params.split(",") if p.strip()], aliases[result])
    return out


def header_table():
    """{symbol: ([expected Deno FFI types], result)} from the C declarations: host_* and char pointers are host memory."""
    text = open(os.path.join(ROOT, "include", "jsgrad_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    scalars = {"int": "i32", "int32_t": "i32", "uint32_t": "u32", "float": "f32", "double": "f64", "size_t": "usize", "uint64_t": "u64"}
    out = {}
    for ret, name, params in re.findall(r"([\w \*]+?)\b(jsgrad_hip_\w+)\s*\(([^)]*)\)\s*;", text):
        types = []
        params = " ".join(params.split())
        for p in ([] if params == "void" else params.split(",")):
            p = p.strip()
            pname = re.search(r"(\w+)\s*(\[\d*\])?$", p).group(1)
            if "*" in p or "[" in p:
                types.append("buffer" if pname.startswith("host_") or "char" in p else "pointer")
            else:
                types.append(scalars[re.sub(r"\bconst\b|\bunsigned\b", "", p[: p.rindex(pname)]).strip()])
        ret = ret.strip()
        out[name] = (types, "pointer" if "*" in ret else scalars[ret.replace("const", "").strip()])
    return out


def ctypes_kind(t):
    if t in (C.c_int, C.c_int32):
        return "i32"
    if t is C.c_float:
        return "f32"
    if t is C.c_double:
        return "f64"
    if t in (C.c_size_t, C.c_uint64):      # one ctypes class on this platform
        return "u64"
    if t is C.c_uint32:
        return "u32"
    return "address"       # c_void_p, c_char_p and POINTER(...) all carry an address


def test_ts_table_lists_every_header_symbol_with_the_headers_types():
    ts, hdr = ts_table(), header_table()
    assert sorted(ts) == sorted(hdr)
    assert len(ts) >= 70
    for name in hdr:
        assert ts[name] == hdr[name], f"{name}: hip_bindings.ts {ts[name]} != header {hdr[name]}"


def test_ts_table_agrees_with_the_ctypes_table():
    ts = ts_table()
    assert sorted(ts) == sorted(ffi.SIGNATURES)
    widen = {"pointer": "address", "buffer": "address", "usize": "u64"}
    for name, (argtypes, restype) in ffi.SIGNATURES.items():
        params, result = ts[name]
        assert [widen.get(p, p) for p in params] == [ctypes_kind(t) for t in argtypes], name
        assert widen.get(result, result) == ctypes_kind(restype), name


def test_generated_table_is_up_to_date():
    r = subprocess.run([sys.executable, os.path.join(TS_DIR, "gen_hip_bindings.py"), "--check"])
    assert r.returncode == 0, "run integration/jsgrad/gen_hip_bindings.py"


def split_args(s: str):
    """Top-level comma split of a call's argument text."""
    args, depth, cur = [], 0, ""
    for ch in s:
        if ch in "([{":
            depth += 1
        elif ch in ")]}":
            depth -= 1
        if ch == "," and depth == 0:
            args.append(cur)
            cur = ""
        else:
            cur += ch
    if cur.strip():
        args.append(cur)
    return args


def calls_in(path):
    """[(symbol, number of arguments)] of every `.jsgrad_hip_x(...)` call in a TypeScript file."""
    text = open(path).read()
    text = re.sub(r"//[^\n]*", "", text)
    out = []
    for m in re.finditer(r"\.(jsgrad_hip_\w+)\(", text):
        i, depth = m.end(), 1
        while depth:
            depth += {"(": 1, ")": -1}.get(text[i], 0)
            i += 1
        out.append((m.group(1), len(split_args(text[m.end(): i - 1]))))
    return out


@pytest.mark.parametrize("rel", ["runtime/ops_hip.ts", "engine/hip_lowerer.ts", "models/llama_hip.ts", "runtime/hip_bindings.ts"])
def test_ts_callers_use_existing_symbols_with_the_right_arity(rel):
    ts = ts_table()
    calls = calls_in(os.path.join(TS_DIR, rel))
    if rel != "runtime/hip_bindings.ts":
        assert calls, f"{rel} calls nothing"
    for name, nargs in calls:
        assert name in ts, f"{rel} calls {name}, which the table does not hold"
        assert nargs == len(ts[name][0]), f"{rel}: {name} called with {nargs} arguments, the header declares {len(ts[name][0])}"


def test_ts_files_hold_no_placeholders():
    for dirpath, _, files in os.walk(TS_DIR):
        for f in files:
            if f.endswith(".ts"):
                text = open(os.path.join(dirpath, f)).read()
                code = re.sub(r"//[^\n]*", "", text)
                assert "TODO" not in text and "see include" not in text, f
                assert not re.search(r"\.\.\.(?![\w\[(])", code), f"{f}: an ellipsis that is not a spread"
                assert code.count("{") == code.count("}") and code.count("(") == code.count(")") and code.count("[") == code.count("]"), f"{f}: unbalanced brackets"


def test_step_descriptor_layout_in_ts_is_the_c_layout(tmp_path):
    """pack_step of hip_bindings.ts writes at fixed offsets; they must be the ones gcc gives jsgrad_hip_step_t."""
    src = tmp_path / "layout.c"
    src.write_text('#include <stdio.h>\n#include <stddef.h>\n#include "jsgrad_hip.h"\n'
                   'int main(void){printf("%zu %zu %zu %zu %zu %zu %zu %zu %zu %zu", sizeof(jsgrad_hip_layer_t), sizeof(jsgrad_hip_step_t),'
                   'offsetof(jsgrad_hip_step_t, n_layers), offsetof(jsgrad_hip_step_t, eps), offsetof(jsgrad_hip_step_t, kind), offsetof(jsgrad_hip_step_t, tok_emb),'
                   'offsetof(jsgrad_hip_step_t, tokens_cap), offsetof(jsgrad_hip_step_t, h), offsetof(jsgrad_hip_step_t, workspace), offsetof(jsgrad_hip_step_t, trace));return 0;}\n')
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    got = [int(v) for v in subprocess.run([str(exe)], capture_output=True, text=True, check=True).stdout.split()]
    text = open(BINDINGS).read()
    fields = re.search(r"LAYER_FIELDS = \[([^\]]*)\]", text).group(1).count("'") // 2
    step_bytes = int(re.search(r"STEP_BYTES = (\d+)", text).group(1))
    assert got[0] == fields * 8 and got[1] == step_bytes
    # offsets the comments of pack_step state, in the order of the struct
    assert got[2:] == [8, 40, 44, 64, 128, 136, 184, 192]
    # and the ctypes mirror the GPU tests use has the same size
    assert C.sizeof(ffi.StepDesc) == step_bytes if hasattr(ffi, "StepDesc") else True
