"""Writes the symbol table of integration/jsgrad/runtime/hip_bindings.ts from include/jsgrad_hip.h.

    python integration/jsgrad/gen_hip_bindings.py          # rewrite the table in place
    python integration/jsgrad/gen_hip_bindings.py --check  # exit 1 if the file is out of date

Mapping of C types to Deno FFI types (what jsgrad's env.dlopen takes, /root/reference/dawn/bindings.ts:5-8):
a pointer parameter whose name starts with `host_`, and any `char *`, is host memory -> 'buffer'; every other pointer
is a device address or an opaque handle -> 'pointer'; int / int32_t -> 'i32'; uint32_t -> 'u32'; float -> 'f32';
double -> 'f64'; size_t -> 'usize'; uint64_t -> 'u64'.
"""
import os
import re
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
HEADER = os.path.join(ROOT, "include", "jsgrad_hip.h")
TARGET = os.path.join(ROOT, "integration", "jsgrad", "runtime", "hip_bindings.ts")
SCALARS = {"uint64_t": "U64", "int": "I", "int32_t": "I", "uint32_t": "U32", "float": "F", "double": "D", "size_t": "U"}


def declarations(text: str):
    """[(name, return C type, [(C type, parameter name)])] in header order."""
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    out = []
    for ret, name, params in re.findall(r"([\w \*]+?)\b(jsgrad_hip_\w+)\s*\(([^)]*)\)\s*;", text):
        plist = []
        params = " ".join(params.split())
        if params != "void":
            for p in params.split(","):
                m = re.match(r"\s*(.*?)(\w+)\s*(\[\d*\])?\s*$", p)
                ctype = m.group(1).strip() + ("*" if m.group(3) else "")
                plist.append((ctype, m.group(2)))
        out.append((name, ret.strip(), plist))
    return out


def ffi_type(ctype: str, pname: str) -> str:
    if "*" in ctype:
        return "B" if pname.startswith("host_") or "char" in ctype else "P"
    base = ctype.replace("const", "").replace("unsigned", "").strip()
    return SCALARS[base]


def result_type(ctype: str) -> str:
    return "P" if "*" in ctype else SCALARS[ctype.replace("const", "").strip()]


def table(decls) -> str:
    lines = ["const SYMBOLS = {"]
    for name, ret, params in decls:
        types = ", ".join(ffi_type(t, n) for t, n in params)
        names = ", ".join(n for _, n in params)
        lines.append(f"  {name}: {{ parameters: [{types}], result: {result_type(ret)} }},{' // ' + names if names else ''}")
    lines.append("} as const")
    return "\n".join(lines)


def render(ts: str, decls) -> str:
    head, rest = ts.split("// <symbols>\n", 1)
    _, tail = rest.split("// </symbols>", 1)
    return head + "// <symbols>\n" + table(decls) + "\n// </symbols>" + tail


if __name__ == "__main__":
    decls = declarations(open(HEADER).read())
    old = open(TARGET).read()
    new = render(old, decls)
    if "--check" in sys.argv:
        sys.exit(0 if new == old else 1)
    open(TARGET, "w").write(new)
    print(f"{len(decls)} symbols -> {os.path.relpath(TARGET, ROOT)}")
