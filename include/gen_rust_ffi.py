"""Prints the Rust `extern "C"` block for every entry point that tract_rocm.h declares.

Usage: ``python include/gen_rust_ffi.py`` (the block goes to stdout; the integration notes at the repository
root hold a copy, and tests/test_abi_cpu.py checks that copy against the header, name by name and argument by argument).
"""
from __future__ import annotations

import os
import re

HERE = os.path.dirname(os.path.abspath(__file__))

SCALARS = {"int": "c_int", "int64_t": "i64", "size_t": "usize", "float": "f32", "uint64_t": "u64", "unsigned": "c_uint",
           "void": "c_void", "char": "c_char"}
RUST_KEYWORDS = {"type", "ref", "in", "move", "match", "loop", "mod", "fn", "use", "box"}


def declarations(header_text: str):
    """[(name, return C type, [(C type, parameter name), ...])] in header order."""
    text = re.sub(r"/\*.*?\*/", "", header_text, flags=re.S)
    text = re.sub(r"^\s*#.*$", "", text, flags=re.M)
    out = []
    for m in re.finditer(r"([A-Za-z_][A-Za-z0-9_ \*]*?)\b(trocm_[a-z0-9_]+)\s*\(([^;{}]*?)\)\s*;", text, flags=re.S):
        ret, name, params = m.group(1).strip(), m.group(2), " ".join(m.group(3).split())
        if ret.startswith("typedef"):
            continue
        plist = []
        if params and params != "void":
            for prm in params.split(","):
                prm = prm.strip()
                pm = re.match(r"^(.*?)([A-Za-z_][A-Za-z0-9_]*)$", prm)
                plist.append((pm.group(1).strip(), pm.group(2)))
        out.append((name, ret, plist))
    return out


def rust_type(ctype: str) -> str:
    """C parameter type -> Rust FFI type: `const T *const *` reads right to left."""
    toks = re.findall(r"\*|const|[A-Za-z_][A-Za-z0-9_]*", ctype)
    base = [t for t in toks if t not in ("*", "const")]
    assert len(base) == 1, ctype
    rust = SCALARS.get(base[0], base[0])   # opaque structs keep their names
    stars = [i for i, t in enumerate(toks) if t == "*"]
    if not stars:
        return rust
    # constness of the pointee at each level: a `const` directly before the base or directly after a star
    pointee_const = "const" in toks[:stars[0]]
    for idx, si in enumerate(stars):
        rust = ("*const " if pointee_const else "*mut ") + rust
        nxt = stars[idx + 1] if idx + 1 < len(stars) else len(toks)
        pointee_const = "const" in toks[si + 1:nxt]
    return rust


def rust_block(header_text: str) -> str:
    lines = ['extern "C" {']
    for name, ret, params in declarations(header_text):
        args = ", ".join(f"{(p + '_') if p in RUST_KEYWORDS else p}: {rust_type(t)}" for t, p in params)
        r = rust_type(ret)
        lines.append(f"    pub fn {name}({args}) -> {r};")
    lines.append("}")
    return "\n".join(lines)


if __name__ == "__main__":
    print(rust_block(open(os.path.join(HERE, "tract_rocm.h")).read()))
