#!/usr/bin/env python3
"""Prints the Rust `extern "C"` block that binds every function declared in rstorch_hip.h.

    python include/gen_rust_extern.py            # the block, as it stands in the integration notes
    python include/gen_rust_extern.py --check    # exit 1 if the notes' block is out of date

The reference crate is Rust; this image has no Rust toolchain, so the block is generated from the C
header (the one source of truth for the ABI) instead of being typed by hand, and tests/test_abi.py
checks that the documentation carries exactly this text."""
import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
HEADER = os.path.join(HERE, "rstorch_hip.h")
INTEGRATION = os.path.join(os.path.dirname(HERE), "INTEGRATION.md")

OPAQUE = {"rst_engine": "RstEngine", "rst_model": "RstModel", "rst_event": "RstEvent",
          "rst_stager": "RstStager", "rst_kernel_record": "RstKernelRecord"}
SCALARS = {"int": "c_int", "double": "f64", "size_t": "usize", "uint64_t": "u64", "uint32_t": "u32",
           "char": "c_char", "void": "c_void"}


def rust_type(c):
    """'const double* const*' -> '*const *const f64' (pointers read right to left)."""
    c = c.strip()
    toks = re.findall(r"\*|const|[A-Za-z_][A-Za-z0-9_]*", c)
    base, quals, i = None, [], 0
    # leading qualifiers and the base type
    const_base = False
    while i < len(toks) and toks[i] != "*":
        if toks[i] == "const":
            const_base = True
        else:
            base = toks[i]
        i += 1
    ty = OPAQUE.get(base) or SCALARS[base]
    pointee_const = const_base
    while i < len(toks):
        assert toks[i] == "*"
        i += 1
        ty = ("*const " if pointee_const else "*mut ") + ty
        pointee_const = False
        if i < len(toks) and toks[i] == "const":
            pointee_const = True
            i += 1
    return ty


def declarations():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = text[text.index('extern "C" {'):]
    out = []
    for m in re.finditer(r"([A-Za-z_][A-Za-z0-9_ ]*?\**)\s*\b(rst_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", text):
        ret, name, args = m.group(1).strip(), m.group(2), m.group(3).strip()
        params = []
        if args and args != "void":
            for a in args.split(","):
                a = " ".join(a.split())
                pm = re.match(r"(.*?)([A-Za-z_][A-Za-z0-9_]*)$", a)
                params.append((pm.group(2), rust_type(pm.group(1))))
        out.append((name, params, rust_type(ret)))
    return out


def block():
    lines = ["extern \"C\" {"]
    for name, params, ret in declarations():
        sig = ", ".join("%s: %s" % (("r#%s" % n) if n in ("type", "ref", "move") else n, t) for n, t in params)
        line = "    pub fn %s(%s) -> %s;" % (name, sig, ret)
        if len(line) > 100:
            line = "    pub fn %s(\n        %s,\n    ) -> %s;" % (name, ",\n        ".join(
                "%s: %s" % (n, t) for n, t in params), ret)
        lines.append(line)
    lines.append("}")
    return "\n".join(lines)


if __name__ == "__main__":
    if "--check" in sys.argv:
        sys.exit(0 if block() in open(INTEGRATION).read() else 1)
    print(block())
