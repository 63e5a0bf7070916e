#!/usr/bin/env python3
"""Generates hip/source/dopt/hip/shim.d, the extern(C) D binding of libdopthip.so, from the C headers
include/dopt_hip.h and include/dopt_hip_plan.h: one D prototype per C prototype, the structs, enums
and callback types they use, nothing else.

    python hip/gen_shim.py            # rewrites shim.d
    python hip/gen_shim.py --check    # exit 1 if shim.d is not what the headers give

The headers keep to a small subset of C (plain scalars, pointers, three structs, two enums, two
function-pointer typedefs), which is all this translator understands; it refuses anything else.
"""
import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
HEADERS = [os.path.join(ROOT, "include", "dopt_hip.h"), os.path.join(ROOT, "include", "dopt_hip_plan.h")]
OUT = os.path.join(HERE, "source", "dopt", "hip", "shim.d")

SCALARS = {"int": "int", "unsigned": "uint", "size_t": "size_t", "float": "float", "double": "double", "void": "void",
           "char": "char", "int32_t": "int", "uint32_t": "uint", "uint64_t": "ulong", "unsigned char": "ubyte"}
D_KEYWORDS = {"in", "out", "ref", "function", "delegate", "module", "import", "version", "debug", "body", "alias"}


def strip_comments(text):
    return re.sub(r"/\*.*?\*/", " ", text, flags=re.S)


def d_type(c, structs):
    """'const float *const *' -> 'const(float*)*' etc."""
    c = " ".join(c.replace("*", " * ").split())
    toks = c.split(" ")
    stars = toks.count("*")
    words = [t for t in toks if t != "*"]
    # `const` binds to what is left of it unless it comes first
    base_words = [w for w in words if w not in ("const", "struct")]
    base = " ".join(base_words)
    if base in SCALARS:
        d = SCALARS[base]
    elif base in structs:
        d = base
    else:
        raise ValueError("unknown C type %r" % c)
    if stars == 0:
        return d
    # walk the declarator left to right: [const] base * [const] * ...
    pos, out, pending_const = 0, d, False
    seq = toks
    first_const = seq[0] == "const"
    i = 1 if first_const else 0
    # skip base words
    while i < len(seq) and seq[i] != "*":
        if seq[i] == "const":
            first_const = True
        i += 1
    if first_const:
        out = "const(%s)" % out
    while i < len(seq):
        if seq[i] == "*":
            out += "*"
        elif seq[i] == "const":       # const pointer
            out = "const(%s)" % out
        i += 1
    return out


def d_name(n):
    return n + "_" if n in D_KEYWORDS else n


def parse(text):
    text = strip_comments(text)
    text = re.sub(r"#.*", "", text)
    text = text.replace('extern "C" {', "").replace("}\n", "}\n")
    items = []
    structs = {}
    # enums
    for m in re.finditer(r"(typedef\s+)?enum\s*\{(.*?)\}\s*(\w*)\s*;", text, flags=re.S):
        names = []
        for part in m.group(2).split(","):
            part = part.strip()
            if not part:
                continue
            k, _, v = part.partition("=")
            names.append((k.strip(), v.strip()))
        items.append(("enum", m.group(3), names))
    text = re.sub(r"(typedef\s+)?enum\s*\{.*?\}\s*\w*\s*;", "", text, flags=re.S)
    # function-pointer typedefs
    fptrs = []
    for m in re.finditer(r"typedef\s+(\w[\w\s\*]*?)\(\*(\w+)\)\s*\((.*?)\)\s*;", text, flags=re.S):
        fptrs.append((m.group(2), m.group(1).strip(), m.group(3)))
    text = re.sub(r"typedef\s+\w[\w\s\*]*?\(\*\w+\)\s*\(.*?\)\s*;", "", text, flags=re.S)
    # structs
    for m in re.finditer(r"typedef\s+struct\s*\w*\s*\{(.*?)\}\s*(\w+)\s*;", text, flags=re.S):
        structs[m.group(2)] = m.group(1)
    text = re.sub(r"typedef\s+struct\s*\w*\s*\{.*?\}\s*\w+\s*;", "", text, flags=re.S)
    known = set(structs) | {n for n, _, _ in fptrs}

    def params(plist):
        plist = " ".join(plist.split())
        if plist in ("", "void"):
            return []
        out = []
        for p in plist.split(","):
            p = p.strip()
            m = re.match(r"(.*?)(\w+)$", p)
            ctype, name = m.group(1).strip(), m.group(2)
            if not ctype:        # unnamed parameter
                ctype, name = p, "arg%d" % len(out)
            out.append((d_type(ctype, known), d_name(name)))
        return out

    for name, body in structs.items():
        fields = []
        for decl in body.split(";"):
            decl = " ".join(decl.split())
            if not decl:
                continue
            fm = re.match(r"(\w[\w\s\*]*?)\(\*(\w+)\)\s*\((.*)\)$", decl)
            if fm:   # function-pointer member
                ps = ", ".join("%s %s" % p for p in params(fm.group(3)))
                fields.append("%s function(%s) %s" % (d_type(fm.group(1).strip(), known), ps, d_name(fm.group(2))))
                continue
            tm = re.match(r"(.*?)([\w\s,\*]+)$", decl)
            # "size_t N, C, H, W" or "const float *partial"
            first = re.match(r"((?:const\s+)?(?:unsigned\s+)?\w+)\s*(.*)$", decl)
            ctype, rest = first.group(1), first.group(2)
            for piece in rest.split(","):
                piece = piece.strip()
                stars = piece.count("*")
                nm = piece.replace("*", "").strip()
                am = re.match(r"(\w+)\s*\[(\d+)\]$", nm)
                if am:   # a fixed-size array member: `int dims[4]` is `int[4] dims` in D
                    fields.append("%s[%s] %s" % (d_type(ctype + " " + "*" * stars, known), am.group(2), d_name(am.group(1))))
                    continue
                fields.append("%s %s" % (d_type(ctype + " " + "*" * stars, known), d_name(nm)))
        items.append(("struct", name, fields))
    for name, ret, plist in fptrs:
        ps = ", ".join("%s %s" % p for p in params(plist))
        items.append(("fptr", name, "%s function(%s)" % (d_type(ret, known), ps)))
    # prototypes
    for m in re.finditer(r"([\w][\w\s\*]*?)\b(dopt_hip_\w+)\s*\(([^;{}]*?)\)\s*;", text, flags=re.S):
        ret, name, plist = m.group(1).strip(), m.group(2), m.group(3)
        ps = ", ".join("%s %s" % p for p in params(plist))
        items.append(("func", name, "%s %s(%s);" % (d_type(ret, known), name, ps)))
    return items


def render():
    out = ["/**", "    extern(C) binding of libdopthip.so, the MI355X kernel library and host mirror behind the dopt.hip backend.",
           "    ",
           "    GENERATED by hip/gen_shim.py from include/dopt_hip.h and include/dopt_hip_plan.h: one declaration per C",
           "    declaration, in header order.  What each function does, and which call site of the reference's CUDA backend",
           "    it replaces, is documented in those headers.  Written where no D compiler exists: never compiled.", "*/",
           "module dopt.hip.shim;", "", "extern(C) @nogc nothrow:", ""]
    for path in HEADERS:
        out.append("// ---- %s" % os.path.relpath(path, ROOT))
        for kind, name, payload in parse(open(path).read()):
            if kind == "enum":
                if name:   # a C enum is an int whose enumerators are visible unqualified
                    out.append("alias %s = int;" % name)
                out.append("enum\n{")
                for k, v in payload:
                    out.append("    %s%s," % (k, " = " + v if v else ""))
                out.append("}")
                out.append("")
            elif kind == "struct":
                out.append("struct %s\n{" % name)
                out.extend("    %s;" % f for f in payload)
                out.append("}")
                out.append("")
            elif kind == "fptr":
                out.append("alias %s = %s;" % (name, payload))
            else:
                out.append(payload)
        out.append("")
    return "\n".join(out).rstrip("\n") + "\n"


def main():
    text = render()
    if "--check" in sys.argv:
        same = os.path.exists(OUT) and open(OUT).read() == text
        sys.exit(0 if same else 1)
    if "--print" in sys.argv:
        sys.stdout.write(text)
        return
    os.makedirs(os.path.dirname(OUT), exist_ok=True)
    with open(OUT, "w") as f:
        f.write(text)


if __name__ == "__main__":
    main()
