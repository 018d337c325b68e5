"""Writes src/lib.rs of the foundry_attn_sys crate from include/foundry_attn.h (the single source of truth of the
boundary): every exported function as an `extern "C"` declaration, every struct as `#[repr(C)]` with its fields in the
header's order, every enumerator as a constant.

    python ffi/foundry_attn_sys/generate.py            # rewrites src/lib.rs
    python ffi/foundry_attn_sys/generate.py --check    # exit 1 if src/lib.rs is not what the header gives

The header's grammar is small (no function pointers, no nested structs, no bit-fields), so a few regular expressions
read it. No Rust toolchain is needed to run this; the crate itself was not compiled in the image this library is
built in (it has no rustc).
"""
import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
HEADER = os.path.join(HERE, "..", "..", "include", "foundry_attn.h")
OUT = os.path.join(HERE, "src", "lib.rs")

SCALARS = {"int": "c_int", "uint32_t": "u32", "uint64_t": "u64", "int32_t": "i32", "uint16_t": "u16", "size_t": "usize",
           "float": "f32", "double": "f64", "char": "c_char", "void": "c_void", "fa_status": "fa_status"}


def strip_comments(text):
    return re.sub(r"/\*.*?\*/", " ", text, flags=re.S)


def rust_type(base, const, stars, known):
    """C `const base ***` -> Rust."""
    t = SCALARS.get(base)
    if t is None:
        if base not in known:
            raise ValueError("unknown C type %r" % base)
        t = base
    for i in range(stars):
        t = ("*const " if (const and i == 0) else "*mut ") + t
    return t


def parse(text):
    """-> (opaque, enums, defines, structs, functions) in header order."""
    text = strip_comments(text)
    opaque = re.findall(r"typedef\s+struct\s+(\w+)\s+(\w+)\s*;", text)
    opaque = [a for a, b in opaque if a == b]
    enums = []
    for body, name in re.findall(r"typedef\s+enum\s+\w*\s*\{(.*?)\}\s*(\w+)\s*;", text, flags=re.S):
        items = [(k, int(v, 0)) for k, v in re.findall(r"(\w+)\s*=\s*(-?\w+)", body)]
        enums.append((name, items))
    defines = [(k, int(v.rstrip("uU"), 0)) for k, v in re.findall(r"#define\s+(FA_\w+)\s+(\d+[uU]?)\s*$", text, flags=re.M)]
    structs = []
    for body, name in re.findall(r"typedef\s+struct\s+\w+\s*\{(.*?)\}\s*(\w+)\s*;", text, flags=re.S):
        fields = []
        for decl in [d.strip() for d in body.split(";") if d.strip()]:
            m = re.match(r"(const\s+)?(\w+)\s+(.*)$", decl, flags=re.S)
            const, base, rest = bool(m.group(1)), m.group(2), m.group(3)
            for d in [x.strip() for x in rest.split(",")]:
                dm = re.match(r"(\**)\s*(\w+)\s*(?:\[(\d+)\])?$", d)
                stars, fname, arr = len(dm.group(1)), dm.group(2), dm.group(3)
                fields.append((fname, base, const, stars, int(arr) if arr else 0))
        structs.append((name, fields))
    functions = []
    no_types = re.sub(r"typedef\s+(struct|enum)\s+\w*\s*\{.*?\}\s*\w+\s*;", " ", text, flags=re.S)
    for ret, name, args in re.findall(r"^\s*((?:const\s+)?\w+\s*\**)\s*\b(fa_\w+)\s*\(([^;{}]*?)\)\s*;", no_types, flags=re.S | re.M):
        rm = re.match(r"(const\s+)?(\w+)\s*(\**)", ret.strip())
        params = []
        if args.strip() != "void":
            for a in [x.strip() for x in args.split(",")]:
                am = re.match(r"(const\s+)?(\w+)\s*(\**)\s*(\w+)$", " ".join(a.split()))
                params.append((am.group(4), am.group(2), bool(am.group(1)), len(am.group(3))))
        functions.append((name, (rm.group(2), bool(rm.group(1)), len(rm.group(3))), params))
    return opaque, enums, defines, structs, functions


RUST_KEYWORDS = {"type", "in", "ref", "fn", "mod", "use", "match", "move", "box", "as", "loop", "where", "self"}


def ident(name):
    return "r#" + name if name in RUST_KEYWORDS else name


def render(parsed):
    opaque, enums, defines, structs, functions = parsed
    known = set(opaque) | {n for n, _ in structs} | {n for n, _ in enums}
    o = []
    o.append("//! Raw FFI declarations of libfoundry_attn.so: the KV-cache attention path of metallic-foundry (KvPrepFused,")
    o.append("//! FlashAttention and the ops either side of them) on AMD MI355X. GENERATED from include/foundry_attn.h by")
    o.append("//! ffi/foundry_attn_sys/generate.py - edit the header, not this file. The header's comments name, for every entry")
    o.append("//! point, the interface of crates/metallic-foundry it stands in for.")
    o.append("#![allow(non_camel_case_types, non_upper_case_globals)]")
    o.append("use std::os::raw::{c_char, c_int, c_void};")
    o.append("")
    o.append("/// 0 = ok; the other values are the variants of MetalError this path raises (src/error.rs:22-75).")
    o.append("pub type fa_status = i32;")
    for name, items in enums:
        if name == "fa_status":
            o.append("")
        else:
            o.append("")
            o.append("pub type %s = u32;" % name)
        ty = "fa_status" if name == "fa_status" else name
        for k, v in items:
            o.append("pub const %s: %s = %d;" % (k, ty, v))
    if defines:
        o.append("")
        for k, v in defines:
            o.append("pub const %s: u32 = %d;" % (k, v))
    for name in opaque:
        o.append("")
        o.append("#[repr(C)]")
        o.append("pub struct %s {" % name)
        o.append("    _private: [u8; 0],")
        o.append("}")
    for name, fields in structs:
        o.append("")
        o.append("#[repr(C)]")
        o.append("#[derive(Clone, Copy, Debug)]")
        o.append("pub struct %s {" % name)
        for fname, base, const, stars, arr in fields:
            t = rust_type(base, const, stars, known)
            if arr:
                t = "[%s; %d]" % (t, arr)
            o.append("    pub %s: %s," % (ident(fname), t))
        o.append("}")
    o.append("")
    o.append('#[link(name = "foundry_attn")]')
    o.append('extern "C" {')
    for name, (rbase, rconst, rstars), params in functions:
        ps = ", ".join("%s: %s" % (ident(p), rust_type(b, c, s, known)) for p, b, c, s in params)
        ret = "" if (rbase == "void" and rstars == 0) else " -> " + rust_type(rbase, rconst, rstars, known)
        line = "    pub fn %s(%s)%s;" % (name, ps, ret)
        if len(line) <= 120:
            o.append(line)
        else:
            o.append("    pub fn %s(" % name)
            for p, b, c, s in params:
                o.append("        %s: %s," % (ident(p), rust_type(b, c, s, known)))
            o.append("    )%s;" % ret)
    o.append("}")
    return "\n".join(o) + "\n"


def main():
    text = render(parse(open(HEADER).read()))
    if "--check" in sys.argv:
        if not os.path.exists(OUT) or open(OUT).read() != text:
            sys.stderr.write("src/lib.rs is out of date: run ffi/foundry_attn_sys/generate.py\n")
            return 1
        return 0
    os.makedirs(os.path.dirname(OUT), exist_ok=True)
    open(OUT, "w").write(text)
    return 0


if __name__ == "__main__":
    sys.exit(main())
