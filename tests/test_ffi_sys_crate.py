"""CPU: the Rust `-sys` crate (ffi/foundry_attn_sys/src/lib.rs) agrees with include/foundry_attn.h and with what
libfoundry_attn.so exports. No Rust toolchain is involved: the Rust text is read with this file's own small parser, the C
side comes from the C compiler (struct sizes and field offsets of the real header) and from the dynamic symbol table, and
the two are compared. The checker is then run on deliberately broken copies of the crate text (a dropped function, a
dropped argument, two swapped struct fields, a changed field type) and has to reject each."""
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "foundry_attn.h")
CRATE = os.path.join(ROOT, "ffi", "foundry_attn_sys")
LIB_RS = os.path.join(CRATE, "src", "lib.rs")
LIB_SO = os.path.join(ROOT, "test-burn_amd", "libfoundry_attn.so")

# Rust scalar -> (size, alignment) on x86-64 / aarch64 Linux (LP64)
RUST_SCALARS = {"u8": (1, 1), "i8": (1, 1), "u16": (2, 2), "u32": (4, 4), "i32": (4, 4), "u64": (8, 8), "usize": (8, 8),
                "f32": (4, 4), "f64": (8, 8), "c_int": (4, 4), "c_char": (1, 1), "fa_status": (4, 4)}
# C parameter type (spaces squeezed) -> the Rust spelling it must have
C_TO_RUST = {"int": "c_int", "uint32_t": "u32", "uint64_t": "u64", "int32_t": "i32", "uint16_t": "u16", "size_t": "usize",
             "float": "f32", "double": "f64", "char": "c_char", "void": "c_void", "fa_status": "fa_status"}


# ------------------------------------------------------------------------------------------------ Rust side
def rust_parse(text):
    """-> (structs {name: [(field, type)]}, functions {name: ([arg types], return type or None)})"""
    text = re.sub(r"//[^\n]*", "", text)
    structs = {}
    for name, body in re.findall(r"#\[repr\(C\)\](?:\s*#\[[^\]]*\])*\s*pub struct (\w+)\s*\{(.*?)\}", text, flags=re.S):
        structs[name] = [(f, " ".join(t.split())) for f, t in re.findall(r"(?:pub\s+)?(\w+)\s*:\s*([^,]+),", body)]
    block = re.search(r'extern "C"\s*\{(.*)\}', text, flags=re.S).group(1)
    functions = {}
    for name, args, ret in re.findall(r"pub fn (\w+)\s*\((.*?)\)\s*(?:->\s*([^;]+?))?\s*;", block, flags=re.S):
        types = [" ".join(a.split(":", 1)[1].split()) for a in args.split(",") if ":" in a]
        functions[name] = (types, " ".join(ret.split()) if ret else None)
    return structs, functions


def rust_layout(fields, structs):
    """repr(C) layout: [(field, offset)], size."""
    def size_align(t):
        m = re.match(r"\[(.+); (\d+)\]$", t)
        if m:
            s, a = size_align(m.group(1))
            return s * int(m.group(2)), a
        if t.startswith("*const ") or t.startswith("*mut "):
            return 8, 8
        if t in RUST_SCALARS:
            return RUST_SCALARS[t]
        if t in structs:
            _, size, align = rust_layout(structs[t], structs)
            return size, align
        raise AssertionError("no layout rule for Rust type %r" % t)

    off, out, amax = 0, [], 1
    for f, t in fields:
        s, a = size_align(t)
        off = (off + a - 1) // a * a
        out.append((f, off))
        off += s
        amax = max(amax, a)
    return out, (off + amax - 1) // amax * amax, amax


# ------------------------------------------------------------------------------------------------ C side
def c_prototypes():
    """Function prototypes of the header, by this file's own reading: {name: ([arg types in Rust spelling], return)}."""
    text = re.sub(r"/\*.*?\*/", " ", open(HEADER).read(), flags=re.S)
    text = re.sub(r"typedef\s+(?:struct|enum)\s+\w*\s*\{.*?\}\s*\w+\s*;", " ", text, flags=re.S)
    text = re.sub(r"^\s*#.*$", " ", text, flags=re.M)
    body = text[text.index('extern "C" {') + len('extern "C" {'):]
    out = {}
    for stmt in body.split(";"):
        stmt = " ".join(stmt.split())
        m = re.match(r"(.+?)\b(fa_\w+) ?\((.*)\)$", stmt)
        if not m or stmt.startswith("typedef"):
            continue

        def spell(decl, has_name):
            toks = decl.replace("*", " * ").split()
            if has_name:
                toks = toks[:-1]
            const = toks[0] == "const"
            base = toks[1] if const else toks[0]
            stars = toks.count("*")
            t = C_TO_RUST.get(base, base)
            for i in range(stars):
                t = ("*const " if const and i == 0 else "*mut ") + t
            return t

        ret = spell(m.group(1), False)
        args = [] if m.group(3).strip() == "void" else [spell(a, True) for a in m.group(3).split(",")]
        out[m.group(2)] = (args, None if ret == "c_void" else ret)
    return out


def c_struct_layouts(struct_fields):
    """Compiles the real header and asks the C compiler for sizeof / offsetof of every field the Rust side names."""
    src = ["#include <stdio.h>", "#include <stddef.h>", '#include "foundry_attn.h"', "int main(void) {"]
    for name, fields in struct_fields.items():
        src.append('printf("S %s %%zu\\n", sizeof(%s));' % (name, name))
        for f, _ in fields:
            src.append('printf("F %s %s %%zu\\n", offsetof(%s, %s));' % (name, f, name, f))
    src.append("return 0; }")
    import tempfile
    with tempfile.TemporaryDirectory() as d:
        c, exe = os.path.join(d, "layout.c"), os.path.join(d, "layout")
        open(c, "w").write("\n".join(src))
        subprocess.check_call(["gcc", "-std=c99", "-I", os.path.join(ROOT, "include"), c, "-o", exe])
        lines = subprocess.check_output([exe], text=True).splitlines()
    sizes, offsets = {}, {}
    for ln in lines:
        p = ln.split()
        if p[0] == "S":
            sizes[p[1]] = int(p[2])
        else:
            offsets.setdefault(p[1], []).append((p[2], int(p[3])))
    return sizes, offsets


def c_struct_names():
    text = re.sub(r"/\*.*?\*/", " ", open(HEADER).read(), flags=re.S)
    return re.findall(r"typedef\s+struct\s+\w+\s*\{.*?\}\s*(\w+)\s*;", text, flags=re.S)


def exported_symbols():
    out = subprocess.check_output(["nm", "-D", "--defined-only", LIB_SO], text=True)
    return {ln.split()[-1] for ln in out.splitlines() if " T fa_" in ln}


# ------------------------------------------------------------------------------------------------ the check
def problems(rust_text):
    """Every disagreement between the crate text and the C side, as strings."""
    bad = []
    structs, functions = rust_parse(rust_text)
    protos = c_prototypes()
    for name in sorted(set(protos) - set(functions)):
        bad.append("function %s is declared in the header but not in lib.rs" % name)
    for name in sorted(set(functions) - set(protos)):
        bad.append("function %s is declared in lib.rs but not in the header" % name)
    for name in sorted(set(protos) & set(functions)):
        (ca, cr), (ra, rr) = protos[name], functions[name]
        if len(ca) != len(ra):
            bad.append("%s: %d arguments in the header, %d in lib.rs" % (name, len(ca), len(ra)))
        elif ca != ra:
            bad.append("%s: argument types differ: header %s, lib.rs %s" % (name, ca, ra))
        if cr != rr:
            bad.append("%s: return type %s in the header, %s in lib.rs" % (name, cr, rr))
    cnames = c_struct_names()
    data_structs = {n: f for n, f in structs.items() if not (len(f) == 1 and f[0][0] == "_private")}
    for name in sorted(set(cnames) - set(data_structs)):
        bad.append("struct %s is in the header but not in lib.rs" % name)
    for name in sorted(set(data_structs) - set(cnames)):
        bad.append("struct %s is in lib.rs but not in the header" % name)
    common = {n: data_structs[n] for n in cnames if n in data_structs}
    try:
        sizes, offsets = c_struct_layouts(common)
    except subprocess.CalledProcessError:
        bad.append("lib.rs names a struct field the header does not have (the C layout program does not compile)")
        return bad
    for name, fields in common.items():
        lay, size, _ = rust_layout(fields, structs)
        if lay != offsets.get(name, []):
            bad.append("struct %s: field offsets differ: C %s, Rust %s" % (name, offsets.get(name), lay))
        if size != sizes[name]:
            bad.append("struct %s: sizeof %d in C, %d by the Rust layout (a field is missing or has another type)" % (name, sizes[name], size))
    return bad


def test_sys_crate_matches_header():
    assert problems(open(LIB_RS).read()) == []


def test_sys_crate_covers_every_export():
    _, functions = rust_parse(open(LIB_RS).read())
    exported = exported_symbols()
    assert set(functions) == exported, (sorted(set(functions) - exported), sorted(exported - set(functions)))


def test_sys_crate_is_what_the_generator_writes():
    assert subprocess.call([sys.executable, os.path.join(CRATE, "generate.py"), "--check"]) == 0


@pytest.mark.parametrize("what", ["dropped function", "dropped argument", "swapped fields", "field type", "extra function"])
def test_checker_rejects_broken_crates(what):
    text = open(LIB_RS).read()
    if what == "dropped function":
        broken = re.sub(r"    pub fn fa_u32_add\(.*?;\n", "", text, flags=re.S)
    elif what == "dropped argument":
        broken = text.replace("kv_seq_len: u32, m: u32, kv_head_major: c_int", "kv_seq_len: u32, kv_head_major: c_int")
        if broken == text:
            broken = re.sub(r"(pub fn fa_flash_attention\(.*?)        m: u32,\n", r"\1", text, flags=re.S)
    elif what == "swapped fields":
        broken = text.replace("    pub seq_len: u32,\n    pub position_offset: u32,", "    pub position_offset: u32,\n    pub seq_len: u32,")
    elif what == "field type":
        broken = text.replace("    pub offset: usize,", "    pub offset: u32,")
    else:
        broken = text.replace('extern "C" {', 'extern "C" {\n    pub fn fa_not_in_the_header(ctx: *mut fa_ctx) -> fa_status;')
    assert broken != text
    assert problems(broken), what
