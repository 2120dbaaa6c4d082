"""Generates the raw Rust bindings of the C ABI (`dflash-hip-sys/src/lib.rs`) from `include/dflash_hip.h`.

The reference engine is Rust; this is the `-sys` crate its maintainers would link (constants, `#[repr(C)]` structs and
the `extern "C"` block, one item per declaration of the header, in the header's order).  The header is written in a
regular subset of C (opaque struct typedefs, anonymous enums, typedef'd plain structs, prototypes), which is all this
parser understands; anything else raises.  Run:  python qwen-llm_amd/rust/gen_sys.py  (rewrites lib.rs);
`--check` exits non-zero if lib.rs is not what the header generates."""
import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
HEADER = os.path.join(HERE, "..", "..", "include", "dflash_hip.h")
OUT = os.path.join(HERE, "dflash-hip-sys", "src", "lib.rs")

PRIM = {"int8_t": "i8", "uint8_t": "u8", "int16_t": "i16", "uint16_t": "u16", "int32_t": "i32", "uint32_t": "u32",
        "int64_t": "i64", "uint64_t": "u64", "size_t": "usize", "float": "f32", "double": "f64", "char": "c_char",
        "void": "c_void", "int": "i32"}
KEYWORDS = {"type", "dyn", "in", "ref", "loop", "match", "move", "fn", "impl", "box", "mod", "use", "self", "super", "where",
            "as", "let", "mut", "pub", "trait", "struct", "enum", "unsafe", "extern", "crate", "const", "static", "yield"}


def strip_comments(text):
    return re.sub(r"/\*.*?\*/", " ", text, flags=re.S)


def ident(name):
    return name + "_" if name in KEYWORDS else name


class Gen:
    def __init__(self, text):
        self.consts, self.opaque, self.structs, self.funcs, self.aliases = [], [], [], [], {}
        self.order = []
        self.parse(strip_comments(text))

    def rust_type(self, base, stars, consts):
        """base: C type name; stars: number of pointer levels; consts[i]: whether level i (0 = the base) is const."""
        if base in self.aliases and stars == 0:
            return self.aliases[base]
        t = self.aliases.get(base) or PRIM.get(base) or base
        if base not in PRIM and base not in self.aliases and base not in self.opaque and base not in [s[0] for s in self.structs]:
            raise ValueError(f"unknown type {base}")
        for level in range(stars):
            t = ("*const " if consts[level] else "*mut ") + t
        return t

    def parse_decl(self, decl):
        """'const float *a, *b' or 'int32_t x[16]' -> [(name, rust type)] (several declarators share the base type)."""
        decl = decl.strip()
        m = re.match(r"(const\s+)?(struct\s+)?(\w+)\s*(.*)$", decl, flags=re.S)
        base_const, base, rest = bool(m.group(1)), m.group(3), m.group(4)
        out = []
        for d in [x.strip() for x in rest.split(",")]:
            dm = re.match(r"((?:\*\s*(?:const\s*)?)*)\s*(\w+)?\s*((?:\[[^\]]+\])*)$", d)
            if not dm:
                raise ValueError(f"cannot parse declarator {d!r} in {decl!r}")
            ptrs, name, arrays = dm.group(1), dm.group(2), dm.group(3)
            levels = re.findall(r"\*\s*(const)?", ptrs)
            # constness of what each pointer level points at: level 0 points at the base
            consts = [base_const] + [bool(c) for c in levels[:-1]] if levels else []
            t = self.rust_type(base, len(levels), consts)
            for dim in reversed(re.findall(r"\[([^\]]+)\]", arrays)):
                dim = dim.strip()
                t = f"[{t}; {dim if dim.isdigit() else dim + ' as usize'}]"
            out.append((name, t))
        return out

    def parse(self, text):
        text = re.sub(r"^\s*#.*$", lambda m: self.define(m.group(0)), text, flags=re.M)
        text = text.replace('extern "C" {', "").strip()
        pos = 0
        while pos < len(text):
            m = re.compile(r"\s*").match(text, pos)
            pos = m.end()
            if pos >= len(text) or text[pos] == "}":
                pos += 1
                continue
            if text.startswith("enum", pos):
                end = text.index("};", pos)
                body = text[text.index("{", pos) + 1:end]
                nxt = 0
                for item in [x.strip() for x in body.split(",") if x.strip()]:
                    name, _, val = item.partition("=")
                    nxt = int(val.strip(), 0) if val.strip() else nxt
                    self.consts.append((name.strip(), "i32", nxt))
                    self.order.append(("const", len(self.consts) - 1))
                    nxt += 1
                pos = end + 2
            elif text.startswith("typedef struct {", pos):
                end = text.index("}", pos)
                body = text[text.index("{", pos) + 1:end]
                semi = text.index(";", end)
                name = text[end + 1:semi].strip()
                fields = []
                for line in [x.strip() for x in body.split(";") if x.strip()]:
                    fields.extend(self.parse_decl(line))
                self.structs.append((name, fields))
                self.order.append(("struct", len(self.structs) - 1))
                pos = semi + 1
            elif text.startswith("typedef", pos):
                semi = text.index(";", pos)
                stmt = text[pos:semi]
                m = re.match(r"typedef\s+struct\s+(\w+)\s+(\w+)$", stmt.strip())
                if m:
                    self.opaque.append(m.group(2))
                    self.order.append(("opaque", len(self.opaque) - 1))
                else:
                    m = re.match(r"typedef\s+void\s*\*\s*(\w+)$", stmt.strip())
                    if not m:
                        raise ValueError(f"unsupported typedef: {stmt}")
                    self.aliases[m.group(1)] = "*mut c_void"
                pos = semi + 1
            else:
                semi = text.index(";", pos)
                stmt = " ".join(text[pos:semi].split())
                m = re.match(r"(.*?)(\w+)\s*\((.*)\)$", stmt)
                if not m:
                    raise ValueError(f"unsupported statement: {stmt}")
                ret, name, params = m.group(1).strip(), m.group(2), m.group(3).strip()
                rt = None if ret == "void" else self.parse_decl(ret + " _")[0][1]
                args = [] if params in ("void", "") else [self.parse_decl(p)[0] for p in params.split(",")]
                self.funcs.append((name, args, rt))
                self.order.append(("fn", len(self.funcs) - 1))
                pos = semi + 1

    def define(self, line):
        m = re.match(r"\s*#define\s+(\w+)\s+(-?\d+)\s*$", line)
        if m:
            self.consts.append((m.group(1), "i64", int(m.group(2))))
            self.order.append(("const", len(self.consts) - 1))
        return ""

    def emit(self):
        L = ["//! Raw bindings of `libdflash_hip.so` (the C ABI of `include/dflash_hip.h`): generated by",
             "//! `qwen-llm_amd/rust/gen_sys.py`, one item per declaration of the header, in its order.  Do not edit.",
             "#![allow(non_camel_case_types, non_upper_case_globals)]",
             "use std::os::raw::{c_char, c_void};", ""]
        in_extern = False

        def close():
            nonlocal in_extern
            if in_extern:
                L.append("}")
                L.append("")
                in_extern = False

        for kind, i in self.order:
            if kind == "fn":
                if not in_extern:
                    L.append('extern "C" {')
                    in_extern = True
                name, args, rt = self.funcs[i]
                a = ", ".join(f"{ident(n)}: {t}" for n, t in args)
                L.append(f"    pub fn {name}({a}){' -> ' + rt if rt else ''};")
                continue
            close()
            if kind == "const":
                name, t, v = self.consts[i]
                L.append(f"pub const {name}: {t} = {v};")
            elif kind == "opaque":
                L.append("#[repr(C)]")
                L.append(f"pub struct {self.opaque[i]} {{ _private: [u8; 0] }}")
            elif kind == "struct":
                name, fields = self.structs[i]
                L.append("#[repr(C)]")
                L.append("#[derive(Clone, Copy)]")
                L.append(f"pub struct {name} {{")
                for n, t in fields:
                    L.append(f"    pub {ident(n)}: {t},")
                L.append("}")
        close()
        return "\n".join(L).rstrip() + "\n"


def generate():
    return Gen(open(HEADER).read()).emit()


if __name__ == "__main__":
    text = generate()
    if "--check" in sys.argv:
        sys.exit(0 if os.path.exists(OUT) and open(OUT).read() == text else 1)
    with open(OUT, "w") as f:
        f.write(text)
    print(f"wrote {OUT}: {text.count('pub fn ')} functions, {text.count('pub struct ')} structs")
