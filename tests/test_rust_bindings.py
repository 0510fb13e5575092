"""rust/cutile-hip-sys/src/lib.rs against include/cutile_hip.h, declaration by declaration.

The image has no Rust toolchain, so nothing compiles the crate here.  Instead both files are read by the small readers
below (independent of the generator's) into one neutral description — per function: name, return class, and per
argument a class such as ("ptr", const, pointee) / ("int", bits, signed) / ("float", bits) / ("fnptr", n) — and the
two descriptions must be equal.  Record layouts are checked three ways: the header's, as the C compiler lays them out
(a probe program built with gcc prints sizeof / offsetof); the Rust file's, laid out by the repr(C) rules; and the
ctypes records of the Python binding.  What the reference has in this place: cuda-bindings/src/lib.rs:16 (generated
declarations) under cuda-core/src/cudarc_shim.rs:28-807.
"""
import ctypes as C
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "cutile_hip.h")
CRATE = os.path.join(ROOT, "rust", "cutile-hip-sys")
LIB_RS = os.path.join(CRATE, "src", "lib.rs")

C_INT = {"int8_t": (8, True), "uint8_t": (8, False), "int16_t": (16, True), "uint16_t": (16, False), "int32_t": (32, True),
         "uint32_t": (32, False), "int64_t": (64, True), "uint64_t": (64, False), "size_t": (64, False), "int": (32, True),
         "char": (8, True), "unsigned char": (8, False)}
R_INT = {"i8": (8, True), "u8": (8, False), "i16": (16, True), "u16": (16, False), "i32": (32, True), "u32": (32, False),
         "i64": (64, True), "u64": (64, False), "usize": (64, False), "isize": (64, True), "c_int": (32, True), "c_uint": (32, False),
         "c_char": (8, True)}


# ---------------------------------------------------------------------------------------------- the C side
def _c_text():
    t = open(HEADER).read()
    t = re.sub(r"/\*.*?\*/", " ", t, flags=re.S)
    t = re.sub(r"//[^\n]*", " ", t)
    t = re.sub(r"^[ \t]*#[ \t]*(?:if|ifdef|ifndef|endif|else|include)\b[^\n]*$", " ", t, flags=re.M)
    return t.replace('extern "C" {', " ")


class CSide:
    def __init__(self):
        t = _c_text()
        self.defines = {m.group(1): int(m.group(2), 0) for m in re.finditer(r"#\s*define\s+(\w+)\s+(-?\d\w*)\s*\n", t)}
        self.opaque = dict((m.group(2), m.group(1)) for m in re.finditer(r"typedef\s+struct\s+(\w+)\s*\*\s*(\w+)\s*;", t))
        self.alias = {}
        for m in re.finditer(r"typedef\s+([\w\s]+?\**)\s*(\w+)\s*;", t):
            if m.group(2) not in self.opaque and "struct" not in m.group(1) and "enum" not in m.group(1):
                self.alias[m.group(2)] = " ".join(m.group(1).split())
        self.fnptr = {m.group(2): (m.group(1).strip(), self._params(m.group(3)))
                      for m in re.finditer(r"typedef\s+([\w\s\*]+?)\(\s*\*\s*(\w+)\s*\)\s*\(([^)]*)\)\s*;", t)}
        self.enums, self.consts = set(), {}
        for m in re.finditer(r"(typedef\s+)?enum\s*\{([^}]*)\}\s*(\w*)\s*;", t):
            if m.group(3):
                self.enums.add(m.group(3))
            nxt = 0
            for e in filter(None, (x.strip() for x in m.group(2).split(","))):
                if "=" in e:
                    e, v = (x.strip() for x in e.split("="))
                    nxt = int(v, 0)
                self.consts[e] = nxt
                nxt += 1
        self.structs = {}
        for m in re.finditer(r"typedef\s+struct\s*\{([^}]*)\}\s*(\w+)\s*;", t):
            fields = []
            for f in filter(None, (x.strip() for x in m.group(1).split(";"))):
                names = f.split(",")
                head = re.match(r"^(.*?)(\w+)\s*(\[\s*\w+\s*\])?$", names[0].strip())
                ty = head.group(1).strip()
                for j, nm in enumerate(names):
                    nmm = re.match(r"^(?:.*?)(\w+)\s*(?:\[\s*(\w+)\s*\])?$", nm.strip())
                    fields.append((nmm.group(1), ty, nmm.group(2)))
            self.structs[m.group(2)] = fields
        body = re.sub(r"^[ \t]*#[ \t]*define\b[^\n]*$", " ", t, flags=re.M)
        body = re.sub(r"typedef[^;{]*(\{[^}]*\})?[^;]*;", " ", body)
        body = re.sub(r"enum\s*\{[^}]*\}\s*;", " ", body)
        self.functions = {}
        for m in re.finditer(r"([\w\s\*]+?)\b(cutile_\w+)\s*\(([^)]*)\)\s*;", body):
            self.functions[m.group(2)] = (self.classify(m.group(1).strip()), [self.classify(*p) for p in self._params(m.group(3))])

    @staticmethod
    def _params(text):
        text = text.strip()
        if text in ("", "void"):
            return []
        out = []
        for p in text.split(","):
            m = re.match(r"^(.*?)(\w+)\s*(\[\s*\w*\s*\])?$", p.strip())
            out.append((m.group(1).strip(), m.group(3) is not None))
        return out

    def dim(self, d):
        return self.defines[d] if d in self.defines else int(d, 0)

    def classify(self, ty, is_array=False):
        ty = " ".join(ty.replace("*", " * ").split())
        if is_array:
            ty += " *"
        toks = ty.split(" ")
        const = "const" in toks[:2] and (toks[0] == "const" or toks[1] == "const")
        toks = [x for i, x in enumerate(toks) if not (x == "const" and i < 2 and "*" not in toks[:i])]
        base = toks[0]
        rest = toks[1:]
        if base == "unsigned" and rest and rest[0] in ("char", "int"):
            base, rest = base + " " + rest[0], rest[1:]
        cls = self._base(base)
        pointee_const = const
        for tok in rest:
            if tok == "*":
                cls = ("ptr", pointee_const, cls)
                pointee_const = False
            elif tok == "const":
                pointee_const = True
            else:
                raise AssertionError(f"cannot classify C type {ty!r}")
        return cls

    def _base(self, base):
        if base == "void":
            return ("void",)
        if base in C_INT:
            return ("int",) + C_INT[base]
        if base == "float":
            return ("float", 32)
        if base == "double":
            return ("float", 64)
        if base in self.enums:
            return ("int", 32, True)
        if base in self.opaque:
            return ("ptr", False, ("opaque", self.opaque[base]))
        if base in self.fnptr:
            ret, params = self.fnptr[base]
            return ("fnptr", self.classify(ret), tuple(self.classify(*p) for p in params))
        if base in self.structs:
            return ("struct", base)
        if base in self.alias:
            return self.classify(self.alias[base])
        raise AssertionError(f"unknown C type {base!r}")


# ---------------------------------------------------------------------------------------------- the Rust side
class RustSide:
    def __init__(self):
        t = open(LIB_RS).read()
        t = re.sub(r"//[^\n]*", "", t)
        self.consts = {m.group(1): (m.group(2), int(m.group(3))) for m in re.finditer(r"pub const (\w+): (\w+) = (-?\d+);", t)}
        self.alias = {m.group(1): m.group(2).strip() for m in re.finditer(r"pub type (\w+) = ([^;]+);", t)}
        self.structs, self.opaque = {}, set()
        for m in re.finditer(r"#\[repr\(C\)\]\s*(?:#\[derive\([^)]*\)\]\s*)?pub struct (\w+) \{([^}]*)\}", t):
            fields = [(f.group(1), f.group(2).strip()) for f in re.finditer(r"(?:pub )?(\w+): ([^,\n]+),", m.group(2))]
            if [n for n, _ in fields] == ["_private"]:
                self.opaque.add(m.group(1))
            else:
                self.structs[m.group(1)] = fields
        ext = re.search(r'extern "C" \{(.*?)\n\}', t, flags=re.S).group(1)
        self.functions = {}
        for m in re.finditer(r"pub fn (\w+)\((.*?)\)( -> ([^;]+))?;", ext):
            args = [a.split(":", 1)[1].strip() for a in self._split(m.group(2))]
            self.functions[m.group(1)] = (self.classify(m.group(4).strip()) if m.group(4) else ("void",), [self.classify(a) for a in args])

    @staticmethod
    def _split(text):
        out, depth, cur = [], 0, ""
        for ch in text:
            if ch in "([<":
                depth += 1
            elif ch in ")]>":
                depth -= 1
            if ch == "," and depth == 0:
                out.append(cur)
                cur = ""
            else:
                cur += ch
        if cur.strip():
            out.append(cur)
        return out

    def classify(self, ty):
        ty = ty.strip()
        if ty.startswith("*const "):
            return ("ptr", True, self.classify(ty[7:]))
        if ty.startswith("*mut "):
            return ("ptr", False, self.classify(ty[5:]))
        m = re.match(r'^Option<unsafe extern "C" fn\((.*)\)( -> (.+))?>$', ty)
        if m:
            args = tuple(self.classify(a.split(":", 1)[1]) for a in self._split(m.group(1)))
            return ("fnptr", self.classify(m.group(3)) if m.group(3) else ("void",), args)
        if ty in ("c_void", "()"):
            return ("void",)
        if ty in R_INT:
            return ("int",) + R_INT[ty]
        if ty == "f32":
            return ("float", 32)
        if ty == "f64":
            return ("float", 64)
        if ty in self.opaque:
            return ("opaque", ty)
        if ty in self.structs:
            return ("struct", ty)
        if ty in self.alias:
            return self.classify(self.alias[ty])
        raise AssertionError(f"unknown Rust type {ty!r}")

    def layout(self, ty):
        """(size, align) under repr(C) on x86-64 / LP64"""
        ty = ty.strip()
        m = re.match(r"^\[(.+); (\w+)\]$", ty)
        if m:
            size, align = self.layout(m.group(1))
            n = self.consts[m.group(2)][1] if m.group(2) in self.consts else int(m.group(2))
            return size * n, align
        if ty.startswith(("*const ", "*mut ", "Option<unsafe extern")):
            return 8, 8
        if ty in R_INT:
            return R_INT[ty][0] // 8, R_INT[ty][0] // 8
        if ty in ("f32", "f64"):
            return int(ty[1:]) // 8, int(ty[1:]) // 8
        if ty in self.structs:
            return self.struct_layout(ty)[:2]
        if ty in self.alias:
            return self.layout(self.alias[ty])
        raise AssertionError(f"no layout for {ty!r}")

    def struct_layout(self, name):
        off, max_align, offsets = 0, 1, []
        for fname, fty in self.structs[name]:
            size, align = self.layout(fty)
            off = (off + align - 1) // align * align
            offsets.append((fname, off, size))
            off += size
            max_align = max(max_align, align)
        return (off + max_align - 1) // max_align * max_align, max_align, offsets


@pytest.fixture(scope="module")
def c_side():
    return CSide()


@pytest.fixture(scope="module")
def rust_side():
    return RustSide()


def test_generated_file_is_current():
    """src/lib.rs is what gen_bindings.py makes of today's header (nobody edited one without the other)"""
    res = subprocess.run([sys.executable, os.path.join(CRATE, "gen_bindings.py"), "--check"], stderr=subprocess.PIPE, text=True)
    assert res.returncode == 0, res.stderr


def test_same_functions_with_the_same_argument_classes(c_side, rust_side):
    assert len(c_side.functions) >= 150
    assert set(c_side.functions) == set(rust_side.functions)
    for name, (c_ret, c_args) in c_side.functions.items():
        r_ret, r_args = rust_side.functions[name]
        assert c_ret == r_ret, (name, "return", c_ret, r_ret)
        assert len(c_args) == len(r_args), (name, len(c_args), len(r_args))
        for i, (a, b) in enumerate(zip(c_args, r_args)):
            assert a == b, (name, i, a, b)


def test_every_export_of_the_header_is_a_symbol_of_the_library_and_of_the_crate(c_side, rust_side):
    lib = os.path.join(ROOT, "cutile-rs_amd", "lib", "libcutile_hip.so")
    if not os.path.exists(lib):
        pytest.skip("library not built")
    dll = C.CDLL(lib)
    for name in rust_side.functions:
        assert hasattr(dll, name), name


def test_constants_agree(c_side, rust_side):
    for name, value in c_side.consts.items():
        assert name in rust_side.consts and rust_side.consts[name][1] == value, name
    for name, value in c_side.defines.items():
        assert rust_side.consts[name][1] == value, name
    # a named enum's constants carry the enum's type; it is a C int
    assert rust_side.consts["CUTILE_DTYPE_BF16"][0] == "cutile_dtype_t" and rust_side.alias["cutile_dtype_t"] == "c_int"
    assert rust_side.consts["CUTILE_ERR_OUT_OF_SLOTS"] == ("i32", -7)


def test_records_have_the_same_fields_in_the_same_order(c_side, rust_side):
    assert set(c_side.structs) == set(rust_side.structs) and len(c_side.structs) == 8
    for name, fields in c_side.structs.items():
        r_fields = rust_side.structs[name]
        assert [f[0] for f in fields] == [f[0] for f in r_fields], name
        for (fname, cty, dim), (_, rty) in zip(fields, r_fields):
            m = re.match(r"^\[(.+); (\w+)\]$", rty)
            if dim is None:
                assert m is None, (name, fname)
                assert c_side.classify(cty) == rust_side.classify(rty), (name, fname)
            else:
                assert m is not None, (name, fname)
                n = rust_side.consts[m.group(2)][1] if m.group(2) in rust_side.consts else int(m.group(2))
                assert n == c_side.dim(dim) and c_side.classify(cty) == rust_side.classify(m.group(1)), (name, fname)


def test_record_layouts_match_what_the_c_compiler_gives(c_side, rust_side, tmp_path):
    """sizeof / offsetof from gcc on the header itself, against the repr(C) layout of the Rust records and the ctypes
    records of the Python binding"""
    lines = ['#include <stdio.h>', '#include <stddef.h>', f'#include "{HEADER}"', "int main(void) {"]
    for name, fields in c_side.structs.items():
        lines.append(f'  printf("{name} %zu\\n", sizeof({name}));')
        for fname, _, _ in fields:
            lines.append(f'  printf("{name}.{fname} %zu\\n", offsetof({name}, {fname}));')
    lines += ["  return 0;", "}"]
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.check_call(["gcc", "-std=c99", "-o", str(exe), str(src)])
    got = dict(l.split() for l in subprocess.check_output([str(exe)], text=True).splitlines())
    for name in c_side.structs:
        size, _, offsets = rust_side.struct_layout(name)
        assert size == int(got[name]), (name, size, got[name])
        for fname, off, _ in offsets:
            assert off == int(got[f"{name}.{fname}"]), (name, fname)
    import __graft_entry__ as entry

    ct = entry.load_package()
    for py, cname in ((ct.TensorArg, "cutile_tensor_arg_t"), (ct.PartitionArg, "cutile_partition_arg_t"), (ct.LaunchOpts, "cutile_launch_opts_t")):
        assert C.sizeof(py) == int(got[cname]), cname


def test_the_crate_has_its_manifest_and_build_script():
    manifest = open(os.path.join(CRATE, "Cargo.toml")).read()
    assert 'name = "cutile-hip-sys"' in manifest and 'links = "cutile_hip"' in manifest
    build = open(os.path.join(CRATE, "build.rs")).read()
    assert "rustc-link-lib=dylib=cutile_hip" in build and "CUTILE_HIP_LIB_DIR" in build
