"""CPU-side checks of the boundary: the shared library loads and exports every symbol the
header declares, and argument errors come back as status codes without a GPU."""
import ctypes as C
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    text = open(os.path.join(ROOT, "include", "autograph_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(agh_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from autograph_amd import _ffi
    syms = header_symbols()
    assert len(syms) >= 30
    for s in syms:
        assert hasattr(_ffi.lib, s), f"{s} declared in the header but not exported"
    # and the ctypes table covers the header exactly
    assert sorted(_ffi.SIGNATURES) == syms


def test_calls_before_init_fail_with_status_not_crash():
    from autograph_amd import _ffi
    p = C.c_void_p()
    rc = _ffi.lib.agh_malloc(C.byref(p), 16)
    if rc == 0:  # a GPU is present and another test initialised the library
        _ffi.lib.agh_free(p)
        return
    assert rc == -2  # AGH_ENOINIT
    assert b"agh_init" in _ffi.lib.agh_last_error_string()
    assert _ffi.lib.agh_gemm_f32(1, 1, 1, 1.0, None, 0, 1, 1, None, 0, 1, 1, 0.0, None, 0, 1, 1) == -2


def test_option_shape_formulas():
    from autograph_amd import Col2ImConv2Options, Im2ColConv2Options, MaxPool2Options
    import oracle as orc
    o = Im2ColConv2Options(filter=(3, 5), padding=(1, 0), stride=(2, 1), dilation=(1, 2))
    assert o.output_shape((9, 14)) == (orc.conv_out(9, 3, 1, 2, 1), orc.conv_out(14, 5, 0, 1, 2))
    c = Col2ImConv2Options(shape=(5, 6), filter=(3, 5), padding=(1, 0), stride=(2, 1), dilation=(1, 2))
    assert c.output_shape() == (orc.col2im_out(5, 3, 1, 2, 1), orc.col2im_out(6, 5, 0, 1, 2))
    assert MaxPool2Options((2, 3), (2, 2)).output_shape((9, 8)) == (orc.pool_out(9, 2, 2), orc.pool_out(8, 3, 2))


_C_TO_RUST = {"int": "c_int", "int64_t": "i64", "float": "f32", "size_t": "usize", "char": "c_char", "void": "c_void"}


def _rust_type_of(ctype):
    """The Rust FFI spelling of a C parameter type: pointers keep their depth and the constness of the pointee."""
    const = re.search(r"\bconst\b", ctype) is not None
    base = re.sub(r"\bconst\b|\*", " ", ctype).split()
    assert len(base) == 1, ctype
    out = _C_TO_RUST[base[0]]
    for level in range(ctype.count("*")):
        out = ("*const " if const and level == 0 else "*mut ") + out
    return out


def test_rust_sys_crate_declares_the_header():
    """rust/autograph-hip-sys/src/lib.rs (source only, no Rust toolchain here) must declare every entry
    point of the header with the same argument TYPES in the same order (int64_t <-> i64, int <-> c_int,
    float <-> f32, size_t <-> usize, pointers with their constness and depth) and the same return type."""
    text = open(os.path.join(ROOT, "include", "autograph_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    c_decls = {}
    for ret, name, args in re.findall(r"^\s*([a-z_0-9 ]+?\s*\**)\s*\b(agh_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", text, flags=re.M):
        types = []
        if args.strip() not in ("", "void"):
            for a in args.split(","):
                a = " ".join(a.split())
                types.append(_rust_type_of(re.sub(r"[A-Za-z_][A-Za-z_0-9]*$", "", a)))  # drop the parameter name
        c_decls[name] = (types, _rust_type_of(ret))
    rs = open(os.path.join(ROOT, "rust", "autograph-hip-sys", "src", "lib.rs")).read()
    rs_decls = {}
    for name, args, ret in re.findall(r"pub fn (agh_[a-z0-9_]+)\(([^)]*)\) -> ([^;]+);", rs):
        types = [a.split(":", 1)[1].strip() for a in args.split(",")] if args.strip() else []
        rs_decls[name] = (types, ret.strip())
    assert sorted(rs_decls) == sorted(c_decls)
    for name in c_decls:
        assert rs_decls[name] == c_decls[name], name
    assert sorted(c_decls) == header_symbols()
    # the ctypes table agrees too (same width and kind per argument)
    from autograph_amd import _ffi
    kind = {"c_int": C.c_int, "i64": C.c_int64, "f32": C.c_float, "usize": C.c_size_t}
    for name, (types, _) in c_decls.items():
        argtypes = _ffi.SIGNATURES[name][0]
        assert len(argtypes) == len(types), name
        for t, ct in zip(types, argtypes):
            if t.startswith("*"):
                assert C.sizeof(ct) == C.sizeof(C.c_void_p) and not issubclass(ct, (C.c_int64, C.c_size_t, C.c_float)) or ct is C.c_void_p, (name, t, ct)
            else:
                assert ct is kind[t] or (C.sizeof(ct) == C.sizeof(kind[t]) and ct._type_ == kind[t]._type_), (name, t, ct)
