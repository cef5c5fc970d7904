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


def test_rust_sys_crate_declares_the_header():
    """rust/autograph-hip-sys/src/lib.rs (source only, no Rust toolchain here) must declare every entry
    point of the header with the same number of arguments."""
    text = open(os.path.join(ROOT, "include", "autograph_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    c_decls = {n: (0 if a.strip() in ("", "void") else a.count(",") + 1)
               for n, a in re.findall(r"\b(agh_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", text)}
    rs = open(os.path.join(ROOT, "rust", "autograph-hip-sys", "src", "lib.rs")).read()
    rs_decls = {n: (0 if not a.strip() else a.count(",") + 1) for n, a in re.findall(r"pub fn (agh_[a-z0-9_]+)\(([^)]*)\)", rs)}
    assert rs_decls == c_decls
    assert sorted(c_decls) == header_symbols()
