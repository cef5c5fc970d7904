"""ctypes front end of libagh_calib.so: the calibration launches of `bench.py --calib` (an MFMA-only loop, copy / read /
read:write-mix streams).  Measurement code, not part of the product package: `autograph_amd` never imports this."""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libagh_calib.so")
if not os.path.exists(LIB_PATH):
    raise ImportError(f"{LIB_PATH} is missing: build it with `make -C {_HERE}` (or __graft_entry__.build())")
lib = C.CDLL(LIB_PATH)

_p, _i, _z = C.c_void_p, C.c_int, C.c_size_t
SIGNATURES = {
    "calib_mfma_bf16": [_p, _p, _i, _i, _i, _i],
    "calib_copy": [_p, _p, _p, _z, _i],
    "calib_read": [_p, _p, _p, _z, _i],
    "calib_mix": [_p, _p, _p, _z, _i, _i],
    "calib_mfma_dma": [_p, _p, _z, _p, _i, _z, _i, _i],
}
for _name, _args in SIGNATURES.items():
    _f = getattr(lib, _name)
    _f.argtypes = _args
    _f.restype = C.c_int
lib.calib_last_error_string.restype = C.c_char_p


class CalibError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(f"[{code}] {msg}")
        self.code = code


def check(code):
    if code != 0:
        raise CalibError(code, lib.calib_last_error_string().decode(errors="replace"))
