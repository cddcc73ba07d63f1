"""ctypes prototypes of the C ABI declared in include/infmoe.h.

The library is looked for next to this package (infmoe_amd/lib/libinfmoe.so); it is never
built implicitly and there is no fallback: without it every entry point raises.
"""
from __future__ import annotations

import ctypes as C
import os

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libinfmoe.so")

OK = 0
ERR_INVALID_ARGUMENT, ERR_UNKNOWN_FIELD, ERR_MISSING_FIELD, ERR_UNSUPPORTED = 1, 2, 3, 4
ERR_IO, ERR_STATE, ERR_HIP, ERR_NAN = 5, 6, 7, 8
FIELD_FLOAT32, FIELD_INT32, FIELD_CHAR, FIELD_UNKNOWN = 1, 5, 6, 8
NORM_NONE, NORM_RMS, NORM_CENTERED = 0, 1, 2
FFN_RELU, FFN_GATED_GELU = 0, 1
NORM_KINDS = {"none": NORM_NONE, "rms": NORM_RMS, "centered": NORM_CENTERED}
FFN_KINDS = {"relu": FFN_RELU, "gated_gelu": FFN_GATED_GELU}


class Field(C.Structure):
    _fields_ = [("name", C.c_char_p), ("data", C.c_void_p), ("type", C.c_int32), ("length", C.c_int32)]


class InfMoEError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"infmoe status {status}: {message}")
        self.status = status
        self.message = message


_vp, _i32, _sz = C.c_void_p, C.c_int32, C.c_size_t
_pi32, _pf = C.POINTER(C.c_int32), C.c_void_p  # device pointers travel as integers

# name -> (restype, argtypes); every symbol include/infmoe.h declares
PROTOTYPES = {
    "infmoe_create": (_i32, [C.c_char_p, C.POINTER(Field), _i32, C.POINTER(_vp)]),
    "infmoe_clone": (_i32, [_vp, C.POINTER(_vp)]),
    "infmoe_set_expert_weights": (_i32, [_vp, _i32, C.c_char_p, _vp, _sz]),
    "infmoe_set_score_bias": (_i32, [_vp, _vp]),
    "infmoe_configure": (_i32, [_vp, _pi32, _i32]),
    "infmoe_workspace_size": (_i32, [_vp, _pi32, _i32, C.POINTER(_sz)]),
    "infmoe_initialize": (_i32, [_vp]),
    "infmoe_enqueue": (_i32, [_vp, _pi32, _i32, C.POINTER(_vp), C.POINTER(_vp), _vp, _vp]),
    "infmoe_terminate": (_i32, [_vp]),
    "infmoe_destroy": (None, [_vp]),
    "infmoe_last_routing": (_i32, [_vp, _pi32, _pi32]),
    "infmoe_last_streaming": (_i32, [_vp, _pi32, _pi32]),
    "infmoe_set_timing": (_i32, [_vp, _i32]),
    "infmoe_timing_history": (_i32, [_vp, _pf, _i32, _pi32]),
    "infmoe_last_timing": (_i32, [_vp, C.POINTER(C.c_float)]),
    "infmoe_serialization_size": (_i32, [_vp, C.POINTER(_sz)]),
    "infmoe_serialize": (_i32, [_vp, _vp, _sz]),
    "infmoe_deserialize": (_i32, [C.c_char_p, _vp, _sz, C.POINTER(_vp)]),
    "infmoe_npz_read_f32": (_i32, [C.c_char_p, C.c_char_p, _vp, _sz, _sz]),
    "infmoe_last_error": (C.c_char_p, []),
    "infmoe_plugin_name": (C.c_char_p, []),
    "infmoe_plugin_version": (C.c_char_p, []),
    "infmoe_gate_top1_scratch_bytes": (_sz, [_i32, _i32, _i32]),
    "infmoe_gate_top1": (_i32, [_i32, _i32, _i32, _pf, _pf, _pf, _i32, _pf, _vp, _pf, _vp, _vp, _vp]),
    "infmoe_expert_count_scratch_bytes": (_sz, [_i32, _i32]),
    "infmoe_expert_count": (_i32, [_i32, _i32, _vp, _vp, _vp, _vp, _vp, _vp]),
    "infmoe_expert_count_noalloc": (_i32, [_i32, _i32, _vp, _vp, _vp, _vp, _vp]),
    "infmoe_expert_scatter": (_i32, [_i32, _i32, _pf, _pf, _vp, _pf, _pf, _vp]),
    "infmoe_expert_gather": (_i32, [_i32, _i32, _pf, _vp, _pf, _vp]),
    "infmoe_expert_mix_gather": (_i32, [_i32, _i32, _vp, _pf, _pf, _pf, _pf, _vp]),
    "infmoe_layernorm": (_i32, [_pf, _pf, _i32, _i32, _pf, _i32, _vp]),
    "infmoe_t5ff_weight_bytes": (_sz, [_i32, _i32, _i32]),
    "infmoe_t5ff_workspace_bytes": (_sz, [_i32, _i32, _i32, _i32]),
    "infmoe_t5ff_run": (_i32, [_i32, _i32, _i32, _i32, _i32, _vp, _pf, _pf, _vp, _vp]),
}

_lib = None


def load(path: str | None = None) -> C.CDLL:
    """dlopen the library and attach prototypes.  Raises if it has not been built."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    path = path or LIB_PATH
    if not os.path.isfile(path):
        raise FileNotFoundError(
            f"{path} not found: build it with `python -m infmoe_amd.build` (there is no CPU fallback)")
    lib = C.CDLL(path, mode=C.RTLD_GLOBAL)
    for name, (restype, argtypes) in PROTOTYPES.items():
        fn = getattr(lib, name)  # AttributeError if a declared symbol is not exported
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(status: int) -> None:
    if status != OK:
        raise InfMoEError(status, load().infmoe_last_error().decode("utf-8", "replace"))
