"""ctypes loader of oracle/libmoe_cpu.so (the C/OpenMP restatement; test infrastructure only)."""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libmoe_cpu.so")
_lib = None
NORM = {"none": 0, "rms": 1, "centered": 2}
FFN = {"relu": 0, "gated_gelu": 1}


def load():
    global _lib
    if _lib is None:
        if not os.path.isfile(LIB):
            raise FileNotFoundError(f"{LIB} not built: run `make -C oracle`")
        _lib = C.CDLL(LIB)
        _lib.moe_cpu_threads.restype = C.c_int
        _lib.moe_cpu_layer.restype = C.c_int
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def pack_slot(w, ffn_kind):
    keys = ("layer_norm_weight", "wi_0_weight", "wi_1_weight", "wo_weight") if ffn_kind == "gated_gelu" \
        else ("layer_norm_weight", "wi_weight", "wo_weight")
    return np.concatenate([np.asarray(w[k], np.float32).ravel() for k in keys])


def layer(x, centroids, variant, slots, *, gamma=None, bias=None, h=0, norm_kind="rms", ffn_kind="relu"):
    """slots: list of packed float32 expert slots, or None for the Identity sub-layer.
    Returns (y [T,d] float32, sel int32[T], count int32[E])."""
    lib = load()
    x = np.ascontiguousarray(x, np.float32)
    centroids = np.ascontiguousarray(centroids, np.float32)
    T, d = x.shape
    E = centroids.shape[0]
    y = np.empty_like(x)
    sel = np.empty(T, np.int32)
    count = np.empty(E, np.int32)
    ln_before, mix = {"cpm_2": (1, 0), "base_layer": (0, 1), "default": (0, 0)}[variant]
    wptr = None
    if slots is not None:
        wptr = (C.c_void_p * E)(*[s.ctypes.data for s in slots])
    g = None if gamma is None else np.ascontiguousarray(gamma, np.float32)
    b = None if bias is None else np.ascontiguousarray(bias, np.float32)
    rc = lib.moe_cpu_layer(T, d, h, E, _p(x), _p(centroids), _p(g), _p(b), ln_before, mix, NORM[norm_kind],
                           FFN[ffn_kind], wptr, _p(y), _p(sel), _p(count))
    if rc != 0:
        raise FloatingPointError("row with no orderable score (NaN)")
    return y, sel, count
