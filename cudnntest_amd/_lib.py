"""ctypes binding of libwino_amd.so (the C ABI declared in include/wino_amd.h).

The library is the product; there is no fallback: if it is missing, loading
raises and every operator fails.
"""
import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
# WINO_AMD_LIB selects another build of the same library (kernel experiments)
LIB_PATH = os.environ.get("WINO_AMD_LIB") or os.path.join(_HERE, "libwino_amd.so")
CSRC = os.path.join(_HERE, "csrc")

_vp = ctypes.c_void_p
_i = ctypes.c_int
_u = ctypes.c_uint
_l = ctypes.c_long



class StackLayer(ctypes.Structure):
    """wino_stack_layer_t"""
    _fields_ = [("K", _i), ("layout_in", _i), ("layout_out", _i), ("flags", _u), ("algo", _i)]


_ip = ctypes.POINTER(_i)

# every symbol include/wino_amd.h declares: name -> (restype, argtypes)
SYMBOLS = {
    "wino_stack_create": (_i, [_i] * 6 + [ctypes.POINTER(StackLayer), ctypes.POINTER(_vp)]),
    "wino_stack_set_layer": (_i, [_vp, _i, _vp, _vp, _vp]),
    "wino_stack_output": (_i, [_vp, _ip, _ip, _ip, _ip, _ip]),
    "wino_stack_forward": (_i, [_vp, _vp, _vp, _vp]),
    "wino_stack_forward_graph": (_i, [_vp, _vp, _vp, _vp]),
    "wino_stack_destroy": (_i, [_vp]),
    "wino_conv": (_i, [_i, _i, _i, _i, _u] + [_i] * 6 + [_vp, _vp, _vp, _vp]),
    "wino_conv_prepared": (_i, [_i, _i, _i, _i, _u] + [_i] * 6 + [_vp, _vp, _vp, _vp]),
    "wino_conv_ex": (_i, [_i, _i, _i, _i, _u] + [_i] * 6 + [_vp, _vp, _vp, _vp, _vp]),
    "wino_conv_prepared_ex": (_i, [_i, _i, _i, _i, _u] + [_i] * 6 + [_vp, _vp, _vp, _vp, _vp]),
    "wino_conv_noalloc": (_i, [_i, _i, _i, _i, _u] + [_i] * 6 + [_vp, _vp, _vp, _vp, _vp]),
    "wino_pick_algo": (_i, [_i] * 8),
    "wino_geometry": (_i, [_i] * 7 + [ctypes.POINTER(_i), ctypes.POINTER(_i), ctypes.POINTER(_l),
                                     ctypes.POINTER(_i), ctypes.POINTER(_i), ctypes.POINTER(_l)]),
    "wino_workspace_bytes": (ctypes.c_size_t, [_i] * 7),
    "wino_set_workspace": (_i, [_vp, ctypes.c_size_t]),
    "wino_filter_transform": (_i, [_i, _i, _i, _i, _vp, _vp, _vp]),
    "wino_input_transform": (_i, [_i] * 8 + [_vp, _vp, _vp]),
    "wino_batched_gemm": (_i, [_i, _i, _i, _i, _l, _vp, _vp, _vp, _vp]),
    "wino_output_transform": (_i, [_i, _i, _i, _i, _u, _i, _i, _i, _i, _vp, _vp, _vp]),
    "wino_gemm_output": (_i, [_i, _i, _i, _u, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp]),
    "wino_f4_geometry": (_i, [_i] * 7 + [ctypes.POINTER(_i), ctypes.POINTER(_i), ctypes.POINTER(_l),
                                        ctypes.POINTER(_i), ctypes.POINTER(_i), ctypes.POINTER(_l)]),
    "wino_f4_filter_transform": (_i, [_i, _i, _i, _i, _vp, _vp, _vp]),
    "wino_f4_input_transform": (_i, [_i] * 8 + [_vp, _vp, _vp]),
    "wino_f4_batched_gemm": (_i, [_i, _i, _i, _i, _l, _vp, _vp, _vp, _vp]),
    "wino_f4_output_transform": (_i, [_i, _i, _i, _i, _u, _i, _i, _i, _i, _vp, _vp, _vp]),
    "wino_f4_gemm_output": (_i, [_i, _i, _i, _u, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp]),
    "wino_layout_transform": (_i, [_i] * 7 + [_vp, _vp, _vp]),
    "wino_stage_timing": (_i, [_i]),
    "wino_stage_times": (_i, [ctypes.POINTER(ctypes.c_float), ctypes.POINTER(_l)]),
    "wino_stage_stats": (_i, [ctypes.POINTER(ctypes.c_float)] * 3 + [ctypes.POINTER(_l)]),
    "wino_warmup": (_i, []),
    "wino_sync": (_i, [_vp]),
    "wino_last_error": (ctypes.c_char_p, []),
    "wino_version": (ctypes.c_char_p, []),
}

_lib = None


def build():
    """Compile the HIP sources for gfx950 (hipcc cross-compiles without a GPU)."""
    subprocess.check_call(["make", "-s", "-B", "-C", CSRC])
    return LIB_PATH


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `make -C {CSRC}` (there is no non-HIP fallback)")
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


class WinoError(RuntimeError):
    def __init__(self, code, what):
        msg = load().wino_last_error().decode()
        super().__init__(f"{what} failed with status {code}: {msg}")
        self.code = code


def check(code, what):
    if code != 0:
        raise WinoError(code, what)
