"""ctypes front end of the CPU oracle (oracle/wino_oracle.c).

Test infrastructure only: imported by tests/, by the smoke test and by the
benchmark's CPU-baseline leg, never by the product package.  Arrays are numpy
float32, C-contiguous, already in the memory order of the layout they are
declared with (NCHW: [N,C,H,W]; NHWC: [N,H,W,C]; CHWN: [C,H,W,N]; filters
NCHW: [K,C,3,3]; NHWC: [K,3,3,C]; CHWN: [C,3,3,K] -- the conventions of
comparison/wrapedConv_NCHW.cuh:869, wrapedConv_NHWC.cuh:341,
wrapedConv_CHWN.cuh:288).
"""
import ctypes
import os
import subprocess

import numpy as np

NCHW, NHWC, CHWN = 0, 1, 2
LAYOUT_NAMES = {NCHW: "NCHW", NHWC: "NHWC", CHWN: "CHWN"}

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libwino_oracle.so")
_lib = None

_fp = ctypes.POINTER(ctypes.c_float)
_i = ctypes.c_int


def build(force=False):
    """Compile the C oracle with gcc (a few seconds)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "libwino_oracle.so"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        L.oracle_direct_conv3x3.argtypes = [_i] * 8 + [_fp, _fp, _fp]
        L.oracle_direct_conv3x3_f32.argtypes = [_i] * 8 + [_fp, _fp, _fp, _i]
        L.oracle_permute_act.argtypes = [_i] * 6 + [_fp, _fp]
        L.oracle_permute_flt.argtypes = [_i] * 4 + [_fp, _fp]
        L.oracle_wino_tiles.argtypes = [_i] * 4 + [ctypes.POINTER(_i)] * 2
        L.oracle_wino_filter_transform.argtypes = [_i] * 4 + [_fp, _fp]
        L.oracle_wino_input_transform.argtypes = [_i] * 7 + [_fp, _fp]
        L.oracle_wino_gemm.argtypes = [_i, _i, _i, ctypes.c_long, _fp, _fp, _fp]
        L.oracle_wino_output_transform.argtypes = [_i] * 6 + [_fp, _fp]
        L.oracle_wino_conv3x3.argtypes = [_i] * 9 + [_fp, _fp, _fp]
        L.oracle_rel_l2.argtypes = [_fp, _fp, ctypes.c_long]
        L.oracle_rel_l2.restype = ctypes.c_double
        L.oracle_round_bf16.argtypes = [_fp, _fp, ctypes.c_long]
        L.oracle_round_f16.argtypes = [_fp, _fp, ctypes.c_long]
        L.oracle_num_threads.restype = _i
        _lib = L
    return _lib


def _p(a):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_fp)


def act_shape(layout, N, C, H, W):
    return {NCHW: (N, C, H, W), NHWC: (N, H, W, C), CHWN: (C, H, W, N)}[layout]


def flt_shape(layout, K, C):
    return {NCHW: (K, C, 3, 3), NHWC: (K, 3, 3, C), CHWN: (C, 3, 3, K)}[layout]


def act_dims(layout, a):
    """(N, C, H, W) of an activation array stored in `layout`."""
    s = a.shape
    return {NCHW: (s[0], s[1], s[2], s[3]), NHWC: (s[0], s[3], s[1], s[2]),
            CHWN: (s[3], s[0], s[1], s[2])}[layout]


def flt_dims(layout, w):
    s = w.shape
    return {NCHW: (s[0], s[1]), NHWC: (s[0], s[3]), CHWN: (s[3], s[0])}[layout]


def _ck(rc, what):
    if rc != 0:
        raise RuntimeError(f"{what} failed with code {rc}")


def permute_act(src, dst, a):
    N, C, H, W = act_dims(src, a)
    out = np.empty(act_shape(dst, N, C, H, W), np.float32)
    _ck(lib().oracle_permute_act(src, dst, N, C, H, W, _p(a), _p(out)), "permute_act")
    return out


def permute_flt(src, dst, w):
    K, C = flt_dims(src, w)
    out = np.empty(flt_shape(dst, K, C), np.float32)
    _ck(lib().oracle_permute_flt(src, dst, K, C, _p(w), _p(out)), "permute_flt")
    return out


def direct_conv(x, w, pad=1, src=NCHW, dst=None):
    """Gold direct 3x3 cross-correlation, double accumulation."""
    dst = src if dst is None else dst
    N, C, H, W = act_dims(src, x)
    K, C2 = flt_dims(src, w)
    assert C == C2
    y = np.empty(act_shape(dst, N, K, H + 2 * pad - 2, W + 2 * pad - 2), np.float32)
    _ck(lib().oracle_direct_conv3x3(src, dst, N, C, K, H, W, pad, _p(x), _p(w), _p(y)), "direct_conv")
    return y


def direct_conv_f32(x, w, pad=1, src=NCHW, dst=None, relu=False):
    """Fast fp32 OpenMP direct conv: the timed host baseline."""
    dst = src if dst is None else dst
    N, C, H, W = act_dims(src, x)
    K, C2 = flt_dims(src, w)
    assert C == C2
    y = np.empty(act_shape(dst, N, K, H + 2 * pad - 2, W + 2 * pad - 2), np.float32)
    _ck(lib().oracle_direct_conv3x3_f32(src, dst, N, C, K, H, W, pad, _p(x), _p(w), _p(y), int(relu)),
        "direct_conv_f32")
    return y


def wino_tiles(m, H, W, pad):
    th, tw = _i(), _i()
    _ck(lib().oracle_wino_tiles(m, H, W, pad, ctypes.byref(th), ctypes.byref(tw)), "wino_tiles")
    return th.value, tw.value


def wino_filter_transform(w, layout=NCHW, m=2):
    """U[t*t][C][K]."""
    K, C = flt_dims(layout, w)
    t = m + 2
    U = np.empty((t * t, C, K), np.float32)
    _ck(lib().oracle_wino_filter_transform(m, layout, K, C, _p(w), _p(U)), "filter_transform")
    return U


def wino_input_transform(x, pad=1, layout=NCHW, m=2):
    """V[t*t][C][P], p = (n*th + ty)*tw + tx."""
    N, C, H, W = act_dims(layout, x)
    th, tw = wino_tiles(m, H, W, pad)
    t = m + 2
    V = np.empty((t * t, C, N * th * tw), np.float32)
    _ck(lib().oracle_wino_input_transform(m, layout, N, C, H, W, pad, _p(x), _p(V)), "input_transform")
    return V


def wino_gemm(U, V, m=2):
    """Mo[t*t][K][P] = sum_c U[xi][c][k] V[xi][c][p]."""
    nxi, C, K = U.shape
    P = V.shape[2]
    assert nxi == (m + 2) ** 2 and V.shape[:2] == (nxi, C), "all coordinate planes of both operands"
    assert U.flags.c_contiguous and V.flags.c_contiguous and U.dtype == np.float32 and V.dtype == np.float32
    Mo = np.empty((nxi, K, P), np.float32)
    _ck(lib().oracle_wino_gemm(m, C, K, P, _p(U), _p(V), _p(Mo)), "gemm")
    return Mo


def wino_output_transform(Mo, N, Ho, Wo, layout=NCHW, m=2):
    K = Mo.shape[1]
    y = np.empty(act_shape(layout, N, K, Ho, Wo), np.float32)
    _ck(lib().oracle_wino_output_transform(m, layout, N, K, Ho, Wo, _p(Mo), _p(y)), "output_transform")
    return y


def wino_conv(x, w, pad=1, src=NCHW, dst=None, m=2):
    dst = src if dst is None else dst
    N, C, H, W = act_dims(src, x)
    K, _ = flt_dims(src, w)
    y = np.empty(act_shape(dst, N, K, H + 2 * pad - 2, W + 2 * pad - 2), np.float32)
    _ck(lib().oracle_wino_conv3x3(m, src, dst, N, C, K, H, W, pad, _p(x), _p(w), _p(y)), "wino_conv")
    return y


def rel_l2(got, want):
    got = np.ascontiguousarray(got, np.float32)
    want = np.ascontiguousarray(want, np.float32)
    assert got.shape == want.shape
    return float(lib().oracle_rel_l2(_p(got), _p(want), got.size))


def round_bf16(a):
    a = np.ascontiguousarray(a, np.float32)
    out = np.empty_like(a)
    lib().oracle_round_bf16(_p(a), _p(out), a.size)
    return out


def round_f16(a):
    a = np.ascontiguousarray(a, np.float32)
    out = np.empty_like(a)
    lib().oracle_round_f16(_p(a), _p(out), a.size)
    return out


def num_threads():
    return int(lib().oracle_num_threads())
