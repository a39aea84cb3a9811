"""Operators over libwino_amd.so.

Two levels:
  * the reference's names -- wrapedConv_NCHW / _NHWC / _CHWN
    (comparison/wrapedConv_NCHW.cuh:335, wrapedConv_NHWC.cuh:24,
    wrapedConv_CHWN.cuh:16), the six convLayoutTrans_X_to_Y and layoutManager
    with DataLayout (comparison/DataLayoutTrans.cuh:9-651) -- same argument
    order and meaning: (bat4Conv, inside, chn, numOfFilter, padding, m1, m2,
    inputTran_gpu, filterTran_gpu, gemmOutput_gpu, output).  They are blocking,
    like the reference's (each ends in a device sync).  `chn` is a C++ int&
    there, overwritten with numOfFilter; here the new value is returned.  The
    three scratch arguments are accepted and ignored: the library owns its
    scratch, because F(2x2) intermediates are larger than the F(4x4) buffers a
    reference caller allocates.
  * stage-level and whole-layer functions that take torch tensors and derive
    sizes from them.
"""
import enum

import torch

from . import _lib

NCHW, NHWC, CHWN = 0, 1, 2
F32, F16, BF16 = 0, 1, 2
ALGO_AUTO, ALGO_STAGED, ALGO_EPILOGUE, ALGO_FUSED, ALGO_STAGED_F4, ALGO_DIRECT, ALGO_EPILOGUE_F4 = 0, 1, 2, 3, 4, 5, 6
TILES_BATCH_MAJOR, TILES_BATCH_MINOR = 0, 1
PRODUCT_KP, PRODUCT_PK = 0, 1
FLAG_RELU = 1
FLAG_POOL2 = 2


class DataLayout(enum.IntEnum):
    NCHW = 0
    NHWC = 1
    CHWN = 2


_DTYPES = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}
_TORCH_DTYPES = {v: k for k, v in _DTYPES.items()}


def _dt(t):
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {t.dtype}") from None


def _ptr(t):
    if not t.is_cuda:
        raise ValueError("tensor must live on the GPU")
    if not t.is_contiguous():
        raise ValueError("tensor must be contiguous in its layout's memory order")
    return t.data_ptr()


def _stream():
    return torch.cuda.current_stream().cuda_stream


def act_shape(layout, N, C, H, W):
    return {NCHW: (N, C, H, W), NHWC: (N, H, W, C), CHWN: (C, H, W, N)}[int(layout)]


def act_dims(layout, t):
    s = t.shape
    return {NCHW: (s[0], s[1], s[2], s[3]), NHWC: (s[0], s[3], s[1], s[2]),
            CHWN: (s[3], s[0], s[1], s[2])}[int(layout)]


def flt_dims(layout, w):
    s = w.shape
    return {NCHW: (s[0], s[1]), NHWC: (s[0], s[3]), CHWN: (s[3], s[0])}[int(layout)]


def geometry(dtype, N, C, K, H, W, pad):
    import ctypes
    th, tw, Cp, Kp = (ctypes.c_int() for _ in range(4))
    P, Pp = ctypes.c_long(), ctypes.c_long()
    _lib.check(_lib.load().wino_geometry(dtype, N, C, K, H, W, pad, th, tw, P, Cp, Kp, Pp), "wino_geometry")
    return dict(th=th.value, tw=tw.value, P=P.value, Cp=Cp.value, Kp=Kp.value, Pp=Pp.value)


ALGO_NAMES = {ALGO_AUTO: "auto", ALGO_STAGED: "staged", ALGO_EPILOGUE: "epilogue", ALGO_FUSED: "fused",
              ALGO_STAGED_F4: "staged_f4", ALGO_DIRECT: "direct", ALGO_EPILOGUE_F4: "epilogue_f4"}


def pick_algo(layout, dtype, N, C, K, H, W, pad=1):
    """The algorithm ALGO_AUTO resolves to for this problem (layout: that of the input tensor)."""
    rc = _lib.load().wino_pick_algo(layout, dtype, N, C, K, H, W, pad)
    if rc < 0:
        _lib.check(rc, "wino_pick_algo")
    return rc


def workspace_bytes(dtype, N, C, K, H, W, pad):
    return int(_lib.load().wino_workspace_bytes(dtype, N, C, K, H, W, pad))


def warmup():
    _lib.check(_lib.load().wino_warmup(), "wino_warmup")


STAGES = ("filter", "input", "gemm", "output")


def stage_timing(enable):
    _lib.check(_lib.load().wino_stage_timing(int(bool(enable))), "wino_stage_timing")


def stage_times():
    """{stage: (total_ms, spans)} accumulated since the last call; blocks on the recorded events."""
    import ctypes
    ms = (ctypes.c_float * 4)()
    calls = (ctypes.c_long * 4)()
    _lib.check(_lib.load().wino_stage_times(ms, calls), "wino_stage_times")
    return {name: (float(ms[i]), int(calls[i])) for i, name in enumerate(STAGES)}


def stage_stats():
    """{stage: (total_ms, min_ms, max_ms, spans)} since the last call: the average / minimum / maximum of the
    reference's per-stage harness (delayTest/testbench/src/M1/M1Test.h:100-151) from the library's own events."""
    import ctypes
    tot, lo, hi = ((ctypes.c_float * 4)() for _ in range(3))
    calls = (ctypes.c_long * 4)()
    _lib.check(_lib.load().wino_stage_stats(tot, lo, hi, calls), "wino_stage_stats")
    return {name: (float(tot[i]), float(lo[i]), float(hi[i]), int(calls[i])) for i, name in enumerate(STAGES)}


# ---- whole layer -------------------------------------------------------------

def _out_for(dst, x, N, K, Ho, Wo, pool, out):
    if pool:
        Ho, Wo = Ho // 2, Wo // 2
    shape = act_shape(dst, N, K, Ho, Wo)
    if out is None:
        return torch.empty(shape, dtype=x.dtype, device=x.device)
    if tuple(out.shape) != tuple(shape):
        raise ValueError(f"out has shape {tuple(out.shape)}, the layer writes {tuple(shape)}")
    return out


def _check_bias(bias, x, K):
    if bias is None:
        return None
    if bias.dtype != x.dtype or bias.numel() != K or not bias.is_contiguous():
        raise TypeError("bias must hold K contiguous elements of x's dtype")
    return bias


def conv(x, w, pad=1, src=NCHW, dst=None, algo=ALGO_AUTO, relu=False, out=None, bias=None, pool=False):
    """y = pool2x2?(relu?(conv3x3(x, w) + bias)); x, w in `src`'s conventions, y in `dst`'s.  Asynchronous."""
    dst = src if dst is None else dst
    N, C, H, W = act_dims(src, x)
    K, C2 = flt_dims(src, w)
    if C2 != C:
        raise ValueError(f"filter bank has {C2} channels, input has {C}")
    if w.dtype != x.dtype:
        raise TypeError("x and w must share a dtype")
    bias = _check_bias(bias, x, K)
    out = _out_for(dst, x, N, K, H + 2 * pad - 2, W + 2 * pad - 2, pool, out)
    flags = (FLAG_RELU if relu else 0) | (FLAG_POOL2 if pool else 0)
    rc = _lib.load().wino_conv_ex(int(src), int(dst), _dt(x), algo, flags, N, C, K, H, W, pad,
                                  _ptr(x), _ptr(w), _ptr(bias) if bias is not None else None, _ptr(out), _stream())
    _lib.check(rc, "wino_conv_ex")
    return out


def conv_noalloc(x, w, out, pad=1, src=NCHW, dst=None, algo=ALGO_AUTO, relu=False, bias=None, pool=False):
    """conv() into the caller's `out` through wino_conv_noalloc: the library's scratch is its built-in fixed buffer,
    nothing is allocated (not here either: `out` is required).  Problems that need more scratch are refused."""
    dst = src if dst is None else dst
    N, C, H, W = act_dims(src, x)
    K, C2 = flt_dims(src, w)
    if C2 != C:
        raise ValueError(f"filter bank has {C2} channels, input has {C}")
    if w.dtype != x.dtype:
        raise TypeError("x and w must share a dtype")
    bias = _check_bias(bias, x, K)
    out = _out_for(dst, x, N, K, H + 2 * pad - 2, W + 2 * pad - 2, pool, out)
    flags = (FLAG_RELU if relu else 0) | (FLAG_POOL2 if pool else 0)
    rc = _lib.load().wino_conv_noalloc(int(src), int(dst), _dt(x), algo, flags, N, C, K, H, W, pad, _ptr(x), _ptr(w),
                                       _ptr(bias) if bias is not None else None, _ptr(out), _stream())
    _lib.check(rc, "wino_conv_noalloc")
    return out


def conv_prepared(x, U, K, pad=1, src=NCHW, dst=None, algo=ALGO_AUTO, relu=False, out=None, bias=None, pool=False):
    """Same with the filter bank already transformed by filter_transform()."""
    dst = src if dst is None else dst
    N, C, H, W = act_dims(src, x)
    bias = _check_bias(bias, x, K)
    out = _out_for(dst, x, N, K, H + 2 * pad - 2, W + 2 * pad - 2, pool, out)
    flags = (FLAG_RELU if relu else 0) | (FLAG_POOL2 if pool else 0)
    rc = _lib.load().wino_conv_prepared_ex(int(src), int(dst), _dt(x), algo, flags, N, C, K, H, W, pad, _ptr(x),
                                           _ptr(U), _ptr(bias) if bias is not None else None, _ptr(out), _stream())
    _lib.check(rc, "wino_conv_prepared_ex")
    return out


class ConvStack:
    """A stack of 3x3 / pad 1 convolution layers with cached filter transforms and bias, ReLU and 2x2
    pooling in each layer's output stage (wino_stack_*): the convolution part of the reference's
    classify_example_modified (netTest/cudnn_test_0124/VGG_Batched/Network.h:603-669).

    layers: list of dicts {K, layout_in, layout_out, relu, pool, algo}; `layout_in` of a layer defaults to
    the previous layer's `layout_out` (the first: NCHW), `layout_out` to its own `layout_in`."""

    def __init__(self, dtype, N, C, H, W, layers):
        import ctypes
        descs = (_lib.StackLayer * len(layers))()
        prev = None
        self._ck = []                      # (C, K) of every layer: what set_layer's tensors must hold
        c = C
        for d, L in zip(descs, layers):
            d.K = int(L["K"])
            self._ck.append((c, d.K))
            c = d.K
            d.layout_in = int(L.get("layout_in", prev if prev is not None else NCHW))
            d.layout_out = int(L.get("layout_out", d.layout_in))
            d.flags = (FLAG_RELU if L.get("relu", False) else 0) | (FLAG_POOL2 if L.get("pool", False) else 0)
            d.algo = int(L.get("algo", ALGO_AUTO))
            prev = d.layout_out
        self._descs = descs
        self._h = ctypes.c_void_p()
        self.dtype = dtype
        self.in_shape = act_shape(descs[0].layout_in, N, C, H, W)
        _lib.check(_lib.load().wino_stack_create(_DTYPES[dtype], N, C, H, W, len(layers), descs, self._h),
                   "wino_stack_create")
        n, k, h, w, lay = (ctypes.c_int() for _ in range(5))
        _lib.check(_lib.load().wino_stack_output(self._h, n, k, h, w, lay), "wino_stack_output")
        self.out_layout = lay.value
        self.out_shape = act_shape(lay.value, n.value, k.value, h.value, w.value)

    def set_layer(self, layer, w, bias=None):
        if w.dtype != self.dtype or (bias is not None and bias.dtype != self.dtype):
            raise TypeError("filters and bias must have the stack's dtype")
        if 0 <= layer < len(self._ck):     # (a layer that does not exist is the library's to refuse)
            C, K = self._ck[layer]
            if w.numel() != 9 * K * C:
                raise ValueError(f"layer {layer} takes a bank of {K} x {C} 3x3 filters, got {w.numel()} elements")
            if bias is not None and bias.numel() != K:
                raise ValueError(f"layer {layer} takes {K} bias values, got {bias.numel()}")
        _lib.check(_lib.load().wino_stack_set_layer(self._h, layer, _ptr(w), _ptr(bias) if bias is not None else None,
                                                    _stream()), "wino_stack_set_layer")

    def forward(self, x, out=None, graph=False):
        """All layers on the current stream.  graph=True replays the pass from a HIP graph recorded on the
        first call for this (x, out) pair: pass the same tensors again to benefit."""
        if tuple(x.shape) != tuple(self.in_shape) or x.dtype != self.dtype:
            raise ValueError(f"input must be {tuple(self.in_shape)} of {self.dtype}")
        if out is None:
            out = torch.empty(self.out_shape, dtype=self.dtype, device=x.device)
        if graph:
            _lib.check(_lib.load().wino_stack_forward_graph(self._h, _ptr(x), _ptr(out), _stream()),
                       "wino_stack_forward_graph")
        else:
            _lib.check(_lib.load().wino_stack_forward(self._h, _ptr(x), _ptr(out), _stream()), "wino_stack_forward")
        return out

    def close(self):
        if self._h:
            _lib.load().wino_stack_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


# ---- stages ------------------------------------------------------------------------

def filter_transform(w, layout=NCHW):
    """U[16][Cp/CV][Kp][CV] = G g G^T (padding zero-filled); CV = 4 (fp32) or 8 (f16/bf16)."""
    K, C = flt_dims(layout, w)
    g = geometry(_dt(w), 1, C, K, 4, 4, 1)
    cv = 16 // w.element_size()
    U = torch.empty((16, g["Cp"] // cv, g["Kp"], cv), dtype=w.dtype, device=w.device)
    _lib.check(_lib.load().wino_filter_transform(int(layout), _dt(w), K, C, _ptr(w), _ptr(U), _stream()),
               "wino_filter_transform")
    return U


def input_transform(x, pad=1, layout=NCHW, tile_order=TILES_BATCH_MAJOR):
    """V[16][Cp/CV][Pp][CV] = B^T d B; columns p >= P are left as allocated (zeros here)."""
    N, C, H, W = act_dims(layout, x)
    g = geometry(_dt(x), N, C, 1, H, W, pad)
    cv = 16 // x.element_size()
    V = torch.zeros((16, g["Cp"] // cv, g["Pp"], cv), dtype=x.dtype, device=x.device)
    _lib.check(_lib.load().wino_input_transform(int(layout), _dt(x), tile_order, N, C, H, W, pad, _ptr(x), _ptr(V),
                                                _stream()), "wino_input_transform")
    return V


def batched_gemm(U, V, C, K, P, product_order=PRODUCT_KP):
    """Mo (fp32) = sum_c U[xi][c][k] V[xi][c][p]; U, V in channel-vector layout.
    Shape [16][Kp][Pp], or [16][Pp][Kp] with PRODUCT_PK."""
    shape = (16, U.shape[2], V.shape[2]) if product_order == PRODUCT_KP else (16, V.shape[2], U.shape[2])
    Mo = torch.empty(shape, dtype=torch.float32, device=U.device)
    _lib.check(_lib.load().wino_batched_gemm(_dt(U), product_order, C, K, P, _ptr(U), _ptr(V), _ptr(Mo), _stream()),
               "wino_batched_gemm")
    return Mo


def output_transform(Mo, N, K, Ho, Wo, layout=NCHW, tile_order=TILES_BATCH_MAJOR, relu=False, dtype=torch.float32,
                     product_order=PRODUCT_KP, pool=False):
    y = torch.empty(act_shape(layout, N, K, Ho // 2, Wo // 2) if pool else act_shape(layout, N, K, Ho, Wo),
                    dtype=dtype, device=Mo.device)
    _lib.check(_lib.load().wino_output_transform(int(layout), _DTYPES[dtype], tile_order, product_order,
                                                 (FLAG_RELU if relu else 0) | (FLAG_POOL2 if pool else 0),
                                                 N, K, Ho, Wo, _ptr(Mo), _ptr(y), _stream()),
               "wino_output_transform")
    return y


def gemm_output(U, V, N, C, K, Ho, Wo, layout=NCHW, tile_order=TILES_BATCH_MAJOR, relu=False, pool=False):
    y = torch.empty(act_shape(layout, N, K, Ho // 2, Wo // 2) if pool else act_shape(layout, N, K, Ho, Wo),
                    dtype=U.dtype, device=U.device)
    _lib.check(_lib.load().wino_gemm_output(int(layout), _dt(U), tile_order,
                                            (FLAG_RELU if relu else 0) | (FLAG_POOL2 if pool else 0), N, C, K, Ho,
                                            Wo, _ptr(U), _ptr(V), _ptr(y), _stream()), "wino_gemm_output")
    return y


# ---- F(4x4,3x3) stages -------------------------------------------------------------------

def f4_geometry(dtype, N, C, K, H, W, pad):
    import ctypes
    th, tw, Cp, Kp = (ctypes.c_int() for _ in range(4))
    P, Pp = ctypes.c_long(), ctypes.c_long()
    _lib.check(_lib.load().wino_f4_geometry(dtype, N, C, K, H, W, pad, th, tw, P, Cp, Kp, Pp), "wino_f4_geometry")
    return dict(th=th.value, tw=tw.value, P=P.value, Cp=Cp.value, Kp=Kp.value, Pp=Pp.value)


def f4_filter_transform(w, layout=NCHW):
    K, C = flt_dims(layout, w)
    g = f4_geometry(_dt(w), 1, C, K, 6, 6, 1)
    cv = 16 // w.element_size()
    U = torch.empty((36, g["Cp"] // cv, g["Kp"], cv), dtype=w.dtype, device=w.device)
    _lib.check(_lib.load().wino_f4_filter_transform(int(layout), _dt(w), K, C, _ptr(w), _ptr(U), _stream()),
               "wino_f4_filter_transform")
    return U


def f4_input_transform(x, pad=1, layout=NCHW, tile_order=TILES_BATCH_MAJOR):
    N, C, H, W = act_dims(layout, x)
    g = f4_geometry(_dt(x), N, C, 1, H, W, pad)
    cv = 16 // x.element_size()
    V = torch.zeros((36, g["Cp"] // cv, g["Pp"], cv), dtype=x.dtype, device=x.device)
    _lib.check(_lib.load().wino_f4_input_transform(int(layout), _dt(x), tile_order, N, C, H, W, pad, _ptr(x),
                                                   _ptr(V), _stream()), "wino_f4_input_transform")
    return V


def f4_batched_gemm(U, V, C, K, P, product_order=PRODUCT_KP):
    shape = (36, U.shape[2], V.shape[2]) if product_order == PRODUCT_KP else (36, V.shape[2], U.shape[2])
    Mo = torch.empty(shape, dtype=torch.float32, device=U.device)
    _lib.check(_lib.load().wino_f4_batched_gemm(_dt(U), product_order, C, K, P, _ptr(U), _ptr(V), _ptr(Mo),
                                                _stream()), "wino_f4_batched_gemm")
    return Mo


def f4_output_transform(Mo, N, K, Ho, Wo, layout=NCHW, tile_order=TILES_BATCH_MAJOR, relu=False,
                        dtype=torch.float32, product_order=PRODUCT_KP, pool=False):
    y = torch.empty(act_shape(layout, N, K, Ho // 2 if pool else Ho, Wo // 2 if pool else Wo), dtype=dtype, device=Mo.device)
    _lib.check(_lib.load().wino_f4_output_transform(int(layout), _DTYPES[dtype], tile_order, product_order,
                                                    (FLAG_RELU if relu else 0) | (FLAG_POOL2 if pool else 0), N, K, Ho, Wo,
                                                    _ptr(Mo), _ptr(y), _stream()), "wino_f4_output_transform")
    return y


def f4_gemm_output(U, V, N, C, K, Ho, Wo, layout=NCHW, tile_order=TILES_BATCH_MAJOR, relu=False, pool=False):
    """y straight from the F(4x4) operands: the 36-way GEMM with the output transform in its epilogue (fp32)."""
    y = torch.empty(act_shape(layout, N, K, Ho // 2 if pool else Ho, Wo // 2 if pool else Wo), dtype=U.dtype, device=U.device)
    _lib.check(_lib.load().wino_f4_gemm_output(int(layout), _dt(U), tile_order,
                                               (FLAG_RELU if relu else 0) | (FLAG_POOL2 if pool else 0), N, C, K, Ho, Wo,
                                               _ptr(U), _ptr(V), _ptr(y), _stream()), "wino_f4_gemm_output")
    return y


def layout_transform(t, src, dst):
    N, C, H, W = act_dims(src, t)
    out = torch.empty(act_shape(dst, N, C, H, W), dtype=t.dtype, device=t.device)
    _lib.check(_lib.load().wino_layout_transform(int(src), int(dst), _dt(t), N, C, H, W, _ptr(t), _ptr(out),
                                                 _stream()), "wino_layout_transform")
    return out


# ---- the reference's call surface --------------------------------------------------------

def _wrapped(src, dst, bat4Conv, inside, chn, numOfFilter, padding, m1, m2, output):
    L = _lib.load()
    rc = L.wino_conv(int(src), int(dst), _dt(m1), ALGO_AUTO, 0, bat4Conv, chn, numOfFilter, inside, inside, padding,
                     _ptr(m1), _ptr(m2), _ptr(output), _stream())
    _lib.check(rc, "wino_conv")
    _lib.check(L.wino_sync(_stream()), "wino_sync")
    return numOfFilter


def wrapedConv_NCHW(bat4Conv, inside, chn, numOfFilter, padding, m1, m2, inputTran_gpu, filterTran_gpu,
                    gemmOutput_gpu, output):
    return _wrapped(NCHW, NCHW, bat4Conv, inside, chn, numOfFilter, padding, m1, m2, output)


def wrapedConv_NHWC(bat4Conv, inside, chn, numOfFilter, padding, m1, m2, inputTran_gpu, filterTran_gpu,
                    gemmOutput_gpu, output):
    return _wrapped(NHWC, NHWC, bat4Conv, inside, chn, numOfFilter, padding, m1, m2, output)


def wrapedConv_CHWN(bat4Conv, inside, chn, numOfFilter, padding, m1, m2, inputTran_gpu, filterTran_gpu,
                    gemmOutput_gpu, output):
    return _wrapped(CHWN, CHWN, bat4Conv, inside, chn, numOfFilter, padding, m1, m2, output)


def _make_cross(src, dst):
    def f(bat4Conv, inside, chn, numOfFilter, padding, m1, m2, inputTran_gpu, filterTran_gpu, gemmOutput_gpu,
          output):
        return _wrapped(src, dst, bat4Conv, inside, chn, numOfFilter, padding, m1, m2, output)
    return f


convLayoutTrans_CHWN_to_NCHW = _make_cross(CHWN, NCHW)
convLayoutTrans_CHWN_to_NHWC = _make_cross(CHWN, NHWC)
convLayoutTrans_NHWC_to_NCHW = _make_cross(NHWC, NCHW)
convLayoutTrans_NHWC_to_CHWN = _make_cross(NHWC, CHWN)
convLayoutTrans_NCHW_to_NHWC = _make_cross(NCHW, NHWC)
convLayoutTrans_NCHW_to_CHWN = _make_cross(NCHW, CHWN)


def layoutManager(srcLayout, dstLayout, bat4Conv, inside, chn, numOfFilter, padding, input, weights, inputTran_gpu,
                  filterTran_gpu, gemmOutput_gpu, output):
    """Dispatch on (src, dst) as comparison/DataLayoutTrans.cuh:594-651 does."""
    return _wrapped(DataLayout(srcLayout), DataLayout(dstLayout), bat4Conv, inside, chn, numOfFilter, padding,
                    input, weights, output)
