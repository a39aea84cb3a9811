"""Seeded synthetic tensors for the convolution workloads.

Counter-based (splitmix64 of seed + index), so a tensor's values depend only on
(seed, logical index) and are identical wherever they are generated.  Values
are produced in the logical NCHW / KCRS order and then permuted, so every
layout sees the same numbers.  Distributions: activations uniform[-1, 1),
weights N(0, sqrt(2 / (9 C))) (He initialisation for a 3x3 filter).
"""
import numpy as np

NCHW, NHWC, CHWN = 0, 1, 2

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)


def _splitmix64(idx, seed):
    with np.errstate(over="ignore"):
        z = (idx + np.uint64(1)) * _GOLDEN + np.uint64(seed)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def uniform_pm1(n, seed):
    """n float32 values in [-1, 1) on a 2^-23 grid."""
    out = np.empty(n, np.float32)
    step = 1 << 22
    for s in range(0, n, step):
        e = min(n, s + step)
        z = _splitmix64(np.arange(s, e, dtype=np.uint64), seed)
        out[s:e] = ((z >> np.uint64(40)).astype(np.float64) * (2.0 ** -23) - 1.0).astype(np.float32)
    return out


def normal(n, seed, std):
    """n float32 normals (Box-Muller on two counter streams)."""
    out = np.empty(n, np.float32)
    step = 1 << 22
    for s in range(0, n, step):
        e = min(n, s + step)
        i = np.arange(s, e, dtype=np.uint64)
        z1 = _splitmix64(i * np.uint64(2), seed)
        z2 = _splitmix64(i * np.uint64(2) + np.uint64(1), seed)
        u1 = ((z1 >> np.uint64(40)).astype(np.float64) + 1.0) * (2.0 ** -24)   # (0, 1]
        u2 = (z2 >> np.uint64(40)).astype(np.float64) * (2.0 ** -24)           # [0, 1)
        out[s:e] = (np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2) * std).astype(np.float32)
    return out


def small_ints(n, seed, lo=-3, hi=3):
    """n float32 integers in [lo, hi]: exact-arithmetic test data."""
    z = _splitmix64(np.arange(n, dtype=np.uint64), seed)
    span = np.uint64(hi - lo + 1)
    return ((z >> np.uint64(33)) % span).astype(np.float32) + np.float32(lo)


def act_to_layout(a_nchw, layout):
    if layout == NCHW:
        return np.ascontiguousarray(a_nchw)
    if layout == NHWC:
        return np.ascontiguousarray(a_nchw.transpose(0, 2, 3, 1))
    if layout == CHWN:
        return np.ascontiguousarray(a_nchw.transpose(1, 2, 3, 0))
    raise ValueError(layout)


def act_from_layout(a, layout):
    """Back to a logical NCHW view (not necessarily contiguous)."""
    if layout == NCHW:
        return a
    if layout == NHWC:
        return a.transpose(0, 3, 1, 2)
    if layout == CHWN:
        return a.transpose(3, 0, 1, 2)
    raise ValueError(layout)


def flt_to_layout(w_kcrs, layout):
    if layout == NCHW:
        return np.ascontiguousarray(w_kcrs)
    if layout == NHWC:
        return np.ascontiguousarray(w_kcrs.transpose(0, 2, 3, 1))
    if layout == CHWN:
        return np.ascontiguousarray(w_kcrs.transpose(1, 2, 3, 0))
    raise ValueError(layout)


def conv_inputs(N, C, K, H, W, seed, layout=NCHW, integer=False):
    """(x, w) for one 3x3 layer, stored in `layout`'s memory order."""
    if integer:
        x = small_ints(N * C * H * W, seed * 2 + 11, -3, 3)
        w = small_ints(K * C * 9, seed * 2 + 12, -2, 2)
    else:
        x = uniform_pm1(N * C * H * W, seed * 2 + 11)
        w = normal(K * C * 9, seed * 2 + 12, float(np.sqrt(2.0 / (9.0 * C))))
    x = x.reshape(N, C, H, W)
    w = w.reshape(K, C, 3, 3)
    return act_to_layout(x, layout), flt_to_layout(w, layout)


# VGG-16's thirteen 3x3 convolutions as (C, K, H); H == W.
VGG16_CONV = [
    (3, 64, 224), (64, 64, 224),
    (64, 128, 112), (128, 128, 112),
    (128, 256, 56), (256, 256, 56), (256, 256, 56),
    (256, 512, 28), (512, 512, 28), (512, 512, 28),
    (512, 512, 14), (512, 512, 14), (512, 512, 14),
]
