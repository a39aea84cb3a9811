"""Writes the golden fixtures of tests/golden/: small seeded problems with their expected results.

The reference keeps no vectors for this path (its inputs were unseeded files outside the repository), so the
expected results come from the definition itself: a float64 zero-padded cross-correlation written out below in
NumPy, y[n,k,i,j] = sum_{c,r,s} x[n,c,i+r-p,j+s-p] * w[k,c,r,s] -- the reference's "Ground-Truth Naive Convolution"
(layoutTest/NCHW/data/WinoTran_NCHW.py:200-228).  Before anything is written the results are checked against two
independent routines: torch.nn.functional.conv2d in float64 and the C oracle.  The Winograd-stage fixtures (U, V,
M of the smallest problem, F(2x2,3x3)) are written from the closed-form matrices in float64; on the integer
problem every entry is a dyadic rational that fp32 holds exactly.

Run from the repository root:  python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from cudnntest_amd import synth  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
SHAPES = [(2, 3, 4, 5, 5), (1, 8, 8, 6, 6), (3, 5, 7, 9, 9), (2, 4, 6, 7, 10)]   # N, C, K, H, W

BT = np.array([[1, 0, -1, 0], [0, 1, 1, 0], [0, -1, 1, 0], [0, 1, 0, -1]], np.float64)
G = np.array([[1, 0, 0], [.5, .5, .5], [.5, -.5, .5], [0, 0, 1]], np.float64)
AT = np.array([[1, 1, 1, 0], [0, 1, -1, -1]], np.float64)


def correlate(x, w, pad):
    N, C, H, W = x.shape
    K = w.shape[0]
    xp = np.zeros((N, C, H + 2 * pad, W + 2 * pad), np.float64)
    xp[:, :, pad:pad + H, pad:pad + W] = x
    Ho, Wo = H + 2 * pad - 2, W + 2 * pad - 2
    y = np.zeros((N, K, Ho, Wo), np.float64)
    for r in range(3):
        for s in range(3):
            y += np.einsum("nchw,kc->nkhw", xp[:, :, r:r + Ho, s:s + Wo], w[:, :, r, s].astype(np.float64))
    return y


def winograd_stages(x, w, pad):
    """U[16][C][K], V[16][C][P] (p = (n*th+ty)*tw+tx), M[16][K][P] in float64."""
    N, C, H, W = x.shape
    K = w.shape[0]
    Ho, Wo = H + 2 * pad - 2, W + 2 * pad - 2
    th, tw = (Ho + 1) // 2, (Wo + 1) // 2
    xp = np.zeros((N, C, 2 * th + 2, 2 * tw + 2), np.float64)
    xp[:, :, pad:pad + H, pad:pad + W] = x
    U = np.einsum("ar,kcrs,bs->abck", G, w.astype(np.float64), G).reshape(16, C, K)
    V = np.zeros((4, 4, C, N, th, tw))
    for ty in range(th):
        for tx in range(tw):
            d = xp[:, :, 2 * ty:2 * ty + 4, 2 * tx:2 * tx + 4]
            V[:, :, :, :, ty, tx] = np.einsum("ai,ncij,bj->abcn", BT, d, BT)
    V = V.reshape(16, C, N * th * tw)
    M = np.einsum("xck,xcp->xkp", U, V)
    # closing the loop: A^T M A must be the correlation
    Y = np.einsum("ai,ijkp,bj->kpab", AT, M.reshape(4, 4, K, -1), AT).reshape(K, N, th, tw, 2, 2)
    Y = Y.transpose(1, 0, 2, 4, 3, 5).reshape(N, K, 2 * th, 2 * tw)[:, :, :Ho, :Wo]
    assert np.allclose(Y, correlate(x, w, pad), rtol=0, atol=1e-9)
    return U, V, M


def main():
    import torch
    import oracle
    out = {}
    for i, (N, C, K, H, W) in enumerate(SHAPES):
        for kind in ("int", "flt"):
            x, w = synth.conv_inputs(N, C, K, H, W, seed=0x601D + i, integer=(kind == "int"))
            tag = f"s{i}_{kind}"
            out[tag + "_x"], out[tag + "_w"] = x.astype(np.float32), w.astype(np.float32)
            for pad in (0, 1):
                y = correlate(x, w, pad)
                t = torch.nn.functional.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(), padding=pad)
                assert np.allclose(y, t.numpy(), rtol=0, atol=1e-12), tag
                o = oracle.direct_conv(x.astype(np.float32), w.astype(np.float32), pad)
                assert np.allclose(y, o, rtol=1e-6, atol=1e-6), tag
                if kind == "int":
                    assert np.array_equal(y, np.round(y)) and np.array_equal(o, y.astype(np.float32))
                out[f"{tag}_y_pad{pad}"] = y.astype(np.float32)
    x, w = out["s0_int_x"], out["s0_int_w"]
    U, V, M = winograd_stages(x, w, 1)
    for name, a in (("U", U), ("V", V), ("M", M)):
        assert np.array_equal(a.astype(np.float32).astype(np.float64), a), name     # exact in fp32
        out["s0_int_" + name] = a.astype(np.float32)
    path = os.path.join(HERE, "conv3x3_fixtures.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
