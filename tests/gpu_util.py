"""Helpers shared by the GPU parity tests (device upload, padded-operand unpacking)."""
import numpy as np
import torch

from cudnntest_amd import ops, synth

TORCH_DT = {ops.F32: torch.float32, ops.F16: torch.float16, ops.BF16: torch.bfloat16}
# relative L2 tolerance of a whole layer against the fp32 direct convolution
TOL = {ops.F32: 1e-4, ops.F16: 2e-2, ops.BF16: 2e-2}


def dev(a, dtype=ops.F32):
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda").to(TORCH_DT[dtype]).contiguous()


def host(t):
    return t.detach().float().cpu().numpy()


def rounded(a, dtype, oracle):
    """What the device sees after storing `a` in `dtype`."""
    if dtype == ops.F16:
        return oracle.round_f16(a)
    if dtype == ops.BF16:
        return oracle.round_bf16(a)
    return a


def batch_minor_perm(N, th, tw):
    """perm[p_minor] = p_major for the two tile orders."""
    n, ty, tx = np.meshgrid(np.arange(N), np.arange(th), np.arange(tw), indexing="ij")
    p_major = ((n * th + ty) * tw + tx).ravel()
    p_minor = ((ty * tw + tx) * N + n).ravel()
    perm = np.empty(N * th * tw, np.int64)
    perm[p_minor] = p_major
    return perm


def unpack_operand(t, dtype=ops.F32):
    """[16][Cp/CV][X][CV] (channel vectors innermost) -> numpy [16][Cp][X]."""
    a = host(t)
    xi, cq, X, cv = a.shape
    return np.ascontiguousarray(a.transpose(0, 1, 3, 2).reshape(xi, cq * cv, X))


def pack_operand(a, dtype=ops.F32):
    """numpy [16][Cp][X] -> device [16][Cp/CV][X][CV]."""
    cv = 4 if dtype == ops.F32 else 8
    xi, Cp, X = a.shape
    assert Cp % cv == 0
    return dev(np.ascontiguousarray(a.reshape(xi, Cp // cv, cv, X).transpose(0, 1, 3, 2)), dtype)
