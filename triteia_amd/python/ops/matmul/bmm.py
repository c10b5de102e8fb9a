import torch

from triteia_amd.python.capi import bmm_2_4
from triteia_amd.python.capi._ffi import lock_workspace
from .sparse_low_precision import matmul_4bit_2_4


def bmm_4bit_2_4_forloop(qweights, xs, metas, ss):
    """One matmul_4bit_2_4 per batch entry (triteia/python/ops/matmul/bmm.py:6-18)."""
    outputs = torch.zeros((xs.shape[0], xs.shape[1], ss.shape[2]), dtype=xs.dtype, device=xs.device)
    for id in range(xs.shape[0]):
        outputs[id] = matmul_4bit_2_4(qweights[id], xs[id], metas[id], ss[id])
    return outputs


def bmm_4bit_2_4(qweights, xs, metas, ss):
    """xs[b] @ W[b] for every b in one launch (triteia/python/ops/matmul/bmm.py:21-35).

    xs fp16 [b, t, k]; qweights [b, k/32, 2m]; metas [b, m, k/16]; ss [b, 1, m] -> [b, t, m]."""
    # every element of C is written by the kernel (unless k = 0); the lock workspace is never touched
    alloc = torch.empty if xs.shape[2] > 0 else torch.zeros
    C = alloc((xs.shape[0], xs.shape[1], ss.shape[2]), dtype=xs.dtype, device=xs.device)
    workspace = lock_workspace(xs.shape[0] * max(ss.shape[2], ss.shape[1]), xs.device)
    bmm_2_4(xs.contiguous(), qweights, metas, C, ss, workspace)
    return C
