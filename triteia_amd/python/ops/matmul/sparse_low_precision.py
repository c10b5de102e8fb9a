import torch

from triteia_amd.python.capi import mul_2_4
from triteia_amd.python.capi._ffi import lock_workspace


def matmul_4bit_2_4(qweight, x, meta, s):
    """x @ W for a 2:4-sparse int4 weight (triteia/python/ops/matmul/sparse_low_precision.py:5-24).

    qweight int32 [k/32, 2m], x fp16 [..., k], meta int16 [m, k/16], s fp16 [1, m] (or [k/128, m], grouped)
    -> fp16 [..., m]."""
    # every element of C is written by the kernel (unless k = 0); the lock workspace is never touched
    alloc = torch.empty if x.shape[-1] > 0 else torch.zeros
    C = alloc((x.shape[:-1] + (s.shape[1],)), dtype=x.dtype, device=x.device)
    workspace = lock_workspace(s.shape[1], x.device)
    x2 = x.reshape(-1, x.shape[-1])
    if not x2.is_contiguous():
        x2 = x2.contiguous()
    mul_2_4(x2, qweight, meta, C.view(-1, C.shape[-1]), s, workspace)
    return C
