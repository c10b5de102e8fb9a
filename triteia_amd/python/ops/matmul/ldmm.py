"""LoRA + Delta mixed multi-model matmul (triteia/python/ops/matmul/ldmm.py:8-174).

indices[t] in [0, M) selects LoRA adapter indices[t]; indices[t] >= M selects the 2:4 int4
delta indices[t] - M; -1 means base model only.
"""
import torch

from triteia_amd.python.capi import route_plan, sbmm_2_4_routed, sgmv_routed
from .lora import lora_forloop
from .sbmm import sbmm_4bit_2_4_forloop


def baseline_ldmm(indices, x, LwA, LwB, DeltaW, metas, ss, base_weight=None, debug=False):
    """Gather / for-loop formulation (ldmm.py:8-48)."""
    x_ = x if x.dtype == torch.float16 else x.to(torch.float16)
    if base_weight is not None:
        y = torch.matmul(x_, base_weight.t())
    else:
        y = torch.zeros(x_.shape[0], LwB.shape[2], dtype=x_.dtype, device=x.device)
    if torch.all(indices == -1):
        return y.to(x.dtype)
    M = LwA.shape[0]
    mask_lora = (indices < M) & (indices != -1)
    mask_sbmm = (indices >= M) & (indices != -1)
    if mask_lora.sum() > 0:
        y[mask_lora] += lora_forloop(LwA.to(torch.float16), LwB.to(torch.float16), x_[mask_lora],
                                     indices[mask_lora].to(torch.long))
    if mask_sbmm.sum() > 0:
        y[mask_sbmm] += sbmm_4bit_2_4_forloop(DeltaW, x_[mask_sbmm], metas, ss, indices[mask_sbmm] - M)
    return y.to(x.dtype)


def ldmm(indices, x, LwA, LwB, DeltaW, metas, ss, base_weight=None, debug=False):
    """One routed LoRA pass (shrink + expand) for the LoRA tokens plus one routed sparse pass for
    the delta tokens, both accumulating in place into the base output; no gathers, no host
    synchronisation.  The reference routes the LoRA tokens through BGMV, which wants every
    adapter transposed on each call (ldmm.py:93-105); the routed SGMV kernels
    read LwA / LwB as they are, one routing pass serving both of its stages.

    indices int [B]; x [B, H1]; LwA [M, H1, R]; LwB [M, R, H2]; DeltaW / metas / ss the stacked
    packed deltas.  Returns [B, H2] in x.dtype."""
    x_ = x.to(torch.float16)
    x_ = x_ if x_.is_contiguous() else x_.contiguous()
    if base_weight is not None:
        y = torch.matmul(x_, base_weight.t())
    else:
        y = torch.zeros(x_.shape[0], LwB.shape[2], dtype=x_.dtype, device=x_.device)
    M = LwA.shape[0]
    idx32 = indices.to(torch.int32)
    if M > 0:
        # the plan over M adapters skips -1 and every index >= M (the delta tokens)
        plan = route_plan(idx32, M)
        v = torch.zeros((x_.shape[0], LwA.shape[2]), dtype=torch.float16, device=x_.device)
        sgmv_routed(v, x_, LwA.to(torch.float16).contiguous(), plan)
        sgmv_routed(y, v, LwB.to(torch.float16).contiguous(), plan)
    if DeltaW.shape[0] > 0:
        sbmm_2_4_routed(x_, DeltaW, metas, y, ss, idx32, index_offset=M, accumulate=True)
    return y.to(x.dtype)
