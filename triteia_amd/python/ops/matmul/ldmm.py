"""LoRA + Delta mixed multi-model matmul (triteia/python/ops/matmul/ldmm.py:8-174).

indices[t] in [0, M) selects LoRA adapter indices[t]; indices[t] >= M selects the 2:4 int4
delta indices[t] - M; -1 means base model only.
"""
import torch

from triteia_amd.python.capi import route_plan, routed_workspace, sbmm_2_4_routed, sgmv_routed
from .lora import lora_forloop
from .sbmm import sbmm_4bit_2_4_forloop


_SIDE_STREAMS = {}


def _side_stream(device):
    """One extra stream per device (default priority), made at first use."""
    key = torch.device(device).index if torch.device(device).index is not None else torch.cuda.current_device()
    if key not in _SIDE_STREAMS:
        _SIDE_STREAMS[key] = torch.cuda.Stream(device=key)
    return _SIDE_STREAMS[key]


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
    M = LwA.shape[0]
    idx32 = indices.to(torch.int32)
    if M > 0:
        A16, B16 = LwA.to(torch.float16).contiguous(), LwB.to(torch.float16).contiguous()
        ws = routed_workspace(x_.shape[0], M, x_.device)
        v = torch.empty((x_.shape[0], LwA.shape[2]), dtype=torch.float16, device=x_.device)
    if M > 0 and base_weight is not None:
        # Routing and the LoRA shrink need only x: they run on a side stream beside the base GEMM (a
        # library GEMM of a few hundred tokens leaves CUs idle); the expand follows the GEMM.  All
        # buffers are allocated on the current stream, which also frees them.
        cur = torch.cuda.current_stream(x_.device)
        side = _side_stream(x_.device)
        side.wait_stream(cur)
        # (the GEMM is enqueued ahead of the side stream's work: recorded into a HIP graph in the other order, the
        # step measured 30 us longer on 256 tokens x 4096 x 11008; launched eagerly the order makes no difference)
        y = torch.matmul(x_, base_weight.t())
        with torch.cuda.stream(side):
            plan = route_plan(idx32, M, workspace=ws)      # skips -1 and every index >= M (the delta tokens)
            sgmv_routed(v, x_, A16, plan, accumulate=False)
        if DeltaW.shape[0] > 0:
            # LoRA tokens and delta tokens are different rows of y (disjoint index ranges): the expand stays
            # on the side stream, beside the delta kernel, and joins at the end
            side.wait_stream(cur)
            with torch.cuda.stream(side):
                sgmv_routed(y, v, B16, plan)
            sbmm_2_4_routed(x_, DeltaW, metas, y, ss, idx32, index_offset=M, accumulate=True)
            cur.wait_stream(side)
            return y.to(x.dtype)
        cur.wait_stream(side)
        sgmv_routed(y, v, B16, plan)
    else:
        if base_weight is not None:
            y = torch.matmul(x_, base_weight.t())
        else:
            y = torch.zeros(x_.shape[0], LwB.shape[2], dtype=x_.dtype, device=x_.device)
        if M > 0:
            plan = route_plan(idx32, M, workspace=ws)
            sgmv_routed(v, x_, A16, plan, accumulate=False)
            sgmv_routed(y, v, B16, plan)
    if DeltaW.shape[0] > 0:
        sbmm_2_4_routed(x_, DeltaW, metas, y, ss, idx32, index_offset=M, accumulate=True)
    return y.to(x.dtype)
