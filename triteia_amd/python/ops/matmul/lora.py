"""LoRA ops: y[t] = base(x[t]) + (x[t] @ A_i) @ B_i with i = indices[t], -1 = none
(triteia/python/ops/matmul/lora.py:4-105)."""
import torch

from triteia_amd.python.capi import add_lora_bgmv, add_lora_sgmv_cutlass, route_plan, sgmv_routed


def _base(x, out_features, base_weight):
    if base_weight is not None:
        return torch.matmul(x, base_weight.t())
    return torch.zeros(x.shape[0], out_features, dtype=x.dtype, device=x.device)


def lora_forloop(weights_A, weights_B, x, indices, base_weight=None):
    """Per-token loop in torch (lora.py:4-20). weights_A [M, k, r], weights_B [M, r, m]."""
    y = _base(x, weights_B.shape[2], base_weight)
    if torch.all(indices == -1):
        return y
    for id in torch.unique(indices).tolist():
        if id != -1:
            idx_mask = indices == id
            y[idx_mask] += torch.matmul(torch.matmul(x[idx_mask], weights_A[id]), weights_B[id])
    return y


def lora_bgmv(weights_A, weights_B, x, indices, base_weight=None, layer_idx=0, scale=1.0):
    """BGMV: one adapter look-up per token (lora.py:22-48).  Tokens with index -1 are skipped
    inside the kernel, so no gather / scatter is needed."""
    y = _base(x, weights_B.shape[2], base_weight)
    weights_A_T = weights_A.transpose(1, 2).contiguous().unsqueeze(1)
    weights_B_T = weights_B.transpose(1, 2).contiguous().unsqueeze(1)
    add_lora_bgmv(y, x.contiguous(), weights_A_T, weights_B_T, indices.to(torch.long), layer_idx, scale)
    return y


def lora_sgmv(weights_A, weights_B, x, indices, base_weight=None, layer_idx=0):
    """SGMV on a host-built segment table, as lora.py:50-105 (needs ascending grouped indices)."""
    y = _base(x, weights_B.shape[2], base_weight)
    if torch.all(indices == -1):
        return y
    rank = weights_A.shape[2]
    counts = torch.bincount(indices[indices >= 0].to(torch.long), minlength=weights_A.shape[0])
    s = torch.zeros(weights_A.shape[0] + 1, dtype=torch.int32, device=x.device)
    s[1:] = torch.cumsum(counts, 0).to(torch.int32)
    skip = int((indices == -1).sum())          # the -1 run leads a sorted vector
    input_x, input_y = x[skip:], y[skip:]
    weights_A = weights_A.unsqueeze(1)
    weights_B = weights_B.unsqueeze(1)
    wa_ptr = torch.tensor([t.data_ptr() for t in weights_A], dtype=torch.int64, device=x.device)
    wb_ptr = torch.tensor([t.data_ptr() for t in weights_B], dtype=torch.int64, device=x.device)
    add_lora_sgmv_cutlass(input_y, input_x.contiguous(), wa_ptr, wb_ptr, s, layer_idx, rank)
    return y


def lora_sgmv_routed(weights_A, weights_B, x, indices, base_weight=None, plan=None):
    """SGMV with device-side grouping: any index order, no host synchronisation; `plan`
    (from capi.route_plan with n_deltas = number of adapters) can be shared with other ops."""
    y = _base(x, weights_B.shape[2], base_weight)
    n_adapters, _, rank = weights_A.shape
    if plan is None:
        plan = route_plan(indices.to(torch.int32), n_adapters)
    x = x if x.is_contiguous() else x.contiguous()
    v = torch.empty((x.shape[0], rank), dtype=x.dtype, device=x.device)
    sgmv_routed(v, x, weights_A.contiguous(), plan, accumulate=False)    # (the expand reads back routed rows only)
    sgmv_routed(y, v, weights_B.contiguous(), plan)
    return y
