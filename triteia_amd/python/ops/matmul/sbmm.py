"""Selective (index-routed) batched matmul: y[t] = base(x[t]) + x[t] @ W[indices[t]], -1 = no delta.

Function names and arguments follow triteia/python/ops/matmul/sbmm.py:7-142.  The
`forloop` / `multilaunch` variants keep the reference's host-driven structure (and
its requirement that equal indices are adjacent); `native` does all routing on the
device and accepts any order.
"""
import torch

from triteia_amd.python.capi import mul_2_4, sbmm_2_4, sbmm_2_4_multilaunch, sbmm_2_4_routed


def _base(xs, out_features, base_weight):
    if base_weight is not None:
        return torch.matmul(xs, base_weight.t())
    return torch.zeros(xs.shape[0], out_features, dtype=xs.dtype, device=xs.device)


def sbmm_16bit_forloop(weights, xs, indices, base_weight=None):
    """fp16 reference: dense weights [N, k, m] (sbmm.py:7-23)."""
    y = _base(xs, weights.shape[2], base_weight)
    if torch.all(indices == -1):
        return y
    for id in torch.unique(indices).tolist():
        if id != -1:
            idx_mask = indices == id
            y[idx_mask] += torch.matmul(xs[idx_mask], weights[id])
    return y


def sbmm_4bit_2_4_forloop(qweights, xs, metas, ss, indices, base_weight=None):
    """One gather + mul_2_4 + scatter per distinct index (sbmm.py:26-51)."""
    y = _base(xs, ss.shape[2], base_weight)
    if torch.all(indices == -1):
        return y
    workspace = torch.zeros(y.shape[1] // 128 * 16, device=xs.device, dtype=torch.int32)
    for id in torch.unique(indices).tolist():
        if id != -1:
            idx_mask = indices == id
            inp = xs[idx_mask].contiguous()
            output = torch.zeros((inp.shape[0], y.shape[1]), dtype=xs.dtype, device=xs.device)
            mul_2_4(inp, qweights[id], metas[id], output, ss[id], workspace)
            y[idx_mask] += output
    return y


def _runs(indices):
    """(run ids, starts, counts) of a grouped index vector, -1 runs dropped (host sync, as sbmm.py:96-123)."""
    unique_indices, counts = torch.unique_consecutive(indices, return_counts=True)
    starts = torch.cumsum(counts, dim=0) - counts
    keep = unique_indices != -1
    return unique_indices[keep].int(), starts[keep].int(), counts[keep].int()


def sbmm_4bit_2_4_multilaunch(qweights, xs, metas, ss, indices, base_weight=None):
    """One mul_2_4 launch per run of equal indices, driven from the host (sbmm.py:54-86)."""
    y = _base(xs, ss.shape[2], base_weight)
    if torch.all(indices == -1):
        return y
    unique_indices, start, counts = _runs(indices)
    workspace = torch.zeros(len(unique_indices), y.shape[1] // 8, device=xs.device, dtype=torch.int32)
    output = torch.zeros_like(y)
    sbmm_2_4_multilaunch(xs, qweights, metas, output, ss, unique_indices, workspace, start, counts)
    y += output
    return y


def sbmm_4bit_2_4_native(qweights, xs, metas, ss, indices, base_weight=None):
    """Single-launch routed sbmm (sbmm.py:89-142): tokens are grouped by index on the device, each
    delta's weights are read once, and the result is accumulated straight into the base output.
    No host synchronisation; indices may come in any order."""
    y = _base(xs, ss.shape[2], base_weight)
    if indices.dtype != torch.int32:
        indices = indices.to(torch.int32)
    xs = xs if xs.is_contiguous() else xs.contiguous()
    sbmm_2_4_routed(xs, qweights, metas, y, ss, indices, accumulate=base_weight is not None)
    return y


def sbmm_4bit_2_4_runs(qweights, xs, metas, ss, indices, base_weight=None):
    """The reference's native call structure kept verbatim: host-side run table, then one
    `sbmm_2_4` launch over all runs and `y += output` (sbmm.py:112-141).  Needs grouped indices."""
    y = _base(xs, ss.shape[2], base_weight)
    if torch.all(indices == -1):
        return y
    unique_indices, start, counts = _runs(indices)
    workspace = torch.zeros(len(unique_indices), y.shape[1] // 8, device=xs.device, dtype=torch.int32)
    output = torch.zeros((xs.shape[0], ss.shape[2]), dtype=torch.float16, device=xs.device)
    sbmm_2_4(xs, qweights, metas, output, ss, unique_indices, workspace, start, counts)
    y += output
    return y
