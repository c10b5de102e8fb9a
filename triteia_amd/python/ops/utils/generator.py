"""Synthetic data for the multi-model GEMM path (triteia/python/ops/utils/generator.py:7-176).

Same function names and return conventions as the reference; differences:
every function takes `device` and an optional `generator` (seeded
torch.Generator on the CPU; the reference is unseeded and hard-codes CUDA),
and packing records the kept positions explicitly, so a kept value of -8
(nibble 0) survives the round trip.
"""
import numpy as np
import torch

from .sparsity import mask_creator, meta_raw, pack_2_4, positions_from_mask


def _randn(shape, generator, device, dtype=torch.float16):
    return torch.randn(shape, generator=generator, dtype=torch.float32).to(dtype).to(device)


def gen_lora_16_bit(m, n, rank, device="cuda", generator=None):
    A = _randn((m, rank), generator, device)
    B = _randn((rank, n), generator, device)
    return A, B


def gen_batched_lora_16_bit(b, m, n, rank, device="cuda", generator=None):
    As, Bs = zip(*(gen_lora_16_bit(m, n, rank, device, generator) for _ in range(b)))
    return torch.stack(As), torch.stack(Bs)


def fp16_to_sparse(weights, scale, device="cuda", mask=None):
    """Quantise + pack a [k, m] fp16 weight that is (to be made) 2:4 sparse along k.

    Returns (weights, qweight, scales, meta, meta_raw), the reference's five values (generator.py:105-123);
    `meta_raw` is the metadata before the kernel's re-layout: int16 [m, k/16], row = output column."""
    weights = weights.to(device)
    scale = scale.to(device).reshape(1, -1)
    k, m = weights.shape
    if mask is None:
        mask = mask_creator(weights.t().contiguous(), n=2, m=4)
    lo, hi = positions_from_mask(mask)
    q = torch.clamp(torch.round(weights / scale).to(torch.int64) + 8, 0, 15) - 8          # [k, m]
    qt = q.t().reshape(m, k // 4, 4)
    kept = torch.stack([qt.gather(-1, lo.unsqueeze(-1)).squeeze(-1), qt.gather(-1, hi.unsqueeze(-1)).squeeze(-1)], -1)
    qweight, meta, s = pack_2_4(kept.reshape(m, k // 2), lo, hi, scale)
    return weights, qweight, s, meta, meta_raw(lo, hi)


def gen_sparse_quant4_NT(m, k, groupsize=-1, device="cuda", prune_n=2, prune_m=4, generator=None):
    """Random [k, m] weight quantised to int4 with per-column scales and 2:4-pruned along k.

    Returns (uncompress [k, m] fp16 -- the dense weight the packed tensors decode to --,
    qweight, scales [1, m], meta), as generator.py:24-69."""
    if groupsize != -1:
        raise NotImplementedError("only per-channel scales (groupsize=-1)")
    if (prune_n, prune_m) != (2, 4):
        raise NotImplementedError("only 2:4 sparsity")
    maxq = 2 ** 4 - 1
    w = _randn((m, k), generator, device).t()                      # [k, m]
    s = torch.max(torch.abs(w), 0, keepdim=True)[0]
    s = s * (2 / maxq)
    wq = torch.clamp(torch.round(w / s).int() + (maxq + 1) // 2, 0, maxq)
    ref = (wq - (maxq + 1) // 2).half() * s
    mask = mask_creator(wq.t().contiguous(), n=prune_n, m=prune_m)  # on the shifted codes, as the reference does
    uncompress = (mask.to(ref.dtype) * ref.t()).t().contiguous()
    _, q, s_out, meta, _ = fp16_to_sparse(uncompress, s, device=device, mask=mask)
    return uncompress, q, s_out, meta


def gen_batched_sparse_quant4_NT(b, m, n, groupsize=-1, device="cuda:0", generator=None):
    outs = [gen_sparse_quant4_NT(m, n, groupsize=groupsize, device=device, generator=generator) for _ in range(b)]
    unc, qs, scales, metas = (torch.stack(t) for t in zip(*outs))
    return unc, qs, scales, metas


def gen_explicit_sparse_quant4(m, k, device="cuda", generator=None, scale_range=(0.005, 0.02)):
    """The benchmark distribution: kept values uniform integers in [-8, 7], two uniformly chosen
    positions per aligned group of 4 along k, per-column fp16 scale ~ U(scale_range).

    Returns (qweight, scales [1, m], meta, (q [m, k/2], lo, hi))."""
    g = generator
    q = torch.randint(-8, 8, (m, k // 2), generator=g)
    pairs = torch.tensor([(0, 1), (0, 2), (0, 3), (1, 2), (1, 3), (2, 3)])
    sel = torch.randint(0, 6, (m, k // 4), generator=g)
    lo, hi = pairs[sel, 0], pairs[sel, 1]
    s = (torch.rand(m, generator=g) * (scale_range[1] - scale_range[0]) + scale_range[0]).to(torch.float16)
    q, lo, hi, s = q.to(device), lo.to(device), hi.to(device), s.to(device)
    qweight, meta, s_out = pack_2_4(q, lo, hi, s)
    return qweight, s_out, meta, (q, lo, hi)


def generate_model_distribution(distribution, num_queries, num_models, device="cuda", seed=None):
    """Delta index per query over {-1, 0..num_models-1} (generator.py:90-102).

    "uniform", "distinct", "zipf:a" (the reference's law: p_i proportional to i**a over the list
    [-1, 0, 1, ...], i.e. increasing in the index) and, additionally, "rank-zipf:a"
    (p proportional to rank**-a over 0..num_models-1, the usual Zipf law; no -1)."""
    rng = np.random.default_rng(seed)
    to_eval_models = list(range(-1, num_models))
    if distribution == "uniform":
        models = rng.choice(to_eval_models, num_queries)
    elif distribution == "distinct":
        models = to_eval_models
    elif distribution.startswith("zipf"):
        alpha = float(distribution.split(":")[1])
        assert alpha > 1, "alpha must be greater than 1"
        probs = np.array([i ** alpha for i in range(1, len(to_eval_models) + 1)], dtype=np.float64)
        models = rng.choice(to_eval_models, num_queries, p=probs / probs.sum())
    elif distribution.startswith("rank-zipf"):
        alpha = float(distribution.split(":")[1])
        probs = np.array([(i + 1) ** -alpha for i in range(num_models)], dtype=np.float64)
        models = rng.choice(np.arange(num_models), num_queries, p=probs / probs.sum())
    else:
        raise ValueError(f"unknown distribution {distribution!r}")
    return torch.tensor(np.asarray(models), dtype=torch.int32, device=device)


@torch.no_grad()
def torch_weight_to_sparse_marlin(weight, scale, tp_size=1, chunk_by="column", device=None):
    """Pack a [k, m] weight into `tp_size` shards (generator.py:126-176).

    chunk_by="column" splits the output features, "row" the input features.  Each shard
    is packed on its own: metadata of column shards cannot be obtained by slicing."""
    assert chunk_by in ["column", "row"], "chunk_by must be either 'column' or 'row'"
    assert weight.dim() == 2, "weight must be a 2D tensor"
    assert weight.size(0) % tp_size == 0, "out_features must be divisible by tp_size"
    assert weight.size(1) == scale.size(1), "out_features of weight and scale must match"
    device = device if device is not None else weight.device
    qweights, scales, metas = [], [], []
    for i in range(tp_size):
        if chunk_by == "column":
            lo_c, hi_c = i * weight.size(1) // tp_size, (i + 1) * weight.size(1) // tp_size
            tp_weight, tp_scales = weight[:, lo_c:hi_c], scale[:, lo_c:hi_c]
        else:
            lo_r, hi_r = i * weight.size(0) // tp_size, (i + 1) * weight.size(0) // tp_size
            tp_weight, tp_scales = weight[lo_r:hi_r, :], scale
        _, q, s, meta, _ = fp16_to_sparse(tp_weight.contiguous(), tp_scales.contiguous(), device=device)
        qweights.append(q.contiguous())
        scales.append(s.contiguous())
        metas.append(meta.contiguous())
    return qweights, scales, metas
