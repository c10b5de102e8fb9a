import torch
import torch.nn as nn

from triteia_amd.python.capi import mul_2_4
from triteia_amd.python.ops.utils.sparsity import mask_creator, meta_raw, pack_2_4, positions_from_mask


class sparse_low_precision_linear(nn.Module):
    """Sparse (2:4) int4 linear layer (triteia/python/nn/linear.py:18-141).

    Buffers: qweight int32 [k/32, 2m], meta int16 [m, k/16], scale fp16 [1, m],
    workspace int32 [m/128*16] (zeros; kept for layout compatibility)."""

    def __init__(self, infeatures, outfeatures, groupsize=-1):
        super().__init__()
        assert groupsize in [-1], f"Group size must be -1, got {groupsize}"
        assert infeatures % 128 == 0, f"Input features must be a multiple of 128, got {infeatures}"
        assert outfeatures % 256 == 0, f"Output features must be a multiple of 256, got {outfeatures}"
        self.infeatures = infeatures
        self.outfeatures = outfeatures
        self.groupsize = infeatures
        self.register_buffer("qweight", torch.empty((infeatures // 32, outfeatures * 16 // 8), dtype=torch.int32))
        self.register_buffer("meta", torch.empty((outfeatures, infeatures // 16), dtype=torch.int16))
        self.register_buffer("scale", torch.empty((1, outfeatures), dtype=torch.float16))
        self.register_buffer("workspace", torch.zeros(outfeatures // 128 * 16, dtype=torch.int32))

    def forward(self, x):
        C = torch.empty(x.shape[:-1] + (self.outfeatures,), dtype=x.dtype, device=x.device)
        x2 = x.reshape(-1, x.shape[-1])
        x2 = x2 if x2.is_contiguous() else x2.contiguous()
        mul_2_4(x2, self.qweight, self.meta, C.view(-1, C.shape[-1]), self.scale, self.workspace)
        return C

    @torch.no_grad()
    def pack(self, weight, scales, trans=False):
        """Quantise and pack `weight` [k, m] fp16 with per-column `scales` [1, m] (linear.py:79-141).

        Signature and destinations are the reference's: `trans=True` selects the 2:4 layout the kernels read
        (every call site of the reference passes it: generator.py:66,120,173); the default, `trans=False`, is
        the dense-Marlin permutation, which no kernel of this path consumes, and raises.  The result goes where
        the reference puts it -- the attributes `B`, `s` and `meta` that its callers assign beforehand
        (generator.py:60-65), when they exist -- and also into the registered buffers `qweight`, `scale`,
        `meta`, so that `forward` works on a module packed either way; `meta_raw` holds the metadata before
        the kernel's re-layout.  The kept 2-of-4 positions come from the magnitude mask, not from `!= 0`,
        so a kept value that quantises to -8 stays where it was.  Unlike the reference (linear.py:125-126)
        `infeatures` and `groupsize` are left intact and the module can be packed again."""
        if weight.dtype != torch.half:
            raise ValueError("Only `torch.half` weights are supported.")
        if not trans:
            raise NotImplementedError(
                "pack(..., trans=False) asks for the dense-Marlin permutation of the compressed weight, a layout that "
                "no kernel of this path reads; pass trans=True for the 2:4 layout (as every caller in the reference does)")
        k, m = weight.shape
        assert (k, m) == (self.infeatures, self.outfeatures)
        B, s_attr = getattr(self, "B", None), getattr(self, "s", None)
        dev = B.device if isinstance(B, torch.Tensor) else self.qweight.device
        w = weight.to(dev)
        s = scales.to(dev).reshape(1, m)
        mask = mask_creator(w.t().contiguous(), n=2, m=4)
        lo, hi = positions_from_mask(mask)
        q = torch.clamp(torch.round(w / s).to(torch.int64) + 8, 0, 15) - 8
        qt = q.t().reshape(m, k // 4, 4)
        kept = torch.stack([qt.gather(-1, lo.unsqueeze(-1)).squeeze(-1), qt.gather(-1, hi.unsqueeze(-1)).squeeze(-1)], -1)
        qweight, meta, s16 = pack_2_4(kept.reshape(m, k // 2), lo, hi, s)
        self.qweight.copy_(qweight)
        self.meta.copy_(meta)        # (the buffer, or the tensor a caller has put in its place)
        self.scale.copy_(s16)
        if isinstance(B, torch.Tensor):
            B[:, :] = qweight.to(B.device)
        if isinstance(s_attr, torch.Tensor):
            s_attr[:, :] = s16.to(s_attr.device)
        self.meta_raw = meta_raw(lo, hi)


class multi_delta_linear(nn.Module):
    """One linear layer serving many fine-tuned variants of a base model at once: an optional
    dense fp16 base weight plus `n_deltas` stacked 2:4 int4 deltas; every token picks its delta
    (or none, index -1) through an index vector.  The layer a serving engine calls once per
    projection (the reference has the op, ops/matmul/sbmm.py:89-142, but no module around it).

    Buffers: qweight int32 [N, k/32, 2m], meta int16 [N, m, k/16], scale fp16 [N, 1, m],
    base fp16 [m, k] (optional).  `forward(x, indices)` routes on the device; with
    `plan=route_plan(indices, N)` the same routing is shared by all layers of a forward pass."""

    def __init__(self, infeatures, outfeatures, n_deltas, with_base=False):
        super().__init__()
        assert infeatures % 128 == 0, f"Input features must be a multiple of 128, got {infeatures}"
        assert outfeatures % 256 == 0, f"Output features must be a multiple of 256, got {outfeatures}"
        self.infeatures, self.outfeatures, self.n_deltas = infeatures, outfeatures, n_deltas
        self.register_buffer("qweight", torch.zeros((n_deltas, infeatures // 32, outfeatures * 2), dtype=torch.int32))
        self.register_buffer("meta", torch.zeros((n_deltas, outfeatures, infeatures // 16), dtype=torch.int16))
        self.register_buffer("scale", torch.zeros((n_deltas, 1, outfeatures), dtype=torch.float16))
        self.register_buffer("base", torch.zeros((outfeatures, infeatures), dtype=torch.float16) if with_base else None)

    @torch.no_grad()
    def load_delta(self, i, module_or_qweight, meta=None, scale=None):
        """Copy one packed delta into slot i: from a `sparse_low_precision_linear` or from its three tensors."""
        if isinstance(module_or_qweight, sparse_low_precision_linear):
            m = module_or_qweight
            module_or_qweight, meta, scale = m.qweight, m.meta, m.scale
        self.qweight[i].copy_(module_or_qweight)
        self.meta[i].copy_(meta)
        self.scale[i].copy_(scale.reshape(1, -1))

    @torch.no_grad()
    def pack_delta(self, i, weight, scales):
        """Quantise and pack a dense [k, m] fp16 delta with per-column scales into slot i."""
        layer = sparse_low_precision_linear(self.infeatures, self.outfeatures).to(self.qweight.device)
        layer.pack(weight, scales, True)
        self.load_delta(i, layer)

    def forward(self, x, indices, plan=None):
        """x [..., k] fp16, indices int32 [tokens] in {-1, 0..N-1} (any order) -> [..., m]."""
        from triteia_amd.python.capi import sbmm_2_4_planned, sbmm_2_4_routed
        x2 = x.reshape(-1, x.shape[-1])
        x2 = x2 if x2.is_contiguous() else x2.contiguous()
        if self.base is not None:
            y = torch.matmul(x2, self.base.t())
        else:
            y = torch.zeros((x2.shape[0], self.outfeatures), dtype=x.dtype, device=x.device)
        if plan is not None:
            sbmm_2_4_planned(x2, self.qweight, self.meta, y, self.scale, plan, accumulate=True)
        else:
            sbmm_2_4_routed(x2, self.qweight, self.meta, y, self.scale, indices.to(torch.int32), accumulate=True)
        return y.view(x.shape[:-1] + (self.outfeatures,))
