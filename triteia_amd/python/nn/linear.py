import torch
import torch.nn as nn

from triteia_amd.python.capi import mul_2_4
from triteia_amd.python.ops.utils.sparsity import mask_creator, pack_2_4, positions_from_mask


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
    def pack(self, weight, scales, trans=True):
        """Quantise and pack `weight` [k, m] fp16 with per-column `scales` [1, m] into the
        module's buffers.  The kept 2-of-4 positions come from the magnitude mask, not from
        `!= 0`, so a kept value that quantises to -8 stays where it was.  Unlike the reference
        (linear.py:125-126) the module's attributes are left intact and can be packed again."""
        if weight.dtype != torch.half:
            raise ValueError("Only `torch.half` weights are supported.")
        if not trans:
            raise NotImplementedError("only the 2:4 layout (trans=True) is implemented")
        k, m = weight.shape
        assert (k, m) == (self.infeatures, self.outfeatures)
        dev = self.qweight.device
        w = weight.to(dev)
        s = scales.to(dev).reshape(1, m)
        mask = mask_creator(w.t().contiguous(), n=2, m=4)
        lo, hi = positions_from_mask(mask)
        q = torch.clamp(torch.round(w / s).to(torch.int64) + 8, 0, 15) - 8
        qt = q.t().reshape(m, k // 4, 4)
        kept = torch.stack([qt.gather(-1, lo.unsqueeze(-1)).squeeze(-1), qt.gather(-1, hi.unsqueeze(-1)).squeeze(-1)], -1)
        qweight, meta, s16 = pack_2_4(kept.reshape(m, k // 2), lo, hi, s)
        self.qweight.copy_(qweight)
        self.meta.copy_(meta)
        self.scale.copy_(s16)
