"""GPTQ 4-bit checkpoint tensors -> dense weights (triteia/python/utils/quant_utils.py:6-76).

Same results as the reference's helpers, computed with broadcast shifts instead of a Python loop
over rows and columns; nothing here is tied to a device.
"""
import torch


@torch.no_grad()
def unpack_4bit_to_32bit_signed(qweight, qzeros):
    """qweight int32 [k/8, m] -> int8 [k, m] (row 8i+j = nibble j of packed row i);
    qzeros int32 [g, m/8] -> int8 [g, m] + 1.  Raises ValueError unless every stored zero point
    is 7, i.e. the checkpoint is symmetric (quant_utils.py:7-36)."""
    shifts = torch.arange(0, 32, 4, dtype=torch.int32, device=qweight.device)
    w = (qweight.unsqueeze(1) >> shifts.view(1, 8, 1)) & 0xF           # [k/8, 8, m]
    unpacked_weights = w.reshape(qweight.shape[0] * 8, qweight.shape[1]).to(torch.int8)
    z = (qzeros.unsqueeze(2) >> shifts.to(qzeros.device).view(1, 1, 8)) & 0xF   # [g, m/8, 8]
    unpacked_zeros = z.reshape(qzeros.shape[0], qzeros.shape[1] * 8).to(torch.int8)
    if not torch.all(unpacked_zeros == 7):
        raise ValueError(
            "Marlin kernel is compatible only with checkpoints using symmetric quantization."
            "Found non-symmetric quantization for the weight")
    return unpacked_weights, unpacked_zeros + 1


@torch.no_grad()
def dequantize_weight(qweight, qzeros, scales):
    """(q - zero) * scale per group, returned transposed: [m, k] (quant_utils.py:39-46)."""
    unpacked_qweight, unpacked_qzeros = unpack_4bit_to_32bit_signed(qweight, qzeros)
    group_size = unpacked_qweight.shape[0] // scales.shape[0]
    scales = scales.repeat_interleave(group_size, dim=0)
    unpacked_qzeros = unpacked_qzeros.repeat_interleave(group_size, dim=0)
    return ((unpacked_qweight - unpacked_qzeros) * scales).T


@torch.no_grad()
def gptq_unpack(bits, qweight, qzeros, scales, group_size=-1):
    """General GPTQ unpack for 2/4/8 bits: scales * (q - (zero + 1)) as [k, m] (quant_utils.py:49-76).

    qweight int32 [k*bits/32, m] holds 32/bits values per word along k (lowest bits first), qzeros int32
    [g, m*bits/32] the same along m, scales [g, m]; `zero + 1` wraps inside `bits` bits, as in the reference."""
    per_word, mask = 32 // bits, (1 << bits) - 1
    k, m = qweight.shape[0] * per_word, qweight.shape[1]
    if group_size == -1:
        group_size = k
    shifts = torch.arange(per_word, dtype=torch.int32, device=qweight.device) * bits
    q = ((qweight.unsqueeze(1) >> shifts.view(1, per_word, 1)) & mask).reshape(k, m)              # row per_word*i + j
    z = ((qzeros.unsqueeze(2) >> shifts.to(qzeros.device).view(1, 1, per_word)) & mask).reshape(qzeros.shape[0], -1)
    z = (z + 1) & mask
    groups = scales.reshape(-1, scales.shape[-1])
    return groups.repeat_interleave(group_size, dim=0) * (q - z.repeat_interleave(group_size, dim=0))
