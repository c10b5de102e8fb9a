"""2:4 sparsity helpers and the packed-layout codec (torch, any device).

The layout is the reference's (triteia/python/nn/linear.py:79-141 with
trans=True; permutation triteia/python/ops/utils/sparsity.py:35-61; metadata
order sparsity.py:134-161), produced here with reshape/permute index
arithmetic instead of gather tables so that it also runs on the GPU at full
model sizes:

  qweight int32 [k/32, 2m]: per packed row `tr` (32 dense k) and 64-column
      chunk, 32 sixteen-byte vectors; vector i = 4*(i//4) + a holds columns
      8*(i//4)..+7 and compressed-k entries {2a, 2a+1, 2a+8, 2a+9}; in word w
      nibble n = (block, r2, r1) in the order [0,2,4,6,1,3,5,7] of
      p = 4*block + 2*r2 + r1 (column 4*block + w, entry 2a + r1 + 8*r2).
  meta int16 [m, k/16] (physical [k/32][m][2]): 16-bit word of (column r,
      16-k block 2*tr + h) sits at bits [r//64 | b1 b5 b4 b3 b0 h b2] inside
      packed row tr; each word = four (lo | hi << 2) codes, low bits first.
"""
import torch

_NIBBLE_ORDER = (0, 2, 4, 6, 1, 3, 5, 7)


def calculate_sparsity(x: torch.Tensor):
    return 1 - (x != 0).sum().float() / x.numel()


def mask_creator(x: torch.Tensor, n: int = 2, m: int = 4):
    """N:M mask keeping the n largest-magnitude entries of each group of m (flat order).

    Same contract as the reference's mask_creator (sparsity.py:99-118); ties are
    resolved by a stable sort (the reference leaves them unspecified)."""
    if x.numel() % m != 0:
        raise ValueError(f"Tensor of size {x.shape} can't be evenly divided into {m} groups")
    groups = x.detach().abs().reshape(-1, m)
    drop = torch.argsort(groups, dim=1, stable=True)[:, : int(m - n)]
    mask = torch.ones(groups.shape, device=groups.device)
    return mask.scatter_(dim=1, index=drop, value=0).reshape(x.shape)


def positions_from_mask(mask: torch.Tensor):
    """[m, k] 0/1 mask with exactly two ones per aligned group of 4 -> (lo, hi) [m, k/4]."""
    m_, k = mask.shape
    g = mask.reshape(m_, k // 4, 4).to(torch.int64)
    if not bool((g.sum(-1) == 2).all()):
        raise ValueError("mask must keep exactly 2 of every 4 entries")
    pos = torch.arange(4, device=mask.device)
    lo = torch.where(g > 0, pos, 4).amin(-1)
    hi = torch.where(g > 0, pos, -1).amax(-1)
    return lo, hi


def pack_nibbles(nib: torch.Tensor) -> torch.Tensor:
    """[k/2, m] values 0..15 (compressed-k major) -> qweight int32 [k/32, 2m]."""
    k2, m = nib.shape
    if k2 % 16 != 0 or m % 64 != 0:
        raise ValueError("need k % 32 == 0 and m % 64 == 0")
    # entry j = 8*r2 + 2*a + r1 ; column = 64*chunk + 8*i4 + 4*block + w
    t = nib.to(torch.int64).reshape(k2 // 16, 2, 4, 2, m // 64, 8, 2, 4)   # tr r2 a r1 chunk i4 block w
    t = t.permute(0, 4, 5, 2, 7, 6, 1, 3)                                   # tr chunk i4 a w block r2 r1
    t = t.reshape(k2 // 16, m // 64, 8, 4, 4, 8)                            # ... p = 4*block + 2*r2 + r1
    word = torch.zeros(t.shape[:-1], dtype=torch.int64, device=nib.device)
    for n, p in enumerate(_NIBBLE_ORDER):
        word |= t[..., p] << (4 * n)
    word = torch.where(word >= 2 ** 31, word - 2 ** 32, word)
    return word.reshape(k2 // 16, 2 * m).to(torch.int32)


def unpack_nibbles(qweight: torch.Tensor) -> torch.Tensor:
    """qweight int32 [k/32, 2m] -> [k/2, m] values 0..15 (uint8)."""
    kt, m2 = qweight.shape
    m = m2 // 2
    word = qweight.to(torch.int64) & 0xFFFFFFFF
    word = word.reshape(kt, m // 64, 8, 4, 4)                               # tr chunk i4 a w
    cols = [None] * 8
    for n, p in enumerate(_NIBBLE_ORDER):
        cols[p] = (word >> (4 * n)) & 15
    t = torch.stack(cols, dim=-1).reshape(kt, m // 64, 8, 4, 4, 2, 2, 2)    # tr chunk i4 a w block r2 r1
    t = t.permute(0, 6, 3, 7, 1, 2, 5, 4)                                   # tr r2 a r1 chunk i4 block w
    return t.reshape(kt * 16, m).to(torch.uint8)


def _meta_words(lo: torch.Tensor, hi: torch.Tensor) -> torch.Tensor:
    """Kept positions (lo < hi) [m, k/4] -> the 16-bit metadata words as int64 [m, k/16], word (r, c) = the four
    (lo | hi << 2) codes of column r in 16-k block c, low bits first (logical order, before any re-layout)."""
    m, kg = lo.shape
    code = (lo.to(torch.int64) | (hi.to(torch.int64) << 2)).reshape(m, kg // 4, 4)
    return code[..., 0] | (code[..., 1] << 4) | (code[..., 2] << 8) | (code[..., 3] << 12)


def meta_raw(lo: torch.Tensor, hi: torch.Tensor) -> torch.Tensor:
    """The metadata words int16 [m, k/16] in logical order: row = output column, column = 16-k block (what the
    CUTLASS-style compressor yields before the kernel's re-layout, triteia/python/ops/utils/sparsity.py:220-244)."""
    w16 = _meta_words(lo, hi)
    return torch.where(w16 >= 2 ** 15, w16 - 2 ** 16, w16).to(torch.int16)


def pack_meta(lo: torch.Tensor, hi: torch.Tensor) -> torch.Tensor:
    """Kept positions (lo < hi) [m, k/4] -> metadata int16 [m, k/16] in physical order."""
    m, kg = lo.shape
    if m % 64 != 0 or kg % 8 != 0:
        raise ValueError("need m % 64 == 0 and k % 32 == 0")
    w16 = _meta_words(lo, hi)                                   # [m, k/16]
    t = w16.reshape(m // 64, 2, 2, 2, 2, 2, 2, kg // 8, 2)     # R b5 b4 b3 b2 b1 b0 tr h
    t = t.permute(7, 0, 5, 1, 2, 3, 6, 8, 4)                    # tr R b1 b5 b4 b3 b0 h b2
    t = t.reshape(m, kg // 4)
    t = torch.where(t >= 2 ** 15, t - 2 ** 16, t)
    return t.to(torch.int16)


def unpack_meta(meta: torch.Tensor):
    """metadata int16 [m, k/16] (physical order) -> (lo, hi) [m, k/4]."""
    m, nc = meta.shape
    t = (meta.to(torch.int64) & 0xFFFF).reshape(nc // 2, m // 64, 2, 2, 2, 2, 2, 2, 2)  # tr R b1 b5 b4 b3 b0 h b2
    t = t.permute(1, 3, 4, 5, 8, 2, 6, 0, 7)                                             # R b5 b4 b3 b2 b1 b0 tr h
    w16 = t.reshape(m, nc)
    code = torch.stack([(w16 >> (4 * g)) & 15 for g in range(4)], dim=-1).reshape(m, nc * 4)
    return code & 3, code >> 2


def pack_2_4(q: torch.Tensor, lo: torch.Tensor, hi: torch.Tensor, scales: torch.Tensor):
    """Pack explicitly positioned 2:4 int4 weights.

    q [m, k/2]: kept values in [-8, 7], two per group of 4 along k (the one at `lo` first);
    lo, hi [m, k/4]: their positions (lo < hi); scales [m] or [1, m].
    Returns (qweight int32 [k/32, 2m], meta int16 [m, k/16], scales fp16 [1, m])."""
    m = q.shape[0]
    nib = (q.to(torch.int64) + 8)
    if bool((nib < 0).any()) or bool((nib > 15).any()):
        raise ValueError("values must lie in [-8, 7]")
    if not bool((lo < hi).all()):
        raise ValueError("positions must satisfy lo < hi")
    qweight = pack_nibbles(nib.t().contiguous())
    return qweight, pack_meta(lo, hi), scales.reshape(1, m).to(torch.float16).contiguous()


GROUP_K = 128   # dense k per scale group (groupsize 64 in the launchers' unit of compressed k)
_GROUP_SCALE_ORDER = [i * 8 + j for i in range(8) for j in (0, 4, 1, 5, 2, 6, 3, 7)]


def pack_group_scales(scales: torch.Tensor) -> torch.Tensor:
    """Scales by (group of 128 dense k, column), [k/128, m] -> the tensor `mul_2_4` takes as `s`: every run of 64
    columns in the reference's stored order (triteia/python/ops/utils/sparsity.py:54-57, nn/linear.py:117)."""
    g, m = scales.shape
    order = torch.tensor(_GROUP_SCALE_ORDER, device=scales.device)
    return scales.to(torch.float16).reshape(-1, 64)[:, order].reshape(g, m).contiguous()


def unpack_group_scales(stored: torch.Tensor) -> torch.Tensor:
    """Inverse of `pack_group_scales`."""
    g, m = stored.shape
    order = torch.tensor(_GROUP_SCALE_ORDER, device=stored.device)
    out = torch.empty((g * m // 64, 64), dtype=stored.dtype, device=stored.device)
    out[:, order] = stored.reshape(-1, 64)
    return out.reshape(g, m)


def unpack_2_4(qweight: torch.Tensor, meta: torch.Tensor, scales: torch.Tensor = None, dtype=torch.float16):
    """Packed tensors -> dense [k, m] weight (x @ W convention).  With `scales` the result is
    fp16(q) * scale (rounded to fp16 like the reference's dequantised test weight,
    triteia/python/ops/utils/generator.py:40); without, the signed integers as `dtype`."""
    nib = unpack_nibbles(qweight)                     # [k/2, m]
    lo, hi = unpack_meta(meta)                        # [m, k/4]
    k2, m = nib.shape
    q = nib.to(torch.int64).t().reshape(m, k2 // 2, 2) - 8
    dense = torch.zeros((m, k2 // 2, 4), dtype=torch.int64, device=qweight.device)
    dense.scatter_(-1, lo.unsqueeze(-1), q[..., 0:1])
    dense.scatter_(-1, hi.unsqueeze(-1), q[..., 1:2])
    dense = dense.reshape(m, 2 * k2).t().contiguous()
    if scales is None:
        return dense.to(dtype)
    if scales.dim() == 2 and scales.shape[0] > 1:      # grouped: stored scales per (128 dense k, column)
        per_row = unpack_group_scales(scales.to(torch.float16)).repeat_interleave(GROUP_K, dim=0)
        return (dense.to(torch.float16) * per_row).to(dtype)
    return (dense.to(torch.float16) * scales.reshape(1, m).to(torch.float16)).to(dtype)
