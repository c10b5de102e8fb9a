"""CPU oracle for the fp16 x (int4, 2:4-sparse) multi-model GEMM path.

TEST INFRASTRUCTURE ONLY.  This module is a plain numpy restatement of the
algorithm the reference implements for this path.  Only `tests/`,
`__graft_entry__.smoke()` and the `cpu_baseline` leg of `bench.py` may import
it; nothing under `triteia_amd/` does, and the product path never falls back
to it.

What each function follows in the reference (paths relative to the reference
checkout):

  perm_2_4 ...................... triteia/python/ops/utils/sparsity.py:35-61
  meta_scatter_offsets .......... triteia/python/ops/utils/sparsity.py:134-161
  encode_2_4_nonzero ............ triteia/python/ops/utils/sparsity.py:167-290
  mask_2_4 ...................... triteia/python/ops/utils/sparsity.py:99-118
  pack_reference ................ triteia/python/nn/linear.py:79-141
  scale_perm_2_4, store/load_group_scales, pack_reference_grouped
                                  triteia/python/ops/utils/sparsity.py:54-57,
                                  triteia/python/nn/linear.py:104-118 (scales per
                                  column and group of 128 dense k), used by the
                                  kernel as marlin.cuh:199-209,342-346,378-380
  pack_explicit ................. same layout, positions given explicitly
  unpack ........................ inverse of the two packers (the dense weight
                                  the reference's tests multiply by,
                                  triteia/python/ops/utils/generator.py:40,52)
  matmul_4bit_2_4 ............... triteia/python/ops/matmul/sparse_low_precision.py:5-24
  bmm_4bit_2_4 .................. triteia/python/ops/matmul/bmm.py:6-35
  sbmm_4bit_2_4 ................. triteia/python/ops/matmul/sbmm.py:7-23 (per-token form)
  lora .......................... triteia/python/ops/matmul/lora.py:4-20
  ldmm .......................... triteia/python/ops/matmul/ldmm.py:8-48

How each is pinned (see tests/test_oracle_*.py):

  perm_2_4, meta_scatter_offsets: golden tables written from the reference's
      own functions (tests/golden/), bijection checks, closed forms.
  encode_2_4_nonzero: the installed torch library's
      torch.sparse._semi_structured_conversions (same code table) after undoing
      torch's own reorder.
  pack_*/unpack: exact integer round trips, brute force at the minimum legal
      size, single-nonzero closed forms.
  GEMM / routing / LoRA: float64 textbook loops on tiny inputs.
  grouped scales: the stored order against the golden table of the reference's
      own `_get_perms_2_4`; the arithmetic against a plain loop and against the
      per-column form when all groups carry the same scales.  No test, caller or
      fixture of the reference exercises grouped scales on this path (its module
      asserts groupsize == -1, linear.py:27), so which column a stored scale
      multiplies inside the reference's kernel is taken from reading
      marlin.cuh:199-209,378-380 together with the weight permutation: PARITY
      UNPINNED beyond that.
  mask_2_4 tie-breaking (equal magnitudes inside a group): PARITY UNPINNED --
      the reference uses an unstable argsort there; BASELINE workloads give the
      kept positions explicitly and never depend on it.
"""
from __future__ import annotations

import numpy as np

# --------------------------------------------------------------------------
# layout tables
# --------------------------------------------------------------------------

_INTERLEAVE = np.array([0, 2, 4, 6, 1, 3, 5, 7])


def perm_2_4() -> np.ndarray:
    """The 1024-entry nibble permutation of one (16 compressed-k x 64 column) chunk.

    Restates `_get_perms_2_4` (sparsity.py:35-54).  `packed_flat[pos] =
    tiled_flat[perm[pos]]` where `tiled_flat` is four 16x16 tiles laid out
    tile-major (tile, row, col).
    """
    perm = []
    for i in range(32):
        perm1 = []
        col = i // 4
        col_o = col // 2
        for block in (0, 1):
            for row in (2 * (i % 4), 2 * (i % 4) + 1, 2 * (i % 4 + 4), 2 * (i % 4 + 4) + 1):
                perm1.append(16 * row + col_o * 256 + 8 * (col % 2) + 4 * block)
        for j in range(4):
            perm.extend(p + j for p in perm1)
    perm = np.array(perm, dtype=np.int64)
    return perm.reshape(-1, 8)[:, _INTERLEAVE].ravel()


def scale_perm_2_4() -> np.ndarray:
    """Order in which a run of 64 grouped scales is stored (`scale_perm` of `_get_perms_2_4`, sparsity.py:54-57):
    stored[p] = scale[perm[p]], i.e. inside every run of 8 columns the order 0 4 1 5 2 6 3 7."""
    return np.array([i * 8 + j for i in range(8) for j in (0, 4, 1, 5, 2, 6, 3, 7)], dtype=np.int64)


GROUP_K = 128   # dense k per scale group: groupsize 64 in the launcher's unit of compressed k (marlin_nm.cu:68)


def store_group_scales(scales: np.ndarray) -> np.ndarray:
    """[k/128, m] scales by (group, column) -> the stored tensor of the same shape (linear.py:117,124)."""
    g, m = scales.shape
    assert m % 64 == 0
    return np.ascontiguousarray(scales.reshape(-1, 64)[:, scale_perm_2_4()].reshape(g, m))


def load_group_scales(stored: np.ndarray) -> np.ndarray:
    """Inverse of `store_group_scales`."""
    g, m = stored.shape
    out = np.empty((g * m // 64, 64), dtype=stored.dtype)
    out[:, scale_perm_2_4()] = stored.reshape(-1, 64)
    return out.reshape(g, m)


def perm_2_4_closed_form() -> np.ndarray:
    """Same table from the closed form (lane i, word w, nibble n)."""
    out = np.empty(1024, dtype=np.int64)
    for i in range(32):
        for w in range(4):
            for n in range(8):
                p = _INTERLEAVE[n]
                block, rsel = p // 4, p % 4
                row = 2 * (i % 4) + (rsel % 2) + 8 * (rsel // 2)
                col64 = 8 * (i // 4) + 4 * block + w
                tile, cc = col64 // 16, col64 % 16
                out[(4 * i + w) * 8 + n] = tile * 256 + row * 16 + cc
    return out


def meta_scatter_offsets(m: int, ncols: int) -> np.ndarray:
    """Flat destination of logical metadata element (r, c), int16 metadata.

    Restates `_calculate_meta_reordering_scatter_offsets` (sparsity.py:134-161)
    for `meta_dtype.itemsize == 2` (group_x = 64, group_y = 32).
    """
    r = np.repeat(np.arange(m, dtype=np.int64)[:, None], ncols, axis=1)
    c = np.repeat(np.arange(ncols, dtype=np.int64)[None, :], m, axis=0)
    group_x, group_y = 64, 32
    r = (r // group_x * group_x + (r % 2) * 2 + (r % 8) // 4
         + ((r % group_y) % 4) // 2 * 32 + ((r % group_x) // 8) * 4)
    topright = ((r % 2 == 0) & (c % 2 == 1)).astype(np.int64)
    bottomleft = ((r % 2 == 1) & (c % 2 == 0)).astype(np.int64)
    r = r + topright - bottomleft
    c = c - (topright - bottomleft)
    return ((c // 2) * m * 2 + r * 2 + c % 2).ravel()


def meta_offset_closed_form(r: int, c: int, m: int) -> int:
    """Bit-level closed form of `meta_scatter_offsets` for one element.

    Inside one 32-dense-k block (`c // 2`) the metadata of 64 output columns
    is 128 consecutive int16; the position inside that run has bits
    [b1 b5 b4 b3 b0 h b2] (MSB first) with b_i = bit i of r % 64, h = c % 2.
    """
    b = [(r >> i) & 1 for i in range(6)]
    pos = (b[1] << 6) | (b[5] << 5) | (b[4] << 4) | (b[3] << 3) | (b[0] << 2) | ((c % 2) << 1) | b[2]
    return (c // 2) * 2 * m + (r // 64) * 128 + pos


# --------------------------------------------------------------------------
# 2:4 encode
# --------------------------------------------------------------------------

def mask_2_4(x: np.ndarray) -> np.ndarray:
    """Keep the 2 largest-magnitude entries of each aligned group of 4 (flat order).

    Follows `mask_creator` (sparsity.py:99-118).  Ties are broken by a stable
    argsort here; the reference's order for ties is unspecified (unpinned).
    """
    g = np.abs(x.astype(np.float32)).reshape(-1, 4)
    drop = np.argsort(g, axis=1, kind="stable")[:, :2]
    mask = np.ones_like(g, dtype=bool)
    np.put_along_axis(mask, drop, False, axis=1)
    return mask.reshape(x.shape)


def encode_2_4_nonzero(dense: np.ndarray):
    """Compress an [m, k] integer matrix that is zero outside 2-of-4 positions.

    Follows `sparse_semi_structured_from_dense_cutlass` (sparsity.py:167-283)
    for 16-bit metadata, up to (not including) the metadata reorder.  Kept
    positions are inferred from `!= 0`, exactly as the reference does, so a
    kept value that happens to be 0 is treated as pruned.

    Returns (sparse [m, k/2], meta16 [m, k/16] uint16 in logical order).
    """
    m, k = dense.shape
    d4 = dense.reshape(m, k // 4, 4)
    nz = d4 != 0
    m0, m1, _m2, m3 = nz[..., 0], nz[..., 1], nz[..., 2], nz[..., 3]
    expr0 = m0 & m1
    expr1 = ~m0 & m1
    expr2 = ~m0 & ~m1
    bit0 = expr1
    bit1 = expr2
    bit2 = expr0 | expr2 | m3
    bit3 = expr1 | ~m1
    idx0 = bit0.astype(np.int64) | (bit1.astype(np.int64) << 1)
    idx1 = bit2.astype(np.int64) | (bit3.astype(np.int64) << 1)
    s0 = np.take_along_axis(d4, idx0[..., None], axis=-1)
    s1 = np.take_along_axis(d4, idx1[..., None], axis=-1)
    sparse = np.concatenate([s0, s1], axis=-1).reshape(m, k // 2)
    code = (idx0 | (idx1 << 2)).reshape(m, k // 16, 4)
    meta16 = (code[..., 0] | (code[..., 1] << 4) | (code[..., 2] << 8) | (code[..., 3] << 12)).astype(np.uint16)
    return sparse, meta16


def encode_2_4_explicit(values: np.ndarray, lo: np.ndarray, hi: np.ndarray):
    """Metadata from explicit kept positions (lo < hi), one pair per group of 4.

    values: [m, k/2] stored values in k order (value at `lo` first).
    lo, hi: [m, k/4] positions in 0..3.
    The code `lo | hi << 2` equals the reference's table for all six legal
    patterns (sparsity.py:212-218).
    """
    m, kg = lo.shape
    code = (lo.astype(np.int64) | (hi.astype(np.int64) << 2)).reshape(m, kg // 4, 4)
    meta16 = (code[..., 0] | (code[..., 1] << 4) | (code[..., 2] << 8) | (code[..., 3] << 12)).astype(np.uint16)
    return values, meta16


def reorder_meta(meta16: np.ndarray) -> np.ndarray:
    """Scatter logical [m, k/16] metadata to its physical order (sparsity.py:285-290)."""
    m, ncols = meta16.shape
    out = np.empty(m * ncols, dtype=np.uint16)
    out[meta_scatter_offsets(m, ncols)] = meta16.ravel()
    return out.reshape(m, ncols)


def unreorder_meta(meta_phys: np.ndarray) -> np.ndarray:
    m, ncols = meta_phys.shape
    return meta_phys.ravel()[meta_scatter_offsets(m, ncols)].reshape(m, ncols)


# --------------------------------------------------------------------------
# pack / unpack
# --------------------------------------------------------------------------

def _pack_nibbles(sparse_t: np.ndarray) -> np.ndarray:
    """[k/2, m] nibble values (0..15) -> qweight [k/32, 2m] int32 (linear.py:127-139)."""
    k2, m = sparse_t.shape
    w = sparse_t.reshape(k2 // 16, 16, m // 16, 16).transpose(0, 2, 1, 3).reshape(k2 // 16, m * 16)
    perm = perm_2_4()
    res = w.reshape(-1, perm.size)[:, perm].reshape(w.shape).astype(np.uint32)
    q = np.zeros((res.shape[0], res.shape[1] // 8), dtype=np.uint32)
    for i in range(8):
        q |= res[:, i::8] << np.uint32(4 * i)
    return q.view(np.int32)


def pack_reference(weight: np.ndarray, scales: np.ndarray, mask: np.ndarray | None = None):
    """Restatement of `sparse_low_precision_linear.pack(weight, scales, trans=True)`.

    weight: [k, m] fp16 (already 2:4 sparse along k in the reference's use),
    scales: [1, m] fp16.  Returns (qweight [k/32, 2m] int32, meta [m, k/16]
    int16 physical order, scales [1, m] fp16).  `mask` ([m, k] bool) overrides
    the magnitude-based mask (used to avoid the unpinned tie-breaking).
    """
    k, m = weight.shape
    assert k % 128 == 0 and m % 256 == 0 and weight.dtype == np.float16
    if mask is None:
        mask = mask_2_4(np.ascontiguousarray(weight.T))
    w = np.rint((weight / scales).astype(np.float16).astype(np.float32)).astype(np.int32)  # fp16 divide, round-half-even
    w = np.clip(w + 8, 0, 15)
    w = (mask * w.T).astype(np.int32)                       # [m, k], zero where pruned
    sparse, meta16 = encode_2_4_nonzero(np.ascontiguousarray(w))
    q = _pack_nibbles(np.ascontiguousarray(sparse.T))
    return q, reorder_meta(meta16).view(np.int16), scales.reshape(1, m).astype(np.float16)


def pack_reference_grouped(weight: np.ndarray, scales: np.ndarray, mask: np.ndarray | None = None):
    """`pack(weight, scales, trans=True)` of a module with groups of 128 dense k (linear.py:104-124): every
    weight is divided by the scale of its (group, column); `scales` [k/128, m] by (group, column).  Returns
    (qweight, meta, stored scales [k/128, m])."""
    k, m = weight.shape
    assert k % GROUP_K == 0 and scales.shape == (k // GROUP_K, m)
    per_row = np.repeat(scales.astype(np.float16), GROUP_K, axis=0)                     # [k, m]
    if mask is None:
        mask = mask_2_4(np.ascontiguousarray(weight.T))
    w = np.rint((weight / per_row).astype(np.float16).astype(np.float32)).astype(np.int32)
    w = np.clip(w + 8, 0, 15)
    w = (mask * w.T).astype(np.int32)
    sparse, meta16 = encode_2_4_nonzero(np.ascontiguousarray(w))
    q = _pack_nibbles(np.ascontiguousarray(sparse.T))
    return q, reorder_meta(meta16).view(np.int16), store_group_scales(scales.astype(np.float16))


def pack_explicit(q_kept: np.ndarray, lo: np.ndarray, hi: np.ndarray, scales: np.ndarray):
    """Packer with explicit positions (no `!= 0` inference).

    q_kept: [m, k/2] signed int4 values in [-8, 7], two per group in k order
    (the value at position `lo` first); lo/hi: [m, k/4]; scales [m] or [1, m].
    """
    m, k2 = q_kept.shape
    nib = (q_kept.astype(np.int32) + 8)
    assert nib.min() >= 0 and nib.max() <= 15
    assert np.all(lo < hi)
    _, meta16 = encode_2_4_explicit(nib, lo, hi)
    q = _pack_nibbles(np.ascontiguousarray(nib.T))
    return q, reorder_meta(meta16).view(np.int16), np.asarray(scales, dtype=np.float16).reshape(1, m)


def _inverse_perm_table() -> np.ndarray:
    """inv[row, col64] = position (0..1023) inside the packed chunk."""
    perm = perm_2_4()
    inv = np.empty(1024, dtype=np.int64)
    inv[perm] = np.arange(1024)
    # perm values are tile*256 + row*16 + cc ; col64 = tile*16 + cc
    t = np.arange(1024)
    tile, row, cc = t // 256, (t // 16) % 16, t % 16
    table = np.empty((16, 64), dtype=np.int64)
    table[row, tile * 16 + cc] = inv[t]
    return table


def unpack_codes(qweight: np.ndarray, meta: np.ndarray):
    """Packed tensors -> (nibbles S [k/2, m] in 0..15, lo [m, k/4], hi [m, k/4])."""
    qw = np.ascontiguousarray(qweight).view(np.uint32)
    kt, m2 = qw.shape
    m = m2 // 2
    shifts = (4 * np.arange(8, dtype=np.uint32))
    nib = ((qw[:, :, None] >> shifts) & np.uint32(15)).astype(np.uint8)      # [kt, 2m, 8]
    nib = nib.reshape(kt, m // 64, 1024)
    table = _inverse_perm_table()                                             # [16, 64]
    S = nib[:, :, table]                                                      # [kt, m/64, 16, 64]
    S = S.transpose(0, 2, 1, 3).reshape(kt * 16, m)
    meta16 = unreorder_meta(np.ascontiguousarray(meta).view(np.uint16))      # [m, k/16]
    code = np.stack([(meta16 >> (4 * g)) & 15 for g in range(4)], axis=-1).reshape(m, -1)  # [m, k/4]
    lo = (code & 3).astype(np.int64)
    hi = (code >> 2).astype(np.int64)
    return S, lo, hi


def unpack_int(qweight: np.ndarray, meta: np.ndarray) -> np.ndarray:
    """Packed tensors -> dense signed integer weight [k, m] (zeros at pruned positions)."""
    S, lo, hi = unpack_codes(qweight, meta)
    k2, m = S.shape
    k = 2 * k2
    q = S.astype(np.int32) - 8                                               # [k/2, m]
    dense = np.zeros((m, k // 4, 4), dtype=np.int32)
    qt = q.T.reshape(m, k // 4, 2)
    # the second store wins when lo == hi, as a scatter in k order would
    np.put_along_axis(dense, lo[..., None], qt[..., 0:1], axis=-1)
    np.put_along_axis(dense, hi[..., None], qt[..., 1:2], axis=-1)
    return np.ascontiguousarray(dense.reshape(m, k).T)


def unpack(qweight: np.ndarray, meta: np.ndarray, scales: np.ndarray) -> np.ndarray:
    """Packed tensors -> dense fp16 weight W [k, m] with the op computing x @ W.

    W = fp16(q) * fp16(s) rounded to fp16, as generator.py:40 builds its
    reference weight.
    """
    q = unpack_int(qweight, meta)
    s = np.asarray(scales, dtype=np.float16)
    if s.ndim == 2 and s.shape[0] > 1:
        # grouped: the stored scale of (group of 128 dense k, column) multiplies the dequantised weight in fp16, as
        # the reference's kernel does ahead of its MMA (marlin.cuh:378-380)
        assert s.shape[0] * GROUP_K == q.shape[0]
        return (q.astype(np.float16) * np.repeat(load_group_scales(s), GROUP_K, axis=0)).astype(np.float16)
    return (q.astype(np.float16) * s.reshape(1, -1)).astype(np.float16)


# --------------------------------------------------------------------------
# ops (float64 accumulate; outputs left in float64 so callers choose the
# comparison -- the GPU path rounds once to fp16)
# --------------------------------------------------------------------------

def matmul_4bit_2_4(qweight, x, meta, scales) -> np.ndarray:
    W = unpack(qweight, meta, scales).astype(np.float64)
    return x.astype(np.float64) @ W


def bmm_4bit_2_4(qweights, xs, metas, ss) -> np.ndarray:
    return np.stack([matmul_4bit_2_4(qweights[b], xs[b], metas[b], ss[b]) for b in range(xs.shape[0])])


def sbmm_dense(weights, xs, indices, base_weight=None) -> np.ndarray:
    """Per-token routed matmul on dense weights [N, k, m]; -1 -> base only / zeros."""
    T = xs.shape[0]
    m = weights.shape[2]
    x64 = xs.astype(np.float64)
    y = np.zeros((T, m), dtype=np.float64)
    if base_weight is not None:
        # the base GEMM result is rounded to fp16 before the delta is added (sbmm.py:91,141)
        y = (x64 @ base_weight.astype(np.float64).T).astype(np.float16).astype(np.float64)
    for t in range(T):
        d = int(indices[t])
        if d >= 0:
            y[t] += x64[t] @ weights[d].astype(np.float64)
    return y


def sbmm_4bit_2_4(qweights, xs, metas, ss, indices, base_weight=None) -> np.ndarray:
    used = sorted({int(i) for i in indices if i >= 0})
    m = ss.shape[-1]
    dense = {d: unpack(qweights[d], metas[d], ss[d]) for d in used}
    T = xs.shape[0]
    x64 = xs.astype(np.float64)
    y = np.zeros((T, m), dtype=np.float64)
    if base_weight is not None:
        y = (x64 @ base_weight.astype(np.float64).T).astype(np.float16).astype(np.float64)
    for d in used:
        rows = np.nonzero(np.asarray(indices) == d)[0]
        y[rows] += x64[rows] @ dense[d].astype(np.float64)
    return y


def round_bf16(a) -> np.ndarray:
    """Round to the nearest bfloat16 (ties to even), returned as float64: the upper 16 bits of the fp32 pattern."""
    bits = np.asarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    bits = (bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000
    return bits.astype(np.uint32).view(np.float32).astype(np.float64)


def lora(weights_A, weights_B, x, indices, base_weight=None, scale=1.0, intermediate="f16") -> np.ndarray:
    """y[t] = base(x[t]) + scale * fp16(x[t] @ A_i) @ B_i for i = indices[t] >= 0 (lora.py:4-20).

    The rank-r intermediate is rounded to the tensors' type as every reference variant does
    (torch matmul in that type, punica.py:27,64 temporaries of x's dtype): fp16, or bf16 for the
    reference's bfloat16 instantiation (bgmv_all.cu:5, sgmv.cu:10; inputs then come as float32
    arrays holding bf16 values).
    """
    rnd = round_bf16 if intermediate == "bf16" else (lambda a: np.asarray(a).astype(np.float16).astype(np.float64))
    T = x.shape[0]
    m = weights_B.shape[2]
    x64 = x.astype(np.float64)
    y = np.zeros((T, m), dtype=np.float64)
    if base_weight is not None:
        y = rnd(x64 @ base_weight.astype(np.float64).T)
    for t in range(T):
        i = int(indices[t])
        if i >= 0:
            v = rnd(x64[t] @ weights_A[i].astype(np.float64))
            y[t] += scale * (v @ weights_B[i].astype(np.float64))
    return y


def ldmm(indices, x, LwA, LwB, DeltaW, metas, ss, base_weight=None) -> np.ndarray:
    """Mixed routing: 0 <= i < M -> LoRA i, i >= M -> delta i - M, -1 -> base only (ldmm.py:8-48)."""
    indices = np.asarray(indices)
    M = LwA.shape[0]
    T = x.shape[0]
    m = LwB.shape[2]
    x16 = x.astype(np.float16)
    x64 = x16.astype(np.float64)
    y = np.zeros((T, m), dtype=np.float64)
    if base_weight is not None:
        y = (x64 @ base_weight.astype(np.float64).T).astype(np.float16).astype(np.float64)
    lora_idx = np.where((indices >= 0) & (indices < M), indices, -1)
    y += lora(LwA, LwB, x16, lora_idx)
    delta_idx = np.where(indices >= M, indices - M, -1)
    if np.any(delta_idx >= 0):
        y += sbmm_4bit_2_4(DeltaW, x16, metas, ss, delta_idx)
    return y


# --------------------------------------------------------------------------
# error metrics used by the parity tests
# --------------------------------------------------------------------------

def rel_frobenius(got, ref) -> float:
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    den = np.linalg.norm(ref)
    return float(np.linalg.norm(got - ref) / den) if den > 0 else float(np.linalg.norm(got - ref))


def rel_mean_abs(got, ref) -> float:
    """The reference tests' own metric: mean|d| / mean|ref| (tests/ops/test_matmul.py:18-22)."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    den = np.mean(np.abs(ref))
    return float(np.mean(np.abs(got - ref)) / den) if den > 0 else float(np.mean(np.abs(got - ref)))
