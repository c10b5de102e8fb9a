"""Seeded synthetic workloads for the benchmark configurations of this path.

Packed weights are drawn directly in packed form: packing is a bijection between
(kept values, kept positions) and (nibbles, metadata codes), so uniform random nibbles
and uniformly chosen legal 2:4 codes are exactly "values uniform in [-8, 7], positions
uniform among the six 2-of-4 patterns" -- without materialising a dense matrix, which
matters at 5.6 GB of packed deltas.
"""
from dataclasses import dataclass

import numpy as np
import torch

_LEGAL_CODES = (0x4, 0x8, 0x9, 0xC, 0xD, 0xE)   # lo | hi << 2 for (0,1) (0,2) (1,2) (0,3) (1,3) (2,3)


def random_packed_deltas(n, k, m, seed, device):
    """n packed deltas [k x m]: (qweight int32 [n, k/32, 2m], meta int16 [n, m, k/16], scales fp16 [n, 1, m])."""
    g = torch.Generator(device=device).manual_seed(seed)
    qweight = torch.randint(-2 ** 31, 2 ** 31, (n, k // 32, 2 * m), generator=g, device=device, dtype=torch.int64).to(torch.int32)
    table = torch.tensor(_LEGAL_CODES, device=device, dtype=torch.int32)
    meta = torch.empty((n, m, k // 16), dtype=torch.int16, device=device)
    for i in range(n):                               # per delta: bounds the int32 temporaries
        code = table[torch.randint(0, 6, (m, k // 16, 4), generator=g, device=device)]
        w16 = code[..., 0] | (code[..., 1] << 4) | (code[..., 2] << 8) | (code[..., 3] << 12)
        meta[i] = torch.where(w16 >= 2 ** 15, w16 - 2 ** 16, w16).to(torch.int16)
    scales = (torch.rand((n, 1, m), generator=g, device=device) * 0.015 + 0.005).to(torch.float16)
    return qweight, meta, scales


def random_activations(t, k, seed, device):
    g = torch.Generator(device=device).manual_seed(seed)
    return torch.randn((t, k), generator=g, device=device, dtype=torch.float32).to(torch.float16)


def uniform_indices(t, n, seed):
    """int32 indices uniform over {-1, 0..n-1}."""
    return np.random.default_rng(seed).integers(-1, n, size=t).astype(np.int32)


def zipf_indices(t, n, alpha, seed, frac_none=0.0):
    """Rank-frequency Zipf (p_r proportional to r**-alpha over deltas 0..n-1), then `frac_none` of the
    tokens set to -1."""
    rng = np.random.default_rng(seed)
    p = np.arange(1, n + 1, dtype=np.float64) ** -alpha
    idx = rng.choice(np.arange(n), size=t, p=p / p.sum()).astype(np.int32)
    if frac_none > 0:
        idx[rng.random(t) < frac_none] = -1
    return idx


@dataclass
class Workload:
    name: str
    op: str            # matmul | bmm | sbmm | ldmm
    k: int
    m: int
    n_deltas: int
    tokens: int
    seed: int
    indices: np.ndarray = None
    lora_rank: int = 0
    n_lora: int = 0
    with_base: bool = False
    index_offset: int = 0   # ldmm with the reference's split index space: [0, offset) = LoRA adapters, offset + d = delta d

    @property
    def delta_bytes(self):
        # int4 values of the kept half + 2 metadata bits per kept value + fp16 scales
        return self.k * self.m // 4 + self.k * self.m // 8 + 2 * self.m

    def delta_indices(self):
        """Per token: its delta, or -1 (no model, or a LoRA adapter of a split index space)."""
        if self.indices is None:
            return None
        d = self.indices - self.index_offset
        return np.where((self.indices >= self.index_offset) & (d < self.n_deltas), d, -1).astype(np.int32)

    def routed_tokens(self):
        return self.tokens if self.indices is None else int((self.delta_indices() >= 0).sum())

    def lora_tokens(self):
        """Tokens that take a LoRA adapter: all routed ones when LoRA shares the routing of the deltas."""
        if self.n_lora == 0 or self.indices is None:
            return 0
        if self.index_offset == 0:
            return self.routed_tokens()
        return int(((self.indices >= 0) & (self.indices < self.index_offset)).sum())

    def distinct_deltas(self):
        if self.indices is None:
            return self.n_deltas
        d = self.delta_indices()
        return int(len(np.unique(d[d >= 0])))

    def delta_flops(self):
        """dense-equivalent 2*T_routed*k*m, the reference's convention (meta/benchmarks/bench_sbmm.py:17)."""
        return 2.0 * self.routed_tokens() * self.k * self.m

    def delta_algorithmic_bytes(self):
        """every distinct delta once + activations + output + indices."""
        b = self.distinct_deltas() * self.delta_bytes + self.tokens * self.k * 2 + self.tokens * self.m * 2
        if self.indices is not None:
            b += self.tokens * 4
        return b


def config(name, tokens=None, shape=None):
    """The five benchmark configurations (seed = 1000 + index).  `shape` = (k, m) overrides the weight
    shape of cfg0 (the single-matrix op at other layer shapes)."""
    if name == "cfg0":
        t = 16 if tokens is None else tokens
        k, m = (4096, 4096) if shape is None else shape
        return Workload(f"cfg0 matmul_4bit_2_4 x[{t},{k}] W[{k}x{m}]", "matmul", k, m, 1, t, 1000)
    if name == "cfg1":
        return Workload("cfg1 bmm_4bit_2_4 8 deltas 4096x4096, 1 token each", "bmm", 4096, 4096, 8, 8, 1001)
    if name == "cfg2":
        t = 64 if tokens is None else tokens
        return Workload(f"cfg2 sbmm_4bit_2_4 {t} tokens x 16 deltas 4096x4096, idx uniform{{-1..15}}", "sbmm", 4096, 4096,
                        16, t, 1002, indices=uniform_indices(t, 16, 1002))
    if name == "cfg3":
        t = 256 if tokens is None else tokens
        return Workload(f"cfg3 ldmm 4096x11008, 32 deltas, {t} tokens Zipf(1.5) 10% -1, SGMV r=16 x 32", "ldmm", 4096, 11008,
                        32, t, 1003, indices=zipf_indices(t, 32, 1.5, 1003, 0.10), lora_rank=16, n_lora=32, with_base=True)
    if name == "cfg3split":
        # the same layer with the reference's ldmm index space (tests/ops/test_ldmm.py:34-64): a routed token
        # takes either LoRA adapter i (index i) or delta i (index 32 + i), by a fair coin
        t = 256 if tokens is None else tokens
        idx = zipf_indices(t, 32, 1.5, 1003, 0.10)
        coin = np.random.default_rng(2003).random(t) < 0.5
        idx = np.where((idx >= 0) & coin, idx + 32, idx).astype(np.int32)
        return Workload(f"cfg3split ldmm 4096x11008, {t} tokens Zipf(1.5) 10% -1, each to LoRA adapter i (r=16) or delta i of 32",
                        "ldmm", 4096, 11008, 32, t, 1003, indices=idx, lora_rank=16, n_lora=32, with_base=True, index_offset=32)
    if name == "cfg4":
        t = 1024 if tokens is None else tokens
        return Workload(f"cfg4 sbmm 8192x28672, 64 deltas, {t} tokens Zipf(1.2)", "sbmm", 8192, 28672, 64, t, 1004,
                        indices=zipf_indices(t, 64, 1.2, 1004))
    raise ValueError(name)
