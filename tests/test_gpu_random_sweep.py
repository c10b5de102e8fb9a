"""Seeded random sweep over shapes, batch sizes and routings with the library's own dispatch rules
(no knobs set): every entry point against an fp32 product with the weights dequantised by the
torch codec (`unpack_2_4`, which the CPU tests hold bit-exact against the oracle's `unpack`).
The cases are small enough for a few hundred of them to run in seconds; which kernel a case
lands on (routing inside the multiply kernel, a plan, wide tiles, split tokens) follows from
its shape."""
import numpy as np
import pytest
import torch

from triteia_amd import workloads as W
from triteia_amd.python import ops
from triteia_amd.python.capi import routed_workspace, sbmm_2_4_routed
from triteia_amd.python.ops.utils.sparsity import unpack_2_4

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOKENS = [1, 2, 7, 16, 17, 31, 33, 64, 65, 100, 128, 129, 200, 256, 257, 300, 511, 700, 1100]


def _rel(a, b):
    return float((a.float() - b.float()).norm() / max(float(b.float().norm()), 1e-9))


def _routing(rng, T, N, case):
    mode = int(rng.integers(0, 4))
    if mode == 0:
        return rng.integers(-1, N, size=T).astype(np.int32)
    if mode == 1:
        return W.zipf_indices(T, N, 1.5, 300 + case, 0.1)
    if mode == 2:
        return np.full(T, int(rng.integers(0, N)), dtype=np.int32)
    idx = np.full(T, -1, dtype=np.int32)
    idx[: T // 2] = rng.integers(0, N, size=T // 2)
    return idx


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_sparse_entry_points_on_random_cases(seed):
    rng = np.random.default_rng(seed)
    for case in range(120):
        kind = ["routed", "routed", "routed", "matmul", "bmm", "runs"][int(rng.integers(0, 6))]
        k = int(rng.choice([64, 128, 192, 256, 512, 1024, 2048, 4096]))
        m = int(rng.choice([128, 256, 384, 512, 1024, 1536, 2048, 4096, 8192]))
        N = int(rng.integers(1, 9 if k * m >= 2048 * 2048 else 70))
        T = int(rng.choice(TOKENS))
        what = f"seed {seed} case {case}: {kind} T={T} N={N} k={k} m={m}"
        print(f"[case] {what}", flush=True)
        q, me, s = W.random_packed_deltas(N, k, m, 1000 * seed + case, DEV)
        dense = torch.stack([unpack_2_4(q[i], me[i], s[i]).float() for i in range(N)])
        if kind == "matmul":
            x = W.random_activations(T, k, 7 + case, DEV)
            assert _rel(ops.matmul_4bit_2_4(q[0], x, me[0], s[0]), x.float() @ dense[0]) < 2e-3, what
            continue
        if kind == "bmm":
            t = int(rng.choice([1, 1, 3, 16, 40, 64, 130]))
            x = W.random_activations(N * t, k, 7 + case, DEV).view(N, t, k)
            assert _rel(ops.bmm_4bit_2_4(q, x, me, s), torch.bmm(x.float(), dense)) < 2e-3, what
            continue
        x = W.random_activations(T, k, 7 + case, DEV)
        idx = _routing(rng, T, N, case)
        if kind == "runs":
            idx = np.sort(idx)
        gi = torch.from_numpy(idx).to(DEV)
        none = gi < 0
        ref = torch.zeros((T, m), dtype=torch.float32, device=DEV)
        for d in np.unique(idx[idx >= 0]):
            rows = torch.from_numpy(np.nonzero(idx == d)[0]).to(DEV)
            ref[rows] = x[rows].float() @ dense[int(d)]
        if kind == "runs":
            got = ops.sbmm_4bit_2_4_runs(q, x, me, s, gi)
            assert bool((got[none] == 0).all()), what
            if (~none).any():
                assert _rel(got, ref) < 2e-3, what
            continue
        acc = bool(rng.integers(0, 2))
        got = torch.full((T, m), -3.0, dtype=torch.float16, device=DEV)
        sbmm_2_4_routed(x, q, me, got, s, gi, accumulate=acc, workspace=routed_workspace(T, N, DEV))
        assert bool((got[none] == -3.0).all()), what + ": a row without a delta was written"
        if (~none).any():
            # (added onto -3 the sum is rounded to fp16 near 3, which is coarser than near the product alone)
            assert _rel(got[~none].float() + (3.0 if acc else 0.0), ref[~none]) < (4e-3 if acc else 2e-3), what


@pytest.mark.parametrize("seed", [21, 22])
def test_lora_and_ldmm_on_random_cases(seed):
    rng = np.random.default_rng(seed)
    for case in range(100):
        kind = ["bgmv", "sgmv", "sgmv_routed", "ldmm", "ldmm"][int(rng.integers(0, 5))]
        k = int(rng.choice([256, 512, 1024, 2048, 4096]))
        m = int(rng.choice([256, 512, 1024, 1536, 2048, 4096, 11008]))
        r = int(rng.choice([8, 16, 32, 64]))
        M = int(rng.integers(1, 40))
        T = int(rng.choice(TOKENS[:-1]))
        what = f"seed {seed} case {case}: {kind} T={T} M={M} k={k} m={m} r={r}"
        print(f"[case] {what}", flush=True)
        g = torch.Generator(device=DEV).manual_seed(1000 * seed + case)
        A = (torch.randn((M, k, r), generator=g, device=DEV) * 0.05).half()
        B = (torch.randn((M, r, m), generator=g, device=DEV) * 0.05).half()
        x = W.random_activations(T, k, 7 + case, DEV)

        def lora_ref(idx_np):
            ref = torch.zeros((T, m), dtype=torch.float32, device=DEV)
            for d in np.unique(idx_np[(idx_np >= 0) & (idx_np < M)]):
                rows = torch.from_numpy(np.nonzero(idx_np == d)[0]).to(DEV)
                ref[rows] = (x[rows].float() @ A[int(d)].float()).half().float() @ B[int(d)].float()
            return ref

        if kind != "ldmm":
            idx = rng.integers(-1, M, size=T).astype(np.int64)
            if kind == "sgmv":
                idx = np.sort(idx)      # the segment form wants grouped, ascending indices
            gi = torch.from_numpy(idx).to(DEV)
            fn = {"bgmv": ops.lora_bgmv, "sgmv": ops.lora_sgmv, "sgmv_routed": ops.lora_sgmv_routed}[kind]
            got = fn(A, B, x, gi)
            assert torch.allclose(got.float(), lora_ref(idx), rtol=5e-3, atol=5e-3), what
            assert bool((got[gi < 0] == 0).all()), what
            continue
        N = int(rng.integers(1, 9 if k * m >= 2048 * 2048 else 40))
        q, me, s = W.random_packed_deltas(N, k, m, 1000 * seed + case, DEV)
        idx = rng.integers(-1, M + N, size=T).astype(np.int32)
        gi = torch.from_numpy(idx).to(DEV)
        base = (torch.randn((m, k), generator=g, device=DEV) * 0.02).half() if rng.integers(0, 2) else None
        got = ops.ldmm(gi, x, A, B, q, me, s, base_weight=base)
        ref = lora_ref(idx)
        for d in np.unique(idx[idx >= M]):
            rows = torch.from_numpy(np.nonzero(idx == d)[0]).to(DEV)
            ref[rows] = x[rows].float() @ unpack_2_4(q[int(d) - M], me[int(d) - M], s[int(d) - M]).float()
        if base is not None:
            ref = ref + (x @ base.t()).float()
        else:
            assert bool((got[gi < 0] == 0).all()), what
        if float(ref.norm()) > 0:
            assert _rel(got, ref) < 2e-3, what
