"""GPU tests at BASELINE's full sizes (configs 3 and 4), where a CPU dequantise of every delta would
take minutes: size-independent properties plus a torch-on-GPU dequantise-then-matmul of sampled
deltas (the torch codec is itself checked bit-exactly against the oracle in test_codec_cpu.py).

  * routing: every sampled routed row equals, bit for bit, the single-matrix product of that row
    alone with its own delta; rows with index -1 are exactly zero (or exactly the base output);
  * exact scaling: out(2x) == 2 out(x) bit for bit wherever the output is a normal fp16 number
    (powers of two commute with every rounding here);
  * token-order invariance: permuting the batch permutes the output rows bit for bit;
  * sampled deltas against fp32 matmul on their dequantised weights, relative Frobenius <= 2e-3.
"""
import os
import sys

import numpy as np
import pytest
import torch

from tests.helpers import reload_knobs, setknob
from triteia_amd import workloads as W

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def ops():
    from triteia_amd.python import ops as _ops
    return _ops


def _check_properties(ops, q, me, s, x, idx_np, sample_rows, sample_deltas, what):
    from triteia_amd.python.ops.utils.sparsity import unpack_2_4
    idx = torch.from_numpy(idx_np).to(DEV)
    out = ops.sbmm_4bit_2_4_native(q, x, me, s, idx)
    torch.cuda.synchronize()
    assert bool((out[idx < 0] == 0).all()), f"{what}: -1 rows must stay zero"
    # Batches of at least 256 tokens with at least 8 tokens per delta carry 64-token wide tiles for
    # deltas with more than 32 tokens; the wide kernel sums over k in another order than the narrow
    # one, so only rows of deltas with at most 32 tokens are comparable bit for bit.
    T, N = x.shape[0], q.shape[0]
    counts = np.bincount(idx_np[idx_np >= 0], minlength=N)
    may_be_wide = counts > 32 if (T >= 256 and T >= 8 * min(T, N)) else np.zeros(N, dtype=bool)
    exact_rows = torch.from_numpy((idx_np < 0) | ~may_be_wide[np.maximum(idx_np, 0)]).to(DEV)
    # On wide layers a plan's 32-token tiles run on the 32-token build of the wide kernel, which also sums over k
    # in its own order: the row-by-row comparison with a row routed on its own (always the K-split kernel) is made
    # on the K-split kernel's result for the batch, and the default result is held against that one.
    os.environ["TRITEIA_HIP_MID"] = "0"
    reload_knobs()
    try:
        out_ksplit = ops.sbmm_4bit_2_4_native(q, x, me, s, idx)
        torch.cuda.synchronize()
    finally:
        del os.environ["TRITEIA_HIP_MID"]
        reload_knobs()
    assert float((out.float() - out_ksplit.float()).norm()) <= 1e-3 * float(out_ksplit.float().norm()), what
    assert bool((out_ksplit[idx < 0] == 0).all())
    batch = out
    out = out_ksplit
    for t in sample_rows:
        d = int(idx_np[t])
        if d >= 0:
            # the same row routed on its own (same delta index, hence the same walk over k): same bits
            alone = ops.sbmm_4bit_2_4_native(q, x[t:t + 1].contiguous(), me, s, idx[t:t + 1].contiguous())
            if not may_be_wide[d]:
                assert torch.equal(alone[0], out[t]), f"{what}: row {t} differs from the same row routed on its own"
            single = ops.matmul_4bit_2_4(q[d], x[t:t + 1], me[d], s[d])
            err = (single[0].float() - out[t].float()).norm() / single[0].float().norm()
            assert float(err) < 1e-3, f"{what}: row {t} is {float(err):.2e} from the single-matrix op"
    out = batch
    out2 = ops.sbmm_4bit_2_4_native(q, x * 2, me, s, idx)
    normal = out.abs() >= 2.0 ** -13             # fp16 subnormals round differently after doubling
    assert torch.equal(out2[normal], (out * 2)[normal]), f"{what}: out(2x) != 2 out(x)"
    assert float((out2.float() - 2 * out.float()).abs().max()) <= 2.0 ** -23
    perm = torch.randperm(x.shape[0], generator=torch.Generator().manual_seed(1)).to(DEV)
    outp = ops.sbmm_4bit_2_4_native(q, x[perm].contiguous(), me, s, idx[perm].contiguous())
    assert torch.equal(outp[exact_rows[perm]], out[perm][exact_rows[perm]]), f"{what}: token order changes the result"
    assert float((outp.float() - out[perm].float()).norm()) <= 1e-3 * float(out.float().norm())
    for d in sample_deltas:
        rows = torch.nonzero(idx == d).flatten()
        if rows.numel() == 0:
            continue
        Wd = unpack_2_4(q[d], me[d], s[d]).float()
        ref = x[rows].float() @ Wd
        err = (out[rows].float() - ref).norm() / ref.norm()
        assert float(err) <= 2e-3, f"{what}: delta {d} relative Frobenius error {float(err):.3e}"
        del Wd
    return out, out_ksplit


def test_config3_ldmm_shape(ops):
    wl = W.config("cfg3")
    say(wl.name)
    q, me, s = W.random_packed_deltas(wl.n_deltas, wl.k, wl.m, wl.seed, DEV)
    x = W.random_activations(wl.tokens, wl.k, wl.seed + 1, DEV)
    used = np.unique(wl.indices[wl.indices >= 0])
    out, out_ksplit = _check_properties(ops, q, me, s, x, wl.indices, range(0, wl.tokens, 37), [int(used[0]), int(used[-1])], "cfg3 delta")
    # the whole ldmm: base GEMM + LoRA (rank 16, 32 adapters, same routing) + delta
    g = torch.Generator(device=DEV).manual_seed(7)
    base = (torch.randn((wl.m, wl.k), generator=g, device=DEV) * 0.02).half()
    A = (torch.randn((wl.n_lora, wl.k, wl.lora_rank), generator=g, device=DEV) * 0.01).half()
    B = (torch.randn((wl.n_lora, wl.lora_rank, wl.m), generator=g, device=DEV) * 0.01).half()
    idx = torch.from_numpy(wl.indices).to(DEV)
    y_delta = ops.sbmm_4bit_2_4_native(q, x, me, s, idx, base_weight=base)
    y0 = torch.matmul(x, base.t())
    assert torch.equal(y_delta[idx < 0], y0[idx < 0])
    err = ((y_delta.float() - y0.float()) - out.float()).norm() / out.float().norm()
    assert float(err) < 5e-3                       # accumulate-in-place = base + delta up to fp16 rounding of the sum
    lora = ops.lora_sgmv_routed(A, B, x, idx)
    ref_rows = torch.nonzero(idx >= 0).flatten()[:8]
    for t in ref_rows.tolist():
        a = int(idx[t])
        v = (x[t].float() @ A[a].float()).half().float()
        ref = v @ B[a].float()
        assert torch.allclose(lora[t].float(), ref, rtol=5e-3, atol=5e-3 * float(ref.abs().max()))
    assert bool((lora[idx < 0] == 0).all())
    # mixed index space of ldmm: adapters 0..31, deltas 32..63
    mixed = torch.where(idx >= 0, idx + (torch.arange(wl.tokens, device=DEV) % 2).int() * wl.n_lora, idx)
    y = ops.ldmm(mixed, x, A, B, q, me, s)
    is_delta = mixed >= wl.n_lora
    # (the delta half of the batch is routed as a batch of its own size: its rows have the bits of the K-split
    # kernel or of the 32-token wide kernel, whichever that batch size takes)
    assert torch.equal(y[is_delta], out_ksplit[is_delta]) or torch.equal(y[is_delta], out[is_delta])
    is_lora = (mixed >= 0) & ~is_delta
    assert torch.allclose(y[is_lora].float(), lora[is_lora].float(), rtol=5e-3, atol=1e-3)
    assert bool((y[mixed < 0] == 0).all())


@pytest.mark.parametrize("tokens", [1, 16, 64, 256, 1024])
def test_config4_70b_shape(ops, tokens):
    wl = W.config("cfg4", tokens)
    say(wl.name)
    q, me, s = _cfg4_weights(wl)
    x = W.random_activations(wl.tokens, wl.k, wl.seed + 1, DEV)
    used = np.unique(wl.indices[wl.indices >= 0])
    step = max(1, tokens // 5)
    _check_properties(ops, q, me, s, x, wl.indices, range(0, tokens, step), [int(used[0])], f"cfg4 T={tokens}")


@pytest.mark.parametrize("k,m,n,tokens,order", [
    (4096, 14336, 8, 1024, 3),     # Llama-3-8B's MLP: 28 column groups, the padding's idle slots at work
    (8192, 8192, 16, 2048, 1),     # 16 column groups: the padded order as it is
    (5120, 13824, 4, 512, 3),      # Llama-2-13B's MLP: 27 column groups
])
def test_wide_layers_on_the_plans_64_token_tiles(ops, k, m, n, tokens, order):
    """Mid-size batches of many tokens per delta on wide layers: the plan is cut in 32-token tiles and also lists
    64-token tiles, which these layers take on the 64-token build of the wide kernel, in the order of units that
    suits their number of column groups."""
    from triteia_amd.python.capi import _ffi
    lib = _ffi.lib()
    say(f"64-token list of a 32-token plan k={k} m={m} deltas={n} tokens={tokens}")
    assert lib.triteia_hip_plan_tile_tokens(tokens, n) == 32
    assert lib.triteia_hip_planned_tile_kernel(tokens, n, m, k) == 64
    assert lib.triteia_hip_wide_unit_order(m) == order
    q, me, s = W.random_packed_deltas(n, k, m, 4100 + n, DEV)
    x = W.random_activations(tokens, k, 4200 + n, DEV)
    idx = W.uniform_indices(tokens, n, 4300 + n)
    _check_properties(ops, q, me, s, x, idx, range(0, tokens, tokens // 5), [0, n - 1], f"{k}x{m} T={tokens}")


_CFG4 = {}


def _cfg4_weights(wl):
    # 64 deltas of 8192 x 28672 = 5.64 GB packed: built once for the five token counts
    if "w" not in _CFG4:
        _CFG4["w"] = W.random_packed_deltas(wl.n_deltas, wl.k, wl.m, wl.seed, DEV)
    return _CFG4["w"]


def test_bmm_many_tokens_per_matrix(ops):
    say("bmm 3 x 150 tokens, 4096 x 4096 (wide tiles + narrow rest)")
    from triteia_amd.python.ops.utils.sparsity import unpack_2_4
    b, t, k, m = 3, 150, 4096, 4096
    q, me, s = W.random_packed_deltas(b, k, m, 77, DEV)
    x = W.random_activations(b * t, k, 78, DEV).reshape(b, t, k)
    out = ops.bmm_4bit_2_4(q, x, me, s)
    for i in range(b):
        ref = x[i].float() @ unpack_2_4(q[i], me[i], s[i]).float()
        err = (out[i].float() - ref).norm() / ref.norm()
        assert float(err) <= 2e-3


@pytest.mark.parametrize("b,t,k,m", [
    (1, 1024, 4096, 4096),    # 256 units of 32 tokens: 32-token tiles, K split over eight wavefronts
    (1, 1500, 4096, 4096),    # 192 units of 64 tokens, last tile of 28: 64-token tiles, K split over eight wavefronts
    (2, 200, 4096, 11008),    # two matrices, 4 tiles each with a last one of 8 tokens, 22 column groups padded to 24
    (1, 576, 8192, 8192),     # 144 units of 64 tokens, 64 steps per half
])
def test_uniform_launches_of_one_workgroup_per_cu(ops, monkeypatch, b, t, k, m):
    """The launcher's own choice for launches that do not fill the chip (workgroups of eight wavefronts, each half
    on half of the K steps) against a dequantise-then-matmul in fp32 and against the narrow kernel."""
    say(f"bmm {b} x {t} tokens, {k} x {m}: default launch rule")
    from triteia_amd.python.ops.utils.sparsity import unpack_2_4
    q, me, s = W.random_packed_deltas(b, k, m, 91, DEV)
    x = W.random_activations(b * t, k, 92, DEV).reshape(b, t, k)
    out = ops.bmm_4bit_2_4(q, x, me, s)
    torch.cuda.synchronize()
    for i in range(b):
        ref = x[i].float() @ unpack_2_4(q[i], me[i], s[i]).float()
        assert float((out[i].float() - ref).norm() / ref.norm()) <= 2e-3
    setknob(monkeypatch, "TRITEIA_HIP_WIDE", "0")
    narrow = ops.bmm_4bit_2_4(q, x, me, s)
    torch.cuda.synchronize()
    assert float((out.float() - narrow.float()).norm() / narrow.float().norm()) < 1e-4


def test_activations_above_4_gib(ops):
    """The wide kernels address activations with 32-bit byte offsets; a batch whose activations reach
    4 GiB must be kept away from them (and from every other 32-bit shortcut) by the launcher."""
    from triteia_amd.python.capi import routed_workspace, sbmm_2_4_routed
    from triteia_amd.python.ops.utils.sparsity import unpack_2_4
    T, k, m, N = 2 ** 18 + 64, 8192, 128, 2
    say(f"activations of {T * k * 2 / 2 ** 30:.3f} GiB: matmul, then routed over {N} deltas")
    q, me, s = W.random_packed_deltas(N, k, m, 91, DEV)
    x = torch.randn((T, k), generator=torch.Generator(device=DEV).manual_seed(92), device=DEV, dtype=torch.float16)
    dense = [unpack_2_4(q[i], me[i], s[i]).float() for i in range(N)]
    out = ops.matmul_4bit_2_4(q[0], x, me[0], s[0])
    idx = np.random.default_rng(93).integers(-1, N, size=T).astype(np.int32)
    gi = torch.from_numpy(idx).to(DEV)
    got = torch.full((T, m), -3.0, dtype=torch.float16, device=DEV)
    sbmm_2_4_routed(x, q, me, got, s, gi, accumulate=False, workspace=routed_workspace(T, N, DEV))
    assert bool((got[gi < 0] == -3.0).all())
    for a in range(0, T, 32768):          # fp32 references in chunks of the batch
        xx = x[a:a + 32768].float()
        r0, r1 = xx @ dense[0], xx @ dense[1]
        assert float((out[a:a + 32768].float() - r0).norm() / r0.norm()) <= 2e-3, f"matmul rows {a}.."
        g = gi[a:a + 32768]
        ref, sel = torch.where((g == 0)[:, None], r0, r1), g >= 0
        assert float((got[a:a + 32768][sel].float() - ref[sel]).norm() / ref[sel].norm()) <= 2e-3, f"routed rows {a}.."


def test_reference_import_path_alias():
    import triteia.python.ops as ref_ops
    from triteia.python.capi import mul_2_4  # noqa: F401
    from triteia.python.nn.linear import sparse_low_precision_linear  # noqa: F401
    assert hasattr(ref_ops, "sbmm_4bit_2_4_native") and hasattr(ref_ops, "ldmm")
