"""GPU parity tests: the HIP path (through the Python mirror -> ctypes -> C ABI) against the
CPU oracle on the same seeded inputs.

Bounds: relative Frobenius error <= 2e-3 and the reference tests' own metric
mean|d|/mean|ref| < 2e-3 (tests/ops/test_matmul.py:18-22, test_sbmm.py:47-61); LoRA / ldmm
additionally allclose(rtol=atol=5e-3) scaled to the output magnitude (tests/ops/test_ldmm.py:73).
Routing and -1 handling are checked bit-exactly.
"""
import sys

import numpy as np
import pytest
import torch

from oracle import triteia_oracle as orc
from tests.helpers import activations, check_close, delknob, make_deltas, reload_knobs, setknob, to_gpu

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


WIDE_MIN_BATCH = 256          # batch size from which a plan carries wide tiles (the library's default)


@pytest.fixture(params=["shipping rules", "wide tiles forced"])
def plan_rules(request, monkeypatch):
    """The tests that route through a plan run twice: under the rules as shipped, and with the plan's 64-token wide
    tiles forced onto these small shapes (carried from 512 tokens on, and taken by the wide kernel however few they
    are; by default only when they fill the chip)."""
    global WIDE_MIN_BATCH
    if request.param == "wide tiles forced":
        WIDE_MIN_BATCH = 512
        setknob(monkeypatch, "TRITEIA_HIP_WIDE_MIN_BATCH", str(WIDE_MIN_BATCH))
        setknob(monkeypatch, "TRITEIA_HIP_PLAN_WIDE_MIN_UNITS", "1")
    else:
        WIDE_MIN_BATCH = 256
    yield request.param
    WIDE_MIN_BATCH = 256


def say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def ops():
    from triteia_amd.python import ops as _ops
    return _ops


# ------------------------------------------------------------------ matmul

@pytest.mark.parametrize("n,k,m,seed", [
    (1, 128, 256, 1), (3, 512, 256, 2), (16, 512, 256, 3), (17, 512, 256, 4), (64, 512, 384, 5),
    (100, 1024, 256, 6), (5, 192, 128, 7),            # k = 64 (mod 128): the partial last k step
    (2, 64, 128, 13), (70, 64, 128, 14),              # the smallest layer: one partial k step, one column block
    (64, 256, 128, 8), (97, 320, 640, 9), (130, 192, 384, 10), (200, 512, 1408, 12),   # wide tiles, ragged ends
    (16, 4096, 4096, 1000),                           # BASELINE config 0
])
def test_matmul_4bit_2_4(ops, n, k, m, seed):
    say(f"matmul n={n} k={k} m={m} seed={seed}")
    qw, meta, s = make_deltas(1, k, m, seed)
    x = activations(n, k, seed + 1)
    ref = orc.matmul_4bit_2_4(qw[0], x, meta[0], s[0])
    gq, gm, gs, gx = to_gpu(qw[0], meta[0], s[0], x)
    out = ops.matmul_4bit_2_4(gq, gx, gm, gs)
    torch.cuda.synchronize()
    assert out.shape == (n, m) and out.dtype == torch.float16
    check_close(out, ref, what="matmul_4bit_2_4")


@pytest.mark.parametrize("n,k,m,seed", [
    (1, 256, 256, 31), (16, 256, 128, 32), (17, 512, 256, 33), (33, 512, 384, 34), (100, 1024, 640, 35),
    (300, 384, 256, 36),
    (16, 4096, 4096, 37),                             # BASELINE config 0's shape with a scale per 128 k and column
])
def test_matmul_with_scales_per_group_of_k(ops, n, k, m, seed):
    """groupsize 64 of the reference's launcher (marlin_nm.cu:68,102-111): `s` is [k/128, m] in the stored order.
    Against the oracle, which scales the dequantised weight in fp16 as the reference's kernel does; and, with all
    groups alike, against the per-column product of the same weights."""
    say(f"matmul grouped scales n={n} k={k} m={m} seed={seed}")
    rng = np.random.default_rng(seed)
    qw, meta, _ = make_deltas(1, k, m, seed)
    s_true = rng.uniform(0.005, 0.02, size=(k // 128, m)).astype(np.float16)
    stored = orc.store_group_scales(s_true)
    x = activations(n, k, seed + 1)
    ref = orc.matmul_4bit_2_4(qw[0], x, meta[0], stored)
    gq, gm, gs, gx = to_gpu(qw[0], meta[0], stored, x)
    out = ops.matmul_4bit_2_4(gq, gx, gm, gs)
    torch.cuda.synchronize()
    assert out.shape == (n, m) and out.dtype == torch.float16
    check_close(out, ref, what="matmul_4bit_2_4 (grouped scales)")
    # every group with the scales of group 0: the per-column product
    flat = orc.store_group_scales(np.repeat(s_true[:1], k // 128, axis=0))
    one = ops.matmul_4bit_2_4(gq, gx, gm, torch.from_numpy(flat).to(DEV))
    per_column = ops.matmul_4bit_2_4(gq, gx, gm, torch.from_numpy(s_true[:1]).to(DEV))
    torch.cuda.synchronize()
    check_close(one, per_column.float().cpu().numpy().astype(np.float64), tol=1e-3, what="grouped == per-column")


def test_scale_groups_other_than_128_k_are_refused(ops):
    qw, meta, _ = make_deltas(1, 256, 128, 40)
    gq, gm, gx = to_gpu(qw[0], meta[0], activations(4, 256, 41))
    with pytest.raises(RuntimeError, match="groupsize=32"):
        ops.matmul_4bit_2_4(gq, gx, gm, torch.ones((4, 128), dtype=torch.float16, device=DEV))


@pytest.mark.parametrize("kernel", ["wide64", "wide64ks", "tile256", "wide32", "wide32ks"])
@pytest.mark.parametrize("n,k,m,seed", [
    (64, 128, 512, 21), (128, 128, 512, 22), (128, 256, 128, 23),      # one tile, 1 and 2 k steps
    (200, 384, 384, 24), (321, 512, 640, 25), (130, 640, 256, 26),     # ragged tokens, partial column groups
    (256, 1024, 1024, 27), (448, 896, 1152, 28),                       # 7 k steps: every ring phase
    (192, 192, 256, 29),                                               # k = 64 (mod 128): falls back to the narrow kernel
])
def test_matmul_wide_kernels(ops, monkeypatch, kernel, n, k, m, seed):
    """The matrix-core-bound kernels (64- and 128-token tiles) and the 32-token build with two steps of
    weights in flight, forced onto small ragged shapes that the launcher would give to the narrow kernel."""
    say(f"matmul {kernel} n={n} k={k} m={m} seed={seed}")
    setknob(monkeypatch, "TRITEIA_HIP_WIDE_MIN_UNITS", "1")
    setknob(monkeypatch, "TRITEIA_HIP_TILE256_MIN_UNITS", "1")
    setknob(monkeypatch, "TRITEIA_HIP_TILE256", "2" if kernel == "tile256" else "0")   # (2: on layers of any width)
    if kernel in ("wide32", "wide32ks"):   # takes the tokens ahead of the other two whenever its window of units is open
        setknob(monkeypatch, "TRITEIA_HIP_WIDE32_MIN_UNITS", "1")
        setknob(monkeypatch, "TRITEIA_HIP_WIDE32_MAX_UNITS", "1000000000")
    # wide32ks: eight wavefronts per workgroup, each half of them on half of the k steps
    setknob(monkeypatch, "TRITEIA_HIP_WIDE32_KSPLIT_MAX_UNITS", "1000000000" if kernel == "wide32ks" else "0")
    setknob(monkeypatch, "TRITEIA_HIP_WIDE64_KSPLIT_MAX_UNITS", "1000000000" if kernel == "wide64ks" else "0")
    qw, meta, s = make_deltas(1, k, m, seed)
    x = activations(n, k, seed + 1)
    ref = orc.matmul_4bit_2_4(qw[0], x, meta[0], s[0])
    gq, gm, gs, gx = to_gpu(qw[0], meta[0], s[0], x)
    out = ops.matmul_4bit_2_4(gq, gx, gm, gs)
    torch.cuda.synchronize()
    check_close(out, ref, what=f"matmul_4bit_2_4 {kernel}")
    # on these small layers most slots of a padded tile would be idle and the launch puts them to work; the padded order
    # and the order without padding give the same workgroups the same work on other XCDs
    setknob(monkeypatch, "TRITEIA_HIP_WIDE_ORDER_MIN_IDLE", "100")
    padded = ops.matmul_4bit_2_4(gq, gx, gm, gs)
    torch.cuda.synchronize()
    assert torch.equal(padded, out), "the order of the units changed bits"
    # ... and from the padded order on, a block of column groups x a block of token tiles per XCD, in every block size
    # that cuts this layer's padded column groups over the 8 XCDs (sizes that do not are ignored)
    for block in (1, 2, 4, 8, 16):
        setknob(monkeypatch, "TRITEIA_HIP_XCD_CGS", str(block))
        blocks = ops.matmul_4bit_2_4(gq, gx, gm, gs)
        torch.cuda.synchronize()
        assert torch.equal(blocks, out), f"blocks of {block} column groups per XCD changed bits"
    delknob(monkeypatch, "TRITEIA_HIP_XCD_CGS")
    delknob(monkeypatch, "TRITEIA_HIP_WIDE_ORDER_MIN_IDLE")
    setknob(monkeypatch, "TRITEIA_HIP_XCD_SWIZZLE", "2")
    unpadded = ops.matmul_4bit_2_4(gq, gx, gm, gs)
    torch.cuda.synchronize()
    assert torch.equal(unpadded, out), "the order of the units changed bits"
    delknob(monkeypatch, "TRITEIA_HIP_XCD_SWIZZLE")
    # same inputs through the narrow kernel: equal up to the order of fp32 accumulation
    setknob(monkeypatch, "TRITEIA_HIP_WIDE", "0")
    narrow = ops.matmul_4bit_2_4(gq, gx, gm, gs)
    torch.cuda.synchronize()
    rel = ((out.float() - narrow.float()).norm() / narrow.float().norm()).item()
    assert rel < 1e-4, rel


@pytest.mark.parametrize("tile256", ["0", "2"])
def test_matmul_many_tokens_reference_test_shape(ops, monkeypatch, tile256):
    # the reference's own test shape m = n = k = 4096 (tests/ops/test_matmul.py:30): on the 64-token kernel, which the
    # rules give it, and on the 256-token tile kernel, whose window of units it fills
    setknob(monkeypatch, "TRITEIA_HIP_TILE256", tile256)
    n = k = m = 4096
    say(f"matmul n={n} k={k} m={m}")
    qw, meta, s = make_deltas(1, k, m, 77)
    x = activations(n, k, 78)
    W = orc.unpack(qw[0], meta[0], s[0]).astype(np.float32)
    ref = x.astype(np.float32) @ W
    gq, gm, gs, gx = to_gpu(qw[0], meta[0], s[0], x)
    out = ops.matmul_4bit_2_4(gq, gx, gm, gs)
    torch.cuda.synchronize()
    check_close(out, ref, what="matmul 4096^3")


@pytest.mark.parametrize("b,n,k,m,ks,seed", [
    (1, 16, 8192, 256, 0, 40),                          # a long K on a narrow layer: split by the default rule
    (1, 1, 512, 256, 2, 41), (1, 16, 512, 384, 3, 42),  # forced splits; 3 does not divide the 4 steps
    (1, 40, 1024, 256, 4, 43), (1, 100, 448, 128, 2, 44),  # several token passes; a partial last step of K
    (1, 8, 192, 256, 5, 45),                            # more splits asked for than there are steps
    (3, 5, 512, 256, 2, 46), (4, 12, 8192, 128, 0, 47), # bmm, forced and by the rule
])
def test_split_k_across_workgroups(ops, monkeypatch, b, n, k, m, ks, seed):
    """matmul / bmm launches of few workgroups split K across workgroups (fp32 partial sums in a scratch buffer, added
    in a fixed order by a second launch): against the oracle, against the unsplit kernel, and the same bits on every
    one of 20 calls."""
    say(f"split-K b={b} n={n} k={k} m={m} forced={ks} seed={seed}")
    from triteia_amd.python.capi import _ffi
    if ks:
        setknob(monkeypatch, "TRITEIA_HIP_KSPLIT", ks)
    kind = _ffi.lib().triteia_hip_uniform_kernel(m, b, n, k, 1)
    assert kind > 1000, f"this launch is meant to be split (kernel code {kind})"
    qw, meta, s = make_deltas(b, k, m, seed)
    x = activations(b * n, k, seed + 1).reshape(b, n, k)
    gq, gm, gs, gx = to_gpu(qw, meta, s, x)
    if b == 1:
        ref = orc.matmul_4bit_2_4(qw[0], x[0], meta[0], s[0])
        call = lambda: ops.matmul_4bit_2_4(gq[0], gx[0], gm[0], gs[0])
    else:
        ref = orc.bmm_4bit_2_4(qw, x, meta, s)
        call = lambda: ops.bmm_4bit_2_4(gq, gx, gm, gs)
    first = call()
    torch.cuda.synchronize()
    check_close(first, ref, what="split-K")
    for _ in range(19):
        again = call()
        assert torch.equal(again, first), "the K split must not depend on the order in which workgroups finish"
    setknob(monkeypatch, "TRITEIA_HIP_KSPLIT", 0)          # 0 turns the split off
    assert _ffi.lib().triteia_hip_uniform_kernel(m, b, n, k, 1) < 1000
    unsplit = call()
    torch.cuda.synchronize()
    assert float((first.float() - unsplit.float()).norm() / unsplit.float().norm()) < 1e-4


@pytest.mark.parametrize("b,n,k,m,seed", [(1, 16, 512, 384, 71), (1, 5, 4096, 256, 72), (3, 1, 1024, 128, 73), (2, 16, 192, 1152, 74),
                                          (1, 16, 11008, 256, 75),     # 86 steps: three chunks of requests per wavefront, the last ragged
                                          (2, 7, 4096, 2048, 76),      # 32 column blocks in all: the most that take 16-column shares
                                          (1, 3, 320, 128, 77),        # k = 320: a third step of two packed rows
                                          (8, 1, 4096, 512, 78),       # one token on each of eight matrices
                                          (1, 16, 1024, 5632, 79),     # 44 column blocks: shares of 32 columns
                                          (3, 9, 768, 3584, 80),       # 84 column blocks: shares of 64 columns
                                          (1, 2, 11008, 11008, 81)])   # 86 blocks, three chunks of requests
def test_column_shares_keep_the_bits(ops, monkeypatch, b, n, k, m, seed):
    """Small matmul / bmm launches give a workgroup a share of a column block (64, 32 or 16 columns instead of 128).  Every
    output column is still summed by the same wavefronts in the same order: each share width gives the bits of the whole block,
    and the oracle's values.  Left to the rule, these launches run on sparse24_share16_kernel (16-column shares, a share's
    columns as the rows of the MFMA, all requests of a wavefront at once): the same bits again."""
    say(f"column shares b={b} n={n} k={k} m={m} seed={seed}")
    from triteia_amd.python.capi import _ffi
    qw, meta, s = make_deltas(b, k, m, seed)
    x = activations(b * n, k, seed + 1).reshape(b, n, k)
    gq, gm, gs, gx = to_gpu(qw, meta, s, x)
    if b == 1:
        ref = orc.matmul_4bit_2_4(qw[0], x[0], meta[0], s[0])
        call = lambda: ops.matmul_4bit_2_4(gq[0], gx[0], gm[0], gs[0])
    else:
        ref = orc.bmm_4bit_2_4(qw, x, meta, s)
        call = lambda: ops.bmm_4bit_2_4(gq, gx, gm, gs)
    setknob(monkeypatch, "TRITEIA_HIP_KSPLIT", 0)
    setknob(monkeypatch, "TRITEIA_HIP_SUB_SHIFT", 0)
    whole = call()
    torch.cuda.synchronize()
    check_close(whole, ref, what="whole column blocks")
    for shift in (1, 2, 3):
        if b * ((((m // 128) << shift) + 7) // 8 * 8) > 256:
            continue        # (past one workgroup per CU the streaming kernel splits K over four wavefronts, not eight)
        setknob(monkeypatch, "TRITEIA_HIP_SUB_SHIFT", shift)
        assert torch.equal(call(), whole), f"shares of {128 >> shift} columns changed the result"
    delknob(monkeypatch, "TRITEIA_HIP_SUB_SHIFT")
    assert _ffi.lib().triteia_hip_uniform_kernel(m, b, n, k, 0) == 16
    assert torch.equal(call(), whole), "the rule's own choice (16-column shares on their own kernel) changed the result"
    setknob(monkeypatch, "TRITEIA_HIP_SHARE16", 0)
    assert _ffi.lib().triteia_hip_uniform_kernel(m, b, n, k, 0) == 0
    assert torch.equal(call(), whole), "the streaming kernel's own choice of share changed the result"


def test_reference_shaped_entry_points_directly(ops):
    """triteia_hip_mul_2_4, triteia_hip_bmm_2_4 and triteia_hip_sbmm_2_4 called with exactly the reference launchers'
    argument lists (marlin_nm.cu:42-46, triteia_nm_bmm.cu:760-764, triteia_nm_sbmm.cu:809-815), no binding layer."""
    say("reference-shaped C entry points")
    from triteia_amd.python.capi import _ffi
    lib, P = _ffi.lib(), _ffi.ptr
    b, k, m = 6, 512, 384
    qw, meta, s = make_deltas(b, k, m, 61)
    x = activations(b, k, 62)
    gq, gm, gs, gx = to_gpu(qw, meta, s, x)
    ws = torch.zeros(m // 128 * 16 * b, dtype=torch.int32, device=DEV)
    st = _ffi.stream_of(gx)
    # mul_2_4: all rows through matrix 2
    out = torch.zeros(b, m, dtype=torch.float16, device=DEV)
    assert lib.triteia_hip_mul_2_4(P(gx), P(gq[2]), P(gm[2]), P(out), P(gs[2]), m, b, k, P(ws), -1, 0, st, -1, -1, -1, 16) == 0
    check_close(out, orc.matmul_4bit_2_4(qw[2], x, meta[2], s[2]), what="triteia_hip_mul_2_4")
    # bmm_2_4: row i through matrix i
    out = torch.zeros(b, 1, m, dtype=torch.float16, device=DEV)
    assert lib.triteia_hip_bmm_2_4(P(gx), P(gq), P(gm), P(out), P(gs), m, b, k, P(ws), -1, 0, st, -1, -1, -1, 16) == 0
    check_close(out, orc.bmm_4bit_2_4(qw, x.reshape(b, 1, k), meta, s), what="triteia_hip_bmm_2_4")
    # sbmm_2_4: runs {matrix 4: rows 0-1}, {matrix 1: rows 2-4}, {-1: row 5}
    idx = np.array([4, 4, 1, 1, 1, -1], dtype=np.int32)
    run_idx, run_start, run_count = to_gpu(np.array([4, 1, -1], dtype=np.int32), np.array([0, 2, 5], dtype=np.int32),
                                           np.array([2, 3, 1], dtype=np.int32))
    out = torch.zeros(b, m, dtype=torch.float16, device=DEV)
    assert lib.triteia_hip_sbmm_2_4(P(gx), P(gq), P(gm), P(out), P(gs), P(run_idx), P(run_start), P(run_count), m, b, k, 3,
                                    P(ws), -1, 0, st, -1, -1, -1, 16) == 0
    torch.cuda.synchronize()
    check_close(out, orc.sbmm_4bit_2_4(qw, x, meta, s, idx), what="triteia_hip_sbmm_2_4")
    assert bool((out[5] == 0).all()) and int(ws.abs().sum()) == 0


def test_matmul_leading_dims_and_module(ops):
    from triteia_amd.python.nn.linear import sparse_low_precision_linear
    say("matmul leading dims + nn module")
    k, m = 256, 256
    qw, meta, s = make_deltas(1, k, m, 11)
    x = activations(6, k, 12).reshape(2, 3, k)
    ref = orc.matmul_4bit_2_4(qw[0], x.reshape(6, k), meta[0], s[0]).reshape(2, 3, m)
    gq, gm, gs, gx = to_gpu(qw[0], meta[0], s[0], x)
    out = ops.matmul_4bit_2_4(gq, gx, gm, gs)
    assert out.shape == (2, 3, m)
    check_close(out, ref, what="matmul 3-D input")
    layer = sparse_low_precision_linear(k, m).to(DEV)
    layer.qweight.copy_(gq), layer.meta.copy_(gm), layer.scale.copy_(gs)
    check_close(layer(gx), ref, what="sparse_low_precision_linear.forward")


def test_matmul_error_paths(ops):
    say("matmul error paths")
    from triteia_amd.python.capi import mul_2_4
    k, m = 128, 256
    qw, meta, s = make_deltas(1, k, m, 1)
    gq, gm, gs, gx = to_gpu(qw[0], meta[0], s[0], activations(4, k, 2))
    C = torch.zeros(4, m, dtype=torch.float16, device=DEV)
    with pytest.raises(RuntimeError, match="workspace must be of size at least"):
        mul_2_4(gx, gq, gm, C, gs, torch.zeros(1, dtype=torch.int32, device=DEV))
    ws = torch.zeros(m, dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError, match="not compatible"):
        mul_2_4(gx[:, :100].contiguous(), gq, gm, C, gs, ws)
    with pytest.raises(RuntimeError, match="contiguous"):
        mul_2_4(gx.t().contiguous().t(), gq, gm, C, gs, ws)
    with pytest.raises(RuntimeError, match="float16"):
        mul_2_4(gx.float(), gq, gm, C, gs, ws)
    mul_2_4(gx, gq, gm, C, gs, ws)
    torch.cuda.synchronize()
    assert int(ws.abs().sum()) == 0          # the lock workspace is left all-zero


# --------------------------------------------------------------------- bmm

@pytest.mark.parametrize("b,t,k,m,seed", [
    (4, 1, 512, 512, 21), (8, 1, 512, 512, 22), (16, 1, 512, 512, 23),   # tests/ops/test_bmm.py:12-15
    (3, 5, 256, 256, 24), (2, 40, 256, 384, 25),
    (8, 1, 4096, 4096, 1001),                                              # BASELINE config 1
])
def test_bmm_4bit_2_4(ops, b, t, k, m, seed):
    say(f"bmm b={b} t={t} k={k} m={m} seed={seed}")
    qw, meta, s = make_deltas(b, k, m, seed)
    x = activations(b * t, k, seed + 1).reshape(b, t, k)
    ref = orc.bmm_4bit_2_4(qw, x, meta, s)
    gq, gm, gs, gx = to_gpu(qw, meta, s, x)
    out = ops.bmm_4bit_2_4(gq, gx, gm, gs)
    loop = ops.bmm_4bit_2_4_forloop(gq, gx, gm, gs)
    torch.cuda.synchronize()
    tol = 1e-3 if (b, t, k, m) != (8, 1, 4096, 4096) else 2e-3           # test_bmm.py:40-42 uses 1e-3
    check_close(out, ref, tol=2e-3, what="bmm native")
    check_close(loop, ref, tol=2e-3, what="bmm forloop")
    # same kernel; delta b of a batch starts its walk over k at another step than a matrix on its own
    # does, so the two differ in the order of fp32 accumulation only
    assert float((out.float() - loop.float()).norm() / loop.float().norm()) < 1e-4
    assert orc.rel_mean_abs(out.float().cpu().numpy(), ref) < max(tol, 1e-3)


@pytest.mark.parametrize("b,t,k,m,seed", [
    (3, 70, 384, 640, 31),     # two full tiles per matrix and a last one of 6 tokens
    (2, 50, 256, 1152, 32),    # a last tile of 18 tokens
    (5, 32, 128, 128, 33),     # one tile, one step, one column block
])
def test_bmm_32_token_wide_kernel(ops, monkeypatch, b, t, k, m, seed):
    """Uniform groups on the 32-token build of the wide kernel (by default only for launches of 160 to 448 units)."""
    say(f"bmm on 32-token wide tiles b={b} t={t} k={k} m={m} seed={seed}")
    setknob(monkeypatch, "TRITEIA_HIP_WIDE32_MIN_UNITS", "1")
    setknob(monkeypatch, "TRITEIA_HIP_WIDE32_MAX_UNITS", "1000000000")
    qw, meta, s = make_deltas(b, k, m, seed)
    x = activations(b * t, k, seed + 1).reshape(b, t, k)
    gq, gm, gs, gx = to_gpu(qw, meta, s, x)
    out = ops.bmm_4bit_2_4(gq, gx, gm, gs)
    torch.cuda.synchronize()
    check_close(out, orc.bmm_4bit_2_4(qw, x, meta, s), what="bmm on 32-token wide tiles")
    setknob(monkeypatch, "TRITEIA_HIP_WIDE", "0")
    narrow = ops.bmm_4bit_2_4(gq, gx, gm, gs)
    torch.cuda.synchronize()
    assert float((out.float() - narrow.float()).norm() / narrow.float().norm()) < 1e-4


# -------------------------------------------------------------------- sbmm

def _indices(kind, T, N, seed, sort):
    rng = np.random.default_rng(seed)
    if kind == "uniform":
        idx = rng.integers(-1, N, size=T)
    elif kind == "zipf":
        p = np.arange(1, N + 2, dtype=np.float64) ** 1.5     # the reference's law over [-1, 0, ..]
        idx = rng.choice(np.arange(-1, N), size=T, p=p / p.sum())
    elif kind == "none":
        idx = np.full(T, -1)
    elif kind == "single":
        idx = np.full(T, N - 1)
    else:
        raise ValueError(kind)
    idx = idx.astype(np.int32)
    return np.sort(idx) if sort else idx


@pytest.mark.parametrize("kind,T,N,m,k,sort,seed", [
    ("uniform", 10, 5, 256, 512, True, 31),          # tests/ops/test_sbmm.py:69
    ("zipf", 128, 2, 4096, 12288, True, 32),         # tests/ops/test_sbmm.py:70
    ("uniform", 10, 5, 256, 512, False, 33),         # any order
    ("uniform", 100, 7, 384, 256, False, 34),
    ("none", 9, 3, 256, 128, True, 35),              # all -1
    ("single", 40, 3, 256, 256, True, 36),           # one run
    ("uniform", 64, 16, 4096, 4096, False, 1002),    # BASELINE config 2
    ("zipf", 600, 6, 512, 256, False, 37),           # plan with wide (64-token) tiles
    ("zipf", 700, 5, 640, 192, False, 38),           # the same with a partial last K step
])
def test_sbmm_variants(ops, kind, T, N, m, k, sort, seed, plan_rules):
    say(f"sbmm {kind} T={T} N={N} m={m} k={k} sorted={sort} seed={seed}")
    qw, meta, s = make_deltas(N, k, m, seed)
    x = activations(T, k, seed + 1)
    idx = _indices(kind, T, N, seed + 2, sort)
    ref = orc.sbmm_4bit_2_4(qw, x, meta, s, idx)
    gq, gm, gs, gx, gi = to_gpu(qw, meta, s, x, idx)
    native = ops.sbmm_4bit_2_4_native(gq, gx, gm, gs, gi)
    torch.cuda.synchronize()
    check_close(native, ref, what="sbmm native")
    # -1 rows are exactly zero, routed rows are not
    none = torch.from_numpy(idx < 0).to(DEV)
    assert bool((native[none] == 0).all())
    # routing: every row equals the product of that row alone with its own delta -- bit for bit when the
    # row is sent through the same routed entry point as a batch of one (the walk over k starts at
    # a step that depends on the delta's index) and the batch takes the narrow kernel; to the
    # accuracy of fp32 reassociation against the single-matrix op and for rows in 64-token wide tiles
    from triteia_amd.python.capi import sbmm_2_4_routed
    counts = np.bincount(idx[idx >= 0], minlength=N)
    for t in range(0, T, max(1, T // 8)):
        if idx[t] >= 0:
            alone = ops.matmul_4bit_2_4(gq[idx[t]], gx[t:t + 1], gm[idx[t]], gs[idx[t]])
            err = (alone[0].float() - native[t].float()).norm() / alone[0].float().norm()
            assert float(err) < 1e-3, f"row {t}: {float(err):.2e} from its own delta's product"
            one = torch.zeros((1, m), dtype=torch.float16, device=DEV)
            sbmm_2_4_routed(gx[t:t + 1].contiguous(), gq, gm, one, gs, gi[t:t + 1].contiguous())
            if T < 512 or counts[idx[t]] <= 32:
                assert torch.equal(one[0], native[t]), f"row {t} differs from the same row routed on its own"
    forloop = ops.sbmm_4bit_2_4_forloop(gq, gx, gm, gs, gi)
    check_close(forloop, ref, what="sbmm forloop")
    assert float((forloop.float() - native.float()).norm()) <= 1e-3 * float(native.float().norm())
    if sort:
        multi = ops.sbmm_4bit_2_4_multilaunch(gq, gx, gm, gs, gi)
        runs = ops.sbmm_4bit_2_4_runs(gq, gx, gm, gs, gi)
        torch.cuda.synchronize()
        check_close(multi, ref, what="sbmm multilaunch")
        check_close(runs, ref, what="sbmm runs")
        if T < 512:
            assert torch.equal(runs, native)          # the run table carries the delta ids: same walk, same bits


def _exact_problem(T, N, k, m, seed):
    """Integer activations in [-2, 2], int4 weights and a power-of-two scale: every product and every
    partial sum is exact in fp32 and the result is exact in fp16, whatever the order of summation."""
    rng = np.random.default_rng(seed)
    pairs = np.array([(0, 1), (0, 2), (0, 3), (1, 2), (1, 3), (2, 3)])
    qws, metas, ss = [], [], []
    for _ in range(N):
        sel = rng.integers(0, 6, size=(m, k // 4))
        qw, meta, sc = orc.pack_explicit(rng.integers(-8, 8, size=(m, k // 2)), pairs[sel, 0], pairs[sel, 1],
                                         np.full(m, 2.0 ** -6, dtype=np.float16))
        qws.append(qw), metas.append(meta), ss.append(sc)
    x = rng.integers(-2, 3, size=(T, k)).astype(np.float16)
    return np.stack(qws), np.stack(metas), np.stack(ss), x


@pytest.mark.parametrize("T,N,k,m,seed", [(64, 16, 512, 384, 51), (37, 5, 1024, 256, 52), (300, 7, 512, 640, 53), (700, 3, 256, 512, 54),
                                          (128, 16, 512, 256, 55), (97, 3, 256, 384, 56), (256, 32, 256, 256, 60), (193, 2, 512, 128, 61)])
def test_routing_is_bit_exact_on_exact_arithmetic(ops, monkeypatch, T, N, k, m, seed, plan_rules):
    """With inputs on which floating point is exact, every path (fused routing, routing plan with narrow
    and wide tiles, run table, one launch per run, one matmul per delta) must reproduce the oracle bit
    for bit: any token sent to the wrong delta, any row written twice or not at all would show."""
    say(f"exact routing T={T} N={N} k={k} m={m} seed={seed}")
    qw, meta, s, x = _exact_problem(T, N, k, m, seed)
    idx = np.random.default_rng(seed + 1).integers(-1, N, size=T).astype(np.int32)
    ref = orc.sbmm_4bit_2_4(qw, x, meta, s, idx)
    assert np.abs(ref).max() < 2048 * 2.0 ** -6                   # inside fp16's exact-integer range after scaling
    gq, gm, gs, gx, gi = to_gpu(qw, meta, s, x, idx)
    want = torch.from_numpy(ref.astype(np.float16)).to(DEV)
    assert torch.equal(ops.sbmm_4bit_2_4_native(gq, gx, gm, gs, gi), want)
    # a plan with wide tiles also carries a narrow-only cut of the same tokens; the kernels choose on the
    # device (here: a bar no launch reaches, so the narrow-only cut runs and the wide launch returns at once)
    setknob(monkeypatch, "TRITEIA_HIP_PLAN_WIDE_MIN_UNITS", "1000000000")
    assert torch.equal(ops.sbmm_4bit_2_4_native(gq, gx, gm, gs, gi), want)
    setknob(monkeypatch, "TRITEIA_HIP_PLAN_WIDE_MIN_UNITS", "1")
    assert torch.equal(ops.sbmm_4bit_2_4_forloop(gq, gx, gm, gs, gi), want)
    order = np.argsort(idx, kind="stable")
    gxs, gis = to_gpu(x[order], idx[order])
    wants = want[torch.from_numpy(order).to(DEV)]
    assert torch.equal(ops.sbmm_4bit_2_4_runs(gq, gxs, gm, gs, gis), wants)
    assert torch.equal(ops.sbmm_4bit_2_4_multilaunch(gq, gxs, gm, gs, gis), wants)


@pytest.mark.parametrize("T,N,k,m,seed", [
    (1, 16, 4096, 512, 201),       # one token: one delta in use, 16-column shares
    (3, 40, 1024, 1152, 202),      # three tokens over three of 40 deltas: 27 column blocks on the bound
    (16, 4, 640, 2048, 203),       # 16 tokens over four deltas (requested ahead of the routing unless that is switched off)
    (16, 64, 320, 1024, 204),      # up to 16 deltas in use of 64: 128 column blocks on the bound, shares of 64 columns; ragged K
    (7, 5, 11008, 128, 205),       # a long K: three chunks of requests per wavefront
    (5, 3, 256, 3584, 206),        # 84 column blocks on the bound
])
def test_small_routed_batches_on_column_shares(ops, monkeypatch, T, N, k, m, seed):
    """A routed batch of at most 16 tokens over few deltas of a small layer runs on the column-share kernel (routing inside
    the kernel, four wavefronts): against the oracle, the same bits as the streaming kernel, the same bits for a token
    when its batch is larger, rows without a delta untouched, accumulation in place."""
    say(f"small routed batch on column shares T={T} N={N} k={k} m={m} seed={seed}")
    from triteia_amd.python.capi import sbmm_2_4_routed
    setknob(monkeypatch, "TRITEIA_HIP_EAGER", "0")          # (route first: the form that takes the column-share kernel)
    qw, meta, s = make_deltas(N, k, m, seed)
    big = 48
    x = activations(big, k, seed + 1)
    rng = np.random.default_rng(seed + 2)
    idx = rng.integers(-1, N, size=big).astype(np.int32)
    idx[0] = N - 1                                           # (at least one routed token in the small batch)
    if T >= 3:
        idx[1] = -1
    ref = orc.sbmm_4bit_2_4(qw, x, meta, s, idx)
    gq, gm, gs, gx, gi = to_gpu(qw, meta, s, x, idx)

    def run(n_tokens, accumulate=False, base=None):
        out = torch.full((n_tokens, m), 3.0, dtype=torch.float16, device=DEV) if base is None else base.clone()
        sbmm_2_4_routed(gx[:n_tokens], gq, gm, out, gs, gi[:n_tokens], accumulate=accumulate)
        torch.cuda.synchronize()
        return out

    small = run(T)
    none = torch.from_numpy(idx[:T] < 0).to(DEV)
    assert bool((small[none] == 3.0).all())
    check_close(torch.where(none[:, None], torch.zeros_like(small), small), ref[:T], what="column shares, routed")
    setknob(monkeypatch, "TRITEIA_HIP_SHARE16", "0")
    assert torch.equal(run(T), small), "the streaming kernel gives other bits"
    delknob(monkeypatch, "TRITEIA_HIP_SHARE16")
    whole = run(big)                                         # the same tokens inside a batch of 48
    assert torch.equal(torch.where(none[:, None], whole[:T], whole[:T]), torch.where(none[:, None], whole[:T], small))
    base = torch.from_numpy(activations(T, m, seed + 3)).to(DEV)
    acc = run(T, accumulate=True, base=base)
    assert torch.equal(acc[none], base[none])
    check_close(acc.float() - base.float(), ref[:T], tol=4e-3, what="column shares, routed, accumulate")


@pytest.mark.parametrize("T,N,used,seed", [
    (64, 16, [0, 3, 5, 15], 41),        # most deltas without tokens: their prefetched weights are dropped
    (64, 8, list(range(8)), 42),         # every delta in use, some with more than one 16-token pass
    (33, 4, [2], 43),                    # one delta, three passes of 16 tokens
    (40, 64, [7, 63], 44),               # fewer than two tokens per delta: routes first, then requests
    (128, 16, list(range(16)), 45),      # two tokens per lane: groups that span both halves of the batch
    (100, 8, [1, 2, 6], 46),             # ... with a ragged second half and 30-token groups (two 16-token passes)
    (70, 40, [3, 39], 47),               # ... routing first
    (128, 32, list(range(32)), 48),      # the most deltas this form takes above 64 tokens
    (64, 64, list(range(64)), 62),       # as many deltas as a wavefront has lanes
    (65, 2, [0, 1], 49),                 # one token in the second half
    (256, 16, list(range(16)), 50),      # four tokens per lane
    (200, 32, list(range(0, 32, 3)), 57),
    (129, 4, [0, 3], 58),                # one token in the third part
    (250, 3, [1], 59),                   # one delta takes nearly everything: 13 passes of 16 tokens / 4 of 64
])
def test_fused_routing_static_groups(ops, monkeypatch, T, N, used, seed):
    """Batches of at most 256 tokens are routed inside the multiply kernel; with at least two tokens per
    delta every delta is a group of its own and its first weights are requested before the indices
    have arrived.  Same bits as routing first (TRITEIA_HIP_EAGER=0) and as the plan-based path."""
    say(f"fused routing T={T} N={N} used={used} seed={seed}")
    k, m = 512, 384
    qw, meta, s = make_deltas(N, k, m, seed)
    x = activations(T, k, seed + 1)
    rng = np.random.default_rng(seed + 2)
    idx = rng.choice(np.array(used + [-1], dtype=np.int32), size=T).astype(np.int32)
    ref = orc.sbmm_4bit_2_4(qw, x, meta, s, idx)
    gq, gm, gs, gx, gi = to_gpu(qw, meta, s, x, idx)
    outs = {}
    for name, env in (("eager", {"TRITEIA_HIP_EAGER": "1"}), ("route-first", {"TRITEIA_HIP_EAGER": "0"}),
                      ("planned", {"TRITEIA_HIP_FUSED_ROUTE": "0"})):
        for key in ("TRITEIA_HIP_EAGER", "TRITEIA_HIP_FUSED_ROUTE"):
            monkeypatch.delenv(key, raising=False)
        for key, value in env.items():
            monkeypatch.setenv(key, value)
        reload_knobs()
        out = torch.full((T, m), 3.0, dtype=torch.float16, device=DEV)      # rows without a delta must stay as they are
        from triteia_amd.python.capi import sbmm_2_4_routed
        sbmm_2_4_routed(gx, gq, gm, out, gs, gi)
        torch.cuda.synchronize()
        outs[name] = out
    none = torch.from_numpy(idx < 0).to(DEV)
    assert bool((outs["eager"][none] == 3.0).all())
    check_close(torch.where(none[:, None], torch.zeros_like(outs["eager"]), outs["eager"]), ref, what="fused routing")
    assert torch.equal(outs["eager"], outs["route-first"]) and torch.equal(outs["eager"], outs["planned"])


@pytest.mark.parametrize("T,N,k,m,seed", [
    (9000, 300, 128, 128, 91),      # more tokens than the plan kernel keeps in LDS between its passes; many deltas
    (12000, 3, 256, 128, 92),       # long runs: hundreds of wide tiles per delta, the wide kernel takes them
    (8300, 8192, 128, 128, 93),     # the largest delta count a plan accepts, most deltas without a token
])
def test_large_batches_through_the_plan(ops, T, N, k, m, seed, plan_rules):
    """Batches beyond the sizes the other tests use: the plan kernel's second pass re-reads the indices
    of tokens past its LDS cache, tile lists are thousands of entries long."""
    say(f"large batch T={T} N={N} k={k} m={m} seed={seed}")
    rng = np.random.default_rng(seed)
    if N <= 300:
        qw, meta, s = make_deltas(N, k, m, seed)
        idx = rng.integers(-1, N, size=T).astype(np.int32)
    else:
        # 8192 distinct deltas would take minutes to pack: a handful of real ones, addressed through a stack
        # whose other entries are never selected
        real = 6
        qw_r, meta_r, s_r = make_deltas(real, k, m, seed)
        sel = rng.choice(N, size=real, replace=False)
        qw = np.zeros((N,) + qw_r.shape[1:], dtype=qw_r.dtype)
        meta = np.zeros((N,) + meta_r.shape[1:], dtype=meta_r.dtype)
        s = np.ones((N,) + s_r.shape[1:], dtype=s_r.dtype)
        qw[sel], meta[sel], s[sel] = qw_r, meta_r, s_r
        idx = np.where(rng.random(T) < 0.1, -1, sel[rng.integers(0, real, size=T)]).astype(np.int32)
    x = activations(T, k, seed + 1)
    gq, gm, gs, gx, gi = to_gpu(qw, meta, s, x, idx)
    out = ops.sbmm_4bit_2_4_native(gq, gx, gm, gs, gi)
    torch.cuda.synchronize()
    used = np.unique(idx[idx >= 0])
    ref = np.zeros((T, m), dtype=np.float64)
    for d in used:                                   # the oracle, one dense delta at a time
        rows = np.nonzero(idx == d)[0]
        ref[rows] = x[rows].astype(np.float64) @ orc.unpack(qw[d], meta[d], s[d]).astype(np.float64)
    check_close(out, ref, what="large batch")
    assert bool((out[torch.from_numpy(idx < 0).to(DEV)] == 0).all())


@pytest.mark.parametrize("T,N,k,m,seed,hot", [
    (600, 3, 256, 512, 111, False),      # a plan of 32-token tiles that also lists 64-token tiles: that list
    (4000, 3, 256, 640, 112, False),     # a plan of 64-token tiles: its narrow-only list
    (1500, 40, 256, 512, 113, True),     # many deltas with a few tokens each beside a hot one
])
def test_one_list_of_64_token_tiles_instead_of_the_split(ops, monkeypatch, T, N, k, m, seed, hot):
    """A plan with wide tiles, on a layer whose wide launch is on: where one list of 64-token tiles over all tokens
    needs no more rounds of workgroups than the wide tiles alone (on these small layers: always), the wide kernel takes
    that list and the narrow kernel returns -- chosen on the device.  Against the oracle, and against the split
    {wide tiles, narrow rest} (knob off), which adds over K in another order for the rest's rows."""
    say(f"all-64 list T={T} N={N} k={k} m={m} seed={seed}")
    from triteia_amd.python.capi import sbmm_2_4_routed
    qw, meta, s = make_deltas(N, k, m, seed)
    x = activations(T, k, seed + 1)
    rng = np.random.default_rng(seed + 2)
    idx = rng.integers(-1, N, size=T).astype(np.int32)
    if hot:
        idx[rng.random(T) < 0.5] = 1
    ref = orc.sbmm_4bit_2_4(qw, x, meta, s, idx)
    gq, gm, gs, gx, gi = to_gpu(qw, meta, s, x, idx)
    setknob(monkeypatch, "TRITEIA_HIP_PLAN_WIDE_MIN_UNITS", "1")
    setknob(monkeypatch, "TRITEIA_HIP_MID", "0")
    outs = {}
    for all64 in ("1", "0"):
        setknob(monkeypatch, "TRITEIA_HIP_PLAN_ALL64", all64)
        for accumulate in (False, True):
            out = torch.full((T, m), -3.0 if not accumulate else 0.5, dtype=torch.float16, device=DEV)
            sbmm_2_4_routed(gx, gq, gm, out, gs, gi, accumulate=accumulate)
            torch.cuda.synchronize()
            outs[all64, accumulate] = out
    none = torch.from_numpy(idx < 0).to(DEV)
    for all64 in ("1", "0"):
        assert bool((outs[all64, False][none] == -3.0).all()) and bool((outs[all64, True][none] == 0.5).all())
        check_close(torch.where(none[:, None], torch.zeros_like(outs[all64, False]), outs[all64, False]), ref, what=f"all64={all64}")
        check_close(torch.where(none[:, None], torch.zeros_like(outs[all64, True]), outs[all64, True] - 0.5), ref, tol=4e-3, what=f"all64={all64}, added")
    rel = ((outs["1", False].float() - outs["0", False].float()).norm() / outs["0", False].float().norm()).item()
    assert rel < 1e-3, rel


@pytest.mark.parametrize("T,N,k,m,seed", [(64, 1, 512, 384, 95), (150, 2, 256, 640, 96), (100, 1, 320, 128, 97)])
def test_few_deltas_take_their_tiles_in_split_passes(ops, monkeypatch, T, N, k, m, seed, plan_rules):
    """One or two deltas with tens of tokens on a narrow layer: the plan's 64-token tiles are taken in
    16-token passes split over workgroups.  Same bits as whole tiles (the order of the sums over K does not
    depend on the pass width), within the bar of the oracle."""
    say(f"few deltas T={T} N={N} k={k} m={m} seed={seed}")
    from triteia_amd.python.capi import sbmm_2_4_routed
    qw, meta, s = make_deltas(N, k, m, seed)
    x = activations(T, k, seed + 1)
    idx = np.random.default_rng(seed + 2).integers(-1, N, size=T).astype(np.int32)
    ref = orc.sbmm_4bit_2_4(qw, x, meta, s, idx)
    gq, gm, gs, gx, gi = to_gpu(qw, meta, s, x, idx)
    outs = []
    for passes in ("4", "2", "1", None):
        setknob(monkeypatch, "TRITEIA_HIP_FUSED_ROUTE", "0")
        if passes is None:
            delknob(monkeypatch, "TRITEIA_HIP_PASS_NT")
        else:
            setknob(monkeypatch, "TRITEIA_HIP_PASS_NT", passes)
        out = torch.full((T, m), -3.0, dtype=torch.float16, device=DEV)
        sbmm_2_4_routed(gx, gq, gm, out, gs, gi)
        torch.cuda.synchronize()
        outs.append(out)
    none = torch.from_numpy(idx < 0).to(DEV)
    assert bool((outs[0][none] == -3.0).all())
    check_close(torch.where(none[:, None], torch.zeros_like(outs[0]), outs[0]), ref, what="split passes")
    for o in outs[1:]:
        assert torch.equal(o, outs[0])


@pytest.mark.parametrize("T,N,k,m,seed,wide_bar", [
    (100, 7, 256, 640, 101, "200"),        # ragged tiles, a partial last group of column blocks
    (300, 40, 384, 1408, 102, "200"),      # most deltas with a handful of tokens
    (90, 3, 128, 128, 103, "200"),         # one K step, one column block (three of four wavefronts idle)
    (600, 40, 256, 512, 104, "1"),         # plan with wide tiles: this kernel takes the narrow-only list of the plan,
    (600, 40, 256, 512, 105, "100000"),    # whatever the bar for the wide tiles says
    (600, 6, 256, 640, 106, "1"),          # a plan of 64-token tiles: the 64-token build takes its narrow-only list
    (200, 3, 128, 256, 107, "200"),        # the same without wide tiles in the plan
    (150, 5, 640, 384, 108, "200"),        # five K steps: the ring of four stages does not end on a whole turn
    (2600, 10, 640, 384, 109, "200"),     # a plan of 64-token tiles, full and ragged (halves with 32, a few and no tokens)
])
def test_plan_tiles_on_the_32_token_wide_kernel(ops, monkeypatch, T, N, k, m, seed, wide_bar, plan_rules):
    """A plan's 32-token tiles on a wide layer run on the 32-token build of the wide kernel (forced here
    onto small layers).  Against the oracle within the bar; against the K-split kernel within rounding;
    untouched rows stay untouched; accumulation in place."""
    say(f"32-token wide kernel T={T} N={N} k={k} m={m} seed={seed} wide_bar={wide_bar}")
    from triteia_amd.python.capi import sbmm_2_4_routed
    setknob(monkeypatch, "TRITEIA_HIP_FUSED_ROUTE", "0")
    setknob(monkeypatch, "TRITEIA_HIP_PLAN_ALL64", "0")   # (with MID=0 the narrow kernel is to take its share of the plan)
    setknob(monkeypatch, "TRITEIA_HIP_PLAN_WIDE_MIN_UNITS", wide_bar)
    qw, meta, s = make_deltas(N, k, m, seed)
    x = activations(T, k, seed + 1)
    idx = np.random.default_rng(seed + 2).integers(-1, N, size=T).astype(np.int32)
    if wide_bar != "200" and N >= 40:
        idx[: T // 3] = 1                                      # a hot delta: several wide tiles
    ref = orc.sbmm_4bit_2_4(qw, x, meta, s, idx)
    gq, gm, gs, gx, gi = to_gpu(qw, meta, s, x, idx)
    outs = {}
    for mid in ("1", "0"):
        setknob(monkeypatch, "TRITEIA_HIP_MID", mid)
        setknob(monkeypatch, "TRITEIA_HIP_MID_MIN_UNITS", "1")
        setknob(monkeypatch, "TRITEIA_HIP_MID_MIN_COLUMN_GROUPS", "1")
        out = torch.full((T, m), -3.0, dtype=torch.float16, device=DEV)
        sbmm_2_4_routed(gx, gq, gm, out, gs, gi)
        torch.cuda.synchronize()
        outs[mid] = out
    none = torch.from_numpy(idx < 0).to(DEV)
    assert bool((outs["1"][none] == -3.0).all())
    got = torch.where(none[:, None], torch.zeros_like(outs["1"]), outs["1"])
    check_close(got, ref, what="32-token wide kernel")
    assert not torch.equal(outs["1"], outs["0"]) or k <= 128, "the knob did not change the kernel"
    assert float((outs["1"].float() - outs["0"].float()).norm()) <= 1e-3 * float(outs["0"].float().norm())
    # two steps of weights in flight (64-token tiles taken as two halves by the 32-token build): every token's sum
    # over K is formed in the same order
    setknob(monkeypatch, "TRITEIA_HIP_MID", "1")
    setknob(monkeypatch, "TRITEIA_HIP_MID_DEPTH", "2")
    out = torch.full((T, m), -3.0, dtype=torch.float16, device=DEV)
    sbmm_2_4_routed(gx, gq, gm, out, gs, gi)
    torch.cuda.synchronize()
    assert torch.equal(out, outs["1"]), "the two-deep build changed bits"
    setknob(monkeypatch, "TRITEIA_HIP_MID_DEPTH", "1")
    # accumulate in place on top of a base
    base = torch.from_numpy(activations(T, m, seed + 3)).to(DEV)
    acc = base.clone()
    sbmm_2_4_routed(gx, gq, gm, acc, gs, gi, accumulate=True)
    torch.cuda.synchronize()
    assert torch.equal(acc[none], base[none])
    check_close(acc.float() - base.float(), ref, tol=4e-3, what="32-token wide kernel, accumulate")


@pytest.mark.parametrize("T,N,k,m,seed,counts", [
    (2000, 10, 640, 384, 111, None),                        # past two workgroups per CU on the bound as it is
    (700, 6, 256, 640, 112, None),                          # smaller: the two-deep build switched off
    (640, 5, 384, 256, 113, (0, 64, 65, 31, 480)),          # no token, a full tile, one over, half a tile, many tiles
    (1024, 16, 128, 128, 114, (64,) * 16),                  # every tile full, one K step, one column block
])
def test_plan_lists_64_token_tiles_for_wide_layers(ops, monkeypatch, T, N, k, m, seed, counts, plan_rules):
    """A batch of 48 tokens per delta and more whose plan is cut in 32-token tiles also lists its tokens in 64-token
    tiles, which wide layers run on the 64-token build of the wide kernel (forced here onto small layers).  Against
    the oracle within the bar; the same bits as from the 32-token tiles; untouched rows stay untouched."""
    say(f"64-token tiles beside a 32-token plan T={T} N={N} k={k} m={m} seed={seed}")
    from triteia_amd.python.capi import sbmm_2_4_routed, _ffi
    lib = _ffi.lib()
    qw, meta, s = make_deltas(N, k, m, seed)
    x = activations(T, k, seed + 1)
    rng = np.random.default_rng(seed + 2)
    if counts is None:
        idx = rng.integers(-1, N, size=T).astype(np.int32)
    else:
        idx = np.concatenate([np.full(c, d, np.int32) for d, c in enumerate(counts)])
        idx = rng.permutation(idx).astype(np.int32)
        assert idx.size == T
    ref = orc.sbmm_4bit_2_4(qw, x, meta, s, idx)
    gq, gm, gs, gx, gi = to_gpu(qw, meta, s, x, idx)
    outs = {}
    for big in ("1", "0"):
        setknob(monkeypatch, "TRITEIA_HIP_FUSED_ROUTE", "0")
        setknob(monkeypatch, "TRITEIA_HIP_MID_MIN_UNITS", "1")
        setknob(monkeypatch, "TRITEIA_HIP_MID_MIN_COLUMN_GROUPS", "1")
        setknob(monkeypatch, "TRITEIA_HIP_MID_NARROW", "0")
        setknob(monkeypatch, "TRITEIA_HIP_MID_DEPTH", "1")
        setknob(monkeypatch, "TRITEIA_HIP_PLAN_BIG", big)
        assert lib.triteia_hip_plan_tile_tokens(T, N) == 32
        assert lib.triteia_hip_planned_tile_kernel(T, N, m, k) == (64 if big == "1" else 32)
        out = torch.full((T, m), -3.0, dtype=torch.float16, device=DEV)
        sbmm_2_4_routed(gx, gq, gm, out, gs, gi)
        torch.cuda.synchronize()
        outs[big] = out
    none = torch.from_numpy(idx < 0).to(DEV)
    assert bool((outs["1"][none] == -3.0).all())
    check_close(torch.where(none[:, None], torch.zeros_like(outs["1"]), outs["1"]), ref, what="64-token tiles beside a 32-token plan")
    assert torch.equal(outs["1"], outs["0"]), "the 64-token tiles changed bits"
    # (on these small layers the idle slots of the padding work; the padded order gives the same)
    setknob(monkeypatch, "TRITEIA_HIP_PLAN_BIG", "1")
    setknob(monkeypatch, "TRITEIA_HIP_WIDE_ORDER_MIN_IDLE", "100")
    out = torch.full((T, m), -3.0, dtype=torch.float16, device=DEV)
    sbmm_2_4_routed(gx, gq, gm, out, gs, gi)
    torch.cuda.synchronize()
    assert torch.equal(out, outs["1"]), "the order of the units changed bits"
    # blocks of column groups x blocks of tiles per XCD (the blocks of tiles are cut on the device from the plan's real
    # number of tiles, the launch from the host's bound)
    for block in (1, 2, 4, 8):
        setknob(monkeypatch, "TRITEIA_HIP_XCD_CGS", str(block))
        out = torch.full((T, m), -3.0, dtype=torch.float16, device=DEV)
        sbmm_2_4_routed(gx, gq, gm, out, gs, gi)
        torch.cuda.synchronize()
        assert torch.equal(out, outs["1"]), f"blocks of {block} column groups per XCD changed bits"


def test_empty_and_degenerate_inputs(ops, plan_rules):
    """Zero tokens, zero deltas, zero adapters, a batch in which nothing is routed: every op returns the
    shape it should and touches nothing else."""
    say("empty and degenerate inputs")
    N, k, m, r = 3, 256, 256, 16
    qw, meta, s = make_deltas(N, k, m, 98)
    A, B = _lora_weights(2, k, r, m, 99, scale=0.05)
    gq, gm, gs, gA, gB = to_gpu(qw, meta, s, A, B)
    x0 = torch.zeros((0, k), dtype=torch.float16, device=DEV)
    i0 = torch.zeros((0,), dtype=torch.int32, device=DEV)
    assert ops.matmul_4bit_2_4(gq[0], x0, gm[0], gs[0]).shape == (0, m)
    assert ops.sbmm_4bit_2_4_native(gq, x0, gm, gs, i0).shape == (0, m)
    assert ops.sbmm_4bit_2_4_forloop(gq, x0, gm, gs, i0).shape == (0, m)
    assert ops.lora_sgmv_routed(gA, gB, x0, i0).shape == (0, m)
    assert ops.lora_bgmv(gA, gB, x0, i0).shape == (0, m)
    assert ops.ldmm(i0, x0, gA, gB, gq, gm, gs).shape == (0, m)
    assert ops.bmm_4bit_2_4(gq[:0], torch.zeros((0, 4, k), dtype=torch.float16, device=DEV), gm[:0], gs[:0]).shape == (0, 4, m)
    # tokens, but no delta / adapter selected
    x = torch.from_numpy(activations(70, k, 100)).to(DEV)
    none = torch.full((70,), -1, dtype=torch.int32, device=DEV)
    for T in (5, 70):
        assert bool((ops.sbmm_4bit_2_4_native(gq, x[:T], gm, gs, none[:T]) == 0).all())
        assert bool((ops.lora_sgmv_routed(gA, gB, x[:T], none[:T]) == 0).all())
        assert bool((ops.ldmm(none[:T], x[:T], gA, gB, gq, gm, gs) == 0).all())
    # no LoRA adapters at all: ldmm is the routed delta op
    idx = torch.from_numpy(np.random.default_rng(101).integers(-1, N, size=70).astype(np.int32)).to(DEV)
    noA = torch.zeros((0, k, r), dtype=torch.float16, device=DEV)
    noB = torch.zeros((0, r, m), dtype=torch.float16, device=DEV)
    assert torch.equal(ops.ldmm(idx, x, noA, noB, gq, gm, gs), ops.sbmm_4bit_2_4_native(gq, x, gm, gs, idx))
    torch.cuda.synchronize()


def test_sbmm_with_base_weight_accumulates_in_place(ops, plan_rules):
    say("sbmm with base weight")
    T, N, k, m = 24, 4, 256, 256
    qw, meta, s = make_deltas(N, k, m, 41)
    x = activations(T, k, 42)
    base = (np.random.default_rng(43).standard_normal((m, k)) * 0.02).astype(np.float16)
    idx = _indices("uniform", T, N, 44, sort=False)
    gq, gm, gs, gx, gi, gb = to_gpu(qw, meta, s, x, idx, base)
    out = ops.sbmm_4bit_2_4_native(gq, gx, gm, gs, gi, base_weight=gb)
    torch.cuda.synchronize()
    # the base GEMM is a library call on both sides: take its fp16 result as given
    y0 = torch.matmul(gx, gb.t()).float().cpu().numpy().astype(np.float64)
    ref = y0 + orc.sbmm_4bit_2_4(qw, x, meta, s, idx)
    check_close(out, ref, what="sbmm + base")
    none = torch.from_numpy(idx < 0).to(DEV)
    assert torch.equal(out[none], torch.matmul(gx, gb.t())[none])


def test_route_plan_is_a_stable_grouping(plan_rules):
    from triteia_amd.python.capi import _ffi, route_plan
    say("route plan")
    rng = np.random.default_rng(51)
    # (the later cases walk through the numbers of token shares the plan kernel places side by side: 16 up to 512
    # deltas, fewer above, one at 8192; shares of ragged size; more tokens than it keeps in LDS between its passes)
    for T, N, off in [(1, 1, 0), (64, 16, 0), (200, 7, 0), (1000, 300, 0), (130, 5, 3), (70, 100, 0), (700, 3, 0), (520, 40, 0),
                      (4096, 16, 0), (65, 2, 0), (129, 513, 0), (5000, 600, 0), (3000, 1024, 2), (2500, 3000, 0), (1500, 8192, 0),
                      (9000, 4, 0), (8193, 33, 1)]:
        idx = rng.integers(-1, N + off, size=T).astype(np.int32)
        plan = route_plan(torch.from_numpy(idx).to(DEV), N, index_offset=off).cpu().numpy()
        d = idx - off
        valid = (d >= 0) & (d < N)
        tile = _ffi.lib().triteia_hip_plan_tile_tokens(T, N)
        max_tiles, max_wide = min(T, N) + T // 16, T // 33 + 1
        n_tiles, n_routed, n_used, tile_dev, n_wide = plan[0], plan[1], plan[2], plan[3], plan[4]
        o_tiles, o_wide, o_perm = 8, 8 + 4 * max_tiles, 8 + 4 * max_tiles + 4 * max_wide
        tiles = plan[o_tiles:o_tiles + 4 * max_tiles].reshape(max_tiles, 4)[:n_tiles]
        wides = plan[o_wide:o_wide + 4 * max_wide].reshape(max_wide, 4)[:n_wide]
        perm = plan[o_perm:o_perm + T]
        o_all = (o_perm + T + 3) // 4 * 4
        alls = plan[o_all:o_all + 4 * max_tiles].reshape(max_tiles, 4)[:plan[5]]
        used = np.unique(d[valid])
        assert tile_dev == tile and n_used == len(used) and n_routed == valid.sum()
        has_wide = T >= WIDE_MIN_BATCH and T >= 8 * min(T, N)
        pos, ti, wi, ai = 0, 0, 0, 0
        for delta in used:
            rows = np.nonzero(d == delta)[0]                # ascending = original order
            c = len(rows)
            assert np.array_equal(perm[pos:pos + c], rows)
            c_wide = 0
            if has_wide:
                c_wide = c // 64 * 64
                if c - c_wide >= 33:
                    c_wide = c
            for first in range(0, c_wide, 64):               # wide tiles first ...
                assert list(wides[wi]) == [delta, pos + first, min(64, c_wide - first), 0]
                wi += 1
            for first in range(c_wide, c, tile):             # ... then the narrow rest
                assert list(tiles[ti]) == [delta, pos + first, min(tile, c - first), 0]
                ti += 1
            if has_wide:                                     # and the same tokens in narrow tiles only
                for first in range(0, c, tile):
                    assert list(alls[ai]) == [delta, pos + first, min(tile, c - first), 0]
                    ai += 1
            pos += c
        assert ti == n_tiles and wi == n_wide and ai == plan[5]
        assert has_wide == (n_wide > 0 or plan[5] > 0) or not valid.any()


# ------------------------------------------------------------- lora / ldmm

def _lora_weights(M, k, r, m, seed, scale=1.0):
    rng = np.random.default_rng(seed)
    A = (rng.standard_normal((M, k, r)) * scale).astype(np.float16)
    B = (rng.standard_normal((M, r, m)) * scale).astype(np.float16)
    return A, B


def _assert_allclose_scaled(got, ref, what):
    # torch.allclose(rtol=atol=5e-3) of tests/ops/test_ldmm.py:73, with atol scaled by the
    # typical output magnitude (the reference's inputs are O(1) weights, outputs O(sqrt(k r)))
    got = got.float().cpu().numpy().astype(np.float64)
    scale = max(1.0, float(np.sqrt(np.mean(ref ** 2))))
    bad = np.abs(got - ref) > 5e-3 * scale + 5e-3 * np.abs(ref)
    assert not bad.any(), f"{what}: {bad.sum()} of {bad.size} elements outside tolerance"


@pytest.mark.parametrize("T,M,k,m,r,seed", [
    (10, 5, 768, 256, 64, 61),        # tests/ops/test_lora_bgmv.py:73
    (128, 2, 4096, 12288, 64, 62),    # tests/ops/test_lora_bgmv.py:74
    (33, 4, 512, 1024, 8, 63), (33, 4, 512, 1024, 16, 64), (33, 4, 512, 1000, 32, 65),
    # segments longer than one pass of the row slots, ragged tails, a rank that is no power of two, the widest rank
    (301, 3, 1024, 2048, 16, 66), (71, 3, 512, 520, 24, 67), (41, 2, 1024, 512, 128, 68),
])
def test_lora_ops(ops, T, M, k, m, r, seed):
    say(f"lora T={T} M={M} k={k} m={m} r={r} seed={seed}")
    A, B = _lora_weights(M, k, r, m, seed, scale=0.1)
    x = activations(T, k, seed + 1)
    idx = np.sort(np.random.default_rng(seed + 2).integers(-1, M, size=T)).astype(np.int32)
    ref = orc.lora(A, B, x, idx)
    gA, gB, gx, gi = to_gpu(A, B, x, idx)
    for name in ("lora_bgmv", "lora_sgmv", "lora_sgmv_routed", "lora_forloop"):
        out = getattr(ops, name)(gA, gB, gx, gi)
        torch.cuda.synchronize()
        check_close(out, ref, tol=2e-3, what=name)
        _assert_allclose_scaled(out, ref, name)
        assert bool((out[torch.from_numpy(idx < 0).to(DEV)] == 0).all())
    # unsorted indices: the per-token and the routed variants do not care
    perm = np.random.default_rng(seed + 3).permutation(T)
    gi2 = torch.from_numpy(idx[perm].copy()).to(DEV)
    gx2 = gx[torch.from_numpy(perm).to(DEV)].contiguous()
    ref2 = ref[perm]
    check_close(ops.lora_bgmv(gA, gB, gx2, gi2), ref2, what="lora_bgmv unsorted")
    check_close(ops.lora_sgmv_routed(gA, gB, gx2, gi2), ref2, what="lora_sgmv_routed unsorted")


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("T,M,k,m,r,seed", [
    (128, 2, 4096, 12288, 64, 181),      # tests/ops/test_lora_bgmv.py:74
    (300, 3, 1024, 2048, 32, 182), (70, 2, 512, 520, 128, 183), (41, 5, 768, 256, 64, 184), (200, 4, 1024, 1000, 32, 185),
    (10, 5, 768, 768, 64, 186),          # short segments through the same kernels
    (97, 3, 2048, 384, 16, 187),         # rank 16: the shrink only
])
def test_lora_on_the_matrix_cores(ops, monkeypatch, T, M, k, m, r, seed, dtype):
    """SGMV and routed SGMV with every launch the matrix-core kernels can take sent to them (by default: ranks 32 / 64 /
    128 with 16 rows per group and more), against the oracle; in bf16 with the oracle's bf16 intermediate.  The same
    calls with those kernels switched off agree to the rounding of the intermediate."""
    say(f"lora mfma T={T} M={M} k={k} m={m} r={r} seed={seed} {dtype}")
    rng = np.random.default_rng(seed)
    idx = np.sort(rng.integers(-1, M, size=T)).astype(np.int32)
    if dtype == "f16":
        A, B = _lora_weights(M, k, r, m, seed, scale=0.1)
        x = activations(T, k, seed + 1)
        ref = orc.lora(A, B, x, idx)
        gA, gB, gx = to_gpu(A, B, x)
        tol = 2e-3
    else:
        A = orc.round_bf16(rng.standard_normal((M, k, r)) * 0.1).astype(np.float32)
        B = orc.round_bf16(rng.standard_normal((M, r, m)) * 0.1).astype(np.float32)
        x = orc.round_bf16(rng.standard_normal((T, k))).astype(np.float32)
        ref = orc.lora(A, B, x, idx, intermediate="bf16")
        gA, gB, gx = (torch.from_numpy(a).to(DEV).to(torch.bfloat16) for a in (A, B, x))
        tol = 1e-2
    gi = torch.from_numpy(idx).to(DEV)
    outs = {}
    for mode in ("2", "0"):
        setknob(monkeypatch, "TRITEIA_HIP_LORA_MFMA", mode)
        for name in ("lora_sgmv", "lora_sgmv_routed"):
            out = getattr(ops, name)(gA, gB, gx, gi)
            torch.cuda.synchronize()
            check_close(out, ref, tol=tol, what=f"{name} (LORA_MFMA={mode})")
            assert bool((out[torch.from_numpy(idx < 0).to(DEV)] == 0).all())
            outs[(name, mode)] = out
    for name in ("lora_sgmv", "lora_sgmv_routed"):
        d = (outs[(name, "2")].float() - outs[(name, "0")].float()).norm() / outs[(name, "0")].float().norm()
        assert float(d) < tol, f"{name}: matrix-core and VALU kernels differ by {float(d):.2e}"
    # unsorted indices through the routed form
    setknob(monkeypatch, "TRITEIA_HIP_LORA_MFMA", "2")
    perm = rng.permutation(T)
    gi2 = torch.from_numpy(idx[perm].copy()).to(DEV)
    gx2 = gx[torch.from_numpy(perm).to(DEV)].contiguous()
    check_close(ops.lora_sgmv_routed(gA, gB, gx2, gi2), ref[perm], tol=tol, what="lora_sgmv_routed unsorted (matrix cores)")


@pytest.mark.parametrize("T,M,d_in,d_out,seed", [
    (37, 4, 1024, 16, 171), (37, 4, 16, 1024, 172), (90, 3, 512, 64, 173), (90, 3, 64, 520, 174), (20, 2, 768, 128, 175),
    (64, 5, 32, 2048, 176), (50, 3, 24, 256, 177),
])
@pytest.mark.parametrize("mfma", ["0", "2"])
def test_lora_kernels_store_instead_of_add(monkeypatch, T, M, d_in, d_out, seed, mfma):
    """The stored form of BGMV / SGMV / routed SGMV (no counterpart in the reference; the intermediate of a LoRA pair then
    needs no clearing): rows that take an adapter hold the product alone, whatever the output held before; the others
    keep what they held.  Both directions (wide -> narrow, narrow -> wide), against a plain fp32 product."""
    from triteia_amd.python.capi import route_plan, sgmv_routed
    from triteia_amd.python.capi.punica import dispatch_bgmv, sgmv, sgmv_tmp_size
    say(f"lora store T={T} M={M} d_in={d_in} d_out={d_out} seed={seed} LORA_MFMA={mfma}")
    setknob(monkeypatch, "TRITEIA_HIP_LORA_MFMA", mfma)
    rng = np.random.default_rng(seed)
    W = (rng.standard_normal((M, d_in, d_out)) * 0.1).astype(np.float16)
    x = (rng.standard_normal((T, d_in))).astype(np.float16)
    idx = np.sort(rng.integers(-1, M, size=T)).astype(np.int32)
    ref = np.full((T, d_out), 7.0)
    for t in range(T):
        if idx[t] >= 0:
            ref[t] = x[t].astype(np.float64) @ W[idx[t]].astype(np.float64)
    gW, gx, gi = to_gpu(W, x, idx)
    routed = torch.from_numpy(idx >= 0).to(DEV)

    def check(y, what):
        torch.cuda.synchronize()
        assert bool((y[~routed] == 7).all()), what + ": a row without an adapter was written"
        check_close(y[routed], ref[idx >= 0], tol=2e-3, what=what)

    y = torch.full((T, d_out), 7.0, dtype=torch.float16, device=DEV)
    sgmv_routed(y, gx, gW, route_plan(gi, M), accumulate=False)
    check(y, "routed SGMV, stored")
    y = torch.full((T, d_out), 7.0, dtype=torch.float16, device=DEV)
    dispatch_bgmv(y, gx, gW.transpose(1, 2).contiguous().unsqueeze(1), gi.to(torch.long), 0, 1.0, accumulate=False)
    check(y, "BGMV, stored")
    # SGMV on a segment table: rows of the leading -1 run lie outside every segment
    y = torch.full((T, d_out), 7.0, dtype=torch.float16, device=DEV)
    skip = int((idx < 0).sum())
    counts = np.bincount(idx[idx >= 0], minlength=M)
    seg = torch.from_numpy(np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)).to(DEV)
    w_ptr = torch.tensor([gW[i].data_ptr() for i in range(M)], dtype=torch.int64, device=DEV)
    tmp = torch.empty((sgmv_tmp_size(M),), dtype=torch.uint8, device=DEV)
    sgmv(y[skip:], gx[skip:], w_ptr, seg, tmp, 0, accumulate=False)
    check(y, "SGMV, stored")
    # and added on top of what is there, as before
    y = torch.full((T, d_out), 7.0, dtype=torch.float16, device=DEV)
    sgmv_routed(y, gx, gW, route_plan(gi, M))
    torch.cuda.synchronize()
    check_close(y[routed].float() - 7.0, ref[idx >= 0], tol=2e-2, what="routed SGMV, added")


@pytest.mark.parametrize("T,M,k,m,r,seed", [
    (10, 5, 768, 256, 64, 161), (33, 4, 512, 1024, 16, 162), (71, 3, 512, 520, 24, 163), (41, 2, 1024, 512, 128, 164),
])
def test_lora_ops_bf16(ops, T, M, k, m, r, seed):
    """The bfloat16 instantiation of BGMV / SGMV (the reference builds both element types: bgmv_all.cu:4-5,
    sgmv.cu:10).  bf16 keeps 8 significant bits: one rounding of an output is up to 2^-9 relative (1.1e-3 rms),
    and the rank-r intermediate, rounded to bf16 as well, can fall on the other side of a rounding boundary when
    the fp32 sums are taken in another order; the bound here is 1e-2 relative Frobenius error."""
    say(f"lora bf16 T={T} M={M} k={k} m={m} r={r} seed={seed}")
    rng = np.random.default_rng(seed)
    A = orc.round_bf16(rng.standard_normal((M, k, r)) * 0.1).astype(np.float32)
    B = orc.round_bf16(rng.standard_normal((M, r, m)) * 0.1).astype(np.float32)
    x = orc.round_bf16(rng.standard_normal((T, k))).astype(np.float32)
    idx = np.sort(rng.integers(-1, M, size=T)).astype(np.int32)
    ref = orc.lora(A, B, x, idx, intermediate="bf16")
    gA, gB, gx = (torch.from_numpy(a).to(DEV).to(torch.bfloat16) for a in (A, B, x))
    gi = torch.from_numpy(idx).to(DEV)
    for name in ("lora_bgmv", "lora_sgmv", "lora_sgmv_routed", "lora_forloop"):
        out = getattr(ops, name)(gA, gB, gx, gi)
        torch.cuda.synchronize()
        assert out.dtype == torch.bfloat16
        check_close(out, ref, tol=1e-2, what=name + " bf16")
        assert bool((out[torch.from_numpy(idx < 0).to(DEV)] == 0).all())
    with pytest.raises(RuntimeError, match="bfloat16"):
        ops.lora_sgmv_routed(gA.half(), gB, gx, gi)          # mixed element types are refused


@pytest.mark.parametrize("T,M,N,m,k,r,seed", [
    (10, 5, 5, 768, 768, 8, 71), (10, 5, 5, 768, 768, 64, 72),          # tests/ops/test_ldmm.py:103
    (128, 2, 3, 4096, 2048, 16, 73), (128, 16, 16, 1024, 1024, 32, 74),
])
def test_ldmm(ops, T, M, N, m, k, r, seed, plan_rules):
    say(f"ldmm T={T} M={M} N={N} m={m} k={k} r={r} seed={seed}")
    qw, meta, s = make_deltas(N, k, m, seed)
    A, B = _lora_weights(M, k, r, m, seed + 1, scale=0.05)
    x = activations(T, k, seed + 2)
    idx = np.random.default_rng(seed + 3).integers(-1, M + N, size=T).astype(np.int32)
    ref = orc.ldmm(idx, x, A, B, qw, meta, s)
    gq, gm, gs, gA, gB, gx, gi = to_gpu(qw, meta, s, A, B, x, idx)
    out = ops.ldmm(gi, gx, gA, gB, gq, gm, gs)
    base = ops.baseline_ldmm(gi, gx, gA, gB, gq, gm, gs)
    torch.cuda.synchronize()
    check_close(out, ref, what="ldmm")
    check_close(base, ref, what="baseline_ldmm")
    _assert_allclose_scaled(out, ref, "ldmm")
    assert bool((out[torch.from_numpy(idx < 0).to(DEV)] == 0).all())
    # the two index ranges really go to the two kinds of model
    only_delta = ops.sbmm_4bit_2_4_native(gq, gx, gm, gs, torch.where(gi >= M, gi - M, -1).int())
    rows = torch.from_numpy(idx >= M).to(DEV)
    assert torch.equal(out[rows], only_delta[rows])
    # with a dense base weight (routing and the LoRA shrink then run on a side stream beside the base GEMM):
    # the library GEMM's fp16 result is taken as given, the routed parts are added to it in place
    base_w = (np.random.default_rng(seed + 4).standard_normal((m, k)) * 0.02).astype(np.float16)
    gb = torch.from_numpy(base_w).to(DEV)
    for _ in range(3):                                   # several calls in a row share the side stream
        with_base = ops.ldmm(gi, gx, gA, gB, gq, gm, gs, base_weight=gb)
    torch.cuda.synchronize()
    y0 = torch.matmul(gx, gb.t())
    ref_b = y0.float().cpu().numpy().astype(np.float64) + ref
    check_close(with_base, ref_b, what="ldmm + base")
    assert torch.equal(with_base[torch.from_numpy(idx < 0).to(DEV)], y0[torch.from_numpy(idx < 0).to(DEV)])
