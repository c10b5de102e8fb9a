"""The entry points under HIP graph capture: a serving loop records one decode step once and
replays it for every batch, with new activations and routing written into the same buffers.
Every replay must give the bits of the eager call on the same inputs."""
import numpy as np
import pytest
import torch

from oracle import triteia_oracle as orc
from tests.helpers import activations, check_close, make_deltas, setknob, to_gpu

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _capture(fn):
    """Record fn() into a graph on a side stream (capture needs a non-default stream)."""
    graph = torch.cuda.CUDAGraph()
    s = torch.cuda.Stream()                      # default priority
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        with torch.cuda.graph(graph, stream=s):
            fn()
    torch.cuda.synchronize()
    return graph


@pytest.mark.parametrize("T,N,k,m,seed", [
    (24, 6, 256, 384, 201),      # routed inside the multiply kernel
    (200, 9, 256, 256, 202),     # same, four tokens per lane
    (300, 40, 256, 384, 203),    # routing plan + multiply, two launches
    (600, 3, 256, 512, 204),     # plan with wide tiles: three launches
])
def test_routed_sbmm_replays(monkeypatch, T, N, k, m, seed):
    from triteia_amd.python.capi import routed_workspace, sbmm_2_4_routed
    # the wide kernel takes its tiles however few they are (by default only when they fill the chip)
    setknob(monkeypatch, "TRITEIA_HIP_PLAN_WIDE_MIN_UNITS", "1")
    print(f"[case] graph replay of routed sbmm T={T} N={N} k={k} m={m} seed={seed}", flush=True)
    qw, meta, s = make_deltas(N, k, m, seed)
    gq, gm, gs = to_gpu(qw, meta, s)
    x = torch.zeros((T, k), dtype=torch.float16, device=DEV)
    idx = torch.full((T,), -1, dtype=torch.int32, device=DEV)
    out = torch.zeros((T, m), dtype=torch.float16, device=DEV)
    ws = routed_workspace(T, N, DEV)
    torch.cuda.synchronize()

    def step():
        out.zero_()                               # a fill kernel, not a memset node
        sbmm_2_4_routed(x, gq, gm, out, gs, idx, workspace=ws)

    step()                                        # load the code objects before capturing
    torch.cuda.synchronize()
    graph = _capture(step)
    rng = np.random.default_rng(seed + 1)
    for rep in range(4):
        hx = activations(T, k, seed + 10 + rep)
        hidx = rng.integers(-1, N, size=T).astype(np.int32)
        if rep == 2:
            hidx[:] = -1                          # a batch nobody routes: every row stays zero
        x.copy_(torch.from_numpy(hx))
        idx.copy_(torch.from_numpy(hidx))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        replayed = out.clone()
        step()                                    # the program's own eager work between replays
        torch.cuda.synchronize()
        assert torch.equal(replayed, out), f"replay {rep} differs from the eager call"
        ref = orc.sbmm_4bit_2_4(qw, hx, meta, s, hidx)
        if (hidx >= 0).any():
            check_close(replayed, ref, what=f"replay {rep}")
        assert bool((replayed[torch.from_numpy(hidx < 0).to(DEV)] == 0).all())


def test_ldmm_replays():
    """ldmm with a dense base: the routing and the LoRA shrink fork onto a second stream inside
    the captured region and join before the expand."""
    from triteia_amd.python import ops
    T, M, N, k, m, r, seed = 96, 4, 5, 512, 768, 16, 211
    print(f"[case] graph replay of ldmm T={T} M={M} N={N} k={k} m={m} r={r}", flush=True)
    qw, meta, s = make_deltas(N, k, m, seed)
    rng = np.random.default_rng(seed + 1)
    A = (rng.standard_normal((M, k, r)) * 0.05).astype(np.float16)
    B = (rng.standard_normal((M, r, m)) * 0.05).astype(np.float16)
    base_w = (rng.standard_normal((m, k)) * 0.02).astype(np.float16)
    gq, gm, gs, gA, gB, gb = to_gpu(qw, meta, s, A, B, base_w)
    x = torch.zeros((T, k), dtype=torch.float16, device=DEV)
    idx = torch.full((T,), -1, dtype=torch.int32, device=DEV)
    result = torch.zeros((T, m), dtype=torch.float16, device=DEV)

    def step():
        result.copy_(ops.ldmm(idx, x, gA, gB, gq, gm, gs, base_weight=gb))

    step()
    torch.cuda.synchronize()
    graph = _capture(step)
    for rep in range(3):
        hx = activations(T, k, seed + 10 + rep)
        hidx = rng.integers(-1, M + N, size=T).astype(np.int32)
        x.copy_(torch.from_numpy(hx))
        idx.copy_(torch.from_numpy(hidx))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        replayed = result.clone()
        step()
        torch.cuda.synchronize()
        assert torch.equal(replayed, result), f"replay {rep} differs from the eager call"
        y0 = torch.matmul(x, gb.t()).float().cpu().numpy().astype(np.float64)
        check_close(replayed, y0 + orc.ldmm(hidx, hx, A, B, qw, meta, s), what=f"ldmm replay {rep}")


def test_matmul_and_bmm_replay():
    """The uniform entry points (one to three launches each: wide tiles, a narrow rest) in one graph."""
    from triteia_amd.python import ops
    T, B, t, k, m, seed = 300, 3, 40, 512, 1024, 221
    print(f"[case] graph replay of matmul T={T} and bmm {B} x {t}, k={k} m={m}", flush=True)
    qw, meta, s = make_deltas(B, k, m, seed)
    gq, gm, gs = to_gpu(qw, meta, s)
    x = torch.zeros((T, k), dtype=torch.float16, device=DEV)
    xb = torch.zeros((B, t, k), dtype=torch.float16, device=DEV)
    y = torch.zeros((T, m), dtype=torch.float16, device=DEV)
    yb = torch.zeros((B, t, m), dtype=torch.float16, device=DEV)

    def step():
        y.copy_(ops.matmul_4bit_2_4(gq[0], x, gm[0], gs[0]))
        yb.copy_(ops.bmm_4bit_2_4(gq, xb, gm, gs))

    step()
    torch.cuda.synchronize()
    graph = _capture(step)
    for rep in range(3):
        hx, hxb = activations(T, k, seed + 10 + rep), activations(B * t, k, seed + 20 + rep).reshape(B, t, k)
        x.copy_(torch.from_numpy(hx))
        xb.copy_(torch.from_numpy(hxb))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        ry, ryb = y.clone(), yb.clone()
        step()
        torch.cuda.synchronize()
        assert torch.equal(ry, y) and torch.equal(ryb, yb), f"replay {rep} differs from the eager call"
        check_close(ry, orc.matmul_4bit_2_4(qw[0], hx, meta[0], s[0]), what=f"matmul replay {rep}")
        check_close(ryb, orc.bmm_4bit_2_4(qw, hxb, meta, s), what=f"bmm replay {rep}")
