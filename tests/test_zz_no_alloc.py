"""The routed multiply with the routing plan in the library's own device buffer (no workspace argument,
no allocation): same bits as the entry point that takes the caller's workspace, on two calls in a row,
the second one smaller."""
import ctypes

import numpy as np
import pytest
import torch

from tests.helpers import activations, make_deltas, to_gpu
from triteia_amd.python.capi import _ffi

pytestmark = pytest.mark.gpu


def run_both(lib, T, N, k, m, seed, accumulate):
    qw, meta, s = make_deltas(N, k, m, seed)
    x = activations(T, k, seed + 1)
    idx = np.random.default_rng(seed + 2).integers(-1, N, size=T).astype(np.int32)
    gq, gm, gs, gx, gi = to_gpu(qw, meta, s, x, idx)
    start = torch.randn((T, m), device="cuda:0").half()
    P = _ffi.ptr
    stream = _ffi.stream_of(gx)

    want = start.clone()
    nbytes = lib.triteia_hip_sbmm_routed_workspace_bytes(T, N)
    ws = torch.empty((nbytes + 3) // 4, dtype=torch.int32, device="cuda:0")
    rc = lib.triteia_hip_sbmm_2_4_routed(P(gx), P(gq), P(gm), P(want), P(gs), P(gi), 0, N, m, T, k, P(ws), ws.numel() * 4,
                                         accumulate, 0, stream)
    assert rc == 0, _ffi.last_error()

    got = start.clone()
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    rc = lib.triteia_hip_sbmm_2_4_routed_static(P(gx), P(gq), P(gm), P(got), P(gs), P(gi), 0, N, m, T, k, accumulate, 0, stream)
    assert rc == 0, _ffi.last_error()
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.equal(got, want), f"T={T} N={N}: {(got != want).sum().item()} elements differ"
    routed = torch.from_numpy(idx >= 0).to("cuda:0")
    assert torch.equal(got[~routed], start[~routed])          # rows without a delta stay as they were
    return got


def test_static_plan_entry_matches_the_workspace_entry_twice_in_a_row():
    lib = _ffi.lib()
    assert lib.triteia_hip_sbmm_routed_static_max_bytes() == 256 * 1024
    # both batches are routed through a plan (more than 256 tokens / more than 64 deltas): the buffer is in use
    print("static plan: 700 tokens over 40 deltas of 512 x 512", flush=True)
    run_both(lib, 700, 40, 512, 512, 501, accumulate=0)
    print("static plan: 300 tokens over 70 deltas of 512 x 384, accumulating", flush=True)
    run_both(lib, 300, 70, 512, 384, 502, accumulate=1)
    # a small batch routes inside the multiply kernel and leaves the buffer alone: still the same bits
    run_both(lib, 48, 8, 256, 256, 503, accumulate=0)


def test_static_plan_entry_rejects_what_does_not_fit():
    lib = _ffi.lib()
    null = ctypes.c_void_p(0)
    assert lib.triteia_hip_sbmm_routed_workspace_bytes(8192, 1024) <= 256 * 1024
    rc = lib.triteia_hip_sbmm_2_4_routed_static(null, null, null, null, null, null, 0, 64, 4096, 65536, 4096, 0, 0, null)
    assert rc == _ffi.ERR_KERN_SHAPE and "scratch" in _ffi.last_error()
