#!/usr/bin/env python3
"""Benchmark of the multi-model low-precision GEMM path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg0..cfg4|cfg3split] [--tokens T]

A step is one pass of the hot path over one batch of synthetic input that is already
resident in HBM: for the default workload (indexed sbmm, 64 tokens routed over 16 deltas of
4096x4096) one call of `triteia_hip_sbmm_2_4_routed` (routing kernel + grouped sparse-MFMA
kernel).  Successive steps rotate over enough distinct copies of the packed deltas that the
weights come from HBM, not from the 256 MB Infinity Cache.

Prints ONE JSON line.  `value` is dense-equivalent TFLOP/s (2 * routed_tokens * k * m per
step, the reference's convention, meta/benchmarks/bench_sbmm.py:17) over the timed region;
`roofline` scores the dominant kernel against HBM bandwidth (or the sparse-fp16 matrix-core peak,
whichever bounds the workload) with its duration measured live by HIP events; `sweep` holds the
same two measurements for the metric's grid (tokens x deltas at the 7B shapes: the reference's
meta/benchmarks/bench_sbmm.py:117-140 and benchmarks/bench_ldmm.py:97-123 sweep the same axes);
`cpu_baseline` is the reference's CPU-expressible path (dequantise with the package's torch codec,
then torch matmul of the rows routed to each delta) timed on all host cores on a bounded sample.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_SPARSE_F16_TFLOPS = 5000.0  # 2:4 sparse fp16 (dense fp16 2.5 PFLOP/s), dense-equivalent FLOPs


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=200)
    p.add_argument("--warmup", type=int, default=20)
    p.add_argument("--workload", default="cfg2", choices=["cfg0", "cfg1", "cfg2", "cfg3", "cfg3split", "cfg4"])
    p.add_argument("--tokens", type=int, default=None, help="override the token count (cfg0/cfg2/cfg3/cfg4)")
    p.add_argument("--deltas", type=int, default=None, help="override the number of resident deltas (cfg4)")
    p.add_argument("--shape", default=None, help="K,M: override the weight shape (cfg0)")
    p.add_argument("--copies", type=int, default=0, help="distinct weight copies to rotate over (0 = auto)")
    p.add_argument("--no-graph", action="store_true", help="time eager launches instead of one captured HIP graph")
    p.add_argument("--no-cpu-baseline", action="store_true")
    p.add_argument("--no-sweep", action="store_true", help="skip the tokens x deltas sweep (the `sweep` array)")
    p.add_argument("--warm-cache", action="store_true", help="do not rotate weight copies (Infinity-Cache-warm number)")
    p.add_argument("--calibrate-copy", action="store_true",
                   help="also run one plain 256 MiB device copy (a known-size reference for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE)")
    return p.parse_args()


class Problem:
    """Device tensors + bound C-ABI calls for one workload."""

    def __init__(self, wl, copies, torch, ffi, weights=None, rotations=1):
        """`weights`: packed deltas to use instead of drawing `copies` sets of them (several problems on one resident
        set).  `rotations` (routed sbmm only): step i routes with every index shifted by ((i // copies) % rotations) *
        (deltas // rotations), modulo the number of deltas -- the same number of distinct deltas and tokens per delta, other
        deltas: a thin batch on a large resident set then reads cold weights at every step without further copies."""
        from triteia_amd import workloads as W
        self.wl, self.torch, self.ffi = wl, torch, ffi
        dev = "cuda:0"
        self.dev = dev
        self.lib = ffi.lib()
        self.weights = weights if weights is not None else [
            W.random_packed_deltas(wl.n_deltas, wl.k, wl.m, wl.seed + 7919 * c, dev) for c in range(copies)]
        self.copies = len(self.weights)
        self.x = W.random_activations(wl.tokens, wl.k, wl.seed + 1, dev)
        self.out = torch.zeros((wl.tokens, wl.m), dtype=torch.float16, device=dev)
        self.idx = torch.from_numpy(wl.indices).to(dev) if wl.indices is not None else None
        nbytes = self.lib.triteia_hip_sbmm_routed_workspace_bytes(wl.tokens, wl.n_deltas)
        self.ws = torch.zeros((nbytes + 3) // 4, dtype=torch.int32, device=dev)
        self.ws_bytes = self.ws.numel() * 4
        self.rotations = rotations if (wl.op == "sbmm" and wl.indices is not None and not wl.index_offset) else 1
        self.idx_rot, self.ws_rot = [self.idx], [self.ws]
        for r in range(1, self.rotations):
            shift = r * max(1, wl.n_deltas // self.rotations)
            rot = np.where(wl.indices >= 0, (wl.indices + shift) % wl.n_deltas, wl.indices).astype(np.int32)
            self.idx_rot.append(torch.from_numpy(rot).to(dev))
            self.ws_rot.append(torch.zeros_like(self.ws))
        self.lock_ws = torch.zeros(max(wl.m, 16) * max(1, wl.n_deltas), dtype=torch.int32, device=dev)
        # matmul / bmm launches of few workgroups split K across workgroups through a scratch buffer of the caller's
        groups, per_group = (1, wl.tokens) if wl.op == "matmul" else (wl.n_deltas, max(1, wl.tokens // max(1, wl.n_deltas)))
        nb = self.lib.triteia_hip_bmm_scratch_bytes(wl.m, groups, per_group, wl.k) if wl.op in ("matmul", "bmm") else 0
        self.scratch = torch.empty(max(nb, 16), dtype=torch.uint8, device=dev)
        self.scratch_bytes = nb
        if wl.op == "ldmm":
            g = torch.Generator(device=dev).manual_seed(wl.seed + 3)
            self.base = [(torch.randn((wl.m, wl.k), generator=g, device=dev) * 0.02).half() for _ in range(copies)]
            self.lora_a = (torch.randn((wl.n_lora, wl.k, wl.lora_rank), generator=g, device=dev) * 0.01).half()
            self.lora_b = (torch.randn((wl.n_lora, wl.lora_rank, wl.m), generator=g, device=dev) * 0.01).half()
            self.v = torch.zeros((wl.tokens, wl.lora_rank), dtype=torch.float16, device=dev)
            self.side = torch.cuda.Stream(device=dev)      # default priority
            if wl.index_offset:
                nb = self.lib.triteia_hip_sbmm_routed_workspace_bytes(wl.tokens, wl.n_lora)
                self.ws_lora = torch.zeros((nb + 3) // 4, dtype=torch.int32, device=dev)

    def _chk(self, rc):
        if rc != 0:
            raise RuntimeError(f"triteia_hip call failed ({rc}): {self.ffi.last_error()}")

    def stream(self):
        return ctypes.c_void_p(self.torch.cuda.current_stream().cuda_stream)

    def plan(self):
        wl, P = self.wl, self.ffi.ptr
        for idx, ws in zip(self.idx_rot, self.ws_rot):
            self._chk(self.lib.triteia_hip_route_plan(P(idx), wl.index_offset, wl.n_deltas, wl.tokens, P(ws), self.ws_bytes, 0,
                                                      self.stream()))

    def plan_lora(self):
        """Split index space: the LoRA tokens (indices below index_offset) get a plan of their own."""
        wl, P = self.wl, self.ffi.ptr
        self._chk(self.lib.triteia_hip_route_plan(P(self.idx), 0, wl.n_lora, wl.tokens, P(self.ws_lora), self.ws_lora.numel() * 4, 0,
                                                  self.stream()))

    def delta_kernel(self, i, accumulate=0):
        """Only the dominant kernel (on an existing plan for sbmm / ldmm)."""
        wl, P = self.wl, self.ffi.ptr
        q, me, s = self.weights[i % self.copies]
        st = self.stream()
        if wl.op == "matmul" and self.scratch_bytes:
            self._chk(self.lib.triteia_hip_bmm_2_4_tokens_scratch(P(self.x), P(q), P(me), P(self.out), P(s), wl.m, 1, wl.tokens, wl.k,
                                                                  P(self.scratch), self.scratch_bytes, 0, st))
        elif wl.op == "matmul":
            self._chk(self.lib.triteia_hip_mul_2_4(P(self.x), P(q), P(me), P(self.out), P(s), wl.m, wl.tokens, wl.k, P(self.lock_ws),
                                                    -1, 0, st, -1, -1, -1, 16))
        elif wl.op == "bmm" and self.scratch_bytes:
            self._chk(self.lib.triteia_hip_bmm_2_4_tokens_scratch(P(self.x), P(q), P(me), P(self.out), P(s), wl.m, wl.n_deltas, 1, wl.k,
                                                                  P(self.scratch), self.scratch_bytes, 0, st))
        elif wl.op == "bmm":
            self._chk(self.lib.triteia_hip_bmm_2_4(P(self.x), P(q), P(me), P(self.out), P(s), wl.m, wl.n_deltas, wl.k, P(self.lock_ws),
                                                    -1, 0, st, -1, -1, -1, 16))
        else:
            ws = self.ws_rot[(i // self.copies) % self.rotations]
            self._chk(self.lib.triteia_hip_sbmm_2_4_planned(P(self.x), P(q), P(me), P(self.out), P(s), P(ws), wl.n_deltas, wl.m,
                                                            wl.tokens, wl.k, accumulate, 0, st))

    def delta_routed(self, i):
        """Split index space: the routed delta multiply, added in place (indices below index_offset are not its rows)."""
        wl, P = self.wl, self.ffi.ptr
        q, me, s = self.weights[i % self.copies]
        self._chk(self.lib.triteia_hip_sbmm_2_4_routed(P(self.x), P(q), P(me), P(self.out), P(s), P(self.idx), wl.index_offset,
                                                       wl.n_deltas, wl.m, wl.tokens, wl.k, P(self.ws), self.ws_bytes, 1, 0,
                                                       self.stream()))

    def step(self, i):
        """The whole hot path for one batch."""
        wl, P, torch = self.wl, self.ffi.ptr, self.torch
        if wl.op in ("matmul", "bmm"):
            self.delta_kernel(i)
        elif wl.op == "sbmm":
            q, me, s = self.weights[i % self.copies]
            r = (i // self.copies) % self.rotations
            self._chk(self.lib.triteia_hip_sbmm_2_4_routed(P(self.x), P(q), P(me), P(self.out), P(s), P(self.idx_rot[r]), 0, wl.n_deltas,
                                                           wl.m, wl.tokens, wl.k, P(self.ws_rot[r]), self.ws_bytes, 0, 0, self.stream()))
        elif wl.index_offset:
            # ldmm on a split index space, as triteia_amd.python.ops.ldmm runs it: LoRA plan, zero and shrink beside
            # the base GEMM; then the expand (LoRA rows) beside the routed delta multiply (delta rows)
            r = wl.lora_rank
            cur, side = torch.cuda.current_stream(), self.side
            q, me, s = self.weights[i % self.copies]
            side.wait_stream(cur)
            # (the GEMM is enqueued first: recorded into a graph the other way round, the step measured 30 us longer)
            torch.matmul(self.x, self.base[i % self.copies].t(), out=self.out)
            with torch.cuda.stream(side):
                self.plan_lora()
                self._chk(self.lib.triteia_hip_sgmv_routed(P(self.v), r, P(self.x), wl.k, P(self.lora_a), wl.k * r, wl.n_lora,
                                                           wl.k, r, 1.0, P(self.ws_lora), wl.tokens, 0, 0, self.stream()))
            side.wait_stream(cur)
            with torch.cuda.stream(side):
                self._chk(self.lib.triteia_hip_sgmv_routed(P(self.out), wl.m, P(self.v), r, P(self.lora_b), r * wl.m, wl.n_lora, r,
                                                           wl.m, 1.0, P(self.ws_lora), wl.tokens, 1, 0, self.stream()))
            self.delta_routed(i)
            cur.wait_stream(side)
        else:  # ldmm: dense base GEMM (library) + routed LoRA (SGMV) + routed delta, one routing plan for both
            r = wl.lora_rank
            cur = torch.cuda.current_stream()
            side = self.side if os.environ.get("BENCH_LDMM_OVERLAP", "1") == "1" else None
            if side is not None:
                # routing and the LoRA shrink need only x: they run beside the base GEMM, which leaves CUs idle
                side.wait_stream(cur)
                # (the GEMM is enqueued first: recorded into a graph the other way round, the step measured 30 us longer)
                torch.matmul(self.x, self.base[i % self.copies].t(), out=self.out)
                with torch.cuda.stream(side):
                    self.plan()
                    self._chk(self.lib.triteia_hip_sgmv_routed(P(self.v), r, P(self.x), wl.k, P(self.lora_a), wl.k * r, wl.n_lora,
                                                               wl.k, r, 1.0, P(self.ws), wl.tokens, 0, 0, self.stream()))
                cur.wait_stream(side)
            else:
                torch.matmul(self.x, self.base[i % self.copies].t(), out=self.out)
                self.plan()
                self._chk(self.lib.triteia_hip_sgmv_routed(P(self.v), r, P(self.x), wl.k, P(self.lora_a), wl.k * r, wl.n_lora, wl.k, r,
                                                           1.0, P(self.ws), wl.tokens, 0, 0, self.stream()))
            st = self.stream()
            self._chk(self.lib.triteia_hip_sgmv_routed(P(self.out), wl.m, P(self.v), r, P(self.lora_b), r * wl.m, wl.n_lora, r, wl.m,
                                                       1.0, P(self.ws), wl.tokens, 1, 0, st))
            self.delta_kernel(i, accumulate=1)


def cpu_baseline(wl, torch, budget_s=20.0):
    """The reference's CPU-expressible path on the host cores (its tests' own recipe: dequantise to a dense fp16
    matrix, generator.py:40,52, then matmul per delta, sbmm.py:7-23): the package's vectorised torch codec
    `unpack_2_4` and torch.matmul of the rows actually routed to each delta, on every host core, on as many of the
    workload's deltas as fit the time budget (the rate is per delta and carries over to all of them)."""
    from triteia_amd import workloads as W
    from triteia_amd.python.ops.utils.sparsity import unpack_2_4
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    didx = wl.delta_indices()
    used = sorted(set(int(i) for i in didx if i >= 0)) if didx is not None else list(range(wl.n_deltas))
    per_group = max(1, wl.tokens // max(1, wl.n_deltas))
    x = W.random_activations(wl.tokens, wl.k, wl.seed + 1, "cpu")
    t_deq = t_mm = 0.0
    flops = 0.0
    done = 0
    t_begin = time.perf_counter()
    for d in used:
        q, me, s = W.random_packed_deltas(1, wl.k, wl.m, wl.seed + 31 * d, "cpu")
        if didx is not None:
            rows = x[torch.from_numpy(np.nonzero(didx == d)[0])]
        elif wl.op == "bmm":
            rows = x[d * per_group:(d + 1) * per_group]
        else:
            rows = x
        t0 = time.perf_counter()
        dense = unpack_2_4(q[0], me[0], s[0], dtype=torch.float32)
        t1 = time.perf_counter()
        y = rows.float() @ dense
        t2 = time.perf_counter()
        del y, dense
        t_deq += t1 - t0
        t_mm += t2 - t1
        flops += 2.0 * rows.shape[0] * wl.k * wl.m
        done += 1
        if time.perf_counter() - t_begin > budget_s:
            break
    total = t_deq + t_mm
    return {
        "value": round(flops / total / 1e12, 6), "unit": "TFLOP/s", "cores": cores, "kind": "port",
        "sample": f"{done} of {len(used)} routed deltas of the workload: torch dequantise {t_deq:.2f}s + torch fp32 matmul of the "
                  f"rows routed to each delta {t_mm:.3f}s, both on {cores} threads; the rate is per delta and carries over to all of them",
        "dequant_s": round(t_deq, 3), "matmul_s": round(t_mm, 4),
    }


def kernel_name(wl, lib, in_kernel):
    """The kernel that takes most of the workload's rows, as the library itself reports it."""
    if wl.op in ("matmul", "bmm"):
        groups, per_group = (1, wl.tokens) if wl.op == "matmul" else (wl.n_deltas, max(1, wl.tokens // max(1, wl.n_deltas)))
        code = lib.triteia_hip_uniform_kernel(wl.m, groups, per_group, wl.k, 1)
        if code >= 1000:
            return f"sparse24_grouped_kernel (K split over {code - 1000} workgroups) + splitk_reduce_kernel"
        return {0: "sparse24_grouped_kernel", 16: "sparse24_share16_kernel", 32: "sparse24_wide_kernel<32 tokens>", 33: "sparse24_wide_kernel<32 tokens, 8 wavefronts>",
                64: "sparse24_wide_kernel<64 tokens>", 65: "sparse24_wide_kernel<64 tokens, 8 wavefronts>",
                256: "sparse24_tile256_kernel"}.get(code, f"kernel code {code}")
    if in_kernel:
        if lib.triteia_hip_routed_in_kernel(wl.tokens, wl.n_deltas, wl.m, wl.k) == 2:
            return "sparse24_share16_kernel (routes in-kernel)"
        return "sparse24_grouped_kernel (routes in-kernel)"
    if wl.index_offset:
        return "sparse24_grouped_kernel"
    tk = lib.triteia_hip_planned_tile_kernel(wl.tokens, wl.n_deltas, wl.m, wl.k)
    if tk:
        return f"sparse24_wide_kernel<{tk}-token plan tiles>"
    hot = wl.tokens >= 256 and wl.tokens >= 8 * min(wl.tokens, wl.n_deltas)
    return "sparse24_grouped_kernel" + (" + sparse24_wide_kernel<64-token tiles of hot deltas>" if hot else "")


def measure(prob, wl, torch, ffi, steps, warmup, use_graph=True, reps=None):
    """One workload: the step timed over `steps` steps (one captured HIP graph, or eager), and its dominant kernel
    timed on its own by HIP events on the launch stream."""
    lib = ffi.lib()
    for i in range(warmup):
        prob.step(i)
    torch.cuda.synchronize()
    if use_graph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                for i in range(steps):
                    prob.step(warmup + i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        graph.replay()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        del graph
    else:
        t0 = time.perf_counter()
        for i in range(steps):
            prob.step(warmup + i)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
    step_s = elapsed / steps

    # ---- dominant kernel alone: batches of back-to-back launches between two events
    # (a batch that the routed entry point routes inside the multiply kernel is one launch: the whole step; otherwise
    # the multiply runs on a routing plan made beforehand)
    in_kernel = wl.op == "sbmm" and bool(lib.triteia_hip_routed_in_kernel(wl.tokens, wl.n_deltas, wl.m, wl.k))
    kernel_call = prob.step if in_kernel else (prob.delta_routed if wl.index_offset else prob.delta_kernel)
    if wl.indices is not None and not in_kernel:
        prob.plan()
    for i in range(5):
        kernel_call(i)
    torch.cuda.synchronize()
    # one timed batch walks over more distinct weights than the 256 MB Infinity Cache holds (as far as the problem has
    # them), so that the kernel's duration is a cold one like the step's
    touched = max(1, wl.distinct_deltas() * wl.delta_bytes)
    batch = int(max(10, min(prob.copies * prob.rotations, np.ceil(512 * 2 ** 20 / touched))))
    reps = reps or max(3, min(20, steps // 10))
    durs = []
    kgraph = None
    if use_graph:
        # the batch is replayed from a captured graph: launched one by one from Python, kernels shorter than the host's
        # launch interval (about 9 us per call through ctypes) would be timed at that interval
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        kgraph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(kgraph, stream=side):
                for i in range(batch):
                    kernel_call(i)
        torch.cuda.synchronize()
        kgraph.replay()
        torch.cuda.synchronize()
    for r in range(reps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        if kgraph is not None:
            kgraph.replay()
        else:
            for i in range(batch):
                kernel_call(r * batch + i)
        e1.record()
        e1.synchronize()
        durs.append(e0.elapsed_time(e1) / batch * 1e-3)
    del kgraph
    kdur = float(np.median(durs))
    abytes = wl.delta_algorithmic_bytes()
    achieved = abytes / kdur / 1e9
    kflops = wl.delta_flops() / kdur / 1e12
    name = kernel_name(wl, lib, in_kernel)
    hbm_time, mfma_time = abytes / (HBM_PEAK_GBS * 1e9), wl.delta_flops() / (MFMA_SPARSE_F16_TFLOPS * 1e12)
    if mfma_time > hbm_time:
        # many tokens per delta: the matrix cores bound the kernel.  The 2:4-sparse instruction executes
        # half of the dense-equivalent multiply-adds, priced against the dense fp16 peak (same fraction
        # as dense-equivalent work against twice that peak).
        roofline = {
            "bound": "mfma", "achieved": round(kflops / 2, 1), "peak": MFMA_SPARSE_F16_TFLOPS / 2, "unit": "TFLOP/s",
            "frac": round(kflops / MFMA_SPARSE_F16_TFLOPS, 4), "traffic": None, "kernel": name, "kernel_us": round(kdur * 1e6, 2),
            "algorithmic_flops_dense_equivalent": wl.delta_flops(), "kernel_tflops_dense_equivalent": round(kflops, 2),
            "hbm_frac": round(achieved / HBM_PEAK_GBS, 4),
        }
    else:
        roofline = {
            "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": None, "kernel": name, "kernel_us": round(kdur * 1e6, 2), "algorithmic_bytes": abytes,
            "kernel_tflops": round(kflops, 2), "mfma_frac": round(kflops / MFMA_SPARSE_F16_TFLOPS, 4),
        }
    return step_s, roofline


def copies_for(wl, warm=False, asked=0):
    """Distinct weight copies to rotate over: enough bytes to out-run the 256 MB Infinity Cache, within ~12 GB."""
    if warm:
        return 1
    if asked > 0:
        return asked
    touched = wl.distinct_deltas() * wl.delta_bytes
    return max(1, min(64, int(np.ceil(1.5 * 2 ** 30 / max(touched, 1))), int(12 * 2 ** 30 // (wl.n_deltas * wl.delta_bytes)) or 1))


def rotations_for(wl, copies):
    """Index rotations (see Problem) that bring a routed sbmm's distinct weights per cycle of steps to about 1.5 GB where
    the copies alone do not."""
    if wl.op != "sbmm" or wl.indices is None:
        return 1
    touched = max(1, wl.distinct_deltas() * wl.delta_bytes * copies)
    return int(max(1, min(16, wl.n_deltas // max(1, wl.distinct_deltas()), np.ceil(1.5 * 2 ** 30 / touched))))


def sweep_points():
    """The metric's grid: routed sbmm over 16 deltas of 4096 x 4096 and over 32 deltas of 4096 x 11008 against the token
    count, the single-matrix product at three token counts, and the ldmm step of configuration 3."""
    from triteia_amd import workloads as W
    pts = []
    for t in (1, 16, 64, 256, 1024, 4096):
        pts.append((f"sbmm 16 x 4096x4096, {t} tokens", W.config("cfg2", t)))
    for t in (1, 16, 64, 256, 1024, 4096):
        wl = W.config("cfg3", t)
        wl.op, wl.name = "sbmm", f"sbmm 32 x 4096x11008, {t} tokens Zipf(1.5) 10% -1"
        pts.append((f"sbmm 32 x 4096x11008, {t} tokens", wl))
    for t in (16, 1024, 4096):
        pts.append((f"matmul 4096x4096, {t} tokens", W.config("cfg0", t)))
    pts.append(("bmm 8 x 4096x4096, 1 token each (cfg1)", W.config("cfg1")))
    pts.append(("ldmm 4096x11008, 256 tokens (cfg3)", W.config("cfg3")))
    return pts


def cfg4_points():
    """Configuration 4 (Llama-2-70B MLP shape, 64 resident deltas of 8192 x 28672 = 5.64 GB) at its token counts."""
    from triteia_amd import workloads as W
    return [(f"sbmm 64 x 8192x28672, {t} tokens Zipf(1.2) (cfg4)", W.config("cfg4", t)) for t in (1, 16, 64, 256, 1024)]


def run_sweep(torch, ffi):
    from triteia_amd import workloads as W
    out = []
    points = [(label, wl, None) for label, wl in sweep_points()]
    # the 5.64 GB of configuration 4 are drawn once and serve its five token counts
    c4 = cfg4_points()
    shared = [W.random_packed_deltas(c4[0][1].n_deltas, c4[0][1].k, c4[0][1].m, c4[0][1].seed, "cuda:0")]
    points += [(label, wl, shared) for label, wl in c4]
    for label, wl, weights in points:
        copies = 1 if weights is not None else copies_for(wl)
        prob = Problem(wl, copies, torch, ffi, weights=weights, rotations=rotations_for(wl, copies))
        torch.cuda.synchronize()
        # a few milliseconds of steps per point
        est_us = max(10.0, wl.delta_flops() / 1.5e15 * 1e6, wl.delta_algorithmic_bytes() / 4e12 * 1e6)
        steps = int(min(50, max(10, 4000.0 / est_us)))
        step_s, roof = measure(prob, wl, torch, ffi, steps, 3, use_graph=True, reps=5)
        flops = wl.delta_flops()
        if wl.op == "ldmm":
            flops += 2.0 * wl.tokens * wl.k * wl.m + 2.0 * wl.lora_tokens() * wl.lora_rank * (wl.k + wl.m)
        out.append({"workload": label, "tokens": wl.tokens, "tokens_routed": wl.routed_tokens(), "deltas_used": wl.distinct_deltas(),
                    "ms_per_step": round(step_s * 1e3, 5), "tflops": round(flops / step_s / 1e12, 2), "kernel": roof["kernel"],
                    "kernel_us": roof["kernel_us"], "bound": roof["bound"], "frac": roof["frac"]})
        del prob
        torch.cuda.empty_cache()
    del shared, points
    torch.cuda.empty_cache()
    return out


def measure_lora(torch, ffi, tokens=256, adapters=32, k=4096, m=11008, rank=16, calls=20):
    """The LoRA companions at configuration 3's shape (rank-16 adapters on 4096 x 11008, the routing of cfg3): BGMV
    (one adapter look-up per token) and routed SGMV (tokens grouped by a routing plan), each as shrink + expand, timed
    as `calls` pairs in one captured HIP graph.  Bytes: every distinct adapter once, activations, the rank-r
    intermediate written and read, the output read and written."""
    from triteia_amd import workloads as W
    from triteia_amd.python.capi import add_lora_bgmv, route_plan, sgmv_routed
    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(77)
    x = W.random_activations(tokens, k, 78, dev)
    A = (torch.randn((adapters, k, rank), generator=g, device=dev) * 0.01).half()
    B = (torch.randn((adapters, rank, m), generator=g, device=dev) * 0.01).half()
    A_t = A.transpose(1, 2).contiguous().unsqueeze(1)      # BGMV's layout: [n, layers, out, in]
    B_t = B.transpose(1, 2).contiguous().unsqueeze(1)
    idx_np = W.zipf_indices(tokens, adapters, 1.5, 1003, 0.10)
    idx32 = torch.from_numpy(idx_np).to(dev)
    idx64 = idx32.to(torch.long)
    y = torch.zeros((tokens, m), dtype=torch.float16, device=dev)
    v = torch.zeros((tokens, rank), dtype=torch.float16, device=dev)
    plan = route_plan(idx32, adapters)
    used = len(set(int(i) for i in idx_np if i >= 0))
    routed = int((idx_np >= 0).sum())
    nbytes = used * (k * rank + rank * m) * 2 + routed * (k * 2 + 4 * rank + 4 * m)

    def bgmv():
        add_lora_bgmv(y, x, A_t, B_t, idx64, 0, 1.0)

    def sgmv():
        sgmv_routed(v, x, A, plan, accumulate=False)
        sgmv_routed(y, v, B, plan)

    out = []
    for name, fn, kernels in (("lora_bgmv", bgmv, "bgmv_shrink_kernel + bgmv_expand_kernel"),
                              ("lora_sgmv_routed", sgmv, "sgmv_shrink_kernel + sgmv_expand_vec_kernel")):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                for _ in range(calls):
                    fn()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        graph.replay()
        torch.cuda.synchronize()
        us = (time.perf_counter() - t0) / calls * 1e6
        del graph
        out.append({"workload": f"{name} rank {rank}, {adapters} adapters on {k}x{m}, {tokens} tokens Zipf(1.5)", "tokens": tokens,
                    "tokens_routed": routed, "deltas_used": used, "ms_per_step": round(us * 1e-3, 5),
                    "tflops": round(2.0 * routed * rank * (k + m) / (us * 1e-6) / 1e12, 2), "kernel": kernels,
                    "kernel_us": round(us, 2), "bound": "hbm", "frac": round(nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)})
    return out


def host_call_us(prob, wl, torch, n=300):
    """Host time of one `ops.sbmm_4bit_2_4_native` call (Python mirror -> ctypes -> C ABI), launches left to queue up."""
    if wl.op != "sbmm":
        return None
    from triteia_amd.python import ops
    q, me, s = prob.weights[0]
    for _ in range(20):
        ops.sbmm_4bit_2_4_native(q, prob.x, me, s, prob.idx)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(n):
        ops.sbmm_4bit_2_4_native(q, prob.x, me, s, prob.idx)
    host = time.perf_counter() - t0
    torch.cuda.synchronize()
    return round(host / n * 1e6, 2)


def main():
    a = parse()
    if a.gpus != 1:
        print("bench.py: this build runs on ONE GPU (no collectives in this path); use --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    from triteia_amd import workloads as W
    from triteia_amd.python.capi import _ffi as ffi

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    from triteia_amd import build as _build
    _build.ensure_built(verbose=False)   # loads what is built in the tree; compiles only if there is nothing
    ffi.lib()   # fails loudly if the HIP library is missing

    shape = tuple(int(v) for v in a.shape.split(",")) if a.shape else None
    if shape is not None and (a.workload != "cfg0" or len(shape) != 2 or shape[0] % 64 or shape[1] % 128):
        print("bench.py: --shape K,M needs --workload cfg0, K % 64 == 0 and M % 128 == 0", file=sys.stderr)
        sys.exit(2)
    wl = W.config(a.workload, a.tokens, shape)
    if a.deltas is not None and a.workload == "cfg4":
        wl.n_deltas = a.deltas
        wl.indices = W.zipf_indices(wl.tokens, wl.n_deltas, 1.2, wl.seed)
    copies = copies_for(wl, a.warm_cache, a.copies)
    prob = Problem(wl, copies, torch, ffi, rotations=1 if a.warm_cache else rotations_for(wl, copies))
    torch.cuda.synchronize()
    if a.calibrate_copy:
        src = torch.empty(256 * 2 ** 20, dtype=torch.uint8, device="cuda:0").random_(0, 255)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)          # one elementwise copy kernel: reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    # ---- whole-job timing (W warm-up steps, then exactly K steps) and the dominant kernel on its own
    use_graph = not a.no_graph
    step_s, roofline = measure(prob, wl, torch, ffi, a.steps, a.warmup, use_graph)
    # eager launches too (shows the host launch cost next to the graph number)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(a.steps):
        prob.step(a.warmup + i)
    torch.cuda.synchronize()
    eager = time.perf_counter() - t0

    ms_per_step = step_s * 1e3
    flops = wl.delta_flops()
    if wl.op == "ldmm":
        flops += 2.0 * wl.tokens * wl.k * wl.m + 2.0 * wl.lora_tokens() * wl.lora_rank * (wl.k + wl.m)
    value = flops / step_s / 1e12
    abytes = wl.delta_algorithmic_bytes()

    # HBM bytes per launch of the dominant kernel, from the committed rocprofv3 --pmc summary of this workload (two
    # counter runs scaled by a plain copy of known size); the file names the commit it was measured at
    tpath = os.path.join(ROOT, "profiles", f"traffic_{a.workload}.json")
    if os.path.exists(tpath) and a.tokens is None and a.deltas is None and a.shape is None:
        try:
            tj = json.load(open(tpath))
            roofline["traffic"] = tj.get("hbm_bytes_per_launch")
            roofline["traffic_measured_at"] = tj.get("commit")
        except Exception:
            pass

    # what this GPU delivers on a plain device-to-device copy (512 MiB read + 512 MiB written per launch), next to
    # the nominal peak the fractions above are priced against
    src = torch.empty(512 * 2 ** 20, dtype=torch.uint8, device="cuda:0").random_(0, 255)
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(10):
        dst.copy_(src)
    e1.record()
    e1.synchronize()
    roofline["device_copy_gbs"] = round(2 * src.numel() * 10 / (e0.elapsed_time(e1) * 1e-3) / 1e9, 1)
    del src, dst

    res = {
        "metric": "sbmm/ldmm dense-equivalent TFLOP/s at Llama-2-7B shapes (with % of HBM roofline)",
        "value": round(value, 3), "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 (int4 2:4 weights, fp32 accumulate)", "data": "synthetic",
        "config": {"workload": wl.name, "op": wl.op, "k": wl.k, "m": wl.m, "deltas_resident": wl.n_deltas, "deltas_used": wl.distinct_deltas(),
                   "tokens": wl.tokens, "tokens_routed": wl.routed_tokens(), "weight_copies_rotated": copies,
                   "index_rotations": prob.rotations,
                   "launch": "hip-graph" if use_graph else "eager"},
        "eager_ms_per_step": round(eager / a.steps * 1e3, 5),
        "host_us_per_ops_call": host_call_us(prob, wl, torch),
        "step_gbs": round((abytes + (wl.k * wl.m * 2 if wl.op == "ldmm" else 0)) / step_s / 1e9, 1),
        "roofline": roofline,
    }
    del prob
    torch.cuda.empty_cache()
    if not a.no_sweep and a.workload == "cfg2" and a.tokens is None:
        res["sweep"] = run_sweep(torch, ffi) + measure_lora(torch, ffi)
    if not a.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline(wl, torch)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
