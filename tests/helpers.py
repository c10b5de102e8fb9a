"""Shared helpers for the parity tests: seeded workloads as numpy + torch pairs."""
import numpy as np
import torch

from oracle import triteia_oracle as orc


def make_deltas(n, k, m, seed):
    """n packed deltas with the benchmark distribution (values U[-8,7], positions uniform,
    scales U(0.005, 0.02)), packed by the oracle's explicit-position packer."""
    rng = np.random.default_rng(seed)
    pairs = np.array([(0, 1), (0, 2), (0, 3), (1, 2), (1, 3), (2, 3)])
    qws, metas, ss = [], [], []
    for _ in range(n):
        sel = rng.integers(0, 6, size=(m, k // 4))
        lo, hi = pairs[sel, 0], pairs[sel, 1]
        q = rng.integers(-8, 8, size=(m, k // 2))
        s = rng.uniform(0.005, 0.02, size=m).astype(np.float16)
        qw, meta, sc = orc.pack_explicit(q, lo, hi, s)
        qws.append(qw), metas.append(meta), ss.append(sc)
    return np.stack(qws), np.stack(metas), np.stack(ss)


def to_gpu(*arrays, device="cuda:0"):
    return tuple(torch.from_numpy(np.ascontiguousarray(a)).to(device) for a in arrays)


def activations(t, k, seed):
    rng = np.random.default_rng(seed)
    return rng.standard_normal((t, k)).astype(np.float16)


def check_close(got, ref, tol=2e-3, what=""):
    """north-star bound (relative Frobenius error) and the reference tests' own metric."""
    got = got.detach().float().cpu().numpy().astype(np.float64) if isinstance(got, torch.Tensor) else got
    fro = orc.rel_frobenius(got, ref)
    mab = orc.rel_mean_abs(got, ref)
    assert fro <= tol, f"{what}: relative Frobenius error {fro:.3e} > {tol}"
    assert mab <= tol, f"{what}: mean-abs error ratio {mab:.3e} > {tol}"
    return fro


def reload_knobs():
    """The library reads its TRITEIA_HIP_* knobs once; after a change of the environment it is told to read them again."""
    from triteia_amd.python.capi import _ffi
    _ffi.reload_env()


def setknob(monkeypatch, name, value):
    """Set one TRITEIA_HIP_* knob for the rest of the test (conftest restores the library's view afterwards)."""
    monkeypatch.setenv(name, str(value))
    reload_knobs()


def delknob(monkeypatch, name):
    monkeypatch.delenv(name, raising=False)
    reload_knobs()
