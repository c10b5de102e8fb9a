"""fp16 x (int4, 2:4) GEMM entry points with the reference's signatures.

Mirrors triteia/python/capi/marlin.py:4-97 (argument names, order, defaults)
and the checks / error texts of triteia/csrc/ops/ops.cpp:88-116,240-327.
"""
import torch

from . import _ffi


def _gemm_checks(A, B, meta, C, s):
    _ffi.require_gpu(A=A, B=B, meta=meta, C=C, s=s)
    _ffi.require_dtype(A, torch.float16, "A")
    _ffi.require_dtype(C, torch.float16, "C")
    _ffi.require_dtype(s, torch.float16, "s")
    _ffi.require_dtype(B, torch.int32, "B")
    _ffi.require_dtype(meta, torch.int16, "meta")


def _raise(err, prob_m, prob_n, prob_k, thread_k, thread_m, groupsize, knob="thread_m"):
    if err == 0:
        return
    if err == _ffi.ERR_PROB_SHAPE:
        raise RuntimeError(f"Problem (m={prob_m}, n={prob_n}, k={prob_k}) not compatible with "
                           f"thread_k={thread_k}, {knob}={thread_m}. [{_ffi.last_error()}]")
    if err == _ffi.ERR_KERN_SHAPE:
        raise RuntimeError(f"No kernel implementation for thread_k={thread_k}, {knob}={thread_m}, "
                           f"groupsize={groupsize}. [{_ffi.last_error()}]")
    raise RuntimeError(f"triteia_hip error {err}: {_ffi.last_error()}")


def _check_packed(B, meta, s, prob_m, prob_k, lead=()):
    if tuple(B.shape) != (*lead, prob_k // 32, 2 * prob_m):
        raise RuntimeError(f"B has shape {tuple(B.shape)}, expected {(*lead, prob_k // 32, 2 * prob_m)}")
    if tuple(meta.shape) != (*lead, prob_m, prob_k // 16):
        raise RuntimeError(f"meta has shape {tuple(meta.shape)}, expected {(*lead, prob_m, prob_k // 16)}")
    if s.shape[-1] != prob_m:
        raise RuntimeError(f"s has {s.shape[-1]} columns, expected {prob_m}")


def mul_2_4(A, B, meta, C, s, workspace, thread_k=-1, thread_m=-1, sms=-1, max_par=16):
    """C = A @ W for one packed weight.  A [n, k] fp16, B [k/32, 2m] int32,
    meta [m, k/16] int16, C [n, m] fp16, s [1, m] fp16 (or [k/128, m]: scales per group of 128
    dense k in the reference's stored order, `sparsity.pack_group_scales`), workspace >= m/128*max_par zeros
    (kept for signature parity; never touched)."""
    _gemm_checks(A, B, meta, C, s)
    if A.dim() != 2 or C.dim() != 2:
        raise RuntimeError("A and C must be 2-D")
    prob_n, prob_k = A.shape
    prob_m = C.shape[1]
    if C.shape[0] != prob_n:
        raise RuntimeError(f"C has {C.shape[0]} rows, A has {prob_n}")
    groupsize = -1 if s.shape[0] == 1 else prob_k // 2 // s.shape[0]
    if groupsize != -1 and groupsize * s.shape[0] != prob_k // 2:
        raise RuntimeError(f"k={prob_k} not compatible with {s.shape[0]} groups.")
    if workspace.numel() < prob_m // 128 * max_par:
        raise RuntimeError(f"workspace must be of size at least {prob_m // 128 * max_par}.")
    if prob_m % 128 == 0 and prob_k % 64 == 0:
        _check_packed(B, meta, s, prob_m, prob_k)
    lib = _ffi.lib()
    split = lib.triteia_hip_bmm_scratch_bytes(prob_m, 1, prob_n, prob_k) if groupsize == -1 else 0
    if split:
        # a launch of few workgroups: K is split across workgroups through a scratch buffer of this binding's (the
        # reference's lock workspace is too small for partial sums); same entry point as bmm with one matrix
        scratch = _ffi.split_scratch(split, A.device)
        err = lib.triteia_hip_bmm_2_4_tokens_scratch(
            _ffi.ptr(A), _ffi.ptr(B), _ffi.ptr(meta), _ffi.ptr(C), _ffi.ptr(s), prob_m, 1, prob_n, prob_k,
            _ffi.ptr(scratch), scratch.numel(), _ffi.device_index(A), _ffi.stream_of(A))
    else:
        err = lib.triteia_hip_mul_2_4(
            _ffi.ptr(A), _ffi.ptr(B), _ffi.ptr(meta), _ffi.ptr(C), _ffi.ptr(s), prob_m, prob_n, prob_k,
            _ffi.ptr(workspace), groupsize, _ffi.device_index(A), _ffi.stream_of(A), thread_k, thread_m, sms, max_par)
    _raise(err, prob_m, prob_n, prob_k, thread_k, thread_m, groupsize)


def bmm_2_4(A, B, meta, C, s, workspace, thread_k=-1, thread_m=-1, sms=-1, max_par=16):
    """C[b] = A[b] @ W[b].  A [b, t, k], B [b, k/32, 2m], meta [b, m, k/16], C [b, t, m], s [b, 1, m].

    The reference kernel handles t == 1 only; any t is accepted here."""
    _gemm_checks(A, B, meta, C, s)
    if A.dim() != 3 or C.dim() != 3:
        raise RuntimeError("A and C must be 3-D")
    batch, tokens, prob_k = A.shape
    prob_m = C.shape[2]
    if C.shape[0] != batch or C.shape[1] != tokens:
        raise RuntimeError(f"C has shape {tuple(C.shape)}, expected ({batch}, {tokens}, {prob_m})")
    groupsize = -1 if s.shape[1] == 1 else prob_k // s.shape[1]
    if groupsize != -1:
        _raise(_ffi.ERR_KERN_SHAPE, prob_m, batch, prob_k, thread_k, thread_m, groupsize)
    if prob_m % 128 == 0 and prob_k % 64 == 0:
        _check_packed(B, meta, s, prob_m, prob_k, lead=(batch,))
    lib = _ffi.lib()
    split = lib.triteia_hip_bmm_scratch_bytes(prob_m, batch, tokens, prob_k) if prob_m % 128 == 0 and prob_k % 64 == 0 else 0
    if split:
        scratch = _ffi.split_scratch(split, A.device)
        err = lib.triteia_hip_bmm_2_4_tokens_scratch(
            _ffi.ptr(A), _ffi.ptr(B), _ffi.ptr(meta), _ffi.ptr(C), _ffi.ptr(s), prob_m, batch, tokens, prob_k,
            _ffi.ptr(scratch), scratch.numel(), _ffi.device_index(A), _ffi.stream_of(A))
    elif tokens == 1:
        # the reference's own case and argument list (triteia_nm_bmm.cu:760-764)
        if workspace.numel() < prob_m // 128 * max_par:
            raise RuntimeError(f"workspace must be of size at least {prob_m // 128 * max_par}.")
        err = _ffi.lib().triteia_hip_bmm_2_4(
            _ffi.ptr(A), _ffi.ptr(B), _ffi.ptr(meta), _ffi.ptr(C), _ffi.ptr(s), prob_m, batch, prob_k,
            _ffi.ptr(workspace), groupsize, _ffi.device_index(A), _ffi.stream_of(A), thread_k, thread_m, sms, max_par)
    else:
        err = _ffi.lib().triteia_hip_bmm_2_4_tokens(
            _ffi.ptr(A), _ffi.ptr(B), _ffi.ptr(meta), _ffi.ptr(C), _ffi.ptr(s), prob_m, batch, tokens, prob_k,
            _ffi.device_index(A), _ffi.stream_of(A))
    _raise(err, prob_m, batch, prob_k, thread_k, thread_m, groupsize)


def _run_checks(A, B, meta, C, s, indices, starts, counts):
    _gemm_checks(A, B, meta, C, s)
    _ffi.require_gpu(indices=indices, starts=starts, counts=counts)
    for name, t in (("indices", indices), ("starts", starts), ("counts", counts)):
        _ffi.require_dtype(t, torch.int32, name)
    if not (indices.numel() == starts.numel() == counts.numel()):
        raise RuntimeError("indices, starts and counts must have one entry per run")
    if A.dim() != 2 or C.dim() != 2 or B.dim() != 3:
        raise RuntimeError("A and C must be 2-D, B 3-D")


def sbmm_2_4(A, B, meta, C, s, indices, workspace, starts, counts, thread_k=-1, thread_n=-1, sms=-1, max_par=16):
    """Run-list selective bmm: rows starts[r]..+counts[r] of C = same rows of A @ W[indices[r]].

    One launch for all runs; nothing is read back to the host."""
    _run_checks(A, B, meta, C, s, indices, starts, counts)
    prob_n, prob_k = A.shape
    prob_m = C.shape[1]
    groupsize = -1 if s.shape[1] == 1 else prob_k // s.shape[1]
    if prob_m % 128 == 0 and prob_k % 64 == 0 and groupsize == -1:
        _check_packed(B, meta, s, prob_m, prob_k, lead=(B.shape[0],))
    # (the entry point with the reference's exact argument list, triteia_hip_sbmm_2_4, trusts the indices; this
    # binding knows how many matrices B holds and passes it on, so that a stray index is skipped)
    err = _ffi.lib().triteia_hip_sbmm_2_4_bounded(
        _ffi.ptr(A), _ffi.ptr(B), _ffi.ptr(meta), _ffi.ptr(C), _ffi.ptr(s), _ffi.ptr(indices), _ffi.ptr(starts),
        _ffi.ptr(counts), prob_m, prob_n, prob_k, indices.numel(), _ffi.ptr(workspace), groupsize,
        _ffi.device_index(A), _ffi.stream_of(A), thread_k, thread_n, sms, max_par, B.shape[0])
    _raise(err, prob_m, prob_n, prob_k, thread_k, thread_n, groupsize, knob="thread_n")


def sbmm_2_4_multilaunch(A, B, meta, C, s, indices, workspace, starts, counts, thread_k=-1, thread_n=-1, sms=-1,
                         max_par=16):
    """Same result as sbmm_2_4 by one mul_2_4 launch per run, driven from the host
    (the reference's sbmm_forloop, triteia/csrc/ops/ops.cpp:279-293; reads the run
    table back to the host, as the reference does)."""
    _run_checks(A, B, meta, C, s, indices, starts, counts)
    idx, st, ct = indices.tolist(), starts.tolist(), counts.tolist()
    for r, (d, a, n) in enumerate(zip(idx, st, ct)):
        ws = workspace[r] if workspace.dim() > 1 else workspace
        mul_2_4(A[a:a + n], B[d], meta[d], C[a:a + n], s[d], ws, thread_k, thread_n, sms, max_par)


def routed_workspace(n_tokens, n_deltas, device):
    """Scratch for `route_plan` / `sbmm_2_4_routed` (int32 tensor)."""
    nbytes = _ffi.lib().triteia_hip_sbmm_routed_workspace_bytes(int(n_tokens), int(n_deltas))
    return torch.empty((nbytes + 3) // 4, dtype=torch.int32, device=device)


def route_plan(token_indices, n_deltas, index_offset=0, workspace=None):
    """Group tokens by delta on the device; returns the plan workspace."""
    _ffi.require_gpu(token_indices=token_indices)
    _ffi.require_dtype(token_indices, torch.int32, "token_indices")
    n = token_indices.numel()
    if workspace is None:
        workspace = routed_workspace(n, n_deltas, token_indices.device)
    err = _ffi.lib().triteia_hip_route_plan(
        _ffi.ptr(token_indices), int(index_offset), int(n_deltas), n, _ffi.ptr(workspace),
        workspace.numel() * workspace.element_size(), _ffi.device_index(token_indices), _ffi.stream_of(token_indices))
    if err:
        raise RuntimeError(f"triteia_hip error {err}: {_ffi.last_error()}")
    return workspace


def sbmm_2_4_routed(A, B, meta, C, s, token_indices, index_offset=0, accumulate=False, workspace=None):
    """Per-token routed selective bmm (device-side grouping, one weight pass per delta):
    C[t] (+)= A[t] @ W[token_indices[t] - index_offset]; rows whose index falls outside
    [0, n_deltas) are left untouched."""
    _gemm_checks(A, B, meta, C, s)
    _ffi.require_gpu(token_indices=token_indices)
    _ffi.require_dtype(token_indices, torch.int32, "token_indices")
    if A.dim() != 2 or C.dim() != 2 or B.dim() != 3:
        raise RuntimeError("A and C must be 2-D, B 3-D")
    prob_n, prob_k = A.shape
    prob_m = C.shape[1]
    n_deltas = B.shape[0]
    if token_indices.numel() != prob_n or C.shape[0] != prob_n:
        raise RuntimeError("token_indices and C need one entry / row per row of A")
    if prob_m % 128 == 0 and prob_k % 64 == 0:
        _check_packed(B, meta, s, prob_m, prob_k, lead=(n_deltas,))
    if workspace is None:
        workspace = routed_workspace(prob_n, n_deltas, A.device)
    err = _ffi.lib().triteia_hip_sbmm_2_4_routed(
        _ffi.ptr(A), _ffi.ptr(B), _ffi.ptr(meta), _ffi.ptr(C), _ffi.ptr(s), _ffi.ptr(token_indices),
        int(index_offset), n_deltas, prob_m, prob_n, prob_k, _ffi.ptr(workspace),
        workspace.numel() * workspace.element_size(), 1 if accumulate else 0, _ffi.device_index(A), _ffi.stream_of(A))
    _raise(err, prob_m, prob_n, prob_k, -1, -1, -1)
    return workspace


def sbmm_2_4_planned(A, B, meta, C, s, plan, accumulate=False):
    """The multiply step of `sbmm_2_4_routed` on an existing routing plan (from `route_plan`
    with n_deltas = B.shape[0] and as many tokens as A has rows); lets one plan serve many
    layers."""
    _gemm_checks(A, B, meta, C, s)
    _ffi.require_gpu(plan=plan)
    if A.dim() != 2 or C.dim() != 2 or B.dim() != 3:
        raise RuntimeError("A and C must be 2-D, B 3-D")
    prob_n, prob_k = A.shape
    prob_m = C.shape[1]
    n_deltas = B.shape[0]
    need = _ffi.lib().triteia_hip_sbmm_routed_workspace_bytes(prob_n, n_deltas)
    if plan.numel() * plan.element_size() < need:
        raise RuntimeError(f"plan holds {plan.numel() * plan.element_size()} bytes, {need} needed")
    if prob_m % 128 == 0 and prob_k % 64 == 0:
        _check_packed(B, meta, s, prob_m, prob_k, lead=(n_deltas,))
    err = _ffi.lib().triteia_hip_sbmm_2_4_planned(
        _ffi.ptr(A), _ffi.ptr(B), _ffi.ptr(meta), _ffi.ptr(C), _ffi.ptr(s), _ffi.ptr(plan), n_deltas, prob_m, prob_n,
        prob_k, 1 if accumulate else 0, _ffi.device_index(A), _ffi.stream_of(A))
    _raise(err, prob_m, prob_n, prob_k, -1, -1, -1)
