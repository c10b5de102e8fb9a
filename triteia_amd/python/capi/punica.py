"""LoRA entry points with the reference's signatures (triteia/python/capi/punica.py:4-68)."""
import torch

from . import _ffi


_LORA_DTYPES = (torch.float16, torch.bfloat16)


def _lora_dtype(x, **others):
    """fp16 or bf16, the same for every tensor of the call (the reference dispatches on x's dtype and
    checks the others against it: ops.cpp:132-143, 199-214)."""
    if x.dtype not in _LORA_DTYPES:
        raise RuntimeError(f"x must be torch.float16 or torch.bfloat16, got {x.dtype}")
    for name, t in others.items():
        _ffi.require_dtype(t, x.dtype, name)
    return x.dtype


def _check(err):
    if err == _ffi.ERR_KERN_SHAPE:
        raise RuntimeError(_ffi.last_error())
    if err:
        raise RuntimeError(f"triteia_hip error {err}: {_ffi.last_error()}")


def sgmv(y, x, w_ptr, s, tmp, layer_idx, accumulate=True):
    """y[s[i]:s[i+1]] += x[s[i]:s[i+1]] @ deref(w_ptr[i])[layer_idx]
    (the reference's `sgmv_cutlass` binding, triteia/csrc/ops/ops.cpp:120-147).
    `accumulate=False` (no counterpart in the reference) stores the product instead of adding it: y is not read."""
    _ffi.require_gpu(y=y, x=x, w_ptr=w_ptr, s=s, tmp=tmp)
    if y.dim() != 2 or x.dim() != 2 or w_ptr.dim() != 1 or s.dim() != 1 or tmp.dim() != 1:
        raise RuntimeError("y, x must be 2D tensors; w_ptr, s, tmp 1D tensors")
    dtype = _lora_dtype(x, y=y)
    _ffi.require_dtype(w_ptr, torch.int64, "w_ptr")
    _ffi.require_dtype(s, torch.int32, "s")
    num_problems = s.size(0) - 1
    if w_ptr.size(0) != num_problems:
        raise RuntimeError(f"w_ptr has {w_ptr.size(0)} entries, s describes {num_problems} problems")
    if tmp.numel() * tmp.element_size() != sgmv_tmp_size(num_problems):
        raise RuntimeError(f"CHECK_EQ(tmp.size(0), sgmv_tmp_size(num_problems)) failed. "
                           f"{tmp.numel()} vs {sgmv_tmp_size(num_problems)}")
    if not accumulate:
        fn = _ffi.lib().triteia_hip_sgmv_store if dtype == torch.float16 else _ffi.lib().triteia_hip_sgmv_store_bf16
        _check(fn(_ffi.ptr(y), _ffi.ptr(x), _ffi.ptr(w_ptr), _ffi.ptr(s), num_problems, x.size(1), y.size(1),
                  int(layer_idx), _ffi.device_index(x), _ffi.stream_of(x)))
        return
    fn = _ffi.lib().triteia_hip_sgmv if dtype == torch.float16 else _ffi.lib().triteia_hip_sgmv_bf16
    _check(fn(
        _ffi.ptr(y), _ffi.ptr(x), _ffi.ptr(w_ptr), _ffi.ptr(s), _ffi.ptr(tmp), num_problems, x.size(1), y.size(1),
        int(layer_idx), _ffi.device_index(x), _ffi.stream_of(x)))


def sgmv_tmp_size(num_problems):
    return _ffi.lib().triteia_hip_sgmv_tmp_size(int(num_problems))


def dispatch_bgmv(y, x, w, indicies, layer_idx, scale, accumulate=True):
    """y[b] += scale * w[indicies[b], layer_idx] @ x[b]  (triteia/csrc/ops/ops.cpp:177-220).
    `accumulate=False` (no counterpart in the reference) stores the product instead of adding it: y is not read."""
    _ffi.require_gpu(y=y, x=x, w=w, indicies=indicies)
    if y.dim() != 2 or x.dim() != 2 or w.dim() != 4 or indicies.dim() != 1:
        raise RuntimeError("y, x must be 2D tensors, w a 4D tensor, indicies a 1D tensor")
    dtype = _lora_dtype(x, y=y, w=w)
    _ffi.require_dtype(indicies, torch.int64, "indicies")
    B, h_in = x.shape
    h_out = y.size(1)
    for a, b, what in ((w.size(3), h_in, "w.size(3), h_in"), (w.size(2), h_out, "w.size(2), h_out"),
                       (indicies.size(0), B, "indicies.size(0), x.size(0)"), (y.size(0), B, "y.size(0), x.size(0)")):
        if a != b:
            raise RuntimeError(f"CHECK_EQ({what}) failed. {a} vs {b}")
    if accumulate:
        fn = _ffi.lib().triteia_hip_bgmv if dtype == torch.float16 else _ffi.lib().triteia_hip_bgmv_bf16
    else:
        fn = _ffi.lib().triteia_hip_bgmv_store if dtype == torch.float16 else _ffi.lib().triteia_hip_bgmv_store_bf16
    _check(fn(
        _ffi.ptr(y), _ffi.ptr(x), _ffi.ptr(w), _ffi.ptr(indicies), B, h_in, h_out, w.size(1), int(layer_idx),
        float(scale), _ffi.device_index(x), _ffi.stream_of(x)))


def add_lora_sgmv_cutlass(y, x, wa_ptr, wb_ptr, s, layer_idx, lora_rank):
    """y[s[i]:s[i+1]] += x[s[i]:s[i+1]] @ deref(wa_ptr[i]) @ deref(wb_ptr[i])

    y [B, H2] (changed in place), x [B, H1], wa_ptr / wb_ptr int64 [S] device pointers to
    [num_layers, H1, R] / [num_layers, R, H2] fp16 matrices, s int32 [S+1] indptr."""
    tmp_size = sgmv_tmp_size(wa_ptr.size(0))
    tmp = torch.empty((tmp_size,), dtype=torch.uint8, device=x.device)
    # the shrink stores its result: the intermediate needs no clearing, and only rows inside a segment are read back
    v = torch.empty((x.size(0), lora_rank), dtype=x.dtype, device=x.device)
    sgmv(v, x, wa_ptr, s, tmp, layer_idx, accumulate=False)
    sgmv(y, v, wb_ptr, s, tmp, layer_idx)


def add_lora_bgmv(y, x, wa_T_all, wb_T_all, indicies, layer_idx, scale):
    """y[i] += x[i] @ wa_T_all[indicies[i], layer_idx].T @ wb_T_all[indicies[i], layer_idx].T * scale

    y [B, H2] (changed in place), x [B, H1], wa_T_all [n, L, R, H1], wb_T_all [n, L, H2, R],
    indicies int64 [B]."""
    r = wb_T_all.size(-1)
    # the shrink stores its result: the intermediate needs no clearing (rows with a negative index are never read back)
    tmp = torch.empty((x.size(0), r), dtype=x.dtype, device=x.device)
    dispatch_bgmv(tmp, x, wa_T_all, indicies, layer_idx, 1.0, accumulate=False)
    dispatch_bgmv(y, tmp, wb_T_all, indicies, layer_idx, scale)


def sgmv_routed(y, x, weights, plan, scale=1.0, accumulate=True):
    """y[t] += scale * x[t] @ weights[a] for every token t the routing plan lists under adapter a
    (`accumulate=False`: stored instead of added; y is not read, rows the plan does not list keep what they hold).

    weights [n_adapters, d_in, d_out] fp16 or bf16 (as x and y), contiguous; `plan` from capi.route_plan with
    n_deltas == n_adapters."""
    _ffi.require_gpu(y=y, x=x, weights=weights, plan=plan)
    dtype = _lora_dtype(x, y=y, weights=weights)
    n_adapters, d_in, d_out = weights.shape
    if x.size(1) != d_in or y.size(1) != d_out or x.size(0) != y.size(0):
        raise RuntimeError("shape mismatch between x, y and weights")
    fn = _ffi.lib().triteia_hip_sgmv_routed if dtype == torch.float16 else _ffi.lib().triteia_hip_sgmv_routed_bf16
    _check(fn(
        _ffi.ptr(y), y.stride(0), _ffi.ptr(x), x.stride(0), _ffi.ptr(weights), d_in * d_out, n_adapters, d_in, d_out,
        float(scale), _ffi.ptr(plan), x.size(0), 1 if accumulate else 0, _ffi.device_index(x), _ffi.stream_of(x)))
