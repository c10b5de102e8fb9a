"""LoRA entry points with the reference's signatures (triteia/python/capi/punica.py:4-68)."""
import torch

from . import _ffi


def _check(err):
    if err == _ffi.ERR_KERN_SHAPE:
        raise RuntimeError(_ffi.last_error())
    if err:
        raise RuntimeError(f"triteia_hip error {err}: {_ffi.last_error()}")


def sgmv(y, x, w_ptr, s, tmp, layer_idx):
    """y[s[i]:s[i+1]] += x[s[i]:s[i+1]] @ deref(w_ptr[i])[layer_idx]
    (the reference's `sgmv_cutlass` binding, triteia/csrc/ops/ops.cpp:120-147)."""
    _ffi.require_gpu(y=y, x=x, w_ptr=w_ptr, s=s, tmp=tmp)
    if y.dim() != 2 or x.dim() != 2 or w_ptr.dim() != 1 or s.dim() != 1 or tmp.dim() != 1:
        raise RuntimeError("y, x must be 2D tensors; w_ptr, s, tmp 1D tensors")
    _ffi.require_dtype(x, torch.float16, "x")
    _ffi.require_dtype(y, torch.float16, "y")
    _ffi.require_dtype(w_ptr, torch.int64, "w_ptr")
    _ffi.require_dtype(s, torch.int32, "s")
    num_problems = s.size(0) - 1
    if w_ptr.size(0) != num_problems:
        raise RuntimeError(f"w_ptr has {w_ptr.size(0)} entries, s describes {num_problems} problems")
    if tmp.numel() * tmp.element_size() != sgmv_tmp_size(num_problems):
        raise RuntimeError(f"CHECK_EQ(tmp.size(0), sgmv_tmp_size(num_problems)) failed. "
                           f"{tmp.numel()} vs {sgmv_tmp_size(num_problems)}")
    _check(_ffi.lib().triteia_hip_sgmv(
        _ffi.ptr(y), _ffi.ptr(x), _ffi.ptr(w_ptr), _ffi.ptr(s), _ffi.ptr(tmp), num_problems, x.size(1), y.size(1),
        int(layer_idx), _ffi.device_index(x), _ffi.stream_of(x)))


def sgmv_tmp_size(num_problems):
    return _ffi.lib().triteia_hip_sgmv_tmp_size(int(num_problems))


def dispatch_bgmv(y, x, w, indicies, layer_idx, scale):
    """y[b] += scale * w[indicies[b], layer_idx] @ x[b]  (triteia/csrc/ops/ops.cpp:177-220)."""
    _ffi.require_gpu(y=y, x=x, w=w, indicies=indicies)
    if y.dim() != 2 or x.dim() != 2 or w.dim() != 4 or indicies.dim() != 1:
        raise RuntimeError("y, x must be 2D tensors, w a 4D tensor, indicies a 1D tensor")
    _ffi.require_dtype(x, torch.float16, "x")
    _ffi.require_dtype(y, torch.float16, "y")
    _ffi.require_dtype(w, torch.float16, "w")
    _ffi.require_dtype(indicies, torch.int64, "indicies")
    B, h_in = x.shape
    h_out = y.size(1)
    for a, b, what in ((w.size(3), h_in, "w.size(3), h_in"), (w.size(2), h_out, "w.size(2), h_out"),
                       (indicies.size(0), B, "indicies.size(0), x.size(0)"), (y.size(0), B, "y.size(0), x.size(0)")):
        if a != b:
            raise RuntimeError(f"CHECK_EQ({what}) failed. {a} vs {b}")
    _check(_ffi.lib().triteia_hip_bgmv(
        _ffi.ptr(y), _ffi.ptr(x), _ffi.ptr(w), _ffi.ptr(indicies), B, h_in, h_out, w.size(1), int(layer_idx),
        float(scale), _ffi.device_index(x), _ffi.stream_of(x)))


def add_lora_sgmv_cutlass(y, x, wa_ptr, wb_ptr, s, layer_idx, lora_rank):
    """y[s[i]:s[i+1]] += x[s[i]:s[i+1]] @ deref(wa_ptr[i]) @ deref(wb_ptr[i])

    y [B, H2] (changed in place), x [B, H1], wa_ptr / wb_ptr int64 [S] device pointers to
    [num_layers, H1, R] / [num_layers, R, H2] fp16 matrices, s int32 [S+1] indptr."""
    tmp_size = sgmv_tmp_size(wa_ptr.size(0))
    tmp = torch.empty((tmp_size,), dtype=torch.uint8, device=x.device)
    v = torch.zeros((x.size(0), lora_rank), dtype=x.dtype, device=x.device)
    sgmv(v, x, wa_ptr, s, tmp, layer_idx)
    sgmv(y, v, wb_ptr, s, tmp, layer_idx)


def add_lora_bgmv(y, x, wa_T_all, wb_T_all, indicies, layer_idx, scale):
    """y[i] += x[i] @ wa_T_all[indicies[i], layer_idx].T @ wb_T_all[indicies[i], layer_idx].T * scale

    y [B, H2] (changed in place), x [B, H1], wa_T_all [n, L, R, H1], wb_T_all [n, L, H2, R],
    indicies int64 [B]."""
    r = wb_T_all.size(-1)
    tmp = torch.zeros((x.size(0), r), dtype=x.dtype, device=x.device)
    dispatch_bgmv(tmp, x, wa_T_all, indicies, layer_idx, 1.0)
    dispatch_bgmv(y, tmp, wb_T_all, indicies, layer_idx, scale)


def sgmv_routed(y, x, weights, plan, scale=1.0):
    """y[t] += scale * x[t] @ weights[a] for every token t the routing plan lists under adapter a.

    weights [n_adapters, d_in, d_out] fp16 contiguous; `plan` from capi.route_plan with
    n_deltas == n_adapters."""
    _ffi.require_gpu(y=y, x=x, weights=weights, plan=plan)
    _ffi.require_dtype(x, torch.float16, "x")
    _ffi.require_dtype(y, torch.float16, "y")
    _ffi.require_dtype(weights, torch.float16, "weights")
    n_adapters, d_in, d_out = weights.shape
    if x.size(1) != d_in or y.size(1) != d_out or x.size(0) != y.size(0):
        raise RuntimeError("shape mismatch between x, y and weights")
    _check(_ffi.lib().triteia_hip_sgmv_routed(
        _ffi.ptr(y), y.stride(0), _ffi.ptr(x), x.stride(0), _ffi.ptr(weights), d_in * d_out, n_adapters, d_in, d_out,
        float(scale), _ffi.ptr(plan), x.size(0), _ffi.device_index(x), _ffi.stream_of(x)))
