"""ctypes binding of libtriteia_hip.so (declared in include/triteia_hip.h).

The library is built in-tree by `python -m triteia_amd.build`; there is no
fallback implementation: if it cannot be loaded every op raises.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.normpath(os.path.join(_HERE, "..", "..", "lib", "libtriteia_hip.so"))

ERR_PROB_SHAPE = 1
ERR_KERN_SHAPE = 2
ERR_ARGUMENT = 3
ERR_RUNTIME = 4

_c_int, _c_vp, _c_sz, _c_long, _c_float = ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_long, ctypes.c_float

# name -> (restype, argtypes); mirrors include/triteia_hip.h one to one
SIGNATURES = {
    "triteia_hip_version": (_c_int, []),
    "triteia_hip_last_error": (ctypes.c_char_p, []),
    "triteia_hip_mul_2_4": (_c_int, [_c_vp] * 5 + [_c_int] * 3 + [_c_vp, _c_int, _c_int, _c_vp] + [_c_int] * 4),
    "triteia_hip_bmm_2_4": (_c_int, [_c_vp] * 5 + [_c_int] * 3 + [_c_vp, _c_int, _c_int, _c_vp] + [_c_int] * 4),
    "triteia_hip_bmm_2_4_tokens": (_c_int, [_c_vp] * 5 + [_c_int] * 4 + [_c_int, _c_vp]),
    "triteia_hip_reload_env": (None, []),
    "triteia_hip_bmm_2_4_tokens_scratch": (_c_int, [_c_vp] * 5 + [_c_int] * 4 + [_c_vp, _c_sz, _c_int, _c_vp]),
    "triteia_hip_bmm_scratch_bytes": (_c_sz, [_c_int] * 4),
    "triteia_hip_uniform_kernel": (_c_int, [_c_int] * 5),
    "triteia_hip_sbmm_2_4": (_c_int, [_c_vp] * 8 + [_c_int] * 4 + [_c_vp, _c_int, _c_int, _c_vp] + [_c_int] * 4),
    "triteia_hip_sbmm_2_4_bounded": (_c_int, [_c_vp] * 8 + [_c_int] * 4 + [_c_vp, _c_int, _c_int, _c_vp] + [_c_int] * 5),
    "triteia_hip_sbmm_2_4_routed": (_c_int, [_c_vp] * 6 + [_c_int] * 5 + [_c_vp, _c_sz, _c_int, _c_int, _c_vp]),
    "triteia_hip_sbmm_2_4_routed_static": (_c_int, [_c_vp] * 6 + [_c_int] * 5 + [_c_int, _c_int, _c_vp]),
    "triteia_hip_sbmm_routed_static_max_bytes": (_c_sz, []),
    "triteia_hip_sbmm_2_4_planned": (_c_int, [_c_vp] * 6 + [_c_int] * 5 + [_c_int, _c_vp]),
    "triteia_hip_sbmm_routed_workspace_bytes": (_c_sz, [_c_int, _c_int]),
    "triteia_hip_plan_tile_tokens": (_c_int, [_c_int, _c_int]),
    "triteia_hip_routed_in_kernel": (_c_int, [_c_int, _c_int, _c_int, _c_int]),
    "triteia_hip_planned_tile_kernel": (_c_int, [_c_int, _c_int, _c_int, _c_int]),
    "triteia_hip_wide_unit_order": (_c_int, [_c_int]),
    "triteia_hip_wide_grid_units": (ctypes.c_long, [ctypes.c_long, _c_int, _c_int]),
    "triteia_hip_wide_block_grid_units": (ctypes.c_long, [ctypes.c_long, _c_int, _c_int]),
    "triteia_hip_route_plan": (_c_int, [_c_vp, _c_int, _c_int, _c_int, _c_vp, _c_sz, _c_int, _c_vp]),
    "triteia_hip_bgmv": (_c_int, [_c_vp] * 4 + [_c_int] * 5 + [_c_float, _c_int, _c_vp]),
    "triteia_hip_sgmv": (_c_int, [_c_vp] * 5 + [_c_int] * 5 + [_c_vp]),
    "triteia_hip_sgmv_tmp_size": (_c_sz, [_c_int]),
    "triteia_hip_bgmv_bf16": (_c_int, [_c_vp] * 4 + [_c_int] * 5 + [_c_float, _c_int, _c_vp]),
    "triteia_hip_sgmv_bf16": (_c_int, [_c_vp] * 5 + [_c_int] * 5 + [_c_vp]),
    "triteia_hip_sgmv_routed_bf16": (_c_int, [_c_vp, _c_long, _c_vp, _c_long, _c_vp, _c_long] + [_c_int] * 3
                                     + [_c_float, _c_vp, _c_int, _c_int, _c_int, _c_vp]),
    "triteia_hip_sgmv_routed": (_c_int, [_c_vp, _c_long, _c_vp, _c_long, _c_vp, _c_long] + [_c_int] * 3
                                + [_c_float, _c_vp, _c_int, _c_int, _c_int, _c_vp]),
    "triteia_hip_bgmv_store": (_c_int, [_c_vp] * 4 + [_c_int] * 5 + [_c_float, _c_int, _c_vp]),
    "triteia_hip_bgmv_store_bf16": (_c_int, [_c_vp] * 4 + [_c_int] * 5 + [_c_float, _c_int, _c_vp]),
    "triteia_hip_sgmv_store": (_c_int, [_c_vp] * 4 + [_c_int] * 5 + [_c_vp]),
    "triteia_hip_sgmv_store_bf16": (_c_int, [_c_vp] * 4 + [_c_int] * 5 + [_c_vp]),
}

_lib = None


def lib():
    """The loaded library; raises RuntimeError if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} not found: build it with `python -m triteia_amd.build` "
                "(there is no fallback implementation)")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def reload_env() -> None:
    """Make the library read its TRITEIA_HIP_* tuning knobs from the environment again (it reads
    them once, at its first call)."""
    lib().triteia_hip_reload_env()


def last_error() -> str:
    return lib().triteia_hip_last_error().decode("utf-8", "replace")


def stream_of(t: torch.Tensor):
    """Handle of torch's current stream on the tensor's device."""
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def device_index(t: torch.Tensor) -> int:
    return t.device.index if t.device.index is not None else torch.cuda.current_device()


def ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def require_gpu(**tensors):
    dev = None
    for name, t in tensors.items():
        if not isinstance(t, torch.Tensor):
            raise TypeError(f"{name} must be a torch.Tensor")
        if not t.is_cuda:
            raise RuntimeError(f"{name} must be a GPU tensor (this op has no CPU implementation)")
        if not t.is_contiguous():
            raise RuntimeError(f"{name} must be contiguous")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError(f"{name} is on {t.device}, expected {dev}")


def require_dtype(t, dtype, name):
    if t.dtype != dtype:
        raise RuntimeError(f"{name} must be {dtype}, got {t.dtype}")


_SPLIT_SCRATCH = {}          # (device, stream) -> buffer, most recently created last
_SPLIT_SCRATCH_MAX_STREAMS = 16


def split_scratch(nbytes: int, device) -> torch.Tensor:
    """Scratch for the K split of small matmul / bmm launches (fp32 partial sums): one buffer per device and
    stream, grown on demand, so that calls on different streams never share one; the streams seen longest ago
    give theirs up once more than a handful have asked.  A call recorded into a graph gets a buffer of its own
    from the graph's memory pool, which is not kept: it belongs to that graph, not to later calls on the stream."""
    dev = torch.device(device)
    nbytes = (int(nbytes) + 255) // 256 * 256
    if torch.cuda.is_current_stream_capturing():
        return torch.empty(max(nbytes, 256), dtype=torch.uint8, device=dev)
    key = (dev.index if dev.index is not None else torch.cuda.current_device(), torch.cuda.current_stream(dev).cuda_stream)
    buf = _SPLIT_SCRATCH.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=dev)
        _SPLIT_SCRATCH.pop(key, None)
        _SPLIT_SCRATCH[key] = buf
        while len(_SPLIT_SCRATCH) > _SPLIT_SCRATCH_MAX_STREAMS:
            _SPLIT_SCRATCH.pop(next(iter(_SPLIT_SCRATCH)))
    return buf


_LOCK_WORKSPACES = {}


def lock_workspace(numel: int, device) -> torch.Tensor:
    """All-zero int32 tensor of at least `numel` elements for the lock `workspace` argument of
    mul_2_4 / bmm_2_4 / sbmm_2_4.  The library checks its size and never reads or writes it, so
    one tensor per device serves every call (the reference allocates and clears one per call)."""
    dev = torch.device(device)
    if dev.type != "cuda":      # the op itself rejects CPU tensors, with its own message
        return torch.zeros(int(numel), dtype=torch.int32, device=dev)
    key = dev.index if dev.index is not None else torch.cuda.current_device()
    ws = _LOCK_WORKSPACES.get(key)
    if ws is None or ws.numel() < numel:
        ws = torch.zeros(max(int(numel), 4096), dtype=torch.int32, device=dev)
        _LOCK_WORKSPACES[key] = ws
    return ws
