"""CPU-side checks of the C-ABI library: it loads, exports every declared symbol, and rejects
bad problems before touching the GPU."""
import ctypes
import os
import re

import pytest

from triteia_amd.python.capi import _ffi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "triteia_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(triteia_hip_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = declared_symbols()
    assert len(names) >= 12
    handle = ctypes.CDLL(_ffi.LIB_PATH)
    for n in names:
        assert hasattr(handle, n), f"{n} declared in include/triteia_hip.h but not exported"
    assert set(names) == set(_ffi.SIGNATURES), "ctypes table and header disagree"


def test_version_and_error_text():
    lib = _ffi.lib()
    assert lib.triteia_hip_version() >= 1000
    assert isinstance(_ffi.last_error(), str)


@pytest.mark.parametrize("m,n,k,gs,code", [
    (100, 16, 4096, -1, _ffi.ERR_PROB_SHAPE),      # m not a multiple of 128
    (4096, 16, 100, -1, _ffi.ERR_PROB_SHAPE),      # k not a multiple of 64
    (4096, 16, 4096, 32, _ffi.ERR_KERN_SHAPE),     # scale groups other than 128 dense k (groupsize 64) have no kernel
    (4096, 0, 4096, -1, 0),                        # empty problem is a no-op
])
def test_shape_errors_do_not_need_a_gpu(m, n, k, gs, code):
    lib = _ffi.lib()
    null = ctypes.c_void_p(0)
    rc = lib.triteia_hip_mul_2_4(null, null, null, null, null, m, n, k, null, gs, 0, null, -1, -1, -1, 16)
    assert rc == code
    if code:
        assert _ffi.last_error() != ""
    rc = lib.triteia_hip_bmm_2_4(null, null, null, null, null, m, n, k, null, gs, 0, null, -1, -1, -1, 16)
    assert rc == code


def test_grouped_scales_are_for_the_single_matrix_product():
    """groupsize 64 (scales per column and 128 dense k, marlin_nm.cu:68,102-111) is taken by mul_2_4; the batched and
    routed launchers, whose group iteration the reference itself has commented out (triteia_nm_bmm.cu:69-71,
    triteia_nm_sbmm.cu:70-72), answer ERR_KERN_SHAPE; K must be whole groups."""
    lib = _ffi.lib()
    null = ctypes.c_void_p(0)
    assert lib.triteia_hip_mul_2_4(null, null, null, null, null, 4096, 0, 4096, null, 64, 0, null, -1, -1, -1, 16) == 0
    assert lib.triteia_hip_mul_2_4(null, null, null, null, null, 4096, 16, 4096, null, 64, 0, null, -1, -1, -1, 16) == _ffi.ERR_ARGUMENT
    assert lib.triteia_hip_mul_2_4(null, null, null, null, null, 4096, 16, 4160, null, 64, 0, null, -1, -1, -1, 16) == _ffi.ERR_PROB_SHAPE
    assert lib.triteia_hip_bmm_2_4(null, null, null, null, null, 4096, 16, 4096, null, 64, 0, null, -1, -1, -1, 16) == _ffi.ERR_KERN_SHAPE
    assert lib.triteia_hip_sbmm_2_4(*([null] * 8), 4096, 16, 4096, 1, null, 64, 0, null, -1, -1, -1, 16) == _ffi.ERR_KERN_SHAPE


def test_other_argument_errors():
    lib = _ffi.lib()
    null = ctypes.c_void_p(0)
    # bgmv: narrow side too wide / not a multiple of 8
    assert lib.triteia_hip_bgmv(null, null, null, null, 4, 4096, 256, 1, 0, 1.0, 0, null) == _ffi.ERR_KERN_SHAPE
    assert "No suitable kernel" in _ffi.last_error()
    assert lib.triteia_hip_bgmv(null, null, null, null, 4, 4096, 12, 1, 0, 1.0, 0, null) == _ffi.ERR_KERN_SHAPE
    assert lib.triteia_hip_bgmv(null, null, null, null, 4, 4096, 16, 1, 3, 1.0, 0, null) == _ffi.ERR_PROB_SHAPE
    # routed sbmm: workspace too small, too many deltas
    need = lib.triteia_hip_sbmm_routed_workspace_bytes(64, 16)
    assert need == 4 * (8 + 4 * (16 + 64 // 16) + 4 * (64 // 33 + 1) + 64 + 4 * (16 + 64 // 16) + 4 * (16 + 64 // 64))
    assert lib.triteia_hip_plan_tile_tokens(8, 8) == 16
    assert lib.triteia_hip_plan_tile_tokens(64, 16) == 16       # at most 4 tokens per delta on average
    assert lib.triteia_hip_plan_tile_tokens(256, 16) == 32
    assert lib.triteia_hip_plan_tile_tokens(4096, 4) == 64
    assert lib.triteia_hip_planned_tile_kernel(256, 32, 11008, 4096) == 32      # cfg3: wide layer, 32-token tiles
    assert lib.triteia_hip_planned_tile_kernel(256, 16, 4096, 4096) == 0        # narrow layer: the K-split kernel
    assert lib.triteia_hip_planned_tile_kernel(2048, 32, 11008, 4096) == 64
    assert lib.triteia_hip_planned_tile_kernel(2048, 64, 28672, 8192) == 64     # 64-token tiles on a long K as well
    # 1024 tokens over 8 deltas: the plan is cut in 32-token tiles and lists 64-token tiles beside them for wide layers
    assert lib.triteia_hip_plan_tile_tokens(1024, 8) == 32
    assert lib.triteia_hip_planned_tile_kernel(1024, 8, 11008, 4096) == 64
    assert lib.triteia_hip_planned_tile_kernel(1024, 8, 4096, 4096) == 32
    assert lib.triteia_hip_planned_tile_kernel(1024, 32, 11008, 4096) == 32     # 32 tokens per delta: no 64-token tiles
    one = ctypes.c_void_p(16)
    assert lib.triteia_hip_route_plan(one, 0, 16, 64, one, need - 1, 0, null) == _ffi.ERR_ARGUMENT
    assert lib.triteia_hip_route_plan(one, 0, 100000, 64, one, 1 << 30, 0, null) == _ffi.ERR_KERN_SHAPE
    assert lib.triteia_hip_sgmv_tmp_size(7) == 420
    assert lib.triteia_hip_sgmv(null, null, null, null, null, 0, 4096, 16, 0, 0, null) == 0


def test_python_wrappers_refuse_cpu_tensors():
    import torch
    from triteia_amd.python.ops import matmul_4bit_2_4
    x = torch.zeros(2, 128, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        matmul_4bit_2_4(torch.zeros(4, 512, dtype=torch.int32), x, torch.zeros(256, 8, dtype=torch.int16),
                        torch.ones(1, 256, dtype=torch.float16))


def test_product_code_never_reaches_for_the_oracle():
    """The CPU restatement is the checker: nothing in the package, its import alias, the C sources
    or the header may import, read or mention it."""
    import pathlib
    root = pathlib.Path(__file__).resolve().parents[1]
    offenders = []
    for top in ("triteia_amd", "triteia", "include"):
        for path in (root / top).rglob("*"):
            if path.suffix in (".py", ".h", ".hip") and "oracle" in path.read_text(errors="replace"):
                offenders.append(str(path.relative_to(root)))
    assert not offenders, offenders


def test_dispatch_queries_at_the_documented_points():
    """Which kernel a call would run is a pure host-side function of the shapes and the knobs: the answers at the
    benchmark's points, as the documentation states them (no GPU involved)."""
    lib = _ffi.lib()
    _ffi.reload_env()
    uniform = lib.triteia_hip_uniform_kernel          # (m, batch, tokens, k, with_scratch)
    assert uniform(4096, 1, 16, 4096, 1) == 16         # cfg0: K of 4096 is too short for a split across workgroups; 16-column shares
    assert uniform(4096, 1, 17, 4096, 1) == 0          # more than one 16-token pass: the streaming kernel
    assert uniform(11008, 1, 16, 4096, 1) == 16        # 86 column blocks: shares of 64 columns
    assert uniform(28672, 1, 16, 4096, 1) == 0         # 224 column blocks: the streaming kernel
    assert uniform(4096, 8, 1, 4096, 1) == 0           # cfg1: a workgroup per CU already
    assert uniform(8192, 1, 16, 8192, 1) == 1004       # long K, few workgroups: K split in 4 ...
    assert uniform(8192, 1, 16, 8192, 0) == 16         # ... only with a scratch buffer (without: shares of 32 columns)
    assert lib.triteia_hip_bmm_scratch_bytes(8192, 1, 16, 8192) == 4 * 16 * 8192 * 4
    assert lib.triteia_hip_bmm_scratch_bytes(4096, 1, 16, 4096) == 0
    assert uniform(4096, 1, 1024, 4096, 1) == 33       # 32-token tiles on eight wavefronts (one workgroup per CU)
    assert uniform(4096, 1, 1536, 4096, 1) == 65       # 64-token tiles on eight wavefronts
    assert uniform(4096, 1, 4096, 4096, 1) == 64       # 64-token tiles, two workgroups per CU
    assert uniform(2048, 1, 8192, 4096, 1) == 256      # a narrow layer: one round of 256-token tiles
    assert uniform(28672, 1, 4096, 8192, 1) == 64      # several rounds: 64-token tiles, two workgroups per CU
    assert uniform(4096, 1, 128, 4096, 1) == 0
    assert uniform(100, 1, 16, 4096, 1) == -1          # not a legal shape
    routed = lib.triteia_hip_routed_in_kernel          # (tokens, deltas, m, k)
    assert routed(64, 16, 4096, 4096) == 1             # cfg2: one launch, no plan
    assert routed(256, 16, 4096, 4096) == 1
    assert routed(65, 17, 4096, 4096) == 0             # above 64 tokens only up to 16 deltas
    assert routed(64, 32, 4096, 4096) == 1             # a small layer: the plan's launch would not pay
    assert routed(64, 32, 11008, 4096) == 0            # 33 .. 64 tokens over many deltas of a large layer: planned ...
    assert lib.triteia_hip_plan_tile_tokens(64, 32) == 32   # ... in 32-token tiles (a skewed batch's hot delta in one tile)
    assert routed(32, 32, 11008, 4096) == 1
    assert routed(1, 16, 4096, 4096) == 2              # one token: column shares, routed in the kernel
    assert routed(4, 16, 4096, 4096) == 2              # at most four deltas in use: 128 column blocks on the bound
    assert routed(8, 16, 4096, 4096) == 1              # up to eight: the streaming kernel
    assert routed(16, 4, 4096, 4096) == 1              # four tokens per delta: weights requested ahead of the routing
    assert routed(256, 32, 11008, 4096) == 0           # cfg3: planned ...
    assert lib.triteia_hip_planned_tile_kernel(256, 32, 11008, 4096) == 32   # ... and its 32-token tiles go to the wide kernel
    assert lib.triteia_hip_planned_tile_kernel(256, 16, 4096, 4096) == 0     # a narrow layer keeps the streaming kernel
    assert lib.triteia_hip_planned_tile_kernel(1024, 16, 4096, 4096) == 32   # except for a thousand tokens in full tiles
    assert lib.triteia_hip_plan_tile_tokens(64, 16) == 16
    assert lib.triteia_hip_plan_tile_tokens(4096, 16) == 64


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert res.returncode == 2
    assert "ONE GPU" in res.stderr
