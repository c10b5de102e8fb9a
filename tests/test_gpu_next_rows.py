"""GPU tests of the callers and formats either side of the GEMM path: the multi-delta layer,
a converted tensor-parallel checkpoint multiplied shard by shard, and the benchmark schema."""
import numpy as np
import pytest
import torch

from oracle import triteia_oracle as orc
from tests.helpers import activations, check_close, make_deltas, to_gpu
from tests.test_formats_cpu import llama_state_dict

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("with_base,use_plan", [(False, False), (True, False), (True, True)])
def test_multi_delta_linear(with_base, use_plan):
    from triteia_amd.python.capi import route_plan
    from triteia_amd.python.nn import multi_delta_linear, sparse_low_precision_linear
    print(f"[case] multi_delta_linear base={with_base} plan={use_plan}", flush=True)
    k, m, n, t = 256, 512, 5, 37
    qw, meta, s = make_deltas(n, k, m, 77)
    x = activations(t, k, 78)
    rng = np.random.default_rng(79)
    idx = rng.integers(-1, n, size=t).astype(np.int32)
    base = (rng.standard_normal((m, k)) * 0.05).astype(np.float16) if with_base else None
    layer = multi_delta_linear(k, m, n, with_base=with_base).to(DEV)
    single = sparse_low_precision_linear(k, m).to(DEV)
    for i in range(n):
        if i == 0:      # through a single-delta module
            single.qweight.copy_(torch.from_numpy(qw[i])), single.meta.copy_(torch.from_numpy(meta[i])), single.scale.copy_(torch.from_numpy(s[i]))
            layer.load_delta(i, single)
        else:
            layer.load_delta(i, *to_gpu(qw[i], meta[i], s[i]))
    if with_base:
        layer.base.copy_(torch.from_numpy(base))
    gx, gidx = to_gpu(x, idx)
    plan = route_plan(gidx, n) if use_plan else None
    out = layer(gx.view(1, t, k), gidx, plan=plan)
    torch.cuda.synchronize()
    assert out.shape == (1, t, m)
    ref = orc.sbmm_4bit_2_4(qw, x, meta, s, idx, base_weight=base)
    check_close(out.view(t, m), ref, what="multi_delta_linear")
    if not with_base:
        assert torch.all(out.view(t, m)[torch.from_numpy(idx == -1).to(DEV)] == 0)


def test_pack_delta_round_trip():
    from triteia_amd.python.nn import multi_delta_linear
    k, m = 128, 256
    g = torch.Generator().manual_seed(5)
    w = torch.randn((k, m), generator=g, dtype=torch.float32).to(torch.float16)
    scales = (w.abs().amax(0, keepdim=True).float() * 2 / 15).to(torch.float16)
    layer = multi_delta_linear(k, m, 2).to(DEV)
    layer.pack_delta(1, w.to(DEV), scales.to(DEV))
    dense = orc.unpack(layer.qweight[1].cpu().numpy(), layer.meta[1].cpu().numpy(), layer.scale[1].cpu().numpy())
    mask = orc.mask_2_4(np.ascontiguousarray(w.numpy().T)).T                # groups of 4 along k; fp16 normals: ties are rare
    q = np.clip(np.round((w.numpy() / scales.numpy()).astype(np.float32)), -8, 7).astype(np.float16)   # fp16 division, as the packer
    want = (q * scales.numpy()) * mask
    np.testing.assert_array_equal(dense.astype(np.float32), want.astype(np.float32))


def test_converted_checkpoint_shards_agree(tmp_path):
    """tools/verify_weights.py's check on a converted synthetic layer: column shards multiplied one by
    one and concatenated equal the unsharded product (the reference accepts a ratio of 1e-3 scale)."""
    from triteia_amd.python.utils import read_tensors, save_tensors
    from triteia_amd.tools.convert_deltazip import convert_tensors
    from triteia_amd.tools.verify_weights import check_output, modules_of
    sd, _ = llama_state_dict(256, 512, 40)
    for tp in (1, 2):
        save_tensors(convert_tensors(sd, tp_size=tp, device=DEV), str(tmp_path / f"tp{tp}.safetensors"))
    ref = read_tensors(str(tmp_path / "tp1.safetensors"), device=DEV)
    tp2 = read_tensors(str(tmp_path / "tp2.safetensors"), device=DEV)
    fused = [mod for mod in modules_of(tp2) if "qkv_proj" in mod or "gate_up_proj" in mod]
    assert len(fused) == 2
    for mod in fused:
        g = torch.Generator(device=DEV).manual_seed(3)
        assert check_output(tp2, ref, mod, tokens=48, generator=g) == 0.0    # same kernel, same columns: bit-equal


def test_timing_function_schema():
    from triteia_amd.python.ops import matmul_4bit_2_4
    from triteia_amd.python.utils import timing_function
    k, m, t = 256, 256, 16
    qw, meta, s = make_deltas(1, k, m, 91)
    gq, gm, gs, gx = to_gpu(qw[0], meta[0], s[0], activations(t, k, 92))

    def flops(x, qweight):
        return 2 * x.shape[0] * x.shape[1] * qweight.shape[1] // 2

    res = timing_function(matmul_4bit_2_4, flops, {"qweight": gq, "x": gx, "meta": gm, "s": gs, "m": m}, repeats=3)
    assert set(res) == {"output", "elapsed", "func_name", "total_flops", "perf_flops", "mfu", "args", "measurements"}
    assert res["func_name"] == "matmul_4bit_2_4" and len(res["measurements"]["elapsed"]) == 3
    assert res["total_flops"] == flops(gx, gq) / 1e9 and res["elapsed"] > 0
    assert res["mfu"] is not None and res["output"].shape == (t, m)
