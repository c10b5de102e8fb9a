"""CPU tests of the steps either side of the GEMM path: GPTQ dequantisation, the checkpoint
converter and its on-disk key format, safetensors I/O and the benchmark-result schema."""
import json

import numpy as np
import pytest
import torch

from oracle import triteia_oracle as orc
from triteia_amd.python.configs.models import llama
from triteia_amd.python.utils import (dequantize_weight, export_benchmark_results, format_benchmark_results, gptq_unpack,
                                      read_tensors, save_tensors, unpack_4bit_to_32bit_signed)
from triteia_amd.tools.convert_deltazip import convert_tensors


def gptq_tensors(k, m, seed, zero=7):
    """A symmetric 4-bit GPTQ module with one group: codes q in 0..15, stored zero point 7."""
    rng = np.random.default_rng(seed)
    q = rng.integers(0, 16, size=(k, m))
    qweight = np.zeros((k // 8, m), dtype=np.int64)
    for row in range(k):                         # row 8i+j lives in nibble j of packed row i
        qweight[row // 8] |= q[row] << (4 * (row % 8))
    qzeros = np.zeros((1, m // 8), dtype=np.int64)
    for col in range(m):
        qzeros[0, col // 8] |= zero << (4 * (col % 8))
    scales = rng.uniform(0.005, 0.02, size=(1, m)).astype(np.float16)
    as_i32 = lambda a: torch.from_numpy((a & 0xFFFFFFFF).astype(np.uint32).view(np.int32))
    return q, as_i32(qweight), as_i32(qzeros), torch.from_numpy(scales)


def test_gptq_dequantise_matches_a_plain_loop():
    k, m = 64, 32
    q, qweight, qzeros, scales = gptq_tensors(k, m, 1)
    w, z = unpack_4bit_to_32bit_signed(qweight, qzeros)
    assert np.array_equal(w.numpy(), q) and (z.numpy() == 8).all()
    dense = dequantize_weight(qweight, qzeros, scales)                 # [m, k]
    want = (torch.from_numpy(q - 8).to(torch.int8) * scales).T
    assert torch.equal(dense, want)
    assert torch.equal(gptq_unpack(4, qweight, qzeros, scales).T, dense)
    with pytest.raises(ValueError):
        unpack_4bit_to_32bit_signed(qweight, gptq_tensors(k, m, 1, zero=6)[2])


@pytest.mark.parametrize("bits", [2, 4, 8])
def test_gptq_unpack_grouped_against_a_plain_loop(bits):
    """scales[g] * (q - (zero + 1 mod 2^bits)) element by element, two groups along k, any zero point."""
    k, m, per = 64, 32, 32 // bits
    rng = np.random.default_rng(bits)
    q = rng.integers(0, 1 << bits, size=(k, m))
    zero = rng.integers(0, 1 << bits, size=(2, m))
    scales = rng.uniform(0.005, 0.02, size=(2, m)).astype(np.float16)
    qweight = np.zeros((k // per, m), dtype=np.uint64)
    for row in range(k):
        qweight[row // per] |= q[row].astype(np.uint64) << np.uint64(bits * (row % per))
    qzeros = np.zeros((2, m // per), dtype=np.uint64)
    for col in range(m):
        qzeros[:, col // per] |= zero[:, col].astype(np.uint64) << np.uint64(bits * (col % per))
    as_i32 = lambda a: torch.from_numpy(a.astype(np.uint32).view(np.int32))
    got = gptq_unpack(bits, as_i32(qweight), as_i32(qzeros), torch.from_numpy(scales), group_size=k // 2)
    want = np.empty((k, m), dtype=np.float16)
    for row in range(k):
        g = row // (k // 2)
        for col in range(m):
            want[row, col] = scales[g, col] * np.float16(int(q[row, col]) - ((int(zero[g, col]) + 1) % (1 << bits)))
    assert got.shape == (k, m) and np.array_equal(got.numpy(), want)


def llama_state_dict(hidden, inter, seed):
    sd, dense = {}, {}
    shapes = {"self_attn.q_proj": (hidden, hidden), "self_attn.k_proj": (hidden, hidden), "self_attn.v_proj": (hidden, hidden),
              "self_attn.o_proj": (hidden, hidden), "mlp.gate_proj": (hidden, inter), "mlp.up_proj": (hidden, inter),
              "mlp.down_proj": (inter, hidden)}
    for j, (name, (k, m)) in enumerate(shapes.items()):
        q, qweight, qzeros, scales = gptq_tensors(k, m, seed + j)
        mod = f"model.layers.0.{name}"
        sd[mod + ".qweight"], sd[mod + ".qzeros"], sd[mod + ".scales"] = qweight, qzeros, scales
        sd[mod + ".g_idx"] = torch.zeros(k, dtype=torch.int32)
        dense[mod] = ((q - 8).astype(np.float32) * scales.numpy().astype(np.float32)).astype(np.float16)   # [k, m]
    sd["model.embed_tokens.weight"] = torch.arange(64 * hidden, dtype=torch.float16).reshape(64, hidden)
    sd["model.norm.weight"] = torch.ones(hidden, dtype=torch.float16)
    return sd, dense


def check_is_2_4_selection(unpacked, dense):
    """`unpacked` keeps, in every aligned group of 4 along k, two entries of `dense` (the others are 0)
    whose magnitudes are the two largest of the group (independent of how ties are broken)."""
    k, m = dense.shape
    u = unpacked.astype(np.float32).T.reshape(m, k // 4, 4)
    d = dense.astype(np.float32).T.reshape(m, k // 4, 4)
    assert np.all((u == d) | (u == 0))
    assert np.all((u != 0).sum(-1) <= 2)
    top2 = np.sort(np.abs(d), axis=-1)[..., 2:].sum(-1)
    np.testing.assert_allclose(np.abs(u).sum(-1), top2, rtol=0, atol=1e-6)


@pytest.mark.parametrize("tp", [1, 2])
def test_converter_writes_the_reference_key_format(tmp_path, tp):
    hidden, inter = 256, 512
    sd, dense = llama_state_dict(hidden, inter, 10)
    out = convert_tensors(sd, tp_size=tp)
    path = tmp_path / f"tp{tp}.safetensors"
    save_tensors(out, str(path))
    back = read_tensors(str(path))
    assert set(back) == set(out) and all(torch.equal(back[key], out[key]) for key in out)
    layer = "model.layers.0."
    want = {f"{layer}{mod}.{i}.{c}" for mod in ("self_attn.qkv_proj", "self_attn.o_proj", "mlp.gate_up_proj", "mlp.down_proj")
            for i in range(tp) for c in ("qweight", "scales", "meta")} | {f"model.embed_tokens.{i}.weight" for i in range(tp)}
    assert set(out) == want
    # fused, column-split modules: shards side by side give the fused dense matrix, 2:4-pruned
    for fused, parts in llama.fused_modules.items():
        full = np.concatenate([dense[layer + part] for part in parts], axis=1)
        shards = [orc.unpack(out[f"{layer}{fused}.{i}.qweight"].numpy(), out[f"{layer}{fused}.{i}.meta"].numpy(),
                             out[f"{layer}{fused}.{i}.scales"].numpy()) for i in range(tp)]
        assert shards[0].shape == (full.shape[0], full.shape[1] // tp)
        check_is_2_4_selection(np.concatenate(shards, axis=1), full)
    # row-split modules: shards stacked along k
    for mod in llama.row_chunking_modules:
        shards = [orc.unpack(out[f"{layer}{mod}.{i}.qweight"].numpy(), out[f"{layer}{mod}.{i}.meta"].numpy(),
                             out[f"{layer}{mod}.{i}.scales"].numpy()) for i in range(tp)]
        check_is_2_4_selection(np.concatenate(shards, axis=0), dense[layer + mod])
    emb = torch.cat([out[f"model.embed_tokens.{i}.weight"] for i in range(tp)], dim=0)
    assert torch.equal(emb, sd["model.embed_tokens.weight"])
    assert read_tensors(str(path), prefix="model.embed_tokens").keys() == {f"{i}.weight" for i in range(tp)}


def test_benchmark_schema_round_trip(tmp_path):
    def result(name, elapsed, m):
        return {"output": torch.zeros(1), "elapsed": elapsed, "func_name": name, "total_flops": 2.0, "perf_flops": 2.0 / elapsed,
                "mfu": None, "args": {"m": m, "k": 128, "x": torch.zeros(2)}, "measurements": {"elapsed": [elapsed], "perf_flops": [], "mfu": []}}
    results = [[result("fp16", 1.0, 256), result("w4_2_4", 0.5, 256)], [result("fp16", 2.0, 512), result("w4_2_4", 0.7, 512)]]
    path = tmp_path / "bench.json"
    export_benchmark_results(results, str(path))
    data = json.load(open(path))
    assert set(data) == {"gpu_specs", "results"} and len(data["results"]) == 4
    assert data["results"][0] == {"config": {"m": 256, "k": 128}, "elapsed": 1.0, "func_name": "fp16", "total_flops": 2.0,
                                  "perf_flops": 2.0, "mfu": None, "measurements": {"elapsed": [1.0], "perf_flops": [], "mfu": []}}
    specs, df = format_benchmark_results(str(path))
    assert len(df) == 2 and {"m", "k", "fp16_elapsed", "w4_2_4_elapsed", "fp16_perf_flops"} <= set(df.columns)
    assert df[df.m == 512]["w4_2_4_elapsed"].item() == 0.7
