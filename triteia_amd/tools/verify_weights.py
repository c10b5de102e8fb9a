"""Check a tensor-parallel packed checkpoint against the unsharded one
(triteia/tools/verify_weights.py:41-96): the column shards of a fused module, multiplied one by one
and concatenated, must give what the single-shard checkpoint gives.

    python -m triteia_amd.tools.verify_weights --input tp2.safetensors --reference-input tp1.safetensors \\
        --module model.layers.0.self_attn.qkv_proj
"""
import argparse

import torch

from triteia_amd.python.ops import matmul_4bit_2_4
from triteia_amd.python.utils.io import read_tensors


def modules_of(weights):
    """Module names of `<module>.<tp>.<component>` keys."""
    return sorted({".".join(key.split(".")[:-2]) for key in weights})


def check_output(weights, reference_weights, module_name, tokens=128, generator=None):
    """max |ref - concat(shards)| / mean |ref| for `tokens` random activation rows."""
    ref = [reference_weights[f"{module_name}.0.{c}"] for c in ("qweight", "meta", "scales")]
    x = torch.randn((tokens, 32 * ref[0].size(0)), dtype=torch.float16, device=ref[0].device, generator=generator)
    reference_output = matmul_4bit_2_4(ref[0], x, ref[1], ref[2])
    tp_groups = sorted({int(key.split(".")[-2]) for key in weights if key.startswith(module_name + ".")})
    outputs = [matmul_4bit_2_4(weights[f"{module_name}.{tp}.qweight"], x, weights[f"{module_name}.{tp}.meta"],
                               weights[f"{module_name}.{tp}.scales"]) for tp in tp_groups]
    tp_output = torch.cat(outputs, dim=1)
    return (torch.max(torch.abs(reference_output - tp_output)) / torch.mean(torch.abs(reference_output))).item()


def main(argv=None):
    parser = argparse.ArgumentParser(description=__doc__.splitlines()[0])
    parser.add_argument("--input", type=str, required=True)
    parser.add_argument("--reference-input", type=str, required=True)
    parser.add_argument("--module", type=str, default=None, help="default: every fused (column-split) module")
    args = parser.parse_args(argv)
    weights = read_tensors(args.input, device="cuda")
    reference_weights = read_tensors(args.reference_input, device="cuda")
    names = [args.module] if args.module else [m for m in modules_of(weights) if "qkv_proj" in m or "gate_up_proj" in m]
    for name in names:
        print(f"{name}: max diff / mean |ref| = {check_output(weights, reference_weights, name):.3e}")


if __name__ == "__main__":
    main()
