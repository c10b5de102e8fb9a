"""GPTQ-style delta checkpoint -> packed 2:4 int4 checkpoint in the reference's on-disk format
(triteia/tools/converters/convert_deltazip.py:17-138).

Output keys: `<module>.<tp>.qweight`, `<module>.<tp>.scales`, `<module>.<tp>.meta` for every quantised
module (q/k/v and gate/up fused first and split along the output features, o_proj and down_proj
split along the input features), `<module>.<tp>.weight` for the row-split fp16 embeddings.  Each
shard is packed on its own, so a shard file can be loaded by one rank without the others.

    python -m triteia_amd.tools.convert_deltazip --ckpt in.safetensors --tp-size 2 --save-path out.safetensors

The lossless (nvCOMP) input layer of the reference is not part of this build.
"""
import argparse

import torch

from triteia_amd.python.configs.models.llama import (pack_modules, row_chunking_modules,
                                                    uncompressed_row_chunking_modules)
from triteia_amd.python.ops.utils.generator import torch_weight_to_sparse_marlin
from triteia_amd.python.utils.io import read_tensors, save_tensors
from triteia_amd.python.utils.quant_utils import dequantize_weight


def _store(out, name, packed):
    for idx, (qweight, scales, meta) in enumerate(zip(*packed)):
        out[f"{name}.{idx}.qweight"] = qweight
        out[f"{name}.{idx}.scales"] = scales.clone()   # row shards share one scale tensor; a file wants owners
        out[f"{name}.{idx}.meta"] = meta


@torch.no_grad()
def convert_tensors(tensors, tp_size=1, device="cpu"):
    """`tensors`: GPTQ state dict ({module}.qweight / .qzeros / .scales / .g_idx plus plain weights)."""
    out = {}
    dense = {}                      # module -> ([k, m] fp16 weight, [1, m] scales)
    consumed = set()
    for key in tensors:
        if not key.endswith(".qweight"):
            continue
        module = key.removesuffix(".qweight")
        w = dequantize_weight(tensors[key].to(device), tensors[module + ".qzeros"].to(device),
                              tensors[module + ".scales"].to(device)).to(torch.float16).t().contiguous()
        dense[module] = (w, tensors[module + ".scales"].to(device))
        consumed.update(module + suffix for suffix in (".qweight", ".qzeros", ".scales", ".g_idx"))
    fuse_plan = {}                  # fused module -> [(position, source module)]
    for module in dense:
        source = next((src for src in pack_modules if module.endswith(src)), None)
        if source is not None:
            target, pos = pack_modules[source].split(":")
            fuse_plan.setdefault(module.removesuffix(source) + target, []).append((int(pos), module))
        elif any(module.endswith(name) for name in row_chunking_modules):
            _store(out, module, torch_weight_to_sparse_marlin(*dense[module], tp_size=tp_size, chunk_by="row", device=device))
    for target, parts in fuse_plan.items():
        parts = [dense[module] for _, module in sorted(parts)]
        weight = torch.cat([w for w, _ in parts], dim=1)
        scales = torch.cat([s for _, s in parts], dim=1)
        _store(out, target, torch_weight_to_sparse_marlin(weight, scales, tp_size=tp_size, chunk_by="column", device=device))
    for key, weight in tensors.items():
        if key in consumed or not any(name in key for name in uncompressed_row_chunking_modules):
            continue
        name, rows = key.removesuffix(".weight"), weight.shape[0]
        for i in range(tp_size):
            out[f"{name}.{i}.weight"] = weight[i * rows // tp_size:(i + 1) * rows // tp_size, :]
    return out


def main(argv=None):
    parser = argparse.ArgumentParser(description=__doc__.splitlines()[0])
    parser.add_argument("--ckpt", type=str, required=True)
    parser.add_argument("--tp-size", type=int, default=1)
    parser.add_argument("--save-path", type=str, required=True)
    parser.add_argument("--device", type=str, default="cuda:0" if torch.cuda.is_available() else "cpu")
    args = parser.parse_args(argv)
    save_tensors(convert_tensors(read_tensors(args.ckpt), args.tp_size, args.device), args.save_path)


if __name__ == "__main__":
    main()
