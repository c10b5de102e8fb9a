"""Which Llama modules are fused and how they shard across a tensor-parallel group
(same facts as triteia/python/configs/models/llama.py:1-30)."""
# fused module -> its source projections, in the order they are concatenated along the output features
fused_modules = {
    "self_attn.qkv_proj": ["self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj"],
    "mlp.gate_up_proj": ["mlp.gate_proj", "mlp.up_proj"],
}
# source module -> "fused module:position inside it"
pack_modules = {src: f"{dst}:{pos}" for dst, srcs in fused_modules.items() for pos, src in enumerate(srcs)}
# sharded along the output features (after fusing) / along the input features
column_chunking_modules = [src for srcs in fused_modules.values() for src in srcs]
row_chunking_modules = ["self_attn.o_proj", "mlp.down_proj"]
# kept in fp16, rows split across the group
uncompressed_row_chunking_modules = ["embed_tokens", "lm_head"]


def _layer_shapes(hidden, intermediate):
    """(in features, out features) of the four packed matrices of one layer."""
    return [(hidden, 3 * hidden), (hidden, hidden), (hidden, 2 * intermediate), (intermediate, hidden)]


llama_shapes = {"7B": _layer_shapes(4096, 10752), "13B": _layer_shapes(5120, 13568)}
