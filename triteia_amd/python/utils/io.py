"""safetensors I/O with the reference's helpers' names and behaviour (triteia/python/utils/io.py:5-22)."""
import safetensors as st
from safetensors.torch import save_file


def save_tensors(tensors, path):
    """Write a {name: tensor} dict; tensors are made contiguous first (io.py:5-8)."""
    save_file({key: value.contiguous() for key, value in tensors.items()}, path)


def read_tensors(path, prefix=None, device="cpu"):
    """Read all tensors, or those under `prefix.` with the prefix stripped (io.py:11-22)."""
    tensors = {}
    with st.safe_open(path, framework="pt", device=device) as f:
        for key in f.keys():
            if prefix is None:
                tensors[key] = f.get_tensor(key)
            elif key.startswith(prefix):
                tensors[key.removeprefix(prefix + ".")] = f.get_tensor(key)
    return tensors
