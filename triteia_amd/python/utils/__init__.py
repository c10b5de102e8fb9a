"""Host-side helpers either side of the GEMM path: checkpoint I/O, GPTQ dequantisation and the
benchmark-result schema (triteia/python/utils/{io,quant_utils,benchmark}.py)."""
from .io import read_tensors, save_tensors  # noqa: F401
from .quant_utils import dequantize_weight, gptq_unpack, unpack_4bit_to_32bit_signed  # noqa: F401
from .benchmark import export_benchmark_results, format_benchmark_results, timing_function  # noqa: F401
