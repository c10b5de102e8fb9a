"""MI355X-native implementation of Triteia's multi-model low-precision GEMM path.

`triteia_amd.python.ops` / `.capi` / `.nn` mirror the reference's `triteia.python.*` modules.
"""
__version__ = "0.1.0"
