from .linear import multi_delta_linear, sparse_low_precision_linear  # noqa: F401
