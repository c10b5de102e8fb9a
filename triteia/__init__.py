"""Import-path alias: `triteia.python.{ops,capi,nn}` resolve to this repository's
`triteia_amd.python.*`, so code written against the reference's module layout runs unchanged."""
import importlib
import sys

import triteia_amd.python as python  # noqa: F401

sys.modules[__name__ + ".python"] = python
for _sub in ("capi", "capi.marlin", "capi.punica", "ops", "ops.matmul", "ops.matmul.sparse_low_precision",
             "ops.matmul.bmm", "ops.matmul.sbmm", "ops.matmul.lora", "ops.matmul.ldmm", "ops.utils",
             "ops.utils.sparsity", "ops.utils.generator", "nn", "nn.linear", "utils", "utils.io", "utils.quant_utils",
             "utils.benchmark", "configs", "configs.models", "configs.models.llama"):
    sys.modules[f"{__name__}.python.{_sub}"] = importlib.import_module(f"triteia_amd.python.{_sub}")
