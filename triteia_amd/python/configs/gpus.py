"""Device table for the benchmark schema's `gpu_specs` block and its MFU column.

The reference looks the device up with NVML in a table of NVIDIA parts
(triteia/python/configs/gpus/specs.py:1-60); here the name comes from the HIP runtime through torch."""
import torch

amd_mi355x = {
    "name": "AMD Instinct MI355X",
    "compute_capability": "gfx950",
    "memory": 288,        # GB
    "bandwidth": 8000,    # GB/s
    "fp16_tflops": 2500,  # dense matrix peak
    "fp32_tflops": 157.3,
}
amd_gpus = [amd_mi355x]


def get_gpu_device_info():
    """The table entry of device 0, or None when no GPU is visible or it is not in the table."""
    if not torch.cuda.is_available():
        return None
    props = torch.cuda.get_device_properties(0)
    arch = getattr(props, "gcnArchName", "").split(":")[0]
    for gpu in amd_gpus:
        if gpu["name"] in props.name or (arch and arch == gpu["compute_capability"]):
            return gpu
    return None
