"""Benchmark-result schema of the reference (triteia/python/utils/benchmark.py:10-133), so that its
plotting scripts read results measured here: `timing_function` returns the same dict, and
`export_benchmark_results` writes the same JSON ({"gpu_specs": ..., "results": [{"config": ..., ...}]})."""
import inspect
import json

import torch

from triteia_amd.python.configs.gpus import get_gpu_device_info


def timing_function(func, flops_func, kwargs, repeats=1):
    """Time `func(**kwargs restricted to its parameters)` with device events, `repeats` times.

    Units follow the reference: elapsed in ms, total_flops in GFLOP, perf_flops in GFLOP/s,
    mfu in percent of the device's fp16 peak (None without a known device)."""
    func_args_names = inspect.getfullargspec(func).args
    func_args = {arg: kwargs[arg] for arg in func_args_names if arg in kwargs}
    gpu_info = get_gpu_device_info()
    flops_func_args = {}
    if flops_func:
        flops_func_args = {arg: kwargs[arg] for arg in inspect.getfullargspec(flops_func).args if arg in kwargs}
    measurements = {"elapsed": [], "perf_flops": [], "mfu": []}
    output = None
    for _ in range(repeats):
        torch.cuda.synchronize()
        start = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        start.record()
        output = func(**func_args)
        end.record()
        torch.cuda.synchronize()
        elapsed = start.elapsed_time(end)
        measurements["elapsed"].append(elapsed)
        if flops_func:
            total_flops = flops_func(**flops_func_args)
            measurements["perf_flops"].append((total_flops / elapsed) / 1e6)
            if gpu_info:
                measurements["mfu"].append(100 * (total_flops / elapsed) / 1e9 / gpu_info["fp16_tflops"])
    elapsed = sum(measurements["elapsed"]) / repeats
    total_flops = perf_flops = mfu = None
    if flops_func:
        total_flops = flops_func(**flops_func_args)
        perf_flops = total_flops / elapsed
        if gpu_info:
            mfu = 100 * perf_flops / 1e9 / gpu_info["fp16_tflops"]
    return {
        "output": output,
        "elapsed": elapsed,
        "func_name": func.__name__,
        "total_flops": total_flops / 1e9 if flops_func else None,
        "perf_flops": perf_flops / 1e6 if flops_func else None,
        "mfu": mfu,
        "args": kwargs,
        "measurements": measurements,
    }


def export_benchmark_results(results, filepath):
    """`results` = list of lists of `timing_function` dicts; tensors in the arguments are dropped."""
    config_results = []
    for result in results:
        for res in result:
            res = dict(res)
            config = {k: v for k, v in res.pop("args").items() if not isinstance(v, torch.Tensor)}
            res.pop("output")
            config_results.append({"config": config, **res})
    with open(filepath, "w") as f:
        json.dump({"gpu_specs": get_gpu_device_info(), "results": config_results}, f, indent=4)


def format_benchmark_results(filepath):
    """Read an exported file back as (gpu_specs, DataFrame with one row per configuration and
    one `<func>_<field>` column per function and field)."""
    import pandas as pd
    with open(filepath, "r") as f:
        data = json.load(f)
    parsed, configs = [], []
    for result in data["results"]:
        result = dict(result)
        config = result.pop("config")
        func_name = result.pop("func_name")
        parsed.append({"config": config, **{f"{func_name}_{k}": v for k, v in result.items()}})
        configs.append(config)
    rows = []
    for config in configs:
        merged = {}
        for d in parsed:
            if d["config"] == config:
                merged.update({k: v for k, v in d.items() if k != "config"})
        rows.append({**config, **merged})
    df = pd.DataFrame(rows)
    df = df.loc[df.astype(str).drop_duplicates().index]
    return data["gpu_specs"], df
