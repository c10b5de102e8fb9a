"""Benchmark-result schema of the reference (triteia/python/utils/benchmark.py:10-133), so that its
plotting scripts read results measured here: `timing_function` returns the same dict, and
`export_benchmark_results` writes the same JSON ({"gpu_specs": ..., "results": [{"config": ..., ...}]})."""
import inspect
import json

import torch

from triteia_amd.python.configs.gpus import get_gpu_device_info


def _accepted(fn, kwargs):
    """The entries of `kwargs` that `fn` names as parameters."""
    names = inspect.signature(fn).parameters
    return {name: value for name, value in kwargs.items() if name in names}


def timing_function(func, flops_func, kwargs, repeats=1):
    """Time `func` on the entries of `kwargs` it takes, `repeats` times, and report in the reference's
    result schema (triteia/python/utils/benchmark.py:52-61: the keys below; elapsed in ms, total_flops in
    GFLOP, perf_flops in GFLOP/s, mfu in percent of the device's fp16 peak or None for an unknown device).

    All repeats are enqueued back to back, each between its own pair of events, and the events are read
    once at the end: no host synchronisation falls between two timed calls."""
    call_args = _accepted(func, kwargs)
    flops = float(flops_func(**_accepted(flops_func, kwargs))) if flops_func else None
    peak = (get_gpu_device_info() or {}).get("fp16_tflops")

    marks = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(max(repeats, 1))]
    output = None
    torch.cuda.synchronize()
    for begin, end in marks:
        begin.record()
        output = func(**call_args)
        end.record()
    torch.cuda.synchronize()
    times_ms = [begin.elapsed_time(end) for begin, end in marks]

    def rates(ms):
        """(GFLOP/s, % of peak) of one duration."""
        if flops is None:
            return None, None
        gflops = flops / ms / 1e6
        return gflops, (100.0 * gflops / 1e3 / peak if peak else None)

    per_call = [rates(ms) for ms in times_ms]
    mean_ms = sum(times_ms) / len(times_ms)
    mean_gflops, mean_mfu = rates(mean_ms)
    return {
        "output": output,
        "elapsed": mean_ms,
        "func_name": func.__name__,
        "total_flops": flops / 1e9 if flops is not None else None,
        "perf_flops": mean_gflops,
        "mfu": mean_mfu,
        "args": kwargs,
        "measurements": {
            "elapsed": times_ms,
            "perf_flops": [g for g, _ in per_call if g is not None],
            "mfu": [u for _, u in per_call if u is not None],
        },
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
