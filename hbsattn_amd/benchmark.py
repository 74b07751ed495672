"""Timing and error harness with the call shape and result schema of the reference's
``hbsattn/benchmark.py`` (``benchmark`` at :50-105, ``_check_correctness`` at :6-47).

Method (reference benchmark.py:72-87): every run is ``synchronize -> perf_counter -> call ->
synchronize``; the first ``n_warmup`` runs are dropped; the first run's result is compared with
``golden`` when one is given.  The result dictionary has the reference's keys
(``runtime_mean/std/min/max``, ``all_times``, ``error`` with ``max_abs/mean_abs/max_rel/mean_rel``)
so its JSON files can be laid over the reference's.
"""
from __future__ import annotations

import time
from typing import Any, Callable, Dict, Optional

import numpy as np
import torch


def _sync() -> None:
    if torch.cuda.is_available():
        torch.cuda.synchronize()


def _check_correctness(golden: torch.Tensor, result: torch.Tensor, name: str) -> dict:
    """Absolute and relative error of ``result`` against ``golden`` (relative error uses the
    reference's denominator ``1e-4 + max(|golden|, |result|)``, benchmark.py:20)."""
    result = result.to(golden.device)
    if golden.shape != result.shape and golden.ndim == 3 and result.ndim == 4:
        # a [B, H, S, D] result against a packed [B*S, H, D] golden (benchmark.py:11-17)
        b, h, s_len, d = result.shape
        result = result.permute(0, 2, 1, 3).reshape(b * s_len, h, d)
    g, r = golden.float(), result.float()
    abs_err = (g - r).abs()
    rel_err = abs_err / (1e-4 + torch.maximum(g.abs(), r.abs()))
    info = {
        "max_abs": abs_err.max().item(),
        "mean_abs": abs_err.mean().item(),
        "max_rel": rel_err.max().item(),
        "mean_rel": rel_err.mean().item(),
    }
    where_abs = tuple(np.unravel_index(int(abs_err.argmax()), abs_err.shape))
    where_rel = tuple(np.unravel_index(int(rel_err.argmax()), rel_err.shape))
    print(f"[{name}] mean rel {info['mean_rel']:.3e}  mean abs {info['mean_abs']:.3e}")
    print(f"[{name}] max rel {info['max_rel']:.3e} at {tuple(int(i) for i in where_rel)}: "
          f"golden {g[where_rel].item():.6g} result {r[where_rel].item():.6g}")
    print(f"[{name}] max abs {info['max_abs']:.3e} at {tuple(int(i) for i in where_abs)}: "
          f"golden {g[where_abs].item():.6g} result {r[where_abs].item():.6g}")
    return info


def benchmark(benchmark_config: Dict[str, Any], func: Callable, *args, **kwargs) -> dict:
    """Times ``func(*args, **kwargs)``.  ``benchmark_config`` keys: ``golden`` (tensor or None),
    ``n_runs`` (default 1), ``n_warmup`` (default 0), ``name``."""
    golden: Optional[torch.Tensor] = benchmark_config.get("golden")
    if golden is not None:
        assert not torch.isnan(golden).any(), "golden is not None, but it contains NaN"
    n_runs = int(benchmark_config.get("n_runs", 1))
    n_warmup = int(benchmark_config.get("n_warmup", 0))
    name = benchmark_config.get("name", getattr(func, "__name__", "func"))
    print(f"===== benchmarking {name} =====")

    kept, error_info = [], None
    for run in range(n_runs):
        _sync()
        t0 = time.perf_counter()
        result = func(*args, **kwargs)
        _sync()
        elapsed = time.perf_counter() - t0
        if run == 0 and golden is not None:
            error_info = _check_correctness(golden, result, name)
        if run >= n_warmup:
            kept.append(elapsed)
    times = np.asarray(kept, dtype=np.float64)
    stats = {
        "runtime_mean": float(times.mean()),
        "runtime_std": float(times.std()),
        "runtime_min": float(times.min()),
        "runtime_max": float(times.max()),
        "all_times": times.tolist(),
        "error": error_info,
    }
    print(f"{name}: {stats['runtime_mean']:.3e} +- {stats['runtime_std']:.3e} s over {len(kept)} runs "
          f"({n_warmup} warm-up runs dropped)")
    return stats
