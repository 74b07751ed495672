"""Host-side checks of the timing/error harness (schema of reference hbsattn/benchmark.py:98-105)."""
import json

import pytest
import torch

from hbsattn_amd.benchmark import _check_correctness, benchmark
from hbsattn_amd import sweep


def test_benchmark_schema_and_warmup_drop():
    calls = []

    def f(x, scale=1.0):
        calls.append(1)
        return x * scale

    x = torch.arange(6.0).reshape(2, 3)
    res = benchmark({"golden": x * 2, "n_runs": 5, "n_warmup": 2, "name": "f"}, f, x, scale=2.0)
    assert len(calls) == 5
    assert set(res) == {"runtime_mean", "runtime_std", "runtime_min", "runtime_max", "all_times", "error"}
    assert len(res["all_times"]) == 3
    assert res["runtime_min"] <= res["runtime_mean"] <= res["runtime_max"]
    assert res["error"] == {"max_abs": 0.0, "mean_abs": 0.0, "max_rel": 0.0, "mean_rel": 0.0}
    json.dumps(res)   # the sweep stores it as JSON


def test_benchmark_without_golden_and_nan_golden():
    res = benchmark({"n_runs": 1}, lambda: torch.zeros(1))
    assert res["error"] is None and len(res["all_times"]) == 1
    with pytest.raises(AssertionError, match="NaN"):
        benchmark({"golden": torch.tensor([float("nan")])}, lambda: torch.zeros(1))


def test_check_correctness_values_and_layout_conversion():
    golden = torch.tensor([[[1.0, -2.0]], [[0.0, 4.0]]])           # [S=2, H=1, D=2]
    result = torch.tensor([[[1.5, -2.0]], [[0.0, 3.0]]])
    info = _check_correctness(golden, result, "t")
    assert info["max_abs"] == pytest.approx(1.0)
    assert info["mean_abs"] == pytest.approx(1.5 / 4)
    assert info["max_rel"] == pytest.approx(0.5 / (1e-4 + 1.5))
    batched = result.reshape(1, 2, 1, 2).permute(0, 2, 1, 3)        # [B=1, H=1, S=2, D=2]
    assert _check_correctness(golden, batched, "t4") == info


def test_sweep_mask_keeps_first_block_of_own_sequence():
    from hbsattn_amd.utils import calculate_blocks
    cu = torch.tensor([0, 256, 512, 768], dtype=torch.int32)
    nqb, _, qb2b, _ = calculate_blocks(cu, 128)
    nkb, _, _, cu_nkb = calculate_blocks(cu, 128)
    m = sweep.make_block_mask(3, qb2b, cu_nkb, nkb, 0.0, torch.device("cpu"))
    expect = torch.zeros(3, nqb, nkb, dtype=torch.bool)
    for i in range(nqb):
        expect[:, i, 2 * (i // 2)] = True
    assert torch.equal(m, expect)


def test_sweep_skip_logic(tmp_path):
    p = tmp_path / "r.json"
    p.write_text(json.dumps([{"unit_seqlen": 256, "headdim": 128, "nhead_q": 32, "causal": True, "sparse_ratio": 0.9}]))
    def ns(**kw):
        import argparse
        base = dict(unit_seqlen=256, headdim=128, nheads=32, causal=True, sparse_ratio=0.9)
        base.update(kw)
        return argparse.Namespace(**base)

    assert sweep.already_done(str(p), ns())
    assert not sweep.already_done(str(p), ns(causal=False))
    assert not sweep.already_done(str(tmp_path / "missing.json"), ns())
