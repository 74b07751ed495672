"""The speed-sweep harness on the GPU: one reduced configuration through ``hbsattn_amd.sweep.main``
(reference test/test_speedup.py:36-238) and through ``hbsattn_amd.benchmark`` (reference
hbsattn/benchmark.py:50-105), with the golden comparison switched on."""
import json

import pytest
import torch

from hbsattn_amd import HBSAttention, calculate_blocks, sweep
from hbsattn_amd.benchmark import benchmark
from oracle.dense import hbsa_oracle

pytestmark = pytest.mark.gpu

# keys of one entry of the reference's result file (test/test_speedup.py:210-221)
REFERENCE_KEYS = {"flash_attn_base_result", "hbsattn(our fix)", "hbsattn(our auto)", "hanlab_block-sparse-attn",
                  "flexattention", "unit_seqlen", "headdim", "nhead_q", "causal", "sparse_ratio"}
# keys of one timing result (reference hbsattn/benchmark.py:93-103)
RESULT_KEYS = {"runtime_mean", "runtime_std", "runtime_min", "runtime_max", "all_times", "error"}


def test_sweep_writes_the_reference_layout_checks_the_golden_and_skips_what_is_present(tmp_path, capsys):
    path = tmp_path / "sweep.json"
    argv = ["--unit_seqlen", "512", "--batch_size", "2", "--nheads", "4", "--golden_ref", "--nruns", "3", "--nwarmup", "1",
            "--causal", "--sparse_ratio", "0.5", "--save_benchmark_to_file", str(path)]
    sweep.main(argv)
    entries = json.loads(path.read_text())
    assert len(entries) == 1
    e = entries[0]
    assert REFERENCE_KEYS <= set(e) and set(e) - REFERENCE_KEYS == {"dense_baseline", "device"}
    assert (e["unit_seqlen"], e["headdim"], e["nhead_q"], e["causal"], e["sparse_ratio"]) == (512, 128, 4, True, 0.5)
    for key in ("hbsattn(our fix)", "hbsattn(our auto)"):
        r = e[key]
        assert set(r) == RESULT_KEYS
        assert len(r["all_times"]) == 2 and r["runtime_min"] > 0          # 3 runs, 1 warm-up run dropped
        assert set(r["error"]) == {"max_abs", "mean_abs", "max_rel", "mean_rel"}
        assert r["error"]["max_abs"] <= 2e-2 and r["error"]["mean_abs"] <= 2e-3, (key, r["error"])
    assert set(e["flash_attn_base_result"]) == RESULT_KEYS and e["flash_attn_base_result"]["error"] is None
    assert e["hanlab_block-sparse-attn"] == {} and e["flexattention"] == {}
    # the same configuration again: found in the file, nothing is run or appended
    capsys.readouterr()
    sweep.main(argv)
    assert "skipped" in capsys.readouterr().out
    assert len(json.loads(path.read_text())) == 1
    # another configuration is appended to the same file
    sweep.main(argv[:-1] + [str(path), "--headdim", "64"])
    assert [x["headdim"] for x in json.loads(path.read_text())] == [128, 64]


def test_sweep_golden_matches_the_cpu_oracle():
    """``sweep.golden_masked_dense`` (the harness's own fp32 golden, computed on the GPU) against the
    oracle on the sweep's problem shape, causal and not."""
    torch.manual_seed(5)
    batch, unit, heads, d = 2, 384, 4, 64
    dev = torch.device("cuda")
    cu = torch.arange(0, batch + 1, dtype=torch.int32, device=dev) * unit
    q, k, v = (torch.randn(batch * unit, heads, d, device=dev, dtype=torch.bfloat16) for _ in range(3))
    nqb, _, qb2b, _ = calculate_blocks(cu, sweep.BLOCK)
    nkb, _, _, cu_nkb = calculate_blocks(cu, sweep.BLOCK)
    mask = sweep.make_block_mask(heads, qb2b, cu_nkb, nkb, 0.4, dev)
    assert mask[:, torch.arange(nqb), cu_nkb.long()[qb2b.long()]].all()      # first k block of each sequence kept
    for causal in (True, False):
        got = sweep.golden_masked_dense(q, k, v, batch, unit, mask, causal, None)
        ref = hbsa_oracle(q.cpu(), k.cpu(), v.cpu(), cu.tolist(), cu.tolist(), mask.cpu(), sweep.BLOCK, sweep.BLOCK, causal,
                          None)
        assert (got.cpu() - ref).abs().max().item() <= 1e-5, causal


def test_benchmark_harness_times_the_operator_and_reports_its_error():
    torch.manual_seed(6)
    dev = torch.device("cuda")
    cu = torch.tensor([0, 300, 812], dtype=torch.int32, device=dev)
    q, k, v = (torch.randn(812, 4, 64, device=dev, dtype=torch.bfloat16) for _ in range(3))
    nqb, _, qb2b, _ = calculate_blocks(cu, 64)
    nkb, _, _, cu_nkb = calculate_blocks(cu, 64)
    mask = sweep.make_block_mask(4, qb2b, cu_nkb, nkb, 0.5, dev)
    golden = hbsa_oracle(q.cpu(), k.cpu(), v.cpu(), cu.tolist(), cu.tolist(), mask.cpu(), 64, 64, True, None).to(dev)
    res = benchmark({"golden": golden, "n_runs": 4, "n_warmup": 2, "name": "HBSAttention"}, HBSAttention, q, k, v, cu, cu,
                    mask, 64, 64, True, None)
    assert set(res) == RESULT_KEYS and len(res["all_times"]) == 2
    assert res["error"]["max_abs"] <= 2e-2 and res["error"]["mean_abs"] <= 2e-3
