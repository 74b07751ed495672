#!/usr/bin/env python3
"""Benchmark of the block-sparse attention forward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload T|C2|C3|C4|C5]

The default workload is T, the shape the 50 %-of-peak goal is stated on; C2, C3, C4 and C5 are measured
after it and reported under ``other_shapes``.  Every workload runs the library's default, reproducible
ascending walk except C4, whose headline figures use the opt-in clocked walk (``walk`` says which; C4's
ascending-walk kernel time is reported beside it).

A step is one ``HBSAttention`` call (one launch: the attention kernel, whose scheduler reads the mask
itself; pre-pass + attention kernel where that form does not apply; block metadata
pre-computed and passed in as the reference's sweep does, reference
test/test_speedup.py:101-102,152) on a synthetic problem already resident in HBM.  The
timed region is ``synchronize -> K calls -> synchronize`` (reference hbsattn/benchmark.py:72-81
brackets every call; the per-call figure measured that way is reported as
``per_call_sync_ms``).  Prints ONE JSON line.

``value`` is effective TFLOP/s over kept blocks: 4 * D * sum(rows(qb) * cols(kb)) over the
visited block pairs of every q head, computed on the host from the mask, divided by the
time of one step.  ``roofline`` prices the attention kernel alone (its launches are
bracketed by events on the stream they are queued on); ``cpu_baseline`` times the CPU
oracle (a port of the reference's golden implementation) on a bounded sample of the same
workload on this machine's host cores.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA, vendor figure
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E, vendor figure
RIDGE_FLOP_PER_BYTE = PEAK_BF16_TFLOPS * 1e12 / (PEAK_HBM_GBS * 1e9)

DESCRIPTIONS = {
    "C2": "C2: batch 8 x 8192 tokens, Hq=Hk=32, D=128, 128x128 blocks, keep 0.1 + diagonal, causal, bf16",
    "T": "T: batch 8 x 32768 tokens, Hq=Hk=32, D=128, 128x128 blocks, keep 0.1 + diagonal, causal, bf16",
    "C3": "C3: batch 8, lengths U[2048,16384], Hq=32 Hk=8, D=128, 64x128 blocks, keep 0.3 + diagonal, causal, bf16",
    "C4": "C4: batch 8 x 65536 tokens, Hq=Hk=32, D=128, 128x128 blocks, keep 0.3, non-causal, bf16",
    "C5": "C5: q lens 3000/5120/777/4096, k lens 6000/5120/4100/8192, Hq=16 Hk=2, D=64, 80x48 blocks, keep 0.5, causal, scale 0.1, bf16",
}
SHAPES = {"C2": "B8 H32 D128 L=8K", "T": "B8 H32 D128 L=32K", "C3": "B8 Hq32/Hk8 D128 varlen", "C4": "B8 H32 D128 L=64K",
          "C5": "B4 Hq16/Hk2 D64 q!=k"}
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")


def kernel_sources_sha16() -> str:
    """Content hash of the kernel sources (hbsattn_amd/csrc): what a counter measurement belongs to."""
    import hashlib

    h = hashlib.sha256()
    d = os.path.join(ROOT, "hbsattn_amd", "csrc")
    for name in sorted(os.listdir(d)):
        if name.endswith((".hip", ".h", ".cpp")):
            h.update(name.encode())
            with open(os.path.join(d, name), "rb") as f:
                h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic(name):
    """HBM bytes per launch of the attention kernel for a workload, from profiles/traffic.json: rocprofv3
    counter runs of this program (FETCH_SIZE and WRITE_SIZE in KiB per dispatch, scaled by what the same
    counters read for a 1 GiB device-to-device copy).  A counter run needs the profiler, so the figure is
    read, not measured live; it is dropped when the kernel sources have changed since it was taken."""
    try:
        with open(TRAFFIC_FILE) as f:
            table = json.load(f)
    except (OSError, ValueError):
        return None, "profiles/traffic.json missing"
    entry = table.get("workloads", {}).get(name)
    if entry is None:
        return None, "no counter run for this workload"
    if table.get("kernel_sources_sha16") != kernel_sources_sha16():
        return None, f"stale: counters were taken at kernel sources {table.get('kernel_sources_sha16')}"
    return float(entry["bytes"]), entry.get("profile", "")


def time_steps(fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps * 1e3


def time_per_call_sync(fn, steps):
    ts = []
    for _ in range(steps):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        ts.append((time.perf_counter() - t0) * 1e3)
    return sum(ts) / len(ts)


def time_kernel_events(fn, steps):
    """Average device time of ``fn``'s launches, from event pairs recorded on the current
    stream (the stream the library launches on)."""
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for a, b in evs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    return sum(a.elapsed_time(b) for a, b in evs) / steps


CLOCKED_WALK = ("C4",)   # workloads measured with the opt-in clocked walk (K + V of a kv head above 192 MiB)


def measure(name, steps, warmup):
    from hbsattn_amd import HBSAttention, set_deterministic
    from hbsattn_amd.interface import hbsa_prepare, hbsa_run
    from hbsattn_amd.workloads import count_work, make_workload

    w = make_workload(name, device="cuda", gen_device="device")
    work = count_work(w)
    clocked = name in CLOCKED_WALK
    was_deterministic = set_deterministic(not clocked)
    try:
        res = _measure(w, work, name, steps, warmup, HBSAttention, hbsa_prepare, hbsa_run)
        res["walk"] = "clocked (opt-in: set_deterministic(False)); results vary in their last bits from run to run" \
            if clocked else "ascending (the default; bitwise reproducible)"
        if clocked:
            set_deterministic(True)
            prepared = hbsa_prepare(w.cu_q_seqlens, w.cu_k_seqlens, w.block_mask, w.q_block_size, w.k_block_size, w.causal,
                                    w.q_meta[0], w.q_meta[2], w.q_meta[3], w.k_meta[0], w.k_meta[3])
            res["attention_kernel_ms_ascending_walk"] = time_kernel_events(
                lambda: hbsa_run(w.q, w.k, w.v, prepared, w.softmax_scale), max(3, steps // 2))
    finally:
        set_deterministic(was_deterministic)
    return w, res


def settle(fn, seconds=0.25):
    """Set-up before any measurement of a workload: calls until `seconds` of wall time have passed, so that the
    device has left its idle clocks, the allocator holds the output buffer and every page of the tensors has been
    touched.  (Measured without it, the first 20 ms after a workload is built run a tenth slower, which is what a
    short workload's whole measurement takes.)  The W warm-up steps and the K timed steps come after it."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(4):
            fn()
        torch.cuda.synchronize()


def _measure(w, work, name, steps, warmup, HBSAttention, hbsa_prepare, hbsa_run):
    args = w.args()
    step = lambda: HBSAttention(*args)
    settle(step)
    ms = time_steps(step, steps, warmup)
    per_call = time_per_call_sync(step, steps)
    # the same with the prepared mask of the first call reused by the following ones (opt-in mode of the
    # operator for static sparsity patterns): one kernel launch per call
    from hbsattn_amd import clear_prepared_cache, set_prepared_cache_size
    previous = set_prepared_cache_size(2)
    ms_reused = time_steps(step, steps, max(1, warmup))
    set_prepared_cache_size(previous)
    clear_prepared_cache()
    prepared = hbsa_prepare(w.cu_q_seqlens, w.cu_k_seqlens, w.block_mask, w.q_block_size, w.k_block_size, w.causal,
                            w.q_meta[0], w.q_meta[2], w.q_meta[3], w.k_meta[0], w.k_meta[3])
    prepared_kernel_ms = time_kernel_events(lambda: hbsa_run(w.q, w.k, w.v, prepared, w.softmax_scale), steps)
    prep_ms = time_kernel_events(
        lambda: hbsa_prepare(w.cu_q_seqlens, w.cu_k_seqlens, w.block_mask, w.q_block_size, w.k_block_size, w.causal,
                             w.q_meta[0], w.q_meta[2], w.q_meta[3], w.k_meta[0], w.k_meta[3]), steps)
    # the launches a step makes: 1 = the attention kernel alone, its scheduler reading the mask itself (then the
    # events around a whole call bracket exactly that kernel), 2 = pre-pass + attention kernel on a workspace
    from hbsattn_amd import _lib
    launches = _lib.load().hbsa_fwd_launches(_lib.DTYPE_BF16, len(w.cu_q) - 1, w.k.shape[0], w.q.shape[1], w.k.shape[1],
                                             w.q.shape[2], w.q_meta[0], w.k_meta[0], w.q_block_size, w.k_block_size,
                                             w.block_mask.stride(2), torch.cuda.current_stream().cuda_stream)
    kernel_ms = time_kernel_events(step, steps) if launches == 1 else prepared_kernel_ms
    res = {
        "ms_per_step": ms,
        "per_call_sync_ms": per_call,
        "ms_per_step_mask_reused": ms_reused,
        "launches_per_step": launches,
        "attention_kernel_ms": kernel_ms,
        "attention_kernel_ms_on_prepared_mask": prepared_kernel_ms,
        "prepass_ms": prep_ms,
        "tflops": work["flops"] / ms / 1e9,
        "tflops_exact_elements": work["flops_exact"] / ms / 1e9,
        "flops": work["flops"],
        "bytes": work["bytes"],
        "visited_pairs": work["visited_pairs"],
    }
    traffic, traffic_note = measured_traffic(name)
    intensity = work["flops"] / work["bytes"]
    if intensity >= RIDGE_FLOP_PER_BYTE:   # right of the ridge at 2500 TFLOP/s / 8 TB/s = 312.5 FLOP/B
        ach = work["flops"] / kernel_ms / 1e9
        res["roofline"] = {"bound": "mfma", "achieved": ach, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                           "frac": ach / PEAK_BF16_TFLOPS, "traffic": traffic, "traffic_from_profile": traffic_note,
                           "kernel": "hbsa_fwd_kernel", "kernel_ms": kernel_ms, "algorithmic_flops": work["flops"],
                           "flop_per_byte": intensity}
    else:
        ach = work["bytes"] / kernel_ms / 1e6
        res["roofline"] = {"bound": "hbm", "achieved": ach, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                           "frac": ach / PEAK_HBM_GBS, "traffic": traffic, "traffic_from_profile": traffic_note,
                           "kernel": "hbsa_fwd_kernel", "kernel_ms": kernel_ms, "algorithmic_bytes": work["bytes"],
                           "flop_per_byte": intensity,
                           "mfma_frac": work["flops"] / kernel_ms / 1e9 / PEAK_BF16_TFLOPS}
    if traffic is not None:
        # the profiled HBM bytes per launch over this run's kernel time: how much of the 8 TB/s the kernel's
        # actual traffic (re-reads of K/V blocks included) takes, whatever roof the algorithmic figures name
        res["roofline"]["traffic_gb_s"] = traffic / kernel_ms / 1e6
        res["roofline"]["traffic_frac_of_hbm_peak"] = traffic / kernel_ms / 1e6 / PEAK_HBM_GBS
    return res


def measure_backward(w, flops, steps):
    """Device time of one backward call (dq and dk/dv kernels) for the workload's tensors, with
    event pairs on the launch stream; FLOPs counted as 2.5 x the forward's over kept blocks."""
    from hbsattn_amd.interface import hbsa_backward, hbsa_prepare, hbsa_run

    prepared = hbsa_prepare(w.cu_q_seqlens, w.cu_k_seqlens, w.block_mask, w.q_block_size, w.k_block_size, w.causal,
                            w.q_meta[0], w.q_meta[2], w.q_meta[3], w.k_meta[0], w.k_meta[3])
    out, lse = hbsa_run(w.q, w.k, w.v, prepared, w.softmax_scale, return_lse=True)
    dout = torch.randn(out.shape, dtype=torch.float32, device=out.device, generator=torch.Generator(out.device).manual_seed(5)).to(out.dtype)
    step = lambda: hbsa_backward(w.q, w.k, w.v, out, dout, lse, prepared, w.softmax_scale)
    for _ in range(min(3, steps)):
        step()
    ms = time_kernel_events(step, steps)
    return {"ms_per_call": ms, "tflops": 2.5 * flops / ms / 1e9, "flops_counted": "2.5 x forward FLOPs over kept blocks",
            "kernels": "hbsa_bwd_dq_kernel + hbsa_bwd_dkv8_kernel (hbsa_bwd_dkv_kernel below D=128)"}


def cpu_baseline(w, budget_s=20.0):
    """The CPU oracle on (sequence, kv head) pairs of the workload, in sequence-major order, one
    pair at a time until the budget is spent; throughput in the metric's unit from the sample's own
    visited blocks."""
    from hbsattn_amd.workloads import Workload, count_work
    from oracle.dense import hbsa_oracle

    ratio = w.q.shape[1] // w.k.shape[1]
    cu_nqb, cu_nkb = w.q_meta[3].tolist(), w.k_meta[3].tolist()
    threads = torch.get_num_threads()
    done_flops, spent, pairs = 0.0, 0.0, 0
    tokens = ""
    for b in range(len(w.cu_q) - 1):
        qs, qe, ks, ke = w.cu_q[b], w.cu_q[b + 1], w.cu_k[b], w.cu_k[b + 1]
        tokens = f"{qe - qs} q x {ke - ks} k tokens"
        for hk in range(w.k.shape[1]):
            q_heads = list(range(hk * ratio, (hk + 1) * ratio))
            q_b = w.q[qs:qe][:, q_heads].cpu()
            k_b, v_b = w.k[ks:ke][:, hk:hk + 1].cpu(), w.v[ks:ke][:, hk:hk + 1].cpu()
            m_b = w.block_mask[hk:hk + 1, cu_nqb[b]:cu_nqb[b + 1], cu_nkb[b]:cu_nkb[b + 1]].cpu()
            sub = Workload("sample", q_b, k_b, v_b, [0, qe - qs], [0, ke - ks], None, None, m_b, w.q_block_size,
                           w.k_block_size, w.causal, w.softmax_scale)
            t0 = time.perf_counter()
            hbsa_oracle(q_b, k_b, v_b, sub.cu_q, sub.cu_k, m_b, w.q_block_size, w.k_block_size, w.causal,
                        w.softmax_scale)
            spent += time.perf_counter() - t0
            done_flops += count_work(sub)["flops"]
            pairs += 1
            if spent >= budget_s:
                break
        if spent >= budget_s:
            break
    return {
        "value": done_flops / spent / 1e12,
        "unit": "TFLOP/s",
        "cores": threads,
        "kind": "port",
        "sample": f"first {pairs} (sequence, kv head) pairs of the workload in sequence-major order (last one {tokens}, "
                  f"{ratio} q head(s) per kv head), fp32 masked-dense torch oracle, {spent:.1f} s; effective FLOPs "
                  "counted over the sample's visited blocks like the GPU figure",
        "host_cpus": os.cpu_count(),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="T", choices=sorted(DESCRIPTIONS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-others", action="store_true",
                    help="skip the extra measurements at the other full-size shapes (reported under 'other_shapes')")
    ap.add_argument("--others", default="C2,C3,C4,C5", help="comma-separated workloads measured besides --workload")
    ap.add_argument("--cpu-budget", type=float, default=20.0)
    ap.add_argument("--backward", action="store_true", help="also time the backward kernels (reported under 'backward')")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run only a 1 GiB device-to-device copy K times (the known-size kernel the HBM counters "
                         "of a profile are scaled by)")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; sequences and kv heads shard with no exchange, "
                 "so --gpus N>1 is not measured here (use --gpus 1)")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")

    if a.copy_calibration:
        n = 1 << 30
        src = torch.full((n // 4,), 1.0, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        ms = time_steps(lambda: dst.copy_(src), a.steps, a.warmup)
        print(json.dumps({"copy_bytes_read": n, "copy_bytes_written": n, "ms_per_copy": ms,
                          "GBps": 2 * n / ms / 1e6}))
        return

    w, res = measure(a.workload, a.steps, a.warmup)
    line = {
        "metric": f"effective TFLOP/s over kept blocks, block-sparse attention forward ({SHAPES[a.workload]})",
        "value": res["tflops"],
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "ms_per_step": res["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": DESCRIPTIONS[a.workload], "timing": "K calls between two synchronisations, "
                   "block metadata precomputed; one HBSAttention call per step"},
        "roofline": res["roofline"],
        "walk": res["walk"],
        "detail": {k: res[k] for k in ("launches_per_step", "per_call_sync_ms", "ms_per_step_mask_reused", "attention_kernel_ms",
                                       "attention_kernel_ms_on_prepared_mask", "prepass_ms", "tflops_exact_elements",
                                       "flops", "bytes", "visited_pairs")},
    }
    if a.workload == "T":
        line["goal"] = ">= 0.50 of bf16 dense MFMA peak at this shape"
    if a.backward:
        line["backward"] = measure_backward(w, res["flops"], max(1, a.steps // 5))
    if not a.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(w, a.cpu_budget)
    del w
    torch.cuda.empty_cache()
    if not a.no_others:
        line["other_shapes"] = {}
        for name in [n for n in a.others.split(",") if n and n != a.workload]:
            heavy = name == "C4"   # 0.2 s per call: a few steps are enough
            wo, t = measure(name, max(3, a.steps // 5) if heavy else a.steps, min(a.warmup, 2) if heavy else a.warmup)
            del wo
            torch.cuda.empty_cache()
            line["other_shapes"][name] = {"workload": DESCRIPTIONS[name], "ms_per_step": t["ms_per_step"],
                                          "ms_per_step_mask_reused": t["ms_per_step_mask_reused"],
                                          "launches_per_step": t["launches_per_step"],
                                          "tflops": t["tflops"], "attention_kernel_ms": t["attention_kernel_ms"],
                                          "attention_kernel_ms_on_prepared_mask": t["attention_kernel_ms_on_prepared_mask"],
                                          "prepass_ms": t["prepass_ms"], "walk": t["walk"], "roofline": t["roofline"]}
            if "attention_kernel_ms_ascending_walk" in t:
                line["other_shapes"][name]["attention_kernel_ms_ascending_walk"] = t["attention_kernel_ms_ascending_walk"]
    print(json.dumps(line))


if __name__ == "__main__":
    main()
