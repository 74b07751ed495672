"""Speed sweep with the arguments and JSON layout of the reference's ``test/test_speedup.py``.

    python -m hbsattn_amd.sweep --unit_seqlen 8192 --sparse_ratio 0.9 --causal \
        --save_benchmark_to_file sweep.json

One run measures one configuration (uniform sequence length, 128x128 blocks, bf16, as in
test_speedup.py:82-100) and appends one entry to the JSON file; a configuration already in the
file is skipped (test_speedup.py:53-69).  Entry keys are the reference's (test_speedup.py:210-221);
the dense baseline under ``flash_attn_base_result`` is torch's scaled_dot_product_attention on this
GPU (flash_attn is a CUDA package), and the two third-party block-sparse baselines, which do not
exist for this platform, are left empty, exactly as the reference leaves a baseline that failed.
``--sweep`` runs the README's series (unit_seqlen 2^7 .. 2^16) in one process.
"""
from __future__ import annotations

import argparse
import json
import os

import torch

from .benchmark import benchmark
from .interface import HBSAttention
from .utils import calculate_blocks

BLOCK = 128   # the reference fixes both block sizes to 128 for its sweep (test_speedup.py:82-84)


def make_block_mask(nhead_k, q_block_to_batch, cu_num_k_block, num_k_block, keep, device):
    """Random mask with keep probability ``keep``; the first k block of a q block's own sequence is
    always kept (test_speedup.py:104-113), so no query row is left without keys."""
    num_q_block = q_block_to_batch.numel()
    mask = torch.rand(nhead_k, num_q_block, num_k_block, device=device) < keep
    first = cu_num_k_block.to(device=device, dtype=torch.long)[q_block_to_batch.to(device=device, dtype=torch.long)]
    mask[:, torch.arange(num_q_block, device=device), first] = True
    return mask


def golden_masked_dense(q, k, v, batch, unit_seqlen, block_mask, causal, softmax_scale, head_chunk=4):
    """fp32 masked-dense attention on the GPU for the uniform-length sweep problem (the role of
    ``hbsattn_reference_v1_base`` under ``--golden_ref``, test_speedup.py:126-129)."""
    hq, d = q.shape[1], q.shape[2]
    scale = softmax_scale if softmax_scale is not None else d ** -0.5
    nb = unit_seqlen // BLOCK
    out = torch.empty_like(q, dtype=torch.float32)
    tri = torch.ones(unit_seqlen, unit_seqlen, dtype=torch.bool, device=q.device).tril() if causal else None
    for b in range(batch):
        rows = slice(b * unit_seqlen, (b + 1) * unit_seqlen)
        for h0 in range(0, hq, head_chunk):
            hs = slice(h0, min(h0 + head_chunk, hq))
            qq, kk, vv = (t[rows, hs].float().permute(1, 0, 2) for t in (q, k, v))
            s = torch.matmul(qq, kk.transpose(1, 2)) * scale
            keep = block_mask[hs, b * nb:(b + 1) * nb, b * nb:(b + 1) * nb]
            keep = keep.repeat_interleave(BLOCK, 1).repeat_interleave(BLOCK, 2)
            if tri is not None:
                keep = keep & tri
            s.masked_fill_(~keep, float("-inf"))
            out[rows, hs] = torch.matmul(torch.softmax(s, -1), vv).permute(1, 0, 2)
    return out


def dense_sdpa(q, k, v, batch, unit_seqlen, causal, softmax_scale):
    """Dense attention over the same tokens: the sweep's speed-of-dense reference line."""
    hq, d = q.shape[1], q.shape[2]
    qb, kb, vb = (t.view(batch, unit_seqlen, hq, d).transpose(1, 2) for t in (q, k, v))
    o = torch.nn.functional.scaled_dot_product_attention(qb, kb, vb, is_causal=causal, scale=softmax_scale)
    return o.transpose(1, 2).reshape(batch * unit_seqlen, hq, d)


def already_done(path, a) -> bool:
    if not os.path.exists(path):
        return False
    with open(path) as f:
        entries = json.load(f)
    return any(e.get("unit_seqlen") == a.unit_seqlen and e.get("headdim") == a.headdim and e.get("nhead_q") == a.nheads
               and e.get("causal") == a.causal and e.get("sparse_ratio") == a.sparse_ratio for e in entries)


def run_one(a) -> dict:
    assert a.unit_seqlen % BLOCK == 0, "unit_seqlen must be a multiple of the 128 block size"
    device = torch.device("cuda", torch.cuda.current_device())
    cu = torch.arange(0, a.batch_size + 1, dtype=torch.int32, device=device) * a.unit_seqlen
    total = a.batch_size * a.unit_seqlen
    q = torch.randn(total, a.nheads, a.headdim, device=device, dtype=torch.bfloat16)
    k = torch.randn(total, a.nheads, a.headdim, device=device, dtype=torch.bfloat16)
    v = torch.randn(total, a.nheads, a.headdim, device=device, dtype=torch.bfloat16)
    nqb, cu_qb, qb2b, cu_nqb = calculate_blocks(cu, BLOCK)
    nkb, cu_kb, kb2b, cu_nkb = calculate_blocks(cu, BLOCK)
    mask = make_block_mask(a.nheads, qb2b, cu_nkb, nkb, 1.0 - a.sparse_ratio, device)
    golden = (golden_masked_dense(q, k, v, a.batch_size, a.unit_seqlen, mask, a.causal, a.softmax_scale).to(q.dtype)
              if a.golden_ref else None)
    cfg = lambda name: {"golden": golden, "n_runs": a.nruns, "n_warmup": a.nwarmup, "name": name}

    def guarded(name, fn, *args):
        try:
            return benchmark(cfg(name), fn, *args)
        except Exception as e:   # a baseline that cannot run leaves an empty entry (test_speedup.py:140-142)
            print(f"Error benchmarking {name}: {e}")
            return {}

    dense = guarded("dense_sdpa", dense_sdpa, q, k, v, a.batch_size, a.unit_seqlen, a.causal, a.softmax_scale)
    if dense:
        dense["error"] = None   # dense attention is not expected to match the sparse golden
    meta = (nqb, cu_qb, qb2b, cu_nqb, nkb, cu_kb, kb2b, cu_nkb)
    ours = {mode: guarded(f"HBSAttention_{mode}_tilesize", HBSAttention, q, k, v, cu, cu, mask, BLOCK, BLOCK, a.causal,
                          a.softmax_scale, mode, *meta) for mode in ("auto", "fix")}
    return {
        "flash_attn_base_result": dense,
        "hbsattn(our fix)": ours["fix"],
        "hbsattn(our auto)": ours["auto"],
        "hanlab_block-sparse-attn": {},
        "flexattention": {},
        "unit_seqlen": a.unit_seqlen,
        "headdim": a.headdim,
        "nhead_q": a.nheads,
        "causal": a.causal,
        "sparse_ratio": a.sparse_ratio,
        "dense_baseline": "torch.nn.functional.scaled_dot_product_attention",
        "device": torch.cuda.get_device_name(device),
    }


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--causal", action="store_true", default=False)
    ap.add_argument("--softmax_scale", type=float, default=None)
    ap.add_argument("--nruns", type=int, default=15)     # README.md:121 of the reference: 15 runs, 5 dropped
    ap.add_argument("--nwarmup", type=int, default=5)
    ap.add_argument("--headdim", type=int, default=128)
    ap.add_argument("--unit_seqlen", type=int, default=256)
    ap.add_argument("--nheads", type=int, default=32)
    ap.add_argument("--batch_size", type=int, default=8)
    ap.add_argument("--save_benchmark_to_file", type=str, default="./benchmark_all_results.json")
    ap.add_argument("--sparse_ratio", type=float, default=0.3)
    ap.add_argument("--golden_ref", action="store_true", default=False)
    ap.add_argument("--sweep", action="store_true", help="run unit_seqlen = 2^7 .. 2^16 instead of one length")
    a = ap.parse_args(argv)
    if not torch.cuda.is_available():
        raise SystemExit("hbsattn_amd.sweep needs an MI355X; no GPU is visible")
    lengths = [1 << e for e in range(7, 17)] if a.sweep else [a.unit_seqlen]
    for length in lengths:
        a.unit_seqlen = length
        path = a.save_benchmark_to_file
        if path and already_done(path, a):
            print(f"[INFO] unit_seqlen={length} headdim={a.headdim} nheads={a.nheads} causal={a.causal} "
                  f"sparse_ratio={a.sparse_ratio} already in {path}: skipped")
            continue
        entry = run_one(a)
        torch.cuda.empty_cache()
        if path:
            entries = json.load(open(path)) if os.path.exists(path) else []
            entries.append(entry)
            with open(path, "w") as f:
                json.dump(entries, f, indent=4)
            print(f"saved to {path} ({len(entries)} entries)")


if __name__ == "__main__":
    main()
