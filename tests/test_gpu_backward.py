"""Backward parity on an MI355X: dq, dk, dv of the HIP kernels (through the C ABI, via the autograd
operator) against the float32 gradient oracle (``oracle.grads``) on the same seeded inputs.

The reference has no backward to compare with (reference ``hbsattn/hbsa_interface.py:31-32``); the
oracle is pinned in ``tests/test_oracle_grads.py``.  Tolerance for 16-bit tensors against float32:
max-abs error at most 1e-2 of the largest gradient magnitude (at least 1), mean-abs at most 2e-3 or 1e-2
of the mean gradient magnitude, whichever is larger.
"""
import pytest
import torch

from oracle.dense import hbsa_oracle
from oracle.grads import hbsa_oracle_grads

pytestmark = pytest.mark.gpu

MAX_REL_TOL = 1e-2
MEAN_ABS_TOL = 2e-3
MEAN_REL_TOL = 1e-2   # of the mean gradient magnitude, where that is the larger bound (sharp softmax, large gradients)


def _problem(seed, q_lens, k_lens, hq, hk, d, qbs, kbs, keep, dtype):
    from hbsattn_amd import calculate_blocks
    g = torch.Generator().manual_seed(seed)
    cu_q, cu_k = [0], [0]
    for a, b in zip(q_lens, k_lens):
        cu_q.append(cu_q[-1] + a)
        cu_k.append(cu_k[-1] + b)
    q = torch.randn(cu_q[-1], hq, d, generator=g).to(dtype)
    k = torch.randn(cu_k[-1], hk, d, generator=g).to(dtype)
    v = torch.randn(cu_k[-1], hk, d, generator=g).to(dtype)
    do = torch.randn(cu_q[-1], hq, d, generator=g).to(dtype)
    cq = torch.tensor(cu_q, dtype=torch.int32, device="cuda")
    ck = torch.tensor(cu_k, dtype=torch.int32, device="cuda")
    nq, nk = calculate_blocks(cq, qbs)[0], calculate_blocks(ck, kbs)[0]
    mask = torch.rand(hk, nq, nk, generator=g) < keep
    return q, k, v, do, cu_q, cu_k, cq, ck, mask


def _gpu_grads(q, k, v, do, cq, ck, mask, qbs, kbs, causal, scale):
    from hbsattn_amd import HBSAttention
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out = HBSAttention(qd, kd, vd, cq, ck, mask.cuda(), qbs, kbs, causal, scale)
    out.backward(do.cuda())
    torch.cuda.synchronize()
    return out.detach(), qd.grad, kd.grad, vd.grad


def _check(got, ref, what):
    got = got.float().cpu()
    assert torch.isfinite(got).all(), f"{what}: non-finite gradient"
    err = (got - ref).abs()
    lim = MAX_REL_TOL * max(1.0, ref.abs().max().item())
    assert err.max().item() <= lim, f"{what}: max-abs {err.max().item():.3e} > {lim:.3e}"
    mean_lim = max(MEAN_ABS_TOL, MEAN_REL_TOL * ref.abs().mean().item())
    assert err.mean().item() <= mean_lim, f"{what}: mean-abs {err.mean().item():.3e} > {mean_lim:.3e}"


CASES = [
    # seed, q_lens, k_lens, hq, hk, d, qbs, kbs, keep, causal, scale
    (1, [64], [64], 1, 1, 32, 32, 32, 1.1, False, None),
    (2, [64], [64], 1, 1, 128, 32, 32, 1.1, True, None),
    (3, [100, 37], [80, 130], 4, 2, 64, 32, 48, 0.6, True, None),
    (4, [300, 129, 5], [257, 129, 70], 6, 2, 128, 128, 128, 0.5, False, None),
    (5, [300, 129, 5], [257, 129, 70], 6, 2, 128, 64, 256, 0.5, True, 0.2),
    (6, [512, 1000], [512, 1000], 8, 8, 128, 128, 128, 0.3, True, None),
    (7, [200, 1], [1, 333], 8, 1, 64, 80, 48, 0.7, False, -0.1),
    (8, [33, 77, 190], [190, 33, 77], 2, 2, 32, 16, 16, 0.4, True, None),
    (9, [700, 130], [130, 700], 4, 1, 128, 256, 16, 0.5, True, None),
    (10, [513], [1029], 2, 2, 128, 64, 192, 0.5, False, None),
    (11, [200, 150], [180, 260], 16, 8, 64, 64, 64, 0.5, True, None),     # eight kv heads: the grid decoded by XCD
    (12, [300], [300], 16, 16, 128, 128, 128, 0.6, True, None),
    # more than 64 q blocks in a sequence (the dK/dV kernels look at them 64 at a time), many tiles per workgroup
    # (tiles are fetched two ahead), a ragged last block
    (13, [9000, 700], [9000, 450], 2, 2, 128, 128, 128, 0.15, True, None),
    (14, [8500], [8200], 2, 1, 64, 64, 128, 0.2, True, None),
    # more than 2048 k blocks in a sequence (the dQ kernel holds 64 words of its bit row at a time), 16-key blocks
    # (half-empty wave slots in the dK/dV kernels)
    (15, [200], [35000], 2, 1, 128, 64, 16, 0.05, False, None),
    (16, [150, 40], [33000, 100], 2, 2, 64, 32, 16, 0.05, True, None),
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("case", CASES, ids=[f"case{c[0]}" for c in CASES])
def test_gradients_match_oracle(case, dtype):
    seed, q_lens, k_lens, hq, hk, d, qbs, kbs, keep, causal, scale = case
    q, k, v, do, cu_q, cu_k, cq, ck, mask = _problem(seed, q_lens, k_lens, hq, hk, d, qbs, kbs, keep, dtype)
    print(f"backward case {case} {dtype}", flush=True)
    out, dq, dk, dv = _gpu_grads(q, k, v, do, cq, ck, mask, qbs, kbs, causal, scale)
    ref_out = hbsa_oracle(q, k, v, cu_q, cu_k, mask, qbs, kbs, causal, scale)
    assert (out.float().cpu() - ref_out).abs().max().item() <= 2e-2     # the forward that saved the log-sum-exp
    rdq, rdk, rdv = hbsa_oracle_grads(q, k, v, do, cu_q, cu_k, mask, qbs, kbs, causal, scale)
    _check(dq, rdq, "dq")
    _check(dk, rdk, "dk")
    _check(dv, rdv, "dv")


@pytest.mark.parametrize("d", [16, 18, 40, 96])
def test_head_dims_that_run_zero_padded(d):
    q, k, v, do, cu_q, cu_k, cq, ck, mask = _problem(20 + d, [90, 33], [70, 120], 4, 2, d, 32, 32, 0.6, torch.bfloat16)
    print(f"backward padded head dim {d}", flush=True)
    _, dq, dk, dv = _gpu_grads(q, k, v, do, cq, ck, mask, 32, 32, True, None)
    assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape
    rdq, rdk, rdv = hbsa_oracle_grads(q, k, v, do, cu_q, cu_k, mask, 32, 32, True, None)
    _check(dq, rdq, "dq")
    _check(dk, rdk, "dk")
    _check(dv, rdv, "dv")


def test_rows_without_visible_keys_and_unkept_keys_get_exact_zeros():
    # q longer than k under bottom-right causal alignment: the first 32 rows see no key; k block 1 is kept by nobody
    q, k, v, do, cu_q, cu_k, cq, ck, mask = _problem(11, [48], [32], 2, 1, 32, 16, 16, 1.1, torch.bfloat16)
    mask[:, :, 1] = False
    print("backward zero rows", flush=True)
    _, dq, dk, dv = _gpu_grads(q, k, v, do, cq, ck, mask, 16, 16, True, None)
    assert torch.count_nonzero(dq[:16]) == 0          # rows 0-15 see keys <= row - 16 < 0
    assert torch.count_nonzero(dq[16:32]) > 0
    assert torch.count_nonzero(dk[16:]) == 0 and torch.count_nonzero(dv[16:]) == 0
    rdq, rdk, rdv = hbsa_oracle_grads(q, k, v, do, cu_q, cu_k, mask, 16, 16, True, None)
    _check(dq, rdq, "dq")
    _check(dk, rdk, "dk")
    _check(dv, rdv, "dv")


def test_backward_is_deterministic():
    q, k, v, do, cu_q, cu_k, cq, ck, mask = _problem(12, [700, 300], [700, 300], 4, 2, 128, 128, 128, 0.5, torch.bfloat16)
    print("backward determinism", flush=True)
    a = _gpu_grads(q, k, v, do, cq, ck, mask, 128, 128, True, None)
    b = _gpu_grads(q, k, v, do, cq, ck, mask, 128, 128, True, None)
    for x, y in zip(a, b):
        assert torch.equal(x, y)


def test_gqa_gradients_equal_mha_with_repeated_kv_heads():
    # one kv head shared by 4 q heads == 4 identical kv heads; dk, dv of the shared head are the sums over the copies
    q, k, v, do, cu_q, cu_k, cq, ck, mask = _problem(13, [150, 90], [150, 90], 4, 1, 64, 32, 32, 0.6, torch.bfloat16)
    print("backward gqa", flush=True)
    _, dq, dk, dv = _gpu_grads(q, k, v, do, cq, ck, mask, 32, 32, True, None)
    _, dq4, dk4, dv4 = _gpu_grads(q, k.repeat(1, 4, 1), v.repeat(1, 4, 1), do, cq, ck, mask.repeat(4, 1, 1), 32, 32, True, None)
    assert torch.equal(dq, dq4)
    torch.testing.assert_close(dk.float(), dk4.float().sum(dim=1, keepdim=True), atol=3e-2, rtol=2e-2)
    torch.testing.assert_close(dv.float(), dv4.float().sum(dim=1, keepdim=True), atol=3e-2, rtol=2e-2)


@pytest.mark.parametrize("d", [32, 64, 128])
def test_strided_tensors_give_the_gradients_of_their_contiguous_copies(d):
    # q, k, v as slices of one packed [tokens, 3, heads, d] tensor (token stride 3 * heads * d), dout and out stored
    # head-major ([heads, tokens, d] seen through a transpose: token stride d): the kernels address tile rows by
    # 32-bit offsets built from these strides
    from hbsattn_amd import interface as I
    from hbsattn_amd import calculate_blocks
    heads, qbs, kbs = 2, 64, 128
    q, k, v, do, cu_q, cu_k, cq, ck, mask = _problem(40 + d, [300, 130], [300, 130], heads, heads, d, qbs, kbs, 0.6, torch.bfloat16)
    print(f"backward strided d={d}", flush=True)
    packed = torch.stack([q, k, v], dim=1).cuda()                       # [tokens, 3, heads, d]
    qs, ks, vs = packed[:, 0], packed[:, 1], packed[:, 2]
    assert not qs.is_contiguous() and qs.stride(0) == 3 * heads * d
    nq, _, qb2b, cu_nqb = calculate_blocks(cq, qbs)
    nk, _, _, cu_nkb = calculate_blocks(ck, kbs)
    prepared = I.hbsa_prepare(cq, ck, mask.cuda(), qbs, kbs, True, int(nq), qb2b, cu_nqb, int(nk), cu_nkb)
    out, lse = I.hbsa_run(qs, ks, vs, prepared, None, return_lse=True)
    out_hm = out.transpose(0, 1).contiguous().transpose(0, 1)           # same values, [heads, tokens, d] in memory
    do_hm = do.cuda().transpose(0, 1).contiguous().transpose(0, 1)
    assert do_hm.stride(0) == d and not do_hm.is_contiguous()
    got = I.hbsa_backward(qs, ks, vs, out_hm, do_hm, lse, prepared, None)
    want = I.hbsa_backward(qs.contiguous(), ks.contiguous(), vs.contiguous(), out.contiguous(), do.cuda(), lse, prepared, None)
    torch.cuda.synchronize()
    for g, w in zip(got, want):
        assert torch.equal(g, w)
    rdq, rdk, rdv = hbsa_oracle_grads(q, k, v, do, cu_q, cu_k, mask, qbs, kbs, True, None)
    _check(got[0], rdq, "dq")
    _check(got[1], rdk, "dk")
    _check(got[2], rdv, "dv")


@pytest.mark.parametrize("fp32_mode", ["exact", "fast"])
def test_float32_inputs_get_gradients_of_bf16_accuracy(fp32_mode):
    """fp32 q, k, v: the forward runs in the chosen fp32 mode, the gradients come from the bf16 kernels on
    rounded copies with the forward's log-sum-exp, returned as fp32, within the 16-bit tolerance of the oracle."""
    from hbsattn_amd import HBSAttention, set_fp32_mode
    previous = set_fp32_mode(fp32_mode)
    try:
        for n, (q_lens, k_lens, hq, hk, d, qbs, kbs, causal) in enumerate([([300, 64], [400, 64], 4, 2, 64, 48, 80, True),
                                                                          ([512], [512], 2, 2, 128, 128, 128, False),
                                                                          ([130, 70], [130, 90], 4, 2, 18, 32, 16, True)]):
            q, k, v, do, cu_q, cu_k, cq, ck, mask = _problem(140 + n, q_lens, k_lens, hq, hk, d, qbs, kbs, 0.6, torch.float32)
            out, dq, dk, dv = _gpu_grads(q, k, v, do, cq, ck, mask, qbs, kbs, causal, None)
            assert dq.dtype == dk.dtype == dv.dtype == torch.float32
            rdq, rdk, rdv = hbsa_oracle_grads(q, k, v, do, cu_q, cu_k, mask, qbs, kbs, causal, None)
            _check(dq, rdq, f"fp32 {fp32_mode} case {n} dq")
            _check(dk, rdk, f"fp32 {fp32_mode} case {n} dk")
            _check(dv, rdv, f"fp32 {fp32_mode} case {n} dv")
    finally:
        set_fp32_mode(previous)


def test_head_dims_above_128_still_raise_in_the_backward_like_the_reference():
    from hbsattn_amd import HBSAttention
    q, k, v, do, cu_q, cu_k, cq, ck, mask = _problem(14, [64], [64], 2, 2, 160, 32, 32, 1.1, torch.bfloat16)
    qd = q.cuda().requires_grad_(True)
    out = HBSAttention(qd, k.cuda(), v.cuda(), cq, ck, mask.cuda(), 32, 32, False, None)
    with pytest.raises(NotImplementedError):
        out.backward(do.cuda())


def test_seeded_random_shapes_against_the_gradient_oracle():
    import random
    rng = random.Random(4242)
    for case in range(32):
        batch = rng.randint(1, 3)
        q_lens = [rng.randint(1, 500) for _ in range(batch)]
        k_lens = q_lens if rng.random() < 0.3 else [rng.randint(1, 600) for _ in range(batch)]
        hk = rng.choice([1, 2, 3])
        ratio = rng.choice([1, 1, 2, 4])
        d = rng.choice([16, 32, 40, 64, 96, 128, 128])
        qbs = 16 * rng.randint(1, 12)
        kbs = 16 * rng.randint(1, 12)
        dtype = rng.choice([torch.bfloat16, torch.bfloat16, torch.float16])
        causal = rng.random() < 0.6
        scale = rng.choice([None, None, 0.05, 0.3])
        keep = rng.choice([0.15, 0.5, 0.9, 1.1])
        what = (f"case {case}: q={q_lens} k={k_lens} heads={hk * ratio}/{hk} d={d} blocks={qbs}x{kbs} {dtype} "
                f"causal={causal} scale={scale} keep={keep}")
        print("backward random " + what, flush=True)
        q, k, v, do, cu_q, cu_k, cq, ck, mask = _problem(7000 + case, q_lens, k_lens, hk * ratio, hk, d, qbs, kbs, keep, dtype)
        _, dq, dk, dv = _gpu_grads(q, k, v, do, cq, ck, mask, qbs, kbs, causal, scale)
        rdq, rdk, rdv = hbsa_oracle_grads(q, k, v, do, cu_q, cu_k, mask, qbs, kbs, causal, scale)
        _check(dq, rdq, what + " dq")
        _check(dk, rdk, what + " dk")
        _check(dv, rdv, what + " dv")
