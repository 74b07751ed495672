"""Pins the gradient oracle (``oracle.grads``), which has no reference counterpart to restate.

Three independent routes to the same gradients: reverse-mode autograd through the masked-dense
forward oracle, central finite differences of that forward in float64, and autograd through torch's
``scaled_dot_product_attention`` where the mask reduces to it.  A dropped ``scale``, a missing
``- rowsum(dP * P)`` term, ``h % ratio`` head mapping, a transposed ``dS`` or a NaN from a row
without visible keys each fail one of them.
"""
import pytest
import torch
import torch.nn.functional as F

from oracle.dense import calculate_blocks_oracle, hbsa_oracle
from oracle.grads import hbsa_oracle_grads


def _rand(seed, *shape, dtype=torch.float32):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=dtype)


def _problem(seed, q_lens, k_lens, hq, hk, d, qbs, kbs, keep, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    cu_q = [0]
    cu_k = [0]
    for a, b in zip(q_lens, k_lens):
        cu_q.append(cu_q[-1] + a)
        cu_k.append(cu_k[-1] + b)
    q = torch.randn(cu_q[-1], hq, d, generator=g, dtype=dtype)
    k = torch.randn(cu_k[-1], hk, d, generator=g, dtype=dtype)
    v = torch.randn(cu_k[-1], hk, d, generator=g, dtype=dtype)
    do = torch.randn(cu_q[-1], hq, d, generator=g, dtype=dtype)
    nq = calculate_blocks_oracle(cu_q, qbs)[0]
    nk = calculate_blocks_oracle(cu_k, kbs)[0]
    mask = torch.rand(hk, nq, nk, generator=g) < keep
    return q, k, v, do, cu_q, cu_k, mask


def _autograd(q, k, v, do, cu_q, cu_k, mask, qbs, kbs, causal, scale, dtype):
    q, k, v = (t.detach().clone().to(dtype).requires_grad_(True) for t in (q, k, v))
    out = hbsa_oracle(q, k, v, cu_q, cu_k, mask, qbs, kbs, causal, scale, compute_dtype=dtype)
    out.backward(do.to(dtype))
    return q.grad, k.grad, v.grad


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("hq,hk", [(4, 4), (6, 2)])
def test_matches_autograd_of_forward_oracle(causal, hq, hk):
    q, k, v, do, cu_q, cu_k, mask = _problem(3, [37, 64, 5], [50, 64, 33], hq, hk, 16, 16, 32, 0.6)
    got = hbsa_oracle_grads(q, k, v, do, cu_q, cu_k, mask, 16, 32, causal, 0.4)
    want = _autograd(q, k, v, do, cu_q, cu_k, mask, 16, 32, causal, 0.4, torch.float32)
    for g, w, name in zip(got, want, "qkv"):
        torch.testing.assert_close(g, w, atol=2e-5, rtol=1e-4, msg=lambda m: f"d{name}: {m}")


def test_rows_without_visible_keys_give_zero_gradients():
    # q longer than k under the bottom-right causal alignment: the first rows see no key at all
    q, k, v, do, cu_q, cu_k, mask = _problem(5, [48], [16], 2, 1, 8, 16, 16, 1.1)
    dq, dk, dv = hbsa_oracle_grads(q, k, v, do, cu_q, cu_k, mask, 16, 16, True, None)
    assert torch.isfinite(dq).all() and torch.isfinite(dk).all() and torch.isfinite(dv).all()
    assert torch.count_nonzero(dq[:32]) == 0
    assert torch.count_nonzero(dq[32:]) > 0


def test_matches_finite_differences_in_float64():
    q, k, v, do, cu_q, cu_k, mask = _problem(7, [9, 6], [7, 11], 2, 1, 4, 16, 16, 0.7, dtype=torch.float64)
    mask[:] = True
    mask[0, 0, 1] = False
    args = (cu_q, cu_k, mask, 16, 16, True, 0.7)
    dq, dk, dv = hbsa_oracle_grads(q, k, v, do, *args, compute_dtype=torch.float64)

    def loss(q_, k_, v_):
        return (hbsa_oracle(q_, k_, v_, *args, compute_dtype=torch.float64) * do).sum().item()

    eps = 1e-6
    gen = torch.Generator().manual_seed(11)
    for t, g, idx in ((q, dq, 0), (k, dk, 1), (v, dv, 2)):
        for _ in range(12):
            i = tuple(int(torch.randint(0, n, (1,), generator=gen)) for n in t.shape)
            plus, minus = t.clone(), t.clone()
            plus[i] += eps
            minus[i] -= eps
            a = [q, k, v]
            a[idx] = plus
            up = loss(*a)
            a[idx] = minus
            down = loss(*a)
            assert abs((up - down) / (2 * eps) - g[i].item()) < 1e-6, (idx, i)


@pytest.mark.parametrize("causal", [False, True])
def test_all_true_mask_matches_sdpa_autograd(causal):
    q, k, v, do, cu_q, cu_k, mask = _problem(9, [40], [40], 4, 2, 16, 16, 16, 1.1)
    got = hbsa_oracle_grads(q, k, v, do, cu_q, cu_k, mask, 16, 16, causal, None)
    q2, k2, v2 = (t.detach().clone().requires_grad_(True) for t in (q, k, v))
    kk = k2.repeat_interleave(2, dim=1)
    vv = v2.repeat_interleave(2, dim=1)
    o = F.scaled_dot_product_attention(q2.permute(1, 0, 2)[None], kk.permute(1, 0, 2)[None], vv.permute(1, 0, 2)[None],
                                       is_causal=causal)
    o[0].permute(1, 0, 2).backward(do)
    for g, w, name in zip(got, (q2.grad, k2.grad, v2.grad), "qkv"):
        torch.testing.assert_close(g, w, atol=2e-5, rtol=1e-4, msg=lambda m: f"d{name}: {m}")
