"""CPU checks of the seeded problem generators and of the FLOP/byte model the bench uses."""
import torch

from hbsattn_amd.workloads import SPECS, count_work, force_diagonal, make_problem, make_workload
from oracle.dense import calculate_blocks_oracle, visited_block_pairs


def test_c1_geometry_is_the_readme_example():
    w = make_workload("C1", device="cpu")
    assert w.cu_q == [0, 32, 64, 96, 128, 160] and w.cu_k == [0, 32, 61, 100, 134, 157]
    assert w.q.shape == (160, 8, 32) and w.k.shape == (157, 2, 32) and w.block_mask.shape == (2, 5, 12)
    assert w.q_meta[0] == 5 and w.k_meta[0] == 12
    w2 = make_workload("C1", device="cpu")
    assert torch.equal(w.q, w2.q) and torch.equal(w.block_mask, w2.block_mask)      # seeded
    assert len(w.args()) == 19 and len(w.args(with_meta=False)) == 10


def test_force_diagonal_bottom_right():
    cu_q, cu_k = [0, 64, 100], [0, 128, 148]
    nq, nk = calculate_blocks_oracle(cu_q, 32)[0], calculate_blocks_oracle(cu_k, 16)[0]
    m = torch.zeros(1, nq, nk, dtype=torch.bool)
    force_diagonal(m, cu_q, cu_k, 32, 16)
    # seq 0: shift 64 -> q block 0 first row sees key 64 (k block 4), q block 1 key 96 (k block 6)
    # seq 1: q 36 (2 blocks) k 20 (2 blocks), shift -16 -> row 0 -> key clamp(-16)=0 -> block 8; row 32 -> key 16 -> block 9
    assert m[0].nonzero().tolist() == [[0, 4], [1, 6], [2, 8], [3, 9]]


def test_count_work_matches_brute_force():
    for seed, causal, qbs, kbs, q_lens, k_lens, hq, hk in [
        (1, True, 32, 16, [32] * 5, [32, 29, 39, 34, 23], 8, 2),
        (2, False, 48, 80, [100, 37], [64, 200], 2, 2),
        (3, True, 80, 48, [300, 77], [600, 41], 4, 1),
    ]:
        w = make_problem(seed=seed, q_lens=q_lens, k_lens=k_lens, hq=hq, hk=hk, d=16, qbs=qbs, kbs=kbs, keep=0.6,
                         diag=False, causal=causal, scale=None, device="cpu")
        blk, exact = visited_block_pairs(w.cu_q, w.cu_k, w.block_mask, qbs, kbs, causal)
        work = count_work(w)
        ratio = hq // hk
        assert work["flops"] == 4 * 16 * blk * ratio
        assert work["flops_exact"] == 4 * 16 * exact * ratio
        assert work["flops_exact"] <= work["flops"]


def test_target_shape_flops_expectation():
    """The 32K target shape: 901,120 expected visited pairs x 8,388,608 FLOP = 7.56 TFLOP."""
    s = SPECS["T"]
    nb = 32768 // 128
    expected_pairs = (nb + 0.1 * nb * (nb - 1) / 2) * 8 * 32
    assert abs(expected_pairs - 901120) < 1
    assert abs(expected_pairs * 4 * 128 ** 3 / 1e12 - 7.56) < 0.01
    assert s["qbs"] == s["kbs"] == 128 and s["keep"] == 0.1 and s["causal"]
