"""Pins the block-geometry oracle and the product's ``calculate_blocks`` (CPU tensors).

Known answers: the worked example the reference documents (README.md:49-63 of the
reference: cu_k=[0,32,61,100,134,157], block 16 -> blocks per sample 2,2,3,3,2 with last
block sizes 16,13,7,2,7; 12 k blocks and 5 q blocks in total).
"""
import numpy as np
import pytest
import torch
from hypothesis import given, settings, strategies as st

from hbsattn_amd.utils import calculate_blocks
from oracle.dense import calculate_blocks_oracle
from oracle.scalar import calculate_blocks_scalar

README_CU_Q = [0, 32, 64, 96, 128, 160]
README_CU_K = [0, 32, 61, 100, 134, 157]


def test_readme_worked_example_k_side():
    nb, cu_block, b2b, cu_nb = calculate_blocks_oracle(README_CU_K, 16)
    assert nb == 12
    assert cu_block == [0, 16, 32, 48, 61, 77, 93, 100, 116, 132, 134, 150, 157]
    assert b2b == [0, 0, 1, 1, 2, 2, 2, 3, 3, 3, 4, 4]
    assert cu_nb == [0, 2, 4, 7, 10, 12]
    sizes = np.diff(cu_block)
    last = [int(sizes[cu_nb[b + 1] - 1]) for b in range(5)]
    assert last == [16, 13, 7, 2, 7]           # last-block sizes the README lists
    assert list(np.diff(cu_nb)) == [2, 2, 3, 3, 2]


def test_readme_worked_example_q_side():
    nb, cu_block, b2b, cu_nb = calculate_blocks_oracle(README_CU_Q, 32)
    assert (nb, cu_block, b2b, cu_nb) == (5, [0, 32, 64, 96, 128, 160], [0, 1, 2, 3, 4], [0, 1, 2, 3, 4, 5])


@pytest.mark.parametrize("length,bs,batch", [(8192, 128, 8), (100, 16, 3), (48, 48, 2), (17, 16, 4)])
def test_uniform_lengths_closed_form(length, bs, batch):
    cu = [i * length for i in range(batch + 1)]
    nb, cu_block, b2b, cu_nb = calculate_blocks_oracle(cu, bs)
    per = -(-length // bs)
    assert nb == per * batch
    assert cu_nb == [i * per for i in range(batch + 1)]
    expect = [0]
    for b in range(batch):
        expect += [min(b * length + (t + 1) * bs, (b + 1) * length) for t in range(per)]
    assert cu_block == expect
    assert b2b == [b for b in range(batch) for _ in range(per)]


lens_strategy = st.lists(st.integers(min_value=1, max_value=700), min_size=1, max_size=9)


@settings(max_examples=150, deadline=None)
@given(lens=lens_strategy, bs=st.sampled_from([16, 32, 48, 64, 80, 128]))
def test_invariants_and_three_implementations_agree(lens, bs):
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    nb, cu_block, b2b, cu_nb = calculate_blocks_oracle(cu, bs)
    # invariants
    sizes = np.diff(cu_block)
    assert (sizes > 0).all() and (sizes <= bs).all()
    for b in range(len(lens)):
        assert cu_block[cu_nb[b]] == cu[b]
        assert cu_nb[b + 1] - cu_nb[b] == -(-lens[b] // bs)
        assert all(x == b for x in b2b[cu_nb[b]:cu_nb[b + 1]])
        assert (sizes[cu_nb[b]:cu_nb[b + 1] - 1] == bs).all()     # only the last block may be short
    assert cu_block[-1] == cu[-1] and len(b2b) == nb
    # the C restatement
    nb_c, cu_block_c, b2b_c, cu_nb_c = calculate_blocks_scalar(cu, bs)
    assert nb_c == nb and cu_block_c.tolist() == cu_block and b2b_c.tolist() == b2b and cu_nb_c.tolist() == cu_nb
    # the product's torch version on CPU tensors
    nb_t, cu_block_t, b2b_t, cu_nb_t = calculate_blocks(torch.tensor(cu, dtype=torch.int32), bs)
    assert isinstance(nb_t, int) and nb_t == nb
    assert cu_block_t.dtype == torch.int32 and cu_block_t.tolist() == cu_block
    assert b2b_t.dtype == torch.int32 and b2b_t.tolist() == b2b
    assert cu_nb_t.dtype == torch.int32 and cu_nb_t.tolist() == cu_nb


def test_product_calculate_blocks_readme_and_int64():
    nb, cu_block, b2b, cu_nb = calculate_blocks(torch.tensor(README_CU_K, dtype=torch.int32), 16)
    assert nb == 12 and cu_block.tolist() == [0, 16, 32, 48, 61, 77, 93, 100, 116, 132, 134, 150, 157]
    assert b2b.tolist() == [0, 0, 1, 1, 2, 2, 2, 3, 3, 3, 4, 4] and cu_nb.tolist() == [0, 2, 4, 7, 10, 12]
    nb64, cu_block64, b2b64, cu_nb64 = calculate_blocks(torch.tensor(README_CU_K, dtype=torch.int64), 16)
    # cu_block / block_to_batch are int32 whatever the input dtype; cu_num_block follows the input
    assert cu_block64.dtype == torch.int32 and b2b64.dtype == torch.int32 and cu_nb64.dtype == torch.int64
    assert nb64 == 12 and cu_nb64.tolist() == [0, 2, 4, 7, 10, 12]
