"""Host-side behaviour of the operator that needs no GPU: signature, error conventions
(reference hbsattn/hbsa_interface.py:19-32, fwd_triton_auto_tile_size.py:261,267,
fwd_triton_fix_tile_size.py:226) and the refusal to compute anywhere but on the GPU."""
import inspect

import pytest
import torch

import hbsattn
import hbsattn.utils
import hbsattn_amd
from hbsattn_amd.interface import _HBSAttentionFunction


def _toy(dtype=torch.bfloat16, hq=8, hk=2, d=32):
    cu_q = torch.tensor([0, 32, 64, 96, 128, 160], dtype=torch.int32)
    cu_k = torch.tensor([0, 32, 61, 100, 134, 157], dtype=torch.int32)
    q = torch.randn(160, hq, d, dtype=dtype)
    k = torch.randn(157, hk, d, dtype=dtype)
    v = torch.randn(157, hk, d, dtype=dtype)
    mask = torch.rand(hk, 5, 12) < 0.7
    return q, k, v, cu_q, cu_k, mask


def test_signature_matches_reference_positional_order():
    params = list(inspect.signature(_HBSAttentionFunction.forward).parameters)
    assert params == ["ctx", "q", "k", "v", "cu_q_seqlens", "cu_k_seqlens", "block_mask", "q_block_size", "k_block_size",
                      "causal", "softmax_scale", "tile_mode", "num_q_block", "cu_q_block", "q_block_to_batch",
                      "cu_num_q_block", "num_k_block", "cu_k_block", "k_block_to_batch", "cu_num_k_block"]
    sig = inspect.signature(_HBSAttentionFunction.forward)
    assert sig.parameters["tile_mode"].default == "auto"
    assert all(sig.parameters[p].default is None for p in params[12:])


def test_drop_in_package_names():
    assert hbsattn.HBSAttention is hbsattn_amd.HBSAttention
    assert hbsattn.utils.calculate_blocks is hbsattn_amd.calculate_blocks


def test_mask_dtype_and_shape_assertions():
    q, k, v, cu_q, cu_k, mask = _toy()
    with pytest.raises(AssertionError, match="block_mask must be a boolean tensor"):
        hbsattn_amd.HBSAttention(q, k, v, cu_q, cu_k, mask.to(torch.uint8), 32, 16, True, None)
    with pytest.raises(AssertionError, match=r"\(nheads_k, num_q_block, num_k_block\) = \(2, 5, 12\)"):
        hbsattn_amd.HBSAttention(q, k, v, cu_q, cu_k, mask[:, :, :11], 32, 16, True, None)


def test_invalid_tile_mode_raises_value_error():
    q, k, v, cu_q, cu_k, mask = _toy()
    with pytest.raises(ValueError, match="Invalid tile mode: banana"):
        hbsattn_amd.HBSAttention(q, k, v, cu_q, cu_k, mask, 32, 16, True, None, "banana")


def test_fix_mode_keeps_power_of_two_assertion():
    q, k, v, cu_q, cu_k, _ = _toy()
    mask = torch.ones(2, 5, 12, dtype=torch.bool)
    with pytest.raises(AssertionError, match="powers of 2"):
        hbsattn_amd.HBSAttention(q, k, v, cu_q, cu_k, torch.ones(2, 5, 5, dtype=torch.bool), 80, 48, True, None, "fix")


def test_gqa_and_block_size_assertions():
    q, k, v, cu_q, cu_k, mask = _toy(hq=3, hk=2)
    with pytest.raises((AssertionError, RuntimeError)):
        hbsattn_amd.HBSAttention(q, k, v, cu_q, cu_k, mask, 32, 16, True, None)


def test_cpu_tensors_are_refused_not_computed():
    """There is no CPU compute path: the reference's kernels are GPU-only too
    (reference test/test_accuracy.py:31)."""
    q, k, v, cu_q, cu_k, mask = _toy()
    with pytest.raises(RuntimeError, match="no CPU path"):
        hbsattn_amd.HBSAttention(q, k, v, cu_q, cu_k, mask, 32, 16, True, None)


def test_backward_is_not_implemented():
    with pytest.raises(NotImplementedError, match="gradient"):
        _HBSAttentionFunction.backward(None, None)


def test_fp32_mode_switch_validates_and_returns_the_previous_mode():
    import pytest
    from hbsattn_amd import set_fp32_mode
    from hbsattn_amd import interface
    first = set_fp32_mode("fast")
    try:
        assert interface._fp32_mode == "fast"
        assert set_fp32_mode("exact") == "fast"
        with pytest.raises(ValueError):
            set_fp32_mode("tf32")
        assert interface._fp32_mode == "exact"
    finally:
        set_fp32_mode(first)


def test_prepare_rejects_host_metadata_and_bad_masks_before_any_launch():
    """Sequence boundaries or block metadata on the host (or a mask of the wrong dtype / shape) must raise:
    their pointers would be dereferenced on the GPU.  A fake device mask stands in for a GPU tensor; the
    checks run before the library is loaded or anything is launched."""
    from hbsattn_amd import interface

    class FakeMask:
        is_cuda = True
        dtype = torch.bool
        shape = (2, 5, 12)
        device = torch.device("cuda", 0)

        def dim(self):
            return 3

    q, k, v, cu_q, cu_k, mask = _toy()
    nq, _, qb2b, cu_nqb = hbsattn_amd.calculate_blocks(cu_q, 32)
    nk, _, _, cu_nkb = hbsattn_amd.calculate_blocks(cu_k, 16)
    with pytest.raises(RuntimeError, match="cu_q_seqlens must be a tensor on cuda:0"):
        interface.hbsa_prepare(cu_q, cu_k, FakeMask(), 32, 16, True, nq, qb2b, cu_nqb, nk, cu_nkb)
    bad = FakeMask()
    bad.dtype = torch.uint8
    with pytest.raises(TypeError, match="boolean"):
        interface.hbsa_prepare(cu_q, cu_k, bad, 32, 16, True, nq, qb2b, cu_nqb, nk, cu_nkb)
    bad = FakeMask()
    bad.shape = (2, 5, 11)
    with pytest.raises(ValueError, match=r"\(\*, 5, 12\)"):
        interface.hbsa_prepare(cu_q, cu_k, bad, 32, 16, True, nq, qb2b, cu_nqb, nk, cu_nkb)
