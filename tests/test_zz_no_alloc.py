"""The allocation-free entry point ``hbsa_fwd_static`` against ``hbsa_fwd``.

``hbsa_fwd_static`` keeps the work description in a device array inside the library instead of a
caller-provided workspace.  Called through the C ABI twice in a row, the second time on a smaller
problem (the array then still holds the first call's contents), each result must be bit-identical
to ``hbsa_fwd`` on the same inputs (same kernels, same order of operations) and within the forward's
tolerance of the CPU oracle; a problem too large for the array is refused before anything runs.
"""
import ctypes

import pytest
import torch

from hbsattn_amd import _lib
from hbsattn_amd.workloads import make_problem
from tests.helpers import assert_close_to_oracle, oracle_for

pytestmark = pytest.mark.gpu


def _common_args(w):
    nqb, _, qb2b, cu_nqb = w.q_meta
    nkb, _, _, cu_nkb = w.k_meta
    i32 = lambda t: t.to(torch.int32).contiguous()
    meta = tuple(map(i32, (w.cu_q_seqlens, w.cu_k_seqlens, qb2b, cu_nqb, cu_nkb)))
    scale = w.softmax_scale if w.softmax_scale is not None else w.q.shape[2] ** -0.5
    sizes = (len(w.cu_q) - 1, w.q.shape[0], w.k.shape[0], w.q.shape[1], w.k.shape[1], w.q.shape[2], int(nqb), int(nkb),
             w.q_block_size, w.k_block_size, int(w.causal))
    return meta, sizes, scale


def _strides(w, out):
    return (ctypes.c_int64 * 11)(w.q.stride(0), w.q.stride(1), w.k.stride(0), w.k.stride(1), w.v.stride(0), w.v.stride(1),
                                 out.stride(0), out.stride(1), *w.block_mask.stride())


def _fwd_with_workspace(w):
    lib = _lib.load()
    (cu_q, cu_k, qb2b, cu_nqb, cu_nkb), sizes, scale = _common_args(w)
    out = torch.full_like(w.q, float("nan"))
    need = lib.hbsa_fwd_workspace_bytes_dtype(_lib.DTYPE_BF16, *sizes[1:8])
    ws = torch.empty(need, dtype=torch.uint8, device=w.q.device)
    rc = lib.hbsa_fwd(w.q.data_ptr(), w.k.data_ptr(), w.v.data_ptr(), out.data_ptr(), cu_q.data_ptr(), cu_k.data_ptr(),
                      w.block_mask.data_ptr(), qb2b.data_ptr(), cu_nqb.data_ptr(), cu_nkb.data_ptr(), ws.data_ptr(), need,
                      _lib.DTYPE_BF16, *sizes, scale, _strides(w, out), torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert rc == 0, _lib.last_error()
    return out


def _fwd_static(w):
    lib = _lib.load()
    (cu_q, cu_k, qb2b, cu_nqb, cu_nkb), sizes, scale = _common_args(w)
    out = torch.full_like(w.q, float("nan"))
    rc = lib.hbsa_fwd_static(w.q.data_ptr(), w.k.data_ptr(), w.v.data_ptr(), out.data_ptr(), cu_q.data_ptr(),
                             cu_k.data_ptr(), w.block_mask.data_ptr(), qb2b.data_ptr(), cu_nqb.data_ptr(),
                             cu_nkb.data_ptr(), _lib.DTYPE_BF16, *sizes, scale, _strides(w, out),
                             torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return rc, out


def test_static_entry_point_matches_hbsa_fwd_on_two_calls_in_a_row():
    big = make_problem(seed=31, q_lens=[1500, 2048, 700], k_lens=[1800, 2048, 900], hq=8, hk=4, d=128, qbs=128, kbs=128,
                       keep=0.3, diag=True, causal=True, scale=None)
    small = make_problem(seed=32, q_lens=[300, 90], k_lens=[260, 200], hq=4, hk=2, d=64, qbs=48, kbs=80, keep=0.5,
                         diag=True, causal=True, scale=0.2)
    for name, w in (("first call", big), ("second, smaller call", small)):
        rc, got = _fwd_static(w)
        assert rc == 0, _lib.last_error()
        assert torch.equal(got, _fwd_with_workspace(w)), name
        assert_close_to_oracle(got, oracle_for(w), name)


def test_static_entry_point_refuses_problems_beyond_its_array():
    # 64 kv heads x 4096 q blocks x 4096 k blocks: the bit rows alone need 128 MiB
    lib = _lib.load()
    assert lib.hbsa_fwd_workspace_bytes(64, 4096, 4096) > _lib.STATIC_SCRATCH_BYTES
    t = torch.zeros(16, dtype=torch.bfloat16, device="cuda")
    out = torch.full((16,), float("nan"), dtype=torch.bfloat16, device="cuda")
    strides = (ctypes.c_int64 * 11)(64 * 128, 128, 64 * 128, 128, 64 * 128, 128, 64 * 128, 128, 4096 * 4096, 4096, 1)
    rc = lib.hbsa_fwd_static(t.data_ptr(), t.data_ptr(), t.data_ptr(), out.data_ptr(), t.data_ptr(), t.data_ptr(),
                             t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), _lib.DTYPE_BF16, 1, 4096 * 128,
                             4096 * 128, 64, 64, 128, 4096, 4096, 128, 128, 1, 0.1, strides,
                             torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert rc == -3 and "hbsa_fwd_static holds" in _lib.last_error()
    assert torch.isnan(out.float()).all()


def test_static_entry_point_allocates_nothing_and_can_be_captured_into_a_graph():
    """After a first call (which looks up the array's address and the kernels' launch limits) further calls
    leave the device's free memory exactly where it was, and a call recorded into a graph (the case the entry
    point is for: nothing may be allocated under capture) replays to the eager result, every time."""
    lib = _lib.load()
    w = make_problem(seed=33, q_lens=[900, 640], k_lens=[1200, 640], hq=8, hk=4, d=128, qbs=64, kbs=128, keep=0.4,
                     diag=True, causal=True, scale=None)
    (cu_q, cu_k, qb2b, cu_nqb, cu_nkb), sizes, scale = _common_args(w)
    out = torch.full_like(w.q, float("nan"))
    strides = _strides(w, out)

    def call(stream):
        return lib.hbsa_fwd_static(w.q.data_ptr(), w.k.data_ptr(), w.v.data_ptr(), out.data_ptr(), cu_q.data_ptr(),
                                   cu_k.data_ptr(), w.block_mask.data_ptr(), qb2b.data_ptr(), cu_nqb.data_ptr(),
                                   cu_nkb.data_ptr(), _lib.DTYPE_BF16, *sizes, scale, strides, stream)

    main = torch.cuda.current_stream().cuda_stream
    assert call(main) == 0, _lib.last_error()
    torch.cuda.synchronize()
    eager = out.clone()
    assert torch.equal(eager, _fwd_with_workspace(w))
    free_before = torch.cuda.mem_get_info()[0]
    for _ in range(3):
        assert call(main) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "hbsa_fwd_static changed the device's free memory"

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        graph.capture_begin()
        rc = call(side.cuda_stream)
        graph.capture_end()
    assert rc == 0, _lib.last_error()
    torch.cuda.current_stream().wait_stream(side)
    for replay in range(3):
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {replay}"
        assert call(main) == 0                      # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
