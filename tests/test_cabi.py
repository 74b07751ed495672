"""The C-ABI library loads without a GPU and exports every function the header declares.
Only host-side entry points and argument validation are exercised here (no kernel runs)."""
import ctypes
import os
import re

import pytest

from hbsattn_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "hbsattn_amd.h")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hbsa_[a-z_0-9]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = _declared_functions()
    assert {"hbsa_abi_version", "hbsa_last_error", "hbsa_fwd_workspace_bytes", "hbsa_fwd"} <= set(names)


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in _declared_functions():
        assert hasattr(lib, name), f"{name} declared in include/hbsattn_amd.h but not exported"


def test_abi_version_matches_header():
    lib = _lib.load()
    version = int(re.search(r"#define HBSA_ABI_VERSION (\d+)", open(HEADER).read()).group(1))
    assert lib.hbsa_abi_version() == version == _lib.ABI_VERSION


def test_workspace_bytes_is_host_only_and_monotone():
    lib = _lib.load()
    a = lib.hbsa_fwd_workspace_bytes(2, 5, 12)
    b = lib.hbsa_fwd_workspace_bytes(32, 2048, 2048)
    c = lib.hbsa_fwd_workspace_bytes(32, 4096, 4096)
    assert 0 < a < b < c
    assert a % 256 == 0 and b % 256 == 0
    # one bit per k block per (kv head, q block) plus a 48-byte record per q block
    assert b >= 32 * 2048 * (2048 // 8) + 2048 * 48
    assert c < 80 * 2 ** 20


def test_workspace_bytes_per_dtype():
    lib = _lib.load()
    base = lib.hbsa_fwd_workspace_bytes(8, 64, 64)
    args = (1000, 2000, 32, 8, 128, 64, 64)
    assert lib.hbsa_fwd_workspace_bytes_dtype(_lib.DTYPE_BF16, *args) == base
    assert lib.hbsa_fwd_workspace_bytes_dtype(_lib.DTYPE_F16, *args) == base
    assert lib.hbsa_fwd_workspace_bytes_dtype(_lib.DTYPE_F32, *args) == base   # fp32 matrix instructions: no staging
    f32 = lib.hbsa_fwd_workspace_bytes_dtype(_lib.DTYPE_F32_STAGED16, *args)
    staged = (1000 * 32 + 2 * 2000 * 8) * 128 * 2          # fp16 copies of q, k and v
    assert base + staged <= f32 <= base + staged + 3 * 256 and f32 % 256 == 0


def _call_fwd(lib, **over):
    strides = (ctypes.c_int64 * 11)(4096, 128, 4096, 128, 4096, 128, 4096, 128, 1, 1, 1)
    a = dict(q=256, k=256, v=256, out=256, cu_q=256, cu_k=256, mask=256, qb2b=256, cu_nqb=256, cu_nkb=256, ws=256,
             ws_bytes=1 << 30, dtype=0, batch=1, total_q=128, total_k=128, hq=32, hk=32, d=128, nqb=1, nkb=1, qbs=128,
             kbs=128, causal=1, scale=0.1)
    a.update(over)
    return lib.hbsa_fwd(a["q"], a["k"], a["v"], a["out"], a["cu_q"], a["cu_k"], a["mask"], a["qb2b"], a["cu_nqb"],
                        a["cu_nkb"], a["ws"], a["ws_bytes"], a["dtype"], a["batch"], a["total_q"], a["total_k"], a["hq"],
                        a["hk"], a["d"], a["nqb"], a["nkb"], a["qbs"], a["kbs"], a["causal"], a["scale"], strides, None)


@pytest.mark.parametrize("over,code,needle", [
    (dict(q=None), -1, "null"),
    (dict(hq=30, hk=4), -1, "divisible"),
    (dict(qbs=100), -1, "multiples of 16"),
    (dict(kbs=0), -1, "multiples of 16"),
    (dict(d=96), -2, "headdim"),
    (dict(dtype=7), -2, "dtype"),
    (dict(ws_bytes=16), -3, "workspace"),
    (dict(q=264), -1, "aligned"),
    (dict(scale=float("inf")), -1, "finite"),
])
def test_argument_validation_reports_errors_without_touching_the_gpu(over, code, needle):
    lib = _lib.load()
    one = lib.hbsa_set_onepass(0)   # (on a machine with a GPU the one-launch form would need no workspace and launch)
    try:
        rc = _call_fwd(lib, **over)
    finally:
        lib.hbsa_set_onepass(one)
    assert rc == code
    assert needle in _lib.last_error()


def test_empty_problem_is_a_no_op():
    lib = _lib.load()
    assert _call_fwd(lib, total_q=0, q=None) == 0
    assert _lib.last_error() == ""


def _call_bwd(lib, **over):
    values = [4096, 128] * 8
    for i, v in over.pop("strides", {}).items():
        values[i] = v
    strides = (ctypes.c_int64 * 16)(*values)
    a = dict(q=256, k=256, v=256, out=256, dout=256, lse=256, dq=256, dk=256, dv=256, cu_k=256, cu_nqb=256, cu_nkb=256,
             ws=256, ws_bytes=1 << 30, bws=256, bws_bytes=1 << 30, dtype=0, batch=1, total_q=128, total_k=128, hq=32, hk=32,
             d=128, nqb=1, nkb=1, qbs=128, kbs=128, causal=1, scale=0.1)
    a.update(over)
    return lib.hbsa_bwd(a["q"], a["k"], a["v"], a["out"], a["dout"], a["lse"], a["dq"], a["dk"], a["dv"], a["cu_k"],
                        a["cu_nqb"], a["cu_nkb"], a["ws"], a["ws_bytes"], a["bws"], a["bws_bytes"], a["dtype"], a["batch"],
                        a["total_q"], a["total_k"], a["hq"], a["hk"], a["d"], a["nqb"], a["nkb"], a["qbs"], a["kbs"],
                        a["causal"], a["scale"], strides, None)


@pytest.mark.parametrize("over,code,needle", [
    (dict(dout=None), -1, "null"),
    (dict(dtype=2), -2, "bf16 or fp16"),
    (dict(d=96), -2, "headdim"),
    (dict(kbs=40), -1, "multiples of 16"),
    (dict(dq=264), -1, "aligned"),
    (dict(ws_bytes=16), -3, "workspace"),
    (dict(bws_bytes=16), -3, "bwd_workspace"),
    (dict(strides={2: -4096}), -2, "k/v token stride"),          # tile rows are addressed with 32-bit offsets
    (dict(strides={4: 1 << 25}), -2, "k/v token stride"),
    (dict(strides={8: -4096}), -2, "q/dout token stride"),
])
def test_backward_argument_validation_without_touching_the_gpu(over, code, needle):
    lib = _lib.load()
    rc = _call_bwd(lib, **over)
    assert rc == code
    assert needle in _lib.last_error()


def test_backward_workspace_bytes_and_empty_problem():
    lib = _lib.load()
    assert lib.hbsa_bwd_workspace_bytes(100, 8) == 2 * 3328  # two arrays of 100 * 8 floats, each rounded up to 256 bytes
    assert lib.hbsa_bwd_workspace_bytes(0, 8) == 0
    assert _call_bwd(lib, total_q=0) == 0
    assert _lib.last_error() == ""


def _c_calculate_blocks(cu, block_size):
    import numpy as np
    lib = _lib.load()
    cu = np.asarray(cu, dtype=np.int32)
    batch = len(cu) - 1
    nb = ctypes.c_int32(-1)
    cu_nb = np.full(batch + 1, -1, dtype=np.int32)
    rc = lib.hbsa_calculate_blocks(cu.ctypes.data, batch, block_size, ctypes.addressof(nb), cu_nb.ctypes.data, None, None, 0)
    assert rc == 0, _lib.last_error()
    cu_block = np.full(nb.value + 1, -1, dtype=np.int32)
    b2b = np.full(nb.value, -1, dtype=np.int32)
    rc = lib.hbsa_calculate_blocks(cu.ctypes.data, batch, block_size, ctypes.addressof(nb), cu_nb.ctypes.data,
                                   cu_block.ctypes.data, b2b.ctypes.data, nb.value)
    assert rc == 0, _lib.last_error()
    return nb.value, cu_block.tolist(), b2b.tolist(), cu_nb.tolist()


def test_host_calculate_blocks_matches_oracle_and_readme_example():
    import random
    from oracle.dense import calculate_blocks_oracle
    # the reference's worked example (README.md:49-63 of the reference): last-block sizes 16, 13, 7, 2, 7
    nb, cu_block, b2b, cu_nb = _c_calculate_blocks([0, 32, 61, 100, 134, 157], 16)
    assert nb == 12 and cu_nb == [0, 2, 4, 7, 10, 12]
    assert [cu_block[cu_nb[b + 1]] - cu_block[cu_nb[b + 1] - 1] for b in range(5)] == [16, 13, 7, 2, 7]
    rng = random.Random(3)
    for _ in range(50):
        lens = [rng.randrange(0, 300) for _ in range(rng.randrange(0, 7))]
        cu = [0]
        for n in lens:
            cu.append(cu[-1] + n)
        bs = rng.choice([16, 32, 48, 80, 128])
        got = _c_calculate_blocks(cu, bs)
        ref = calculate_blocks_oracle(cu, bs)
        assert got == (ref[0], list(ref[1]), list(ref[2]), list(ref[3])), (cu, bs)


def test_host_calculate_blocks_rejects_bad_input():
    import numpy as np
    lib = _lib.load()
    nb = ctypes.c_int32(0)
    cu = np.asarray([0, 10, 5], dtype=np.int32)
    assert lib.hbsa_calculate_blocks(cu.ctypes.data, 2, 16, ctypes.addressof(nb), None, None, None, 0) == -1
    cu = np.asarray([0, 100], dtype=np.int32)
    assert lib.hbsa_calculate_blocks(cu.ctypes.data, 1, 0, ctypes.addressof(nb), None, None, None, 0) == -1
    small = np.zeros(3, dtype=np.int32)
    assert lib.hbsa_calculate_blocks(cu.ctypes.data, 1, 16, ctypes.addressof(nb), None, small.ctypes.data, None, 2) == -3
    assert nb.value == 7


def test_array_form_entry_point_validates_like_hbsa_fwd():
    """hbsa_fwd_v is hbsa_fwd with its arguments in arrays: same checks, same codes, nothing launched."""
    lib = _lib.load()
    fwd_v = lib.hbsa_fwd_v_locked
    strides = (ctypes.c_int64 * 11)(4096, 128, 4096, 128, 4096, 128, 4096, 128, 1, 1, 1)
    ptrs = (ctypes.c_void_p * 11)(*([256] * 11))
    sizes = (ctypes.c_int32 * 12)(0, 1, 128, 128, 30, 4, 128, 1, 1, 128, 128, 1)          # 30 q heads on 4 kv heads
    a = lambda x: ctypes.addressof(x)
    assert fwd_v(a(ptrs), 1 << 30, a(sizes), 0.1, a(strides), None) == -1 and "divisible" in _lib.last_error()
    sizes[4] = 32; sizes[5] = 32; sizes[6] = 96                                            # head dim 96
    assert fwd_v(a(ptrs), 1 << 30, a(sizes), 0.1, a(strides), None) == -2 and "headdim" in _lib.last_error()
    sizes[6] = 128; sizes[2] = 0                                                           # no queries: nothing to do
    assert fwd_v(a(ptrs), 1 << 30, a(sizes), 0.1, a(strides), None) == 0
    assert fwd_v(None, 0, a(sizes), 0.1, a(strides), None) == -1 and "null" in _lib.last_error()


def test_a_call_without_a_device_reports_two_launches_and_asks_for_its_workspace():
    """Whether a call runs as one launch is a host-side question (sizes, strides, the stream's state); without a
    device to run on the answer is the two-launch form, and hbsa_fwd without a workspace is refused, not launched."""
    lib = _lib.load()
    args = (_lib.DTYPE_BF16, 8, 65536, 32, 32, 128, 512, 512, 128, 128, 1, None)
    assert lib.hbsa_fwd_launches(*args) in (1, 2)                       # 2 here (no GPU), 1 on an MI355X
    assert lib.hbsa_fwd_launches(_lib.DTYPE_F32, *args[1:]) == 2        # fp32 tensors never run as one launch
    assert lib.hbsa_fwd_launches(_lib.DTYPE_BF16, 200, *args[2:]) == 2  # nor do more than 127 sequences
    assert lib.hbsa_fwd_launches(*args[:10], 2, None) == 2              # nor a mask whose k block stride is not 1
    previous = lib.hbsa_set_onepass(0)
    try:
        assert lib.hbsa_fwd_launches(*args) == 2
        assert lib.hbsa_set_onepass(1) == 0
    finally:
        lib.hbsa_set_onepass(previous)
    import torch
    if not torch.cuda.is_available():
        assert _call_fwd(lib, ws=None, ws_bytes=0) == -3 and "workspace" in _lib.last_error()
