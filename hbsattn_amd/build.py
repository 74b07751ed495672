"""Builds ``libhbsattn_amd.so`` in-tree with hipcc for gfx950.

``python -m hbsattn_amd.build`` or ``hbsattn_amd.build.build()``.  hipcc
cross-compiles, so no GPU is needed to build.
"""
from __future__ import annotations

import os
import re
import shutil
import subprocess
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))
_ROOT = os.path.dirname(_HERE)
SOURCES = [os.path.join(_HERE, "csrc", "hbsa_fwd.hip")]
OUTPUT = os.path.join(_HERE, "libhbsattn_amd.so")
HAND_ISSUED_READS = "hbsa_fwd_kernel"   # substring of the mangled names of the kernels with hand-issued LDS reads ...
COMPILER_ISSUED = "hbsa_fwd_kernelILi256E"   # ... except the head dim 256 instantiations, whose reads the compiler issues

# -packed-fp32-ops: keep the compiler from forming v_pk_*_f32 out of scalar float code.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I" + os.path.join(_ROOT, "include"),
]


def _vgpr_spills(remarks: str) -> dict:
    """Kernels with vector-register spills, from the compiler's resource-usage remarks."""
    spills, name = {}, None
    for line in remarks.splitlines():
        m = re.search(r"remark:\s+Function Name: (\S+)", line)
        if m:
            name = m.group(1)
        m = re.search(r"remark:\s+VGPRs Spill: (\d+)", line)
        if m and name is not None and int(m.group(1)) > 0:
            spills[name] = int(m.group(1))
    return spills


def build(verbose: bool = False) -> str:
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    cmd = [hipcc] + HIPCC_FLAGS + ["-Rpass-analysis=kernel-resource-usage"] + SOURCES + ["-o", OUTPUT]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        sys.stderr.write(res.stdout + res.stderr)
        raise RuntimeError("hipcc failed: " + " ".join(cmd))
    # The forward attention kernel issues its LDS reads by hand and waits for them by count.  The
    # compiler does not know that such a register has a read in flight; if it spills one, it saves the
    # register before the data has arrived and the result is wrong now and then.  So a build in which
    # that kernel spills vector registers is refused.  (The other kernels leave every wait to the
    # compiler; a spill there only costs time and is reported.)
    spills = _vgpr_spills(res.stderr)
    fatal = {k: v for k, v in spills.items() if HAND_ISSUED_READS in k and COMPILER_ISSUED not in k}
    if fatal:
        os.remove(OUTPUT)
        raise RuntimeError(f"vector-register spills in {fatal}: reduce register pressure (see the comment here)")
    if spills and verbose:
        print(f"note: vector-register spills in {spills}")
    if verbose:
        print(" ".join(cmd))
    return OUTPUT


EXAMPLE_SOURCE = os.path.join(_HERE, "csrc", "cabi_example.cpp")
EXAMPLE_OUTPUT = os.path.join(_HERE, "cabi_example")


def build_example(verbose: bool = False) -> str:
    """The torch-free C++ caller of the library (``csrc/cabi_example.cpp``); run it on a GPU box as
    ``./hbsattn_amd/cabi_example``."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    cmd = [hipcc, "--offload-arch=gfx950", "-O2", "-std=c++17", "-I" + os.path.join(_ROOT, "include"), EXAMPLE_SOURCE,
           "-L" + _HERE, "-lhbsattn_amd", "-Wl,-rpath,$ORIGIN", "-o", EXAMPLE_OUTPUT]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        sys.stderr.write(res.stdout + res.stderr)
        raise RuntimeError("hipcc failed: " + " ".join(cmd))
    if verbose:
        print(" ".join(cmd))
    return EXAMPLE_OUTPUT


if __name__ == "__main__":
    print(build(verbose=True))
    print(build_example(verbose=True))
