"""Measurements that design decisions of the kernels rest on, as tests: if the hardware behaved otherwise, the kernels
would be built otherwise."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu


def test_fp32_mfma_and_vector_instructions_do_not_overlap():
    """tests/cxx/mfma_valu_overlap.cpp: wavefronts that issue FP32 MFMAs and wavefronts on the same SIMDs that issue
    FP32 multiply-adds take, together, about as long as one after the other (not as long as the slower of the two), and a
    wavefront that interleaves the two kinds takes no less.  This is why the matrix-product and attention kernels count
    every vector instruction inside their MFMA loops (operand offsets in the instructions' immediate fields, addresses
    computed outside the loop, rescaling only when a maximum grew), and why a fused attention backward pass, which would
    recompute the exponentials inside the loop, was decided against."""
    print("[case] MFMA / VALU overlap microbenchmark", flush=True)
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cxx", "mfma_valu_overlap")
    assert os.path.exists(exe), "tests/cxx/mfma_valu_overlap is not built: run __graft_entry__.build()"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    print("  " + r.stdout.strip(), flush=True)
    words = r.stdout.split()
    t = {words[i]: float(words[i + 1]) for i in range(0, 8, 2)}
    assert t["both"] >= 0.85 * (t["mfma"] + t["valu"]), t
    assert t["both"] >= 1.5 * max(t["mfma"], t["valu"]), t
    assert t["mixed"] >= 0.85 * (t["mfma"] + t["valu"]), t
