"""The text of generated element-wise kernels, compiled for the host and run thread by thread, against closed forms
and the oracle (tests/host_kernels.py).  These kernels are the ones the lowering's size bounds exist for: with the
bounds raised (ADHIP_KERNEL_BOUNDS, a diagnostic switch) they read dozens of buffers under hundreds of predicates, and
the gfx950 compiler can only build them by spilling vector registers.  On the GPU three such kernels computed wrong
elements.  Their text is right -- that is what these tests hold -- so the fault lies in the device code of that
regime, which the library therefore never runs (it cuts such a kernel again, or refuses the program)."""
import os

import numpy as np
import pytest

from adhip.core import ValueData
from adhip.device import Device
from host_kernels import CLANG, generated_kernels, launch_of, run_on_host

pytestmark = pytest.mark.skipif(not os.path.exists(CLANG), reason="needs the ROCm clang++ as a host compiler")

# expressions of up to 32 operands, kernels of up to 64 buffers, nothing else bounded: what was in force when the kernel
# of the third failing program (scale 48, seed 81) was generated
OLD_BOUNDS = "100000,100000,32,100000,64,100000,100000"


class Capture(Device):
    def execute(self, proc, deps):
        self.proc, self.deps = proc, deps

    def get_tensor(self, id):
        return ValueData.none()


@pytest.mark.parametrize("name", ["wide_concat", "one_buffer_pieces"])
def test_one_wide_kernel_computes_the_closed_form(name, monkeypatch):
    """With the bounds out of the way a Concat of 2 x 40 buffers, or 100 pieces of one buffer, under one multiplication
    is one kernel; its text computes numpy's answer bit for bit."""
    import adversarial_programs as A
    monkeypatch.setenv("ADHIP_KERNEL_BOUNDS", "100000,100000,100000,100000,100000,100000,100000")
    proc, keep, want = A.wide_concat(40) if name == "wide_concat" else A.one_buffer_pieces(100)
    plan, kernels = generated_kernels(proc, keep)
    assert len(kernels) == 1, list(kernels)
    (entry, (kind, source)), = kernels.items()
    assert kind == "elw"
    grid, block, args = launch_of(plan, entry)
    leaves = {c.id: np.asarray(c.contents, np.float32) for c in proc.walk() if type(c).__name__ == "CreateMat"}
    arrays = [np.zeros(args[0][2], np.float32)] + [leaves[a[0]] for a in args[1:]]
    assert len(arrays) == (81 if name == "wide_concat" else 3)
    out, = run_on_host(entry, source, grid, block, arrays, 1)
    ref = want["y"].astype(np.float32).ravel()
    assert (out == ref).all()


def test_text_of_a_kernel_that_failed_on_the_gpu_is_right(monkeypatch):
    """Random program 81 at scale 48 under the bounds of the time: one element-wise kernel names 59 operand buffers and
    4 results and evaluates some 140 loads under predicates; compiled for gfx950 it takes all 512 vector registers,
    keeps over 200 scalar registers in lanes and spills some 80 vector registers to scratch, and on the GPU it
    produced wrong elements.  Compiled for the host from the same text and fed the oracle's values of its operands, it
    reproduces the oracle's values of all four results bit for bit (every operation in it is exactly rounded and
    evaluated in program order on both sides)."""
    from fuzz_programs import random_program
    from oracle.interp import OracleDevice
    monkeypatch.setenv("ADHIP_KERNEL_BOUNDS", OLD_BOUNDS)
    dev = Capture()
    random_program(dev, 81, scale=48)
    plan, kernels = generated_kernels(dev.proc, dev.deps)
    import re
    entry = max((e for e, (kind, _) in kernels.items() if kind == "elw"),
                key=lambda e: len(set(re.findall(r"\bb\d+\b", kernels[e][1]))))
    source = kernels[entry][1]
    n_out = len(set(re.findall(r"\bo\d+\b", source)))
    assert len(set(re.findall(r"\bb\d+\b", source))) >= 50 and n_out == 4
    grid, block, args = launch_of(plan, entry)
    oracle = OracleDevice()
    random_program(oracle, 81, scale=48)
    written = {}
    for c in dev.proc.walk():
        r = getattr(c, "res", None) or getattr(c, "s", None)
        if r:
            written[r] = written.get(r, 0) + 1
    arrays = []
    for id, _, n in args:
        assert written.get(id, 0) <= 1, f"{id} is written more than once: its final value is not what the kernel saw"
        v = np.asarray(oracle.buf[id] if id in oracle.buf else oracle._value(id), np.float32).ravel()
        assert v.size == n
        arrays.append(v)
    outs = run_on_host(entry, source, grid, block, arrays, n_out)
    for out, ref in zip(outs, arrays[:n_out]):
        assert np.abs(ref).max() > 0
        assert (out == ref).all()
