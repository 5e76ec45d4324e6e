"""Writes tests/golden/wire_every_command.bin: the serialised form of one small program that uses every command of
the wire format once (the 26 variants of reference src/core/ir.rs:8-105 in the reference's field order, plus Max),
nested blocks included, with the CreateMat pointer fields set to zero.  The same program is built a second time in
C++ (tests/cxx/wire_fixture.cpp, through autodiff-ir-rust_amd/host/adhip_device.hpp); tests/test_wire_format.py holds
both writers, and the reader in csrc/ir.cpp, to these bytes.

Run from the repository root:  python tests/golden/make_wire_fixture.py"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path[:0] = [ROOT, os.path.join(ROOT, "autodiff-ir-rust_amd")]

from adhip import ir as IR  # noqa: E402


def every_command_program() -> IR.IRProcedure:
    f32 = np.float32
    body = IR.IRProcedure("loop", [IR.ElwAddEq(s="k", o="m1"), IR.MoreZero(a="k", res="cond")])
    arm0 = IR.IRProcedure("arm0", [IR.ElwMultiplyEq(s="e", o="c")])
    arm1 = IR.IRProcedure("arm1", [IR.CreateConstant(2.0, "two", [2, 3]), IR.ElwAddEq(s="e", o="two")])
    other = IR.IRProcedure("other", [IR.Heading(cmt="neither predicate held")])
    return IR.IRProcedure("main", [
        IR.Heading(cmt="every command once"),
        IR.CreateMat(np.arange(1, 7, dtype=f32), [2, 3], "a"),
        IR.CreateMat(np.array([1, 0, -1, 2, 0.5, 4], dtype=f32), [3, 2], "b"),
        IR.CreateConstant(0.5, "c", [2, 3]),
        IR.ElwMultiply(a="a", b="c", res="d"),
        IR.ElwAdd(a="a", b="d", res="e"),
        IR.ElwMultiplyEq(s="e", o="c"),
        IR.ElwAddEq(s="e", o="a"),
        IR.EqualZero(a="e", res="f"),
        IR.MoreZero(a="e", res="g"),
        IR.LessZero(a="e", res="h"),
        IR.Sum(a="e", res="s"),
        IR.DotProduct(a="a", b="b", res="p"),
        IR.View(a="a", target_dim=[3, 2], res="v"),
        IR.Index(a="a", index=1, dim=0, res="i"),
        IR.Concat(a="a", b="a", dim=0, res="cc"),
        IR.Permute(a="a", p=[1, 0], res="t"),
        IR.View(a="s", target_dim=[2, 1], res="s1"),
        IR.Broadcast(a="s1", dim=1, r=3, res="sb"),
        IR.Contigious(a="t", res="tc"),
        IR.Exp2(a="a", res="x2"),
        IR.Log2(a="x2", res="l2"),
        IR.Sin(a="a", res="sn"),
        IR.Recip(a="x2", res="rc"),
        IR.Sqrt(a="x2", res="sq"),
        IR.CreateMat(np.array([2], dtype=f32), [1], "k"),
        IR.CreateConstant(-1.0, "m1", [1]),
        IR.MoreZero(a="k", res="cond"),
        IR.While(conditional_var="cond", block=body),
        IR.EqualZero(a="k", res="is0"),
        IR.LessZero(a="k", res="neg"),
        IR.If(conditions=[("neg", arm0), ("is0", arm1)], else_proc=other),
        IR.Max(a="e", res="mx"),
        IR.EX(),
    ])


KEEP = ["e", "f", "g", "h", "s", "p", "v", "i", "cc", "sb", "tc", "l2", "sn", "rc", "sq", "k", "mx"]


def blanked(blob: bytes, offsets) -> bytes:
    out = bytearray(blob)
    for o in offsets:
        out[o:o + 8] = bytes(8)
    return bytes(out)


if __name__ == "__main__":
    offs = []
    blob, _keep = IR.serialize(every_command_program(), offs)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "wire_every_command.bin")
    with open(path, "wb") as f:
        f.write(blanked(blob, offs))
    print(path, len(blob), "bytes,", len(offs), "pointer fields blanked")
