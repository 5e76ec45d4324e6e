"""Programs built to strain the size of one generated kernel: many distinct buffers behind one Concat, one buffer read
through many pieces that do not continue one another, many operands gathered against the grain, and an element-wise
pass with many operands whose row and column sums are wanted too.  Each returns (procedure, keep list, numpy closed
form of every kept id), built straight from IR commands (no caller-side graph in between)."""
import numpy as np

from adhip import ir as IR


def _mat(rng, cmds, id, shape):
    data = rng.standard_normal(int(np.prod(shape))).astype(np.float32)
    cmds.append(IR.CreateMat(data, list(shape), id))
    return data.reshape(shape)


def wide_concat(n, rows=64, cols=3, seed=0):
    """y = concat(a0..a(n-1), dim 1) * concat(b0..b(n-1), dim 1): 2n distinct buffers under one multiplication."""
    rng = np.random.default_rng(seed)
    cmds, vals = [], {}
    for c in "ab":
        parts = [_mat(rng, cmds, f"{c}{i}", (rows, cols)) for i in range(n)]
        prev = f"{c}0"
        for i in range(1, n):
            cmds.append(IR.Concat(a=prev, b=f"{c}{i}", dim=1, res=f"{c}c{i}"))
            prev = f"{c}c{i}"
        vals[c] = (prev, np.concatenate(parts, axis=1))
    cmds.append(IR.ElwMultiply(a=vals["a"][0], b=vals["b"][0], res="y"))
    return IR.IRProcedure("main", cmds + [IR.EX()]), {"y"}, {"y": vals["a"][1] * vals["b"][1]}


def one_buffer_pieces(n, rows=256, seed=1):
    """y[:, i] = x[:, 2 (n-1-i)] * w[:, i]: one buffer behind n pieces, none of which continues its neighbour."""
    rng = np.random.default_rng(seed)
    cmds = []
    x = _mat(rng, cmds, "x", (rows, 2 * n))
    w = _mat(rng, cmds, "w", (rows, n))
    prev = None
    for i in range(n):
        cmds.append(IR.Index(a="x", index=2 * (n - 1 - i), dim=1, res=f"c{i}"))
        cmds.append(IR.View(a=f"c{i}", target_dim=[rows, 1], res=f"u{i}"))
        if prev is None:
            prev = f"u{i}"
        else:
            cmds.append(IR.Concat(a=prev, b=f"u{i}", dim=1, res=f"k{i}"))
            prev = f"k{i}"
    cmds.append(IR.ElwMultiply(a=prev, b="w", res="y"))
    return IR.IRProcedure("main", cmds + [IR.EX()]), {"y"}, {"y": x[:, ::2][:, ::-1] * w}


def gathers(n, r=256, c=256, seed=2):
    """s = g0^T + g1^T + ... : n operands read against the grain (too small for the transposing copy)."""
    rng = np.random.default_rng(seed)
    cmds, prev, acc = [], None, None
    for i in range(n):
        g = _mat(rng, cmds, f"g{i}", (c, r))
        cmds.append(IR.Permute(a=f"g{i}", p=[1, 0], res=f"t{i}"))
        if prev is None:
            prev, acc = f"t{i}", g.T.copy()
        else:
            cmds.append(IR.ElwAdd(a=prev, b=f"t{i}", res=f"s{i}"))
            prev, acc = f"s{i}", acc + g.T
    return IR.IRProcedure("main", cmds + [IR.EX()]), {prev}, {prev: acc}


def rider(n, rows=2048, cols=1024, seed=3):
    """m = x0 * x1 * ... * x(n-1) with m.sum(1) and m.sum(0) wanted as well: the sums ride on the pass if it is small
    enough (1024 threads a block leave a lane 128 vector registers)."""
    rng = np.random.default_rng(seed)
    cmds, prev, acc = [], None, None
    for i in range(n):
        x = _mat(rng, cmds, f"x{i}", (rows, cols))
        if prev is None:
            prev, acc = f"x{i}", x.copy()
        else:
            cmds.append(IR.ElwMultiply(a=prev, b=f"x{i}", res=f"m{i}"))
            prev, acc = f"m{i}", acc * x
    cmds.append(IR.Sum(a=prev, res="rs"))
    cmds.append(IR.Permute(a=prev, p=[1, 0], res="pt"))
    cmds.append(IR.Sum(a="pt", res="cs"))
    a64 = acc.astype(np.float64)
    return IR.IRProcedure("main", cmds + [IR.EX()]), {prev, "rs", "cs"}, {prev: acc, "rs": a64.sum(1), "cs": a64.sum(0)}
