"""Every variant of the 256x128 block tile of the matrix-core kernel, value-checked.

The lowering picks that tile only for outputs of at least 4096 x 4096 (512 tiles), so these cases use such an output
with a short inner dimension (k = 256 keeps the float64 reference cheap): the four operand layouts (k- or m-contiguous
A, k- or n-contiguous B: the forward product and the two backward products of reference
src/graph/ops/dot_product.rs:34-42 read their operands that way), each plain and with an element-wise epilogue on the
accumulators.  The kernel each case runs is asserted from the plan, so a change of the selection rule cannot turn the
test into one of another tile without notice.  Tolerance: 1e-5 * sqrt(k) of the largest |a|.|b| dot product."""
import math
import re

import numpy as np
import pytest

from adhip import ir as IR
from adhip.device import lower_describe
from parity import RED_RTOL, assert_close

pytestmark = pytest.mark.gpu

M = N = 4096


def _operands(layout, k, rng):
    """IR commands that define `a` [M,k] and `b` [k,N] with the requested contiguity, and the arrays as float64."""
    cmds = []
    if layout[0] == "k":
        a = rng.standard_normal((M, k), dtype=np.float32)
        cmds.append(IR.CreateMat(a.reshape(-1), [M, k], "a"))
        a64 = a.astype(np.float64)
    else:
        at = rng.standard_normal((k, M), dtype=np.float32)
        cmds += [IR.CreateMat(at.reshape(-1), [k, M], "at"), IR.Permute(a="at", p=[1, 0], res="a")]
        a64 = at.T.astype(np.float64)
    if layout[1] == "n":
        b = rng.standard_normal((k, N), dtype=np.float32)
        cmds.append(IR.CreateMat(b.reshape(-1), [k, N], "b"))
        b64 = b.astype(np.float64)
    else:
        bt = rng.standard_normal((N, k), dtype=np.float32)
        cmds += [IR.CreateMat(bt.reshape(-1), [N, k], "bt"), IR.Permute(a="bt", p=[1, 0], res="b")]
        b64 = bt.T.astype(np.float64)
    return cmds, a64, b64


def _kernels(proc, keep):
    return re.findall(r"launch dot_\w+ \[dot_mfma\] kernel=(\w+)", lower_describe(proc, set(keep)))


@pytest.mark.parametrize("layout", ["kn", "kk", "mn", "mk"])
@pytest.mark.parametrize("k", [256, 272])
def test_256_tile_plain(layout, k, hip_device):
    print(f"[case] 256x128 tile, layout {layout}, k {k}", flush=True)
    rng = np.random.default_rng(100 + k + sum(map(ord, layout)))
    cmds, a64, b64 = _operands(layout, k, rng)
    cmds += [IR.DotProduct(a="a", b="b", res="c"), IR.EX()]
    proc = IR.IRProcedure("main", cmds)
    assert _kernels(proc, ["c"]) == [f"adhip_gemm_{layout}_256"]
    hip_device.execute(proc, {"c"})
    got = hip_device.get_tensor("c")
    assert got.dim == [M, N]
    ref = a64 @ b64
    scale = float((np.abs(a64) @ np.abs(b64)).max())
    assert_close(got.data, ref.reshape(-1), RED_RTOL * math.sqrt(k), f"c ({layout})", scale=scale)


@pytest.mark.parametrize("layout", ["kn", "kk", "mn", "mk"])
@pytest.mark.parametrize("kind", ["update", "activation"])
def test_256_tile_epilogue(layout, kind, hip_device):
    """`update`: W += -0.01 * (A.B), the product itself never stored (the SGD step on a weight gradient);
    `activation`: y = sigmoid-like 1 / (1 + exp2(-(A.B + bias))) with the product also kept."""
    print(f"[case] 256x128 tile epilogue, layout {layout}, {kind}", flush=True)
    k = 256
    rng = np.random.default_rng(200 + sum(map(ord, layout + kind)))
    cmds, a64, b64 = _operands(layout, k, rng)
    d = a64 @ b64
    scale = float((np.abs(a64) @ np.abs(b64)).max())
    tol = RED_RTOL * math.sqrt(k)
    if kind == "update":
        w = rng.standard_normal((M, N), dtype=np.float32)
        cmds += [IR.CreateMat(w.reshape(-1), [M, N], "w"), IR.DotProduct(a="a", b="b", res="d"),
                 IR.CreateConstant(-0.01, "c", [M, N]), IR.ElwMultiply(a="d", b="c", res="t"), IR.ElwAddEq(s="w", o="t"), IR.EX()]
        keep = ["w"]
        proc = IR.IRProcedure("main", cmds)
        names = _kernels(proc, keep)
        assert len(names) == 1 and re.fullmatch(rf"adhip_gemm_{layout}_256_e\d+", names[0]), names
        hip_device.execute(proc, set(keep))
        got = hip_device.get_tensor("w")
        assert_close(got.data, (w.astype(np.float64) - 0.01 * d).reshape(-1), tol, "w", scale=scale)
    else:
        bias = rng.standard_normal(N).astype(np.float32)
        cmds += [IR.CreateMat(bias, [N], "bias"), IR.DotProduct(a="a", b="b", res="p"),
                 IR.View(a="bias", target_dim=[1, N], res="b1"), IR.Broadcast(a="b1", dim=0, r=M, res="bb"),
                 IR.ElwAdd(a="p", b="bb", res="h"), IR.CreateConstant(-1.0 / 64.0, "m1", [M, N]), IR.ElwMultiply(a="h", b="m1", res="nh"),
                 IR.Exp2(a="nh", res="e"), IR.CreateConstant(1.0, "one", [M, N]), IR.ElwAdd(a="e", b="one", res="den"),
                 IR.Recip(a="den", res="y"), IR.EX()]
        keep = ["y", "p"]
        proc = IR.IRProcedure("main", cmds)
        names = _kernels(proc, keep)
        assert len(names) == 1 and re.fullmatch(rf"adhip_gemm_{layout}_256_e\d+", names[0]), names
        hip_device.execute(proc, set(keep))
        assert_close(hip_device.get_tensor("p").data, d.reshape(-1), tol, "p", scale=scale)
        y = 1.0 / (1.0 + np.exp2(-(d + bias) / 64.0))
        # |dy/dh| <= 1/64 * 1/4: the product's error is damped; the chain adds a few roundings of its own
        assert_close(hip_device.get_tensor("y").data, y.reshape(-1), tol * scale / 256.0 + 4e-7, "y", scale=1.0)


def _operand(cmds, name, rows, cols, rows_contiguous, gapped, rng):
    """Defines `name` as a [rows, cols] operand and returns it as float64.  `rows_contiguous`: the rows (not the
    columns) have unit stride.  `gapped`: the operand is every other line of a tensor twice as large, so its leading
    dim is a multiple of four elements although its contiguous extent is not, and the last 128-bit quad of every line
    is only partly inside the operand."""
    lines, run = (cols, rows) if rows_contiguous else (rows, cols)   # memory: `lines` lines of `run` contiguous elements
    if gapped:
        full = rng.standard_normal((lines, 2, run), dtype=np.float32)
        cmds += [IR.CreateMat(full.reshape(-1), [lines, 2, run], name + "_full"), IR.Index(a=name + "_full", index=0, dim=1, res=name + "_m")]
        mem = full[:, 0, :]
    else:
        mem = rng.standard_normal((lines, run), dtype=np.float32)
        cmds.append(IR.CreateMat(mem.reshape(-1), [lines, run], name + "_m"))
    if rows_contiguous:
        cmds.append(IR.Permute(a=name + "_m", p=[1, 0], res=name))
        return mem.T.astype(np.float64)
    cmds.append(IR.Contigious(a=name + "_m", res=name) if False else IR.View(a=name + "_m", target_dim=[rows, cols], res=name))
    return mem.astype(np.float64)


@pytest.mark.parametrize("layout", ["kn", "kk", "mn", "mk"])
@pytest.mark.parametrize("shape", [(200, 136, 100, False, "rim"),     # multiples of 4 that fit no tile: 128-bit loads, checked rim
                                   (130, 70, 50, True, "rim"),        # aligned leading dims, extents end inside a quad
                                   (520, 300, 1030, True, "rim"),     # the same with k cut into slices
                                   (2100, 2100, 260, False, "128x64_rim"), (2050, 4100, 130, True, "128_rim"),   # the larger tiles
                                   (203, 131, 77, False, "rim"),      # nothing aligned: 128-bit loads that start at any element
                                   (2051, 2303, 35, False, "rim"),
                                   (700, 900, 2, False, None), (515, 3, 300, False, None),   # lines of fewer than four elements: single loads
                                   (1, 4096, 64, False, None), (4096, 1, 64, False, None)])
def test_ragged_products(layout, shape, hip_device):
    """Products whose extents fit no tile, in the four operand layouts: the kernel variant with 128-bit loads inside
    and checked single elements on the rim, and the variant with single elements only."""
    m, n, k, gapped, variant = shape
    print(f"[case] ragged product {m}x{n}x{k} layout {layout} gapped {gapped}", flush=True)
    rng = np.random.default_rng(m * 7 + n * 3 + k + sum(map(ord, layout)))
    cmds = []
    a64 = _operand(cmds, "a", m, k, layout[0] == "m", gapped, rng)
    b64 = _operand(cmds, "b", k, n, layout[1] == "k", gapped, rng)
    cmds += [IR.DotProduct(a="a", b="b", res="c"), IR.EX()]
    proc = IR.IRProcedure("main", cmds)
    if variant and m > 1 and n > 1:
        names = _kernels(proc, ["c"])
        assert names and all(("_" + variant) in x for x in names), names
    hip_device.execute(proc, {"c"})
    got = hip_device.get_tensor("c")
    assert got.dim == [m, n]
    ref = a64 @ b64
    scale = float((np.abs(a64) @ np.abs(b64)).max())
    assert_close(got.data, ref.reshape(-1), RED_RTOL * math.sqrt(k), f"c ({layout})", scale=scale)


def _wide_line_product(dev):
    """C = A B with A the first 64 columns of a [64, 2^22] tensor: aligned in every respect, but a line of A is 2^22
    elements long."""
    from adhip import autodiff
    from adhip.core import dot
    autodiff.set_device(dev)
    rng = np.random.default_rng(11)
    wide = np.zeros((64, 1 << 22), np.float32)
    wide[:, :64] = rng.standard_normal((64, 64), dtype=np.float32)
    bn = rng.standard_normal((64, 128), dtype=np.float32)
    x = autodiff.tensor(wide.reshape(-1), [64, 1 << 22])
    b = autodiff.tensor(bn.reshape(-1), [64, 128])
    c = dot(x.r(range(0, 64), 1), b)
    c.forward()
    c.val().keep()
    return c, wide[:, :64].astype(np.float64) @ bn.astype(np.float64)


def test_lines_of_2_to_the_22_take_the_checked_variant(hip_device):
    """The kernel without bounds checks addresses a tile by 32-bit offsets from its corner; an operand whose lines are
    2^22 elements apart is therefore given to the checked variant (64-bit index arithmetic), and the product is right."""
    from adhip import autodiff
    from test_row_chains import Capture
    print("[case] product with a leading dim of 2^22", flush=True)
    cap = Capture()
    _wide_line_product(cap)
    autodiff.execute()
    names = _kernels(cap.proc, cap.deps)
    assert names and all("_rim" in n or "_edge" in n for n in names), names
    c, want = _wide_line_product(hip_device)
    autodiff.execute()
    got = c.val().get()
    assert got.dim == [64, 128]
    assert_close(got.data, want.reshape(-1), RED_RTOL * math.sqrt(64), "c", scale=float(np.abs(want).max()))
