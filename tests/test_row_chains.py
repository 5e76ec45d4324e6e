"""Row chains: a row reduction and what follows it row by row (softmax, LayerNorm, RMS and their backward passes)
lowered to one kernel in which a wavefront or a block owns a row (reference src/nn/activations/softmax.rs:1-30,
src/nn/norm/layer.rs:1-30, src/nn/norm/rms.rs:1-27 are the compositions; the reference runs every command of them as
a kernel of its own)."""
import math
import re

import numpy as np
import pytest

from adhip import autodiff, nn
from adhip.core import ValueData
from adhip.device import Device, lower_describe
from oracle.interp import OracleDevice
from parity import RED_RTOL


class Capture(Device):
    def execute(self, proc, deps):
        self.proc, self.deps = proc, deps

    def get_tensor(self, id):
        return ValueData.none()


def _program(dev, kind, rows, cols, seed=0, backward=True):
    """y = f(x) for f in softmax / LayerNorm / RMS over the last dim of x [rows, cols], L = sum(y * w); keeps y and the
    gradients of x and of the module's parameters."""
    autodiff.set_device(dev)
    rng = np.random.default_rng(seed)
    xn = (rng.standard_normal((rows, cols)) * 3).astype(np.float32)
    wn = rng.standard_normal((rows, cols)).astype(np.float32)
    gn = rng.uniform(0.5, 1.5, cols).astype(np.float32)
    bn = rng.standard_normal(cols).astype(np.float32)
    x = autodiff.tensor(xn, [rows, cols])
    w = autodiff.tensor(wn, [rows, cols])
    params = {}
    if kind == "softmax":
        y = x.softmax(-1)
    elif kind == "layernorm":
        m = nn.LayerNorm.__new__(nn.LayerNorm)
        m.scale, m.bias = autodiff.tensor(gn, [cols]), autodiff.tensor(bn, [cols])
        params = {"dscale": m.scale, "dbias": m.bias}
        y = m.f(x)
    else:
        m = nn.RMS.__new__(nn.RMS)
        m.scale = autodiff.tensor(gn, [cols])
        params = {"dscale": m.scale}
        y = m.f(x)
    L = (y * w).sum(0).sum(0)
    L.forward()
    y.val().keep()
    outs = {"y": y.val()}
    if backward:
        L.backward()
        outs["dx"] = x.grad()
        for k, p in params.items():
            outs[k] = p.grad()
    return outs, (xn, wn, gn, bn)


def _float64(kind, xn, wn, gn, bn):
    import torch
    x = torch.tensor(xn.astype(np.float64), requires_grad=True)
    g = torch.tensor(gn.astype(np.float64), requires_grad=True)
    b = torch.tensor(bn.astype(np.float64), requires_grad=True)
    if kind == "softmax":
        y = torch.softmax(x, dim=-1)
    elif kind == "layernorm":
        y = torch.nn.functional.layer_norm(x, (x.shape[1],), g, b, eps=1e-9)
    else:
        y = g * (x / torch.sqrt(torch.mean(x * x, dim=-1, keepdim=True) + 1e-9))
    (y * torch.tensor(wn.astype(np.float64))).sum().backward()
    out = {"y": y.detach().numpy(), "dx": x.grad.numpy()}
    if kind != "softmax":
        out["dscale"] = g.grad.numpy()
    if kind == "layernorm":
        out["dbias"] = b.grad.numpy()
    return out


def _launches(proc, deps):
    return [(m.group(1), m.group(2)) for m in re.finditer(r"launch (\S+) \[(\w+)\]", lower_describe(proc, deps))]


@pytest.mark.parametrize("kind", ["softmax", "layernorm", "rms"])
def test_forward_is_one_row_kernel(kind, monkeypatch):
    """Forward only, [2048, 768]: the whole normalisation is one launch that reads x once and writes y once; with the
    chains switched off (ADHIP_ROW_CHAINS=0) it is two to four launches (reductions and element-wise passes in turn)."""
    dev = Capture()
    _program(dev, kind, 2048, 768, backward=False)
    autodiff.execute()
    ls = _launches(dev.proc, dev.deps)
    assert [k for _, k in ls] == ["rowchain"], ls
    text = lower_describe(dev.proc, dev.deps)
    chain = [l for l in text.splitlines() if "[rowchain]" in l][0]
    moved = float(re.search(r"bytes=(\d+)", chain).group(1))
    assert moved <= 4.0 * 2048 * 768 * 2 + 4.0 * 768 * 2 + 64, chain   # x in, y out, the parameters
    monkeypatch.setenv("ADHIP_ROW_CHAINS", "0")
    plain = _launches(dev.proc, dev.deps)
    assert not any(k == "rowchain" for _, k in plain) and len(plain) > len(ls), plain


@pytest.mark.parametrize("kind", ["softmax", "layernorm", "rms"])
@pytest.mark.parametrize("rows,cols", [(333, 1000), (64, 8192), (100, 2052)])
def test_chains_compile_without_spills(kind, rows, cols, monkeypatch):
    """Wavefront-per-row and block-per-row forms, ragged rows, eight 128-bit pieces per thread: every kernel compiles
    for gfx950 and none spills a vector register."""
    from test_library_cpu import _compile_check, _vector_spills
    monkeypatch.setenv("ADHIP_CACHE_DIR", "off")
    dev = Capture()
    _program(dev, kind, rows, cols)
    autodiff.execute()
    assert any(k == "rowchain" for _, k in _launches(dev.proc, dev.deps))
    rc, msg = _compile_check(dev.proc, dev.deps)
    assert rc == 0, msg
    assert not _vector_spills(msg) and "tighter kernel bounds" not in msg, msg


def test_softmax_over_columns_is_not_a_row_chain():
    """softmax(0) normalises down the columns: the values between the reductions are not laid out along the rows the
    reductions walk, so the kernels stay separate (and correct)."""
    dev = Capture()
    autodiff.set_device(dev)
    x = autodiff.tensor(np.ones(64 * 48, np.float32), [64, 48])
    y = x.softmax(0)
    y.forward()
    y.val().keep()
    autodiff.execute()
    assert not any(k == "rowchain" for _, k in _launches(dev.proc, dev.deps))


SHAPES = [(2048, 768), (333, 1000), (64, 8192), (100, 2052), (7, 4), (5, 12), (1000, 64)]


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["softmax", "layernorm", "rms"])
@pytest.mark.parametrize("rows,cols", SHAPES)
def test_norm_modules_at_scale_match_float64(kind, rows, cols, hip_device):
    """Forward and backward of softmax / LayerNorm / RMS through the row-chain kernels against float64 torch and the
    oracle.  A value may be 1e-5 sqrt(cols) of its own largest element off, or a few times as far from float64 as the
    oracle's float32 arithmetic is (the gradients of LayerNorm cancel to a fraction of their terms)."""
    print(f"[case] row chain {kind} {rows}x{cols}", flush=True)
    outs, data = _program(hip_device, kind, rows, cols, seed=rows + cols)
    autodiff.execute()
    got = {k: v.get() for k, v in outs.items()}
    o = OracleDevice()
    routs, _ = _program(o, kind, rows, cols, seed=rows + cols)
    autodiff.execute()
    ref = {k: v.get() for k, v in routs.items()}
    exact = _float64(kind, *data)
    tol = RED_RTOL * math.sqrt(max(cols, rows))
    for k, e in exact.items():
        g = np.asarray(got[k].data, np.float64).reshape(e.shape)
        r = np.asarray(ref[k].data, np.float64).reshape(e.shape)
        own = float(np.abs(e).max())
        oracle_err = float(np.abs(r - e).max())
        allowed = max(tol * own, 8.0 * oracle_err)
        assert np.isfinite(g).all()
        assert float(np.abs(g - e).max()) <= allowed, (kind, k, float(np.abs(g - e).max()), allowed, own)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["softmax", "layernorm", "rms"])
def test_chained_equals_unchained(kind, hip_device, monkeypatch):
    """The same program with and without row chains on the device: the chains change which kernel does the arithmetic,
    not the arithmetic (sums are added in another order)."""
    print(f"[case] row chain on/off {kind}", flush=True)
    rows, cols = 777, 516

    def run():
        outs, _ = _program(hip_device, kind, rows, cols, seed=3)
        autodiff.execute()
        return {k: np.asarray(v.get().data, np.float64) for k, v in outs.items()}
    chained = run()
    monkeypatch.setenv("ADHIP_ROW_CHAINS", "0")
    plain = run()
    for k in plain:
        s = float(np.abs(plain[k]).max())
        assert float(np.abs(chained[k] - plain[k]).max()) <= 4 * RED_RTOL * math.sqrt(cols) * s, k


def _in_place_normalise_program(rows, cols, iters, seed=5):
    """x [rows, cols] is replaced by its row softmax `iters` times inside a counted loop, spelled in commands: the chain
    reads the old x and writes the new one into the same buffer."""
    from adhip import ir as IR
    rng = np.random.default_rng(seed)
    xn = rng.standard_normal((rows, cols)).astype(np.float32)
    c = lambda v, id, sh: IR.CreateConstant(float(v), id, list(sh))  # noqa: E731
    body = [
        IR.Max(a="x", res="m"), IR.View(a="m", target_dim=[rows, 1], res="mv"), IR.Broadcast(a="mv", dim=1, r=cols, res="mb"),
        c(-1.0, "neg", [rows, cols]), IR.ElwMultiply(a="mb", b="neg", res="n"), IR.ElwAdd(a="x", b="n", res="d"),
        c(1.4426950408889634, "l2e", [rows, cols]), IR.ElwMultiply(a="d", b="l2e", res="e1"), IR.Exp2(a="e1", res="e"),
        IR.Sum(a="e", res="s"), IR.Recip(a="s", res="r"), IR.View(a="r", target_dim=[rows, 1], res="rv"),
        IR.Broadcast(a="rv", dim=1, r=cols, res="rb"), IR.ElwMultiply(a="e", b="rb", res="x"),
        c(1.0, "one", [1]), IR.ElwAddEq(s="i", o="one"), c(-float(iters), "lim", [1]), IR.ElwAdd(a="i", b="lim", res="t"),
        IR.LessZero(a="t", res="go"),
    ]
    cmds = [IR.CreateMat(xn.reshape(-1), [rows, cols], "x"), IR.CreateMat(np.zeros(1, np.float32), [1], "i"),
            c(-float(iters), "lim0", [1]), IR.ElwAdd(a="i", b="lim0", res="t0"), IR.LessZero(a="t0", res="go"),
            IR.While(conditional_var="go", block=IR.IRProcedure("body", body)), IR.EX()]
    want = xn.astype(np.float64)
    for _ in range(iters):
        e = np.exp(want - want.max(1, keepdims=True))
        want = e / e.sum(1, keepdims=True)
    return IR.IRProcedure("main", cmds), {"x", "i"}, want


def test_in_place_chain_needs_no_copy():
    """The softmax that overwrites its own operand inside a loop is one row-chain launch per iteration, with no copy
    behind it: a chain reads all it needs of a row before it stores any of it."""
    proc, keep, _ = _in_place_normalise_program(512, 256, 3)
    text = lower_describe(proc, keep)
    body = text[text.index("while "):]
    assert body.count("[rowchain]") == 1 and "[copy]" not in body, body


@pytest.mark.gpu
@pytest.mark.parametrize("rows,cols", [(512, 256), (100, 2052), (37, 8192)])
def test_in_place_chain_in_a_loop_matches_float64(rows, cols, hip_device):
    print(f"[case] in-place row chain in a loop {rows}x{cols}", flush=True)
    proc, keep, want = _in_place_normalise_program(rows, cols, 3)
    hip_device.execute(proc, keep)
    assert hip_device.get_tensor("i").data[0] == 3.0
    got = hip_device.get_tensor("x").numpy().astype(np.float64)
    assert np.abs(got - want).max() <= RED_RTOL * math.sqrt(cols) * np.abs(want).max()
    np.testing.assert_allclose(got.sum(1), 1.0, rtol=1e-5)


def _redefining_program(rows, cols, seed=9):
    """`x` [rows, cols] is redefined as the [rows] vector of its rows' sums of exp2(x - max): the chain that reads the
    old x writes a value of another extent under the same id."""
    from adhip import ir as IR
    rng = np.random.default_rng(seed)
    xn = rng.standard_normal((rows, cols)).astype(np.float32)
    cmds = [IR.CreateMat(xn.reshape(-1), [rows, cols], "x"),
            IR.Max(a="x", res="m"), IR.View(a="m", target_dim=[rows, 1], res="mv"), IR.Broadcast(a="mv", dim=1, r=cols, res="mb"),
            IR.CreateConstant(-1.0, "neg", [rows, cols]), IR.ElwMultiply(a="mb", b="neg", res="n"), IR.ElwAdd(a="x", b="n", res="d"),
            IR.Exp2(a="d", res="e"), IR.Sum(a="e", res="x"), IR.EX()]
    x64 = xn.astype(np.float64)
    return IR.IRProcedure("main", cmds), {"x"}, np.exp2(x64 - x64.max(1, keepdims=True)).sum(1)


def test_a_chain_does_not_overwrite_an_operand_of_another_extent():
    """Row x's sum would land on element x of the buffer, which is element (0, x) of the old value that row 0 may still
    be reading: the result goes to a buffer of its own and is copied afterwards."""
    proc, keep, _ = _redefining_program(512, 256)
    text = lower_describe(proc, keep)
    assert "[rowchain]" in text and "launch commit_x [copy]" in text, text


@pytest.mark.gpu
@pytest.mark.parametrize("rows,cols", [(512, 256), (3000, 2052)])
def test_redefinition_with_another_extent_matches_float64(rows, cols, hip_device):
    print(f"[case] row chain redefines its operand's id with another extent {rows}x{cols}", flush=True)
    proc, keep, want = _redefining_program(rows, cols)
    hip_device.execute(proc, keep)
    got = hip_device.get_tensor("x")
    assert got.dim == [rows]
    assert np.abs(got.numpy().astype(np.float64) - want).max() <= RED_RTOL * math.sqrt(cols) * np.abs(want).max()
