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
