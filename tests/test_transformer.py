"""The attention / transformer-encoder modules of the caller side (reference src/nn/transformer.rs) end to end:
forward and every gradient of one encoder layer against a float64 restatement in torch, on the oracle (CPU) and on
the device (GPU), and the device against the oracle."""
import math

import numpy as np
import pytest

from adhip import autodiff
from adhip import workloads as W
from adhip.core import dot
from oracle.interp import OracleDevice
from parity import RED_RTOL, assert_close
from transformer_ref import encoder_layer_reference


def _against_reference(out, inputs, heads, rtol):
    ref = encoder_layer_reference(inputs, heads)
    assert set(out) == set(ref)
    for k, v in out.items():
        assert not v.is_none, k
        assert list(v.dim) == list(ref[k].shape), k
        assert_close(v.data, ref[k].reshape(-1), rtol, k)


@pytest.mark.parametrize("seq,d_model,heads,ff", [(8, 16, 4, 32), (12, 8, 1, 8), (24, 32, 2, 48)])
def test_encoder_layer_oracle_matches_float64_autograd(seq, d_model, heads, ff):
    wl = W.encoder_layer(OracleDevice(), seq, d_model, heads, ff, seed=seq)
    _against_reference(wl.run(), wl.inputs, heads, 2e-5)


def test_leaf_gradients_do_not_alias():
    """v = x + w feeds two consumers: the gradient value handed to x and to w is one and the same IR id, so adding
    the second contribution in place (as the reference does) would change both leaves' gradients twice."""
    autodiff.set_device(OracleDevice())
    rng = np.random.default_rng(3)
    xn, wn = rng.standard_normal((6, 8)).astype(np.float32), rng.standard_normal((6, 8)).astype(np.float32)
    x, w = autodiff.tensor(xn, [6, 8]), autodiff.tensor(wn, [6, 8])
    v = x + w
    L = (v * v).sum(0).sum(0)
    L.forward()
    L.backward()
    gx, gw = x.grad(), w.grad()
    gx.keep()
    gw.keep()
    autodiff.execute()
    expect = 2.0 * (xn.astype(np.float64) + wn)
    assert_close(gx.get().data, expect.reshape(-1), 1e-6, "dx")
    assert_close(gw.get().data, expect.reshape(-1), 1e-6, "dw")


@pytest.mark.gpu
@pytest.mark.parametrize("seq,d_model,heads,ff", [(8, 16, 4, 32), (64, 32, 4, 64), (200, 96, 3, 160)])
def test_encoder_layer_device_matches_oracle_and_reference(seq, d_model, heads, ff, hip_device):
    print(f"[case] encoder layer {seq}x{d_model} heads {heads} ff {ff}", flush=True)
    got = W.encoder_layer(hip_device, seq, d_model, heads, ff, seed=seq).run()
    wl = W.encoder_layer(OracleDevice(), seq, d_model, heads, ff, seed=seq)
    ref = wl.run()
    tol = 4 * RED_RTOL * math.sqrt(max(seq, d_model, ff))
    for k, rv in ref.items():
        assert got[k].dim == rv.dim, k
        assert_close(got[k].data, rv.data, tol, k)
    _against_reference(got, wl.inputs, heads, 1e-4)


@pytest.mark.gpu
def test_encoder_layer_matrix_core_sizes(hip_device):
    """Sizes at which every product goes to the MFMA kernel (aligned and edge variants, epilogues included), checked
    against float64 autograd only (the oracle's one-thread-per-output matmul is too slow here)."""
    print("[case] encoder layer 512x256", flush=True)
    wl = W.encoder_layer(hip_device, 512, 256, 4, 1024, seed=5)
    _against_reference(wl.run(), wl.inputs, 4, 2e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["layernorm", "rms", "softmax"])
@pytest.mark.parametrize("rows,cols", [(2048, 768), (333, 1000)])
def test_norm_modules_at_scale_match_float64_autograd(kind, rows, cols, hip_device):
    """LayerNorm, RMS and softmax over a few thousand rows, forward and backward, against float64 autograd (the small
    known-answer tests of the two norms are in the reference's norm.rs; softmax has none there).  The softmax inputs
    reach +-100: exp alone would overflow at 88."""
    print(f"[case] {kind} {rows}x{cols}", flush=True)
    import torch
    from adhip import nn
    rng = np.random.default_rng(rows + cols)
    xn = rng.standard_normal((rows, cols)).astype(np.float32)
    rn = rng.standard_normal((rows, cols)).astype(np.float32)
    if kind == "softmax":
        xn *= 25.0
        xn[0, :] = 100.0
        xn[1, 0], xn[1, 1] = 100.0, -100.0
    autodiff.set_device(hip_device)
    x = autodiff.tensor(xn, [rows, cols])
    mod = {"layernorm": lambda: nn.LayerNorm(cols), "rms": lambda: nn.RMS(cols), "softmax": lambda: nn.Softmax(-1)}[kind]()
    y = mod.f(x)
    L = (y * autodiff.tensor(rn, [rows, cols])).sum(0).sum(0)
    L.forward()
    L.backward()
    y.val().keep()
    x.grad().keep()
    autodiff.execute()
    got_y, got_dx = y.val().get(), x.grad().get()

    xt = torch.tensor(xn, dtype=torch.float64, requires_grad=True)
    if kind == "layernorm":
        mean = xt.mean(-1, keepdim=True)
        var = ((xt - mean) ** 2).sum(-1) / cols
        yt = (xt - mean) / torch.sqrt(var + 1e-9).unsqueeze(-1)
    elif kind == "rms":
        yt = xt / torch.sqrt((xt ** 2).mean(-1, keepdim=True) + 1e-9)
    else:
        yt = torch.softmax(xt, -1)
    (yt * torch.tensor(rn, dtype=torch.float64)).sum().backward()
    tol = RED_RTOL * math.sqrt(cols)
    assert_close(got_y.data, yt.detach().numpy().reshape(-1), tol, "y")
    assert_close(got_dx.data, xt.grad.numpy().reshape(-1), 4 * tol, "dx")


@pytest.mark.gpu
@pytest.mark.parametrize("seq,d_model,heads,ff", [(128, 128, 2, 256), (96, 144, 3, 200), (16, 16, 4, 32)])
def test_encoder_training_loop_matches_oracle(seq, d_model, heads, ff, hip_device):
    """Three SGD steps on an encoder layer inside an IR for-loop (workloads.encoder_train): grouped per-head products,
    product epilogues and in-place weight updates inside a loop body, where every update must come after the last
    product of the iteration that still reads the old weights.  What is compared is how far each weight moved, which
    is a thousand times smaller than the weight itself."""
    print(f"[case] encoder training loop {seq}x{d_model} heads {heads} ff {ff}", flush=True)
    got = W.encoder_train(hip_device, seq, d_model, heads, ff, iters=3, lr=1.0, seed=seq).run()
    wl = W.encoder_train(OracleDevice(), seq, d_model, heads, ff, iters=3, lr=1.0, seed=seq)
    ref = wl.run()
    assert_close(got["loss"].data, ref["loss"].data, 1e-4, "loss")
    for k, rv in ref.items():
        if k not in wl.inputs:
            continue
        w0 = wl.inputs[k].reshape(-1).astype(np.float64)
        moved_ref = np.asarray(rv.data, dtype=np.float64) - w0
        moved_got = np.asarray(got[k].data, dtype=np.float64) - w0
        assert np.abs(moved_ref).max() > 1e-4, f"{k} did not train"
        err = np.abs(moved_got - moved_ref).max()
        assert err <= 2e-3 * np.abs(moved_ref).max() + 4e-7 * np.abs(w0).max(), (k, err, np.abs(moved_ref).max())
