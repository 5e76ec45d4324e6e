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


# ---- fused attention --------------------------------------------------------------------------------------------

def _attention_float64(q, k, v, d_model, mask=None):
    s = q.astype(np.float64) @ k.astype(np.float64).T / math.sqrt(float(d_model))
    if mask is not None:
        s = s * mask
    e = np.exp(s - s.max(-1, keepdims=True))
    return (e / e.sum(-1, keepdims=True)) @ v.astype(np.float64)


def _attention_program(dev, sq, sk, d, dv, d_model, seed, spread=1.0, mask=False, keep_scores=False):
    """O = Attention(Q, K, V) on tensors handed in as they are: Q [sq, d], K [sk, d], V [sk, dv]."""
    from adhip import nn
    autodiff.set_device(dev)
    rng = np.random.default_rng(seed)
    qn = (spread * rng.standard_normal((sq, d))).astype(np.float32)
    kn = (spread * rng.standard_normal((sk, d))).astype(np.float32)
    vn = rng.standard_normal((sk, dv)).astype(np.float32)
    mn = (rng.random((sq, sk)) < 0.7).astype(np.float32) if mask else None
    Q, K, V = autodiff.tensor(qn, [sq, d]), autodiff.tensor(kn, [sk, d]), autodiff.tensor(vn, [sk, dv])
    if mask:
        o = nn.AttentionMasked(Q, K, V, d_model, autodiff.tensor(mn, [sq, sk]))
    else:
        o = nn.Attention(Q, K, V, d_model)
    o.forward()
    o.val().keep()
    return o, (qn, kn, vn, mn)


_FUSED_SHAPES = [
    # sq, sk, d, dv: one query block and many, ragged in both directions, narrow and wide heads, sq != sk, d != dv
    (64, 64, 16, 16), (100, 100, 48, 48), (1, 7, 4, 16), (65, 129, 8, 32), (300, 77, 64, 64), (257, 640, 128, 128),
    (130, 1000, 36, 80), (96, 200, 256, 256), (200, 96, 20, 240), (33, 31, 16, 16), (64, 33, 64, 48), (2100, 40, 32, 32),
    # 512 row blocks and more: the variant with blocks of four wavefronts
    (33000, 40, 16, 16), (32768, 70, 20, 32),
]


@pytest.mark.parametrize("sq,sk,d,dv", _FUSED_SHAPES)
def test_attention_lowers_to_one_kernel(sq, sk, d, dv):
    from adhip.core import ValueData
    from adhip.device import Device, lower_describe

    class Capture(Device):
        def execute(self, proc, deps):
            self.proc, self.deps = proc, list(deps)

        def get_tensor(self, id):
            return ValueData.none()

    dev = Capture()
    _attention_program(dev, sq, sk, d, dv, 64, 0)
    autodiff.execute()
    launches = [l for l in lower_describe(dev.proc, dev.deps).splitlines() if l.lstrip().startswith("launch")]
    assert len(launches) == 1 and "[attention]" in launches[0], launches
    assert f"adhip_attention_d{d}_v{dv}_k" in launches[0]
    # the kernel of this head width compiles for gfx950 (both score layouts: d % 16 == 0 and not; narrow and wide tiles)
    from test_library_cpu import _compile_check
    rc, msg = _compile_check(dev.proc, dev.deps)
    assert rc == 0, msg


@pytest.mark.parametrize("what", ["mask_of_another_shape", "scores_kept", "head_of_6", "plain_exp"])
def test_attention_that_does_not_match_stays_unfused(what, monkeypatch):
    """A factor between the scaling and the softmax that is not a mask of the scores' shape, a softmax somebody else
    reads, a head width the kernel has no tile for, or the reference's own max-less softmax: none of them is the fused
    kernel's arithmetic."""
    from adhip.core import ValueData
    from adhip.device import Device, lower_describe

    class Capture(Device):
        def execute(self, proc, deps):
            self.proc, self.deps = proc, list(deps)

        def get_tensor(self, id):
            return ValueData.none()

    dev = Capture()
    autodiff.set_device(dev)
    if what == "mask_of_another_shape":
        rng = np.random.default_rng(0)
        Q, K, V = (autodiff.tensor(rng.standard_normal((64, 16)).astype(np.float32), [64, 16]) for _ in range(3))
        row = autodiff.tensor(rng.random(64).astype(np.float32), [64])     # one factor per key, broadcast over the queries
        o = dot((dot(Q, K.t()) / 8.0 * row).softmax(-1), V)
        o.forward()
        o.val().keep()
    elif what == "head_of_6":
        _attention_program(dev, 64, 64, 6, 16, 64, 0)
    else:
        rng = np.random.default_rng(0)
        Q, K, V = (autodiff.tensor(rng.standard_normal((64, 16)).astype(np.float32), [64, 16]) for _ in range(3))
        s = dot(Q, K.t()) / 8.0
        if what == "scores_kept":
            p = s.softmax(-1)
        else:
            e = s.exp()
            p = e / e.sum(-1).unsqueeze(-1)
        o = dot(p, V)
        o.forward()
        o.val().keep()
        if what == "scores_kept":
            p.val().keep()
    autodiff.execute()
    text = lower_describe(dev.proc, dev.deps)
    assert "[attention]" not in text, text


def test_attention_fusion_can_be_switched_off(monkeypatch):
    from adhip.core import ValueData
    from adhip.device import Device, lower_describe

    class Capture(Device):
        def execute(self, proc, deps):
            self.proc, self.deps = proc, list(deps)

        def get_tensor(self, id):
            return ValueData.none()

    dev = Capture()
    _attention_program(dev, 64, 64, 16, 16, 64, 0)
    autodiff.execute()
    assert "[attention]" in lower_describe(dev.proc, dev.deps)
    monkeypatch.setenv("ADHIP_FUSE_ATTENTION", "0")
    assert "[attention]" not in lower_describe(dev.proc, dev.deps)


_MASKED_SHAPES = [(64, 64, 16, 16), (100, 100, 48, 48), (65, 129, 8, 32), (257, 640, 128, 128), (96, 200, 256, 256),
                  (1, 7, 4, 16), (33000, 40, 16, 16)]


@pytest.mark.parametrize("sq,sk,d,dv", _MASKED_SHAPES)
def test_masked_attention_lowers_to_one_kernel(sq, sk, d, dv):
    from adhip.core import ValueData
    from adhip.device import Device, lower_describe
    from test_library_cpu import _compile_check

    class Capture(Device):
        def execute(self, proc, deps):
            self.proc, self.deps = proc, list(deps)

        def get_tensor(self, id):
            return ValueData.none()

    dev = Capture()
    _attention_program(dev, sq, sk, d, dv, 64, 0, mask=True)
    autodiff.execute()
    launches = [l for l in lower_describe(dev.proc, dev.deps).splitlines() if l.lstrip().startswith("launch")]
    assert len(launches) == 1 and "[attention]" in launches[0] and "_mask" in launches[0], launches
    rc, msg = _compile_check(dev.proc, dev.deps)
    assert rc == 0, msg


@pytest.mark.gpu
@pytest.mark.parametrize("sq,sk,d,dv", _MASKED_SHAPES)
def test_fused_masked_attention_matches_oracle_and_float64(sq, sk, d, dv, hip_device):
    """AttentionMasked (the scaled scores times a 0/1 mask, then softmax: reference src/nn/transformer.rs:21-30) through
    the fused kernel, against the oracle running the unfused commands and against float64."""
    print(f"[case] fused masked attention {sq}x{sk} d {d} dv {dv}", flush=True)
    o, (qn, kn, vn, mn) = _attention_program(hip_device, sq, sk, d, dv, 16, sq + sk, spread=2.0, mask=True)
    autodiff.execute()
    got = o.val().get()
    ro, _ = _attention_program(OracleDevice(), sq, sk, d, dv, 16, sq + sk, spread=2.0, mask=True)
    autodiff.execute()
    ref = ro.val().get()
    assert got.dim == ref.dim == [sq, dv]
    tol = RED_RTOL * math.sqrt(max(sk, d))
    assert_close(got.data, ref.data, tol, "o vs oracle")
    assert_close(got.data, _attention_float64(qn, kn, vn, 16, mn).reshape(-1), tol, "o vs float64")


@pytest.mark.gpu
def test_masked_multi_head_attention_fused_equals_unfused(hip_device, monkeypatch):
    """MaskedMultiHeadAttention (every head under the same causal mask) fused and unfused."""
    print("[case] masked multi-head attention 200x96 heads 3", flush=True)
    from adhip import nn
    seq, d_model, heads = 200, 96, 3

    def run():
        autodiff.set_device(hip_device)
        rng = np.random.default_rng(5)
        mask = autodiff.tensor(np.tril(np.ones((seq, seq), dtype=np.float32)), [seq, seq])
        mha = nn.MaskedMultiHeadAttention(d_model, heads, mask)
        for group in (mha.wq, mha.wk, mha.wv):
            for lin in group:
                lin.w = autodiff.tensor((rng.standard_normal((d_model, d_model // heads)) / 10).astype(np.float32), [d_model, d_model // heads])
        mha.wo.w = autodiff.tensor((rng.standard_normal((d_model, d_model)) / 10).astype(np.float32), [d_model, d_model])
        x = autodiff.tensor(rng.standard_normal((seq, d_model)).astype(np.float32), [seq, d_model])
        y = mha.f(x)
        y.forward()
        y.val().keep()
        autodiff.execute()
        return y.val().get()
    fused = run()
    monkeypatch.setenv("ADHIP_FUSE_ATTENTION", "0")
    plain = run()
    assert fused.dim == plain.dim == [seq, d_model]
    assert_close(fused.data, plain.data, RED_RTOL * math.sqrt(seq), "fused vs unfused")


@pytest.mark.gpu
@pytest.mark.parametrize("sq,sk,d,dv", _FUSED_SHAPES)
def test_fused_attention_matches_oracle_and_float64(sq, sk, d, dv, hip_device):
    """The fused kernel against the oracle running the unfused commands, and both against float64.  Scores reach a few
    tens: without the running maximum exp2 would lose the small terms or overflow."""
    print(f"[case] fused attention {sq}x{sk} d {d} dv {dv}", flush=True)
    o, (qn, kn, vn, _) = _attention_program(hip_device, sq, sk, d, dv, 16, sq + sk, spread=2.0)
    autodiff.execute()
    got = o.val().get()
    ro, _ = _attention_program(OracleDevice(), sq, sk, d, dv, 16, sq + sk, spread=2.0)
    autodiff.execute()
    ref = ro.val().get()
    assert got.dim == ref.dim == [sq, dv]
    tol = RED_RTOL * math.sqrt(max(sk, d))
    exact = _attention_float64(qn, kn, vn, 16).reshape(-1)
    print(f"  error / (1e-5 sqrt(N) |o|max): device {np.abs(got.data - exact).max() / np.abs(exact).max() / tol:.2f}, "
          f"oracle {np.abs(ref.data - exact).max() / np.abs(exact).max() / tol:.2f}", flush=True)
    assert_close(got.data, ref.data, tol, "o vs oracle")
    assert_close(got.data, exact, tol, "o vs float64")


@pytest.mark.gpu
def test_fused_attention_survives_extreme_scores(hip_device):
    """Rows whose scores differ by hundreds (one key wins outright), a row of identical scores, and a key block in which
    every score is far below the running maximum."""
    print("[case] fused attention extreme scores", flush=True)
    autodiff.set_device(hip_device)
    sq, sk, d, dv = 70, 200, 16, 32
    rng = np.random.default_rng(11)
    qn = rng.standard_normal((sq, d)).astype(np.float32) * 30.0
    kn = rng.standard_normal((sk, d)).astype(np.float32) * 30.0
    qn[3, :] = 0.0                      # all scores equal: the mean of V
    kn[64:128, :] *= 1e-3               # a whole block of keys that hardly counts
    vn = rng.standard_normal((sk, dv)).astype(np.float32)
    Q, K, V = autodiff.tensor(qn, [sq, d]), autodiff.tensor(kn, [sk, d]), autodiff.tensor(vn, [sk, dv])
    from adhip import nn
    o = nn.Attention(Q, K, V, 4)
    o.forward()
    o.val().keep()
    autodiff.execute()
    got = np.asarray(o.val().get().data, dtype=np.float64).reshape(sq, dv)
    ref = _attention_float64(qn, kn, vn, 4)
    assert np.isfinite(got).all()
    np.testing.assert_allclose(got[3], vn.astype(np.float64).mean(0), rtol=0, atol=2e-6)
    # a product of 16 terms of size 900 carries an absolute error of 1e-4 into the exponent
    np.testing.assert_allclose(got, ref, rtol=0, atol=2e-3)


@pytest.mark.gpu
@pytest.mark.parametrize("seq,d_model,heads", [(100, 96, 2), (128, 64, 4), (320, 512, 2), (2112, 512, 16)])
def test_attention_forward_workload_fused_equals_unfused(seq, d_model, heads, hip_device, monkeypatch):
    """Multi-head attention end to end (projections, fused attention of all heads in one launch, concatenation, output
    projection) against the same program lowered without the fusion, and against the oracle."""
    print(f"[case] attention forward {seq}x{d_model} heads {heads}", flush=True)
    fused = W.attention_forward(hip_device, seq, d_model, heads, seed=seq).run()["y"]
    monkeypatch.setenv("ADHIP_FUSE_ATTENTION", "0")
    plain = W.attention_forward(hip_device, seq, d_model, heads, seed=seq).run()["y"]
    monkeypatch.delenv("ADHIP_FUSE_ATTENTION")
    tol = 4 * RED_RTOL * math.sqrt(max(seq, d_model))
    assert_close(fused.data, plain.data, tol, "fused vs unfused")
    if seq <= 512:  # the oracle's one-thread-per-output products take too long beyond
        ref = W.attention_forward(OracleDevice(), seq, d_model, heads, seed=seq).run()["y"]
        assert_close(fused.data, ref.data, tol, "fused vs oracle")


@pytest.mark.gpu
def test_attention_forward_full_size_matches_float64(hip_device):
    """2048 tokens, d_model 1024, 8 heads of 128: the size the throughput is quoted on, against float64 on sampled
    rows of every head's share of the output."""
    print("[case] attention forward 2048x1024 heads 8", flush=True)
    seq, d_model, heads = 2048, 1024, 8
    wl = W.attention_forward(hip_device, seq, d_model, heads, seed=1, scale_x=3.0)
    got = np.asarray(wl.run()["y"].data, dtype=np.float64).reshape(seq, d_model)
    x = wl.inputs["x"].astype(np.float64)
    d_v = d_model // heads
    rows = [0, 1, 63, 64, 1000, 1027, 2047]
    cat = np.zeros((len(rows), d_model))
    for h in range(heads):
        q = x[rows] @ wl.inputs[f"wq{h}"].astype(np.float64)
        k = x @ wl.inputs[f"wk{h}"].astype(np.float64)
        v = x @ wl.inputs[f"wv{h}"].astype(np.float64)
        cat[:, h * d_v:(h + 1) * d_v] = _attention_float64(q, k, v, d_model)
    ref = cat @ wl.inputs["wo"].astype(np.float64)
    err = np.abs(got[rows] - ref).max()
    assert err <= RED_RTOL * math.sqrt(seq) * np.abs(ref).max() * 4, err
