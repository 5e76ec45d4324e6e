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
    idx = np.array([0, 1, 15, 16, 17, 63, 64, 4095, 4096, 8175, 8176, 8190, 8191])   # block rows are 16 rows
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
    cj = np.array([0, 3, 4, 5, 255, 256, 4097, 8188, 8191])   # a wavefront covers 256 columns, a lane 4
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


def _mlp_host_step(x, t, Ws, bs, lr):
    """One training step of the three-layer network on the host, float32 BLAS products with float64 element-wise
    arithmetic in between (the products are what the tolerance is sized for).  Returns the loss and the gradients."""
    B, d3 = t.shape
    h1 = x @ Ws[0] + bs[0]
    a1 = (1.0 / (1.0 + np.exp(-h1.astype(np.float64)))).astype(np.float32)
    h2 = a1 @ Ws[1] + bs[1]
    a2 = (1.0 / (1.0 + np.exp(-h2.astype(np.float64)))).astype(np.float32)
    y = a2 @ Ws[2] + bs[2]
    d = (y - t).astype(np.float64)
    loss = (d * d).sum() / (B * d3)
    g = (2.0 * d / (B * d3)).astype(np.float32)                       # dL/dy
    dW2, db2 = a2.T @ g, g.astype(np.float64).sum(0)
    g2 = ((g @ Ws[2].T).astype(np.float64) * (a2.astype(np.float64) * (1 - a2.astype(np.float64)))).astype(np.float32)
    dW1, db1 = a1.T @ g2, g2.astype(np.float64).sum(0)
    g1 = ((g2 @ Ws[1].T).astype(np.float64) * (a1.astype(np.float64) * (1 - a1.astype(np.float64)))).astype(np.float32)
    dW0, db0 = x.T @ g1, g1.astype(np.float64).sum(0)
    dx = g1 @ Ws[0].T
    return loss, [dW0, dW1, dW2], [db0, db1, db2], dx


# rows and columns at the edges of the 256x128 block tile, the 64x64 wave tile and the 32x32 MFMA block
_EDGE = np.array([0, 1, 31, 32, 63, 64, 127, 128, 255, 256, 257, 2047, 2048, 4000, 4094, 4095])


def _check_update(name, got, before, grad, lr, tol, rows=None, cols=None):
    """`got - before` against `-lr * grad` on the sampled rows x all columns and all rows x sampled columns."""
    upd = got.astype(np.float64) - before.astype(np.float64)
    want = -lr * grad.astype(np.float64)
    scale = float(np.abs(want).max())
    if upd.ndim == 1:
        assert_close(upd, want, tol, name, scale=scale)
        return
    r = _EDGE[_EDGE < upd.shape[0]] if rows is None else rows
    c = _EDGE[_EDGE < upd.shape[1]] if cols is None else cols
    assert_close(upd[r, :], want[r, :], tol, name + " rows", scale=scale)
    assert_close(upd[:, c], want[:, c], tol, name + " cols", scale=scale)


def test_mlp_train_full_size_one_step(hip_device):
    """One training step at batch 4096, 4096-4096-4096-1024 (the only size at which every product of the step
    takes the 256x128 block tile: forward k-/n-contiguous, dX with W^T read in place, dW with x^T read in place, the
    weight updates as epilogues on the accumulators).  Checked against a host step: the loss, and for every weight and
    bias the update `new - old = -lr * gradient`, on rows and columns at the tile edges; dx likewise.  The update is
    1e-6 of the weight, so it is compared with the float32 rounding of the sum `old + update` in mind: tolerance
    2^-23 * |W|_max / |update|_max relative to the update's largest entry, plus 1e-5*sqrt(k) for the product."""
    print("[case] full mlp_train 1 step", flush=True)
    batch, dims, lr = 4096, (4096, 4096, 4096, 1024), 0.01
    wl = W.mlp_train(hip_device, batch, dims, 1, lr=lr, seed=13)
    out = wl.run()
    x, t = wl.inputs["x"], wl.inputs["t"]
    Ws = [wl.inputs[f"W{i}"] for i in range(3)]
    bs = [wl.inputs[f"b{i}"] for i in range(3)]
    loss, dWs, dbs, dx = _mlp_host_step(x, t, Ws, bs, lr)
    assert_close(out["loss"].data, [loss], RED_RTOL * math.sqrt(4096), "loss")
    ktol = RED_RTOL * math.sqrt(4096)
    for li in range(3):
        for name, got, before, grad in ((f"W{li}", out[f"W{li}"].numpy(), Ws[li], dWs[li]), (f"b{li}", out[f"b{li}"].numpy(), bs[li], dbs[li])):
            rounding = 2.0 ** -23 * float(np.abs(before).max()) / float(np.abs(lr * grad).max())
            _check_update(name + " update", got, before, grad, lr, ktol + rounding)
    got_dx = out["dx"].numpy().astype(np.float64)
    scale = float(np.abs(dx).max())
    assert_close(got_dx[_EDGE, :], dx[_EDGE, :], ktol, "dx rows", scale=scale)
    assert_close(got_dx[:, _EDGE], dx[:, _EDGE], ktol, "dx cols", scale=scale)


def test_mlp_train_full_size_ten_iterations(hip_device):
    """The benchmarked configuration itself: 10 iterations inside the IR for-loop at full size (the unrolled loop
    replayed as a graph, weights updated in place by product epilogues while the next iteration reads them), against
    10 host steps.  Weights move by ~1e-5 of their size in total, so they are compared through their total update."""
    print("[case] full mlp_train 10 iterations", flush=True)
    batch, dims, lr, iters = 4096, (4096, 4096, 4096, 1024), 0.01, 10
    wl = W.mlp_train(hip_device, batch, dims, iters, lr=lr, seed=14)
    out = wl.run()
    x, t = wl.inputs["x"], wl.inputs["t"]
    W0 = [wl.inputs[f"W{i}"] for i in range(3)]
    b0 = [wl.inputs[f"b{i}"] for i in range(3)]
    Ws = [w.copy() for w in W0]
    bs = [b.copy() for b in b0]
    loss = None
    for it in range(iters):
        print(f"  host step {it}", flush=True)
        loss, dWs, dbs, dx = _mlp_host_step(x, t, Ws, bs, lr)
        for li in range(3):
            Ws[li] = (Ws[li] - np.float32(lr) * dWs[li]).astype(np.float32)
            bs[li] = (bs[li].astype(np.float64) - lr * dbs[li]).astype(np.float32)
    ktol = RED_RTOL * math.sqrt(4096) * iters
    assert_close(out["loss"].data, [loss], ktol, "loss after 10 iterations")
    for li in range(3):
        for name, got, before, after in ((f"W{li}", out[f"W{li}"].numpy(), W0[li], Ws[li]), (f"b{li}", out[f"b{li}"].numpy(), b0[li], bs[li])):
            total = after.astype(np.float64) - before.astype(np.float64)
            rounding = iters * 2.0 ** -23 * float(np.abs(before).max()) / float(np.abs(total).max())
            _check_update(name + " total update", got, before, -total / lr, lr, ktol + rounding)
    got_dx = out["dx"].numpy().astype(np.float64)
    scale = float(np.abs(dx).max())
    assert_close(got_dx[_EDGE, :], dx[_EDGE, :], ktol, "dx of the last iteration, rows", scale=scale)


def test_manip_loop_full_size(hip_device):
    print("[case] full manip_loop", flush=True)
    wl = W.manip_loop(hip_device, snapshot_at=10)
    out = wl.run()
    p, q, w = wl.inputs["p"], wl.inputs["q"], wl.inputs["w"]
    expect = np.concatenate([p.transpose(0, 2, 1), q], axis=2)[:, 128:896, :].reshape(64 * 768, 768)
    assert_exact(out["gathered"].data, expect.reshape(-1), "gathered")     # data movement: bit-exact
    assert out["i"].data[0] == 10.0
    r = expect.astype(np.float64) * w.astype(np.float64)
    r0 = r
    for _ in range(10):
        r = r - 0.01 * r.sum(1, keepdims=True)
    # each iteration multiplies the row sums by (1 - 7.68): compare relative to the row scale.  After ten iterations a
    # row is its first sum times a constant, so that sum's relative error carries through: a float32 sum of 768 terms
    # is off by up to RED_RTOL * sqrt(768) of its largest term, which for the few rows whose terms nearly cancel
    # (|sum| down to 2e-4 here, terms up to 1) is large next to the sum whatever the order of the additions
    got = out["r"].numpy().astype(np.float64)
    scale = np.abs(r).max(1, keepdims=True)
    err = np.abs(got - r) / scale
    cancel = np.abs(r0).max(1, keepdims=True) / np.abs(r0.sum(1, keepdims=True))
    tol = RED_RTOL * math.sqrt(768) * (10 + cancel)
    assert (err <= tol).all(), float((err / tol).max())
    assert np.median(err.max(1)) <= RED_RTOL * math.sqrt(768), "the typical row is far inside the bound"


def test_manip_loop_runs_to_the_iteration_limit(hip_device):
    """At the configured 50 iterations the values overflow float32: each iteration scales a row's sum by
    1 - 0.01 * 768 = -6.68 and leaves every element of the row near sum / 768, so a row's elements end finite exactly
    when its 49th sum still fits, i.e. when its first sum is below FLT_MAX / 6.68^49 = 1.3e-2 in size: some fifty rows
    whose terms cancel that far; all others end as inf / NaN.  The loop must still stop at the limit, and the rows
    that end non-finite must be the ones a float32 numpy replay of the loop ends non-finite.  Rows whose first sum
    lies within a factor of 2 of the threshold are left out: a sum that cancels to 1e-2 of its 768 terms is known to
    float32 to a few per cent at best, whatever the order of the additions."""
    print("[case] full manip_loop 50 iterations", flush=True)
    wl = W.manip_loop(hip_device)
    out = wl.run()
    assert out["i"].data[0] == 50.0
    got = out["r"].numpy()
    p, q, w = wl.inputs["p"], wl.inputs["q"], wl.inputs["w"]
    g = np.concatenate([p.transpose(0, 2, 1), q], axis=2)[:, 128:896, :].reshape(64 * 768, 768)
    r = g * w
    assert r.dtype == np.float32
    first = r.astype(np.float64).sum(1)
    with np.errstate(over="ignore", invalid="ignore"):
        for _ in range(50):
            r = r - np.float32(0.01) * r.sum(1, keepdims=True, dtype=np.float32)
    replay_finite = np.isfinite(r).all(1)
    threshold = float(np.finfo(np.float32).max) / 6.68 ** 49
    clear = (np.abs(first) < threshold / 2) | (np.abs(first) > threshold * 2)
    got_finite = np.isfinite(got).all(1)
    assert clear.sum() >= len(first) - 200
    assert (got_finite == np.isfinite(got).any(1))[clear].all(), "a row is either finite throughout or lost throughout"
    assert (got_finite == (np.abs(first) < threshold))[clear].all()
    assert (got_finite == replay_finite)[clear].all()
    assert 0 < got_finite.sum() < 400 and not np.isfinite(got).all()


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
