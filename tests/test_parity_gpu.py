"""Parity of the HIP device with the CPU oracle and with the reference's own known answers.
Everything here goes through the C ABI (`adhip_execute` / `adhip_get_tensor`) on a real GPU."""
import math

import numpy as np
import pytest

from adhip import workloads as W
from oracle.interp import OracleDevice
from parity import ELW_RTOL, RED_RTOL, assert_close, assert_exact, compare_outputs
from programs import KATS, ROUNDED, check_golden

pytestmark = pytest.mark.gpu

EXACT_KATS = {"grd", "eq", "if_ctrl", "if_else_ctrl", "for_ctrl", "evrty_ctrl", "everything"}


@pytest.mark.parametrize("name", sorted(KATS))
def test_reference_kat_on_gpu(name, hip_device):
    print(f"[case] kat {name}", flush=True)
    out = KATS[name](hip_device)
    check_golden(name, out)
    ref = KATS[name](OracleDevice())
    for k, rv in ref.items():
        if name in EXACT_KATS:
            assert_exact(out[k].data, rv.data, f"{name}.{k}")
        else:
            assert_close(out[k].data, rv.data, 4e-6, f"{name}.{k}")


def _both(builder, hip_device):
    got = builder(hip_device).run()
    ref = builder(OracleDevice()).run()
    return got, ref


def test_readme_mlp(hip_device):
    print("[case] readme_mlp", flush=True)
    got, ref = _both(lambda d: W.readme_mlp(d, seed=3), hip_device)
    compare_outputs(got, ref, {}, ("close", RED_RTOL * math.sqrt(5)))


@pytest.mark.parametrize("rows,cols", [(64, 128), (33, 20), (256, 1024), (7, 4), (1, 4096)])
def test_fused_elw_small(rows, cols, hip_device):
    print(f"[case] fused_elw {rows}x{cols}", flush=True)
    got, ref = _both(lambda d: W.fused_elw(d, rows, cols, seed=1), hip_device)
    n = rows * cols
    rules = {"L": ("close", RED_RTOL * math.sqrt(n)), "dbias": ("close", RED_RTOL * math.sqrt(rows))}
    # y and the three full-size gradients are pure element-wise chains
    compare_outputs(got, ref, rules, ("close", 4 * ELW_RTOL))


@pytest.mark.parametrize("rows,cols", [(128, 64), (100, 36), (1024, 512), (5, 3), (3, 2048), (2048, 3)])
def test_reductions_small(rows, cols, hip_device):
    print(f"[case] reductions {rows}x{cols}", flush=True)
    got, ref = _both(lambda d: W.reductions(d, rows, cols, seed=2), hip_device)
    n = rows * cols
    rules = {"s0": ("close", RED_RTOL * math.sqrt(cols)), "s1": ("close", RED_RTOL * math.sqrt(rows)),
             "s2": ("close", RED_RTOL * math.sqrt(n)), "dx": ("close", 4 * ELW_RTOL)}
    compare_outputs(got, ref, rules, ("close", RED_RTOL))
    # closed form, independent of the oracle: float64 sums of the same inputs
    x = W.reductions(OracleDevice(), rows, cols, seed=2).inputs["x"].astype(np.float64)
    assert_close(got["s0"].data, (x * x).sum(1), RED_RTOL * math.sqrt(cols), "s0 vs f64")
    assert_close(got["s1"].data, x.sum(0), RED_RTOL * math.sqrt(rows), "s1 vs f64",
                 scale=float(np.abs(x).sum(0).max()))
    assert_close(got["s2"].data, [(x * x).sum()], RED_RTOL * math.sqrt(n), "s2 vs f64")
    assert_close(got["dx"].data, (4 * x + 1).reshape(-1), 4 * ELW_RTOL, "dx closed form")


@pytest.mark.parametrize("batch,dims,iters", [(32, (16, 24, 16, 8), 3), (64, (48, 40, 56, 24), 2), (5, (7, 3, 9, 2), 4)])
def test_mlp_train_small(batch, dims, iters, hip_device):
    print(f"[case] mlp_train {batch} {dims} {iters}", flush=True)
    got, ref = _both(lambda d: W.mlp_train(d, batch, dims, iters, lr=0.05, seed=4), hip_device)
    k = max(max(dims), batch)
    compare_outputs(got, ref, {}, ("close", RED_RTOL * math.sqrt(k) * iters))


@pytest.mark.parametrize("shape", [(2, 8, 16, 4, 4, 12, 5), (3, 6, 10, 5, 1, 9, 4), (2, 16, 32, 16, 8, 24, 6)])
def test_manip_loop_small(shape, hip_device):
    print(f"[case] manip_loop {shape}", flush=True)
    nb, n1, n2, n3, lo, hi, iters = shape
    got, ref = _both(lambda d: W.manip_loop(d, nb, n1, n2, n3, lo, hi, iters, seed=5), hip_device)
    assert_exact(got["gathered"].data, ref["gathered"].data, "gathered")  # data movement only
    # the gather stage against numpy, independently of the oracle
    wl = W.manip_loop(OracleDevice(), nb, n1, n2, n3, lo, hi, iters, seed=5)
    p, q = wl.inputs["p"], wl.inputs["q"]
    expect = np.concatenate([p.transpose(0, 2, 1), q], axis=2)[:, lo:hi, :].reshape(nb * (hi - lo), n1 + n3)
    assert_exact(got["gathered"].data, expect.reshape(-1), "gathered vs numpy")
    assert_exact(got["i"].data, ref["i"].data, "i")
    assert_close(got["r"].data, ref["r"].data, RED_RTOL * math.sqrt(n1 + n3) * iters, "r")
