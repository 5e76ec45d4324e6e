"""Parity of the HIP device with the CPU oracle and with the reference's own known answers.
Everything here goes through the C ABI (`adhip_execute` / `adhip_get_tensor`) on a real GPU."""
import math
import os

import numpy as np
import pytest

from adhip import workloads as W
from oracle.interp import OracleDevice
from parity import ELW_RTOL, RED_RTOL, assert_close, assert_exact, compare_outputs
from programs import KATS, ROUNDED, check_golden

pytestmark = pytest.mark.gpu


def _sweep(generator):
    """More seeds for a generator's test, for sweeps on a GPU box.  ADHIP_FUZZ_SWEEP holds comma-separated
    `generator:scale:first:last` entries (generator = models | programs | control; for control, scale 1 draws the
    extended command set and 0 the plain one); each adds (scale, seed) for first <= seed < last.  Example:
    ADHIP_FUZZ_SWEEP=models:16:0:200 python -m pytest tests/test_parity_gpu.py -m gpu -x -k random_model_programs"""
    out = []
    for entry in filter(None, os.environ.get("ADHIP_FUZZ_SWEEP", "").split(",")):
        name, scale, first, last = entry.split(":")
        if name == generator:
            out += [(int(scale), s) for s in range(int(first), int(last))]
    return out

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


@pytest.mark.parametrize("rows,cols", [(128, 64), (100, 36), (1024, 512), (5, 3), (3, 2048), (2048, 3), (300, 260), (77, 1028),
                                       (4100, 4100)])   # the pass with riding sums walks two rows per wavefront; ragged in both directions
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


@pytest.mark.parametrize("m,k,n", [(256, 128, 384), (100, 70, 90), (128, 16, 128), (512, 512, 512), (130, 33, 257),
                                   (64, 64, 64), (1, 300, 5), (384, 1024, 128)])
def test_dot_forward_backward(m, k, n, hip_device):
    """C = A.B on the matrix cores, plus the two backward products that read W^T and x^T through
    strides (no transposed copies)."""
    print(f"[case] dot {m}x{k}x{n}", flush=True)
    from adhip import autodiff, dot
    rng = np.random.default_rng(7)
    an = rng.standard_normal((m, k), dtype=np.float32)
    bn = rng.standard_normal((k, n), dtype=np.float32)

    def build(dev):
        autodiff.set_device(dev)
        a = autodiff.tensor(an, [m, k])
        b = autodiff.tensor(bn, [k, n])
        c = dot(a, b)
        c.forward()
        c.backward()
        c.val().keep()
        autodiff.execute()
        return {"c": c.val().get(), "da": a.grad().get(), "db": b.grad().get()}

    got, ref = build(hip_device), build(OracleDevice())
    tol = RED_RTOL * math.sqrt(max(m, k, n))
    compare_outputs(got, ref, {}, ("close", tol))
    a64, b64 = an.astype(np.float64), bn.astype(np.float64)
    ones = np.ones((m, n))
    assert_close(got["c"].data, (a64 @ b64).reshape(-1), tol, "c vs f64")
    assert_close(got["da"].data, (ones @ b64.T).reshape(-1), tol, "da vs f64")
    assert_close(got["db"].data, (a64.T @ ones).reshape(-1), tol, "db vs f64")


@pytest.mark.parametrize("chain", range(6))
def test_data_movement_chains_bit_exact(chain, hip_device):
    """View / permute / index / broadcast / concat chains (including a non-involutive permute and a
    reshape across a permuted boundary) against brute-force index arithmetic."""
    print(f"[case] chain {chain}", flush=True)
    from adhip import ir as IR
    from test_oracle_math import CHAINS, _brute, _to_ir
    rng = np.random.default_rng(chain)
    x = rng.standard_normal((2, 3, 4)).astype(np.float32)
    z = rng.standard_normal((2, 4, 2)).astype(np.float32)
    cmds = CHAINS[chain]
    expect = _brute(cmds, {"x": x, "z": z})
    last = cmds[-1][-1]
    proc = IR.IRProcedure("main", [IR.CreateMat(x.reshape(-1), [2, 3, 4], "x"), IR.CreateMat(z.reshape(-1), [2, 4, 2], "z")]
                          + _to_ir(cmds) + [IR.Contigious(a=last, res="out"), IR.EX()])
    hip_device.execute(proc, {"out", last})
    got = hip_device.get_tensor("out")
    assert got.dim == list(expect.shape)
    assert_exact(got.data, expect.reshape(-1), "contiguous copy")
    # a kept id that is only a view has no buffer in the reference; here it is materialised
    assert_exact(hip_device.get_tensor(last).data, expect.reshape(-1), "kept view id")


def test_control_flow_and_late_bound_views(hip_device):
    print("[case] control flow", flush=True)
    from adhip import ir as IR
    one = np.ones(4, np.float32)
    proc = IR.IRProcedure("main", [
        IR.CreateMat(np.arange(4, dtype=np.float32), [2, 2], "a"), IR.CreateMat(one, [2, 2], "o"),
        IR.Permute(a="a", p=[1, 0], res="t"), IR.ElwAddEq(s="a", o="o"), IR.Contigious(a="t", res="u"), IR.EX()])
    hip_device.execute(proc, {"u"})
    assert_exact(hip_device.get_tensor("u").data, np.array([1, 3, 2, 4], np.float32), "view resolved at use")

    body = IR.IRProcedure("b", [IR.CreateConstant(-1.0, "m", [1]), IR.ElwAddEq(s="c", o="m"),
                                IR.CreateConstant(2.0, "two", [1]), IR.ElwMultiplyEq(s="y", o="two")])
    skipped = IR.IRProcedure("s", [IR.CreateConstant(100.0, "h", [1]), IR.ElwAddEq(s="y", o="h")])
    taken = IR.IRProcedure("t", [IR.CreateConstant(0.5, "q", [1]), IR.ElwAddEq(s="y", o="q")])
    proc = IR.IRProcedure("main", [
        IR.CreateMat(np.array([3.0], np.float32), [1], "c"), IR.CreateMat(np.array([1.0], np.float32), [1], "y"),
        IR.CreateMat(np.array([2.0], np.float32), [1], "nt"), IR.CreateMat(np.array([1.0], np.float32), [1], "yes"),
        IR.While(conditional_var="c", block=body),
        IR.If(conditions=[("nt", skipped), ("yes", taken)], else_proc=skipped),
        IR.EX(),
        IR.ElwAddEq(s="y", o="yes"),
    ])
    hip_device.execute(proc, {"y", "c", "zz"})
    assert hip_device.get_tensor("y").data[0] == 8.5
    assert hip_device.get_tensor("c").data[0] == 0.0
    assert hip_device.get_tensor("zz").is_none


def test_errors_are_reported_not_fatal(hip_device):
    from adhip import ir as IR
    proc = IR.IRProcedure("main", [IR.ElwAdd(a="nope", b="nope", res="y"), IR.EX()])
    with pytest.raises(RuntimeError, match="used before it is defined"):
        hip_device.execute(proc, {"y"})
    # the context stays usable
    proc = IR.IRProcedure("main", [IR.CreateMat(np.ones(3, np.float32), [3], "a"), IR.ElwAdd(a="a", b="a", res="y"), IR.EX()])
    hip_device.execute(proc, {"y"})
    assert_exact(hip_device.get_tensor("y").data, np.full(3, 2.0, np.float32), "y")


def test_predicated_loop_with_branches(hip_device):
    """Data-dependent loop run device-predicated (iterations enqueued ahead, flags on the device),
    including an if/else and a nested if whose arms are predicated too."""
    print("[case] predicated loop", flush=True)
    from programs import predicated_loop_program
    got = predicated_loop_program(hip_device)
    ref = predicated_loop_program(OracleDevice())
    assert [ref["y"].data[0], ref["z"].data[0], ref["i"].data[0]] == [25.0, 8.0, 7.0]
    for k in ref:
        assert_exact(got[k].data, ref[k].data, k)


def test_c_abi_from_cxx():
    """tests/cxx/cabi_smoke.cpp: a C++ host (no Python) builds a program with the header-only mirror of the
    reference's Device interface, runs it through the C ABI and checks the results in double precision."""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cxx", "cabi_smoke")
    assert os.path.exists(exe), "tests/cxx/cabi_smoke is not built: run __graft_entry__.build()"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "cabi_smoke ok" in r.stdout


@pytest.mark.parametrize("seed", list(range(30)) + [369])   # 369: a reduction epilogue that re-uses a split row index
def test_random_programs_match_oracle(seed, hip_device):
    """Differential test: random graphs of element-wise ops, sums, permutes, views, slices, concats and
    matmuls, forward and backward, device vs oracle."""
    print(f"[case] fuzz seed {seed}", flush=True)
    from fuzz_programs import random_program
    got = random_program(hip_device, seed)
    oracle = OracleDevice()
    ref = random_program(oracle, seed)
    assert set(got) == set(ref)
    # the contract's 1e-5 * sqrt(N), N = the most terms any Sum or DotProduct of this program adds; values pass
    # through up to ten such commands in a row (forward, then backward through the same chain)
    tol = RED_RTOL * math.sqrt(oracle.max_terms) * 2
    for k, rv in ref.items():
        assert got[k].dim == rv.dim, f"{k}: dim {got[k].dim} vs {rv.dim}"
        assert_close(got[k].data, rv.data, tol, f"seed {seed} {k}")


@pytest.mark.parametrize("scale,seed", [(16, s) for s in range(12)] + [(16, 23), (16, 122), (16, 343)] + [(48, s) for s in range(6)] + [(48, 31), (48, 81)] +
                         _sweep("programs"))
def test_random_programs_at_scale(scale, seed, hip_device):
    """The same generator with every leaf extent multiplied (tests/fuzz_programs.py, `scale`): tensors of 10^4 to 10^6
    elements, so the kernels are the 128-bit element-wise forms, sums riding along, chunked reductions and matrix-core
    products with extents that fit no tile.  A value is compared relative to its own largest element; a one-element
    value not below 1 % of the largest element of any output: the gradient of a one-element leaf is a sum of thousands
    of terms of the program's magnitude that may cancel (seed 23 at scale 16: -2.5e-3 from terms of order 1).  Seed 122 at scale 16
    slices long dims: views nested more than a thousand deep; seed 343 folds some 300 loads into one expression,
    which the lowering has to cut into kernels of bounded size (seeds 31 and 81 at scale 48 likewise: each held a kernel
    of some 60 buffers that spilled vector registers and computed wrong elements)."""
    print(f"[case] fuzz scale {scale} seed {seed}", flush=True)
    from fuzz_programs import random_program
    got = random_program(hip_device, seed, scale=scale)
    oracle = OracleDevice()
    ref = random_program(oracle, seed, scale=scale)
    assert set(got) == set(ref)
    tol = RED_RTOL * math.sqrt(oracle.max_terms) * 2
    finite = [np.asarray(rv.data)[np.isfinite(rv.data)] for rv in ref.values()]
    largest = max((float(np.max(np.abs(f))) for f in finite if f.size), default=1.0)
    for k, rv in ref.items():
        assert got[k].dim == rv.dim, f"{k}: dim {got[k].dim} vs {rv.dim}"
        f = np.asarray(rv.data)[np.isfinite(rv.data)]
        own = float(np.max(np.abs(f))) if f.size else 0.0
        # the floor is for what it was introduced for: one-element values (the gradient of a one-element leaf is a sum
        # of thousands of terms of the program's magnitude that may cancel); every other value answers for its own size
        floor = 1e-2 * largest if f.size <= 1 else 0.0
        assert_close(got[k].data, rv.data, tol, f"scale {scale} seed {seed} {k}", scale=max(own, floor, 1e-30))


@pytest.mark.parametrize("name", ["wide_concat", "one_buffer_pieces", "gathers", "rider17", "rider19"])
def test_adversarial_programs_match_numpy(name, hip_device):
    """Programs that strain the size of one kernel (tests/adversarial_programs.py) against closed forms in numpy: data
    movement and a single multiplication are bit-exact, the sum of 39 transposed operands is added in program order on
    both sides, the sums are compared with float64."""
    print(f"[case] adversarial {name}", flush=True)
    import adversarial_programs as A
    build = {"wide_concat": lambda: A.wide_concat(100), "one_buffer_pieces": lambda: A.one_buffer_pieces(200),
             "gathers": lambda: A.gathers(39), "rider17": lambda: A.rider(17), "rider19": lambda: A.rider(19)}[name]
    proc, keep, want = build()
    hip_device.execute(proc, set(keep))
    for k, ref in want.items():
        got = hip_device.get_tensor(k)
        assert got.dim == list(ref.shape), (k, got.dim)
        if k in ("rs", "cs"):
            assert_close(got.data.reshape(ref.shape), ref, RED_RTOL * math.sqrt(2048))
        else:  # (the riders' product of up to 19 factors is multiplied in program order on both sides)
            assert_exact(got.data.reshape(ref.shape), ref, f"{name}.{k}")


MODEL_FUZZ = ([(1, s) for s in range(40)] + [(4, s) for s in range(16)] + [(16, s) for s in range(10)] +
              [(48, s) for s in range(4)]) + _sweep("models")


@pytest.mark.parametrize("scale,seed", MODEL_FUZZ)
def test_random_model_programs(scale, seed, hip_device):
    """Random programs out of softmax, row maxima, mean / variance, LayerNorm, RMS, Linear with its in-place bias,
    tensor `*=` / `-=` / `+=`, Attention and AttentionMasked (fused, and unfused where the probabilities are kept),
    and Concats of up to 12 distinct values (tests/fuzz_models.py), forward and backward.  Checked twice: against the
    oracle (same command stream, the reference's arithmetic) and against a float64 torch shadow of the same
    computation that shares no code with the caller side.  Where a value is the outcome of cancellation (the
    gradient of a sum of softmax rows is exactly 0), the oracle's own distance from the float64 answer says how well
    float32 can know it, and the device may be a few times that far from it; otherwise 1e-5 sqrt(N) of the value's own
    largest element, N = the most terms any Sum or DotProduct of the program adds -- and never less than that fraction
    of a thousandth of the program's largest value, below which a number is the rounding noise of larger terms."""
    print(f"[case] model fuzz scale {scale} seed {seed}", flush=True)
    from fuzz_models import random_model_program, shadow_model_program
    got = random_model_program(hip_device, seed, scale)
    oracle = OracleDevice()
    ref = random_model_program(oracle, seed, scale)
    exact = shadow_model_program(seed, scale)
    assert set(got) == set(ref)
    tol = RED_RTOL * math.sqrt(oracle.max_terms) * 2
    for k, rv in ref.items():
        assert got[k].dim == rv.dim, f"{k}: dim {got[k].dim} vs {rv.dim}"
        if k not in exact:
            continue  # the gradient of a leaf that the shadow holds as a constant
        e = exact[k].ravel()
        r = np.asarray(rv.data, np.float64)
        g = np.asarray(got[k].data, np.float64)
        assert e.shape == r.shape, f"{k}: {exact[k].shape} vs {rv.dim}"
        own = float(np.max(np.abs(e))) if e.size else 0.0
        oracle_err = float(np.max(np.abs(r - e))) if e.size else 0.0
        largest = max(float(np.max(np.abs(x))) for x in exact.values())
        assert oracle_err <= tol * max(own, 1e-3 * largest), \
            f"scale {scale} seed {seed} {k}: the oracle is {oracle_err:.3e} from float64 (own scale {own:.3e})"
        allowed = max(tol * own, 8.0 * oracle_err, tol * 1e-3 * largest)
        err = float(np.max(np.abs(g - e))) if e.size else 0.0
        assert err <= allowed, f"scale {scale} seed {seed} {k}: |device - float64| = {err:.3e} > {allowed:.3e} (own scale {own:.3e}, oracle {oracle_err:.3e})"
        assert float(np.max(np.abs(g - r))) <= 2 * allowed if e.size else True


def _run_ir(dev, cmds, keep):
    from adhip import ir as IR
    proc = IR.IRProcedure("main", list(cmds) + [IR.EX()])
    dev.execute(proc, set(keep))
    return {k: dev.get_tensor(k) for k in keep}


def test_edge_shapes(hip_device):
    """Empty tensors, single elements, degenerate matmuls and reductions, high rank."""
    print("[case] edge shapes", flush=True)
    from adhip import ir as IR
    rng = np.random.default_rng(9)
    x = rng.standard_normal(2 * 3 * 2 * 2 * 5).astype(np.float32)
    cmds = [
        IR.CreateMat(np.zeros(0, np.float32), [0, 4], "e"), IR.CreateMat(np.arange(8, dtype=np.float32), [2, 4], "a"),
        IR.Concat(a="e", b="a", dim=0, res="ea"), IR.Concat(a="a", b="e", dim=0, res="ae"),   # empty pieces vanish
        IR.Contigious(a="ea", res="c1"), IR.Contigious(a="ae", res="c2"),
        IR.CreateMat(np.array([3.0], np.float32), [1, 1], "one"), IR.DotProduct(a="one", b="one", res="d11"),
        IR.CreateMat(np.arange(6, dtype=np.float32), [6, 1], "col"), IR.Sum(a="col", res="s1"),           # R = 1
        IR.Permute(a="col", p=[1, 0], res="row"), IR.Sum(a="row", res="s6"),                           # V = 1
        IR.DotProduct(a="col", b="row", res="outer"),                                                     # K = 1
        IR.CreateMat(x, [2, 3, 2, 2, 5], "x5"), IR.Permute(a="x5", p=[4, 2, 0, 3, 1], res="p5"),
        IR.View(a="p5", target_dim=[10, 12], res="v5"), IR.Sum(a="v5", res="s5"),
        IR.Index(a="a", index=1, dim=0, res="a1"), IR.Index(a="a1", index=2, dim=0, res="a12"),          # rank 0
        IR.View(a="a12", target_dim=[1], res="a12v"), IR.Contigious(a="a12v", res="scalar"),
    ]
    out = _run_ir(hip_device, cmds, ["c1", "c2", "d11", "s1", "s6", "outer", "s5", "scalar", "e"])
    assert out["c1"].dim == [2, 4] and out["c2"].dim == [2, 4]
    assert_exact(out["c1"].data, np.arange(8, dtype=np.float32), "empty ++ a")
    assert_exact(out["c2"].data, np.arange(8, dtype=np.float32), "a ++ empty")
    assert out["d11"].data[0] == 9.0
    assert_exact(out["s1"].data, np.arange(6, dtype=np.float32), "sum over one element")
    assert_exact(out["s6"].data, np.array([15.0], np.float32), "sum of one row")
    assert_exact(out["outer"].data, np.outer(np.arange(6), np.arange(6)).astype(np.float32).reshape(-1), "outer product")
    ref5 = x.reshape(2, 3, 2, 2, 5).transpose(4, 2, 0, 3, 1).reshape(10, 12).astype(np.float64).sum(1)
    assert_close(out["s5"].data, ref5, RED_RTOL * math.sqrt(12), "5-D permute + view + sum")
    assert out["scalar"].data[0] == 6.0 and out["scalar"].dim == [1]
    assert out["e"].dim == [0, 4] and out["e"].data.size == 0


def test_shape_errors_are_reported(hip_device):
    from adhip import ir as IR
    a = IR.CreateMat(np.zeros(6, np.float32), [2, 3], "a")
    b = IR.CreateMat(np.zeros(8, np.float32), [2, 4], "b")
    for bad, msg in [
        ([a, b, IR.DotProduct(a="a", b="b", res="c")], "DotProduct"),
        ([a, IR.View(a="a", target_dim=[4, 2], res="v")], "cannot be viewed"),
        ([a, IR.Permute(a="a", p=[0, 0], res="p")], "not a permutation"),
        ([a, IR.Index(a="a", index=5, dim=0, res="i")], "out of range"),
        ([a, b, IR.Concat(a="a", b="b", dim=0, res="c")], "Concat"),
        ([a, IR.Broadcast(a="a", dim=1, r=7, res="r")], "Broadcast"),
        ([a, IR.Sum(a="a", res="s"), IR.Sum(a="s", res="t")], "expected 2-D"),
    ]:
        proc = IR.IRProcedure("main", bad + [IR.EX()])
        with pytest.raises(RuntimeError, match=msg):
            hip_device.execute(proc, {"a"})


@pytest.mark.parametrize("m,k,n", [(2048, 256, 4096), (1024, 64, 8192), (2048, 64, 2048), (2000, 48, 2100)])
def test_dot_large_tile_variant(m, k, n, hip_device):
    """Shapes that select the 128x128 and 128x64 block tiles of the MFMA kernel (the small shapes above take the 64x64
    tile, the full-size MLP test the 256x128 one), all three operand layouts, aligned and bounds-checked."""
    test_dot_forward_backward(m, k, n, hip_device)


@pytest.mark.parametrize("m,k,n", [(128, 4096, 128), (256, 1024, 64), (100, 2000, 70), (64, 520, 192)])
def test_dot_split_k(m, k, n, hip_device):
    """Small outputs with a long inner dimension: k is cut into ranges computed by different blocks and the slices are
    added afterwards (aligned and bounds-checked variants, a last range shorter than the others)."""
    test_dot_forward_backward(m, k, n, hip_device)


def test_single_ops_per_element(hip_device):
    """Every element-wise command on its own (nothing to fuse), compared element by element: add, multiply, the
    in-place forms, reciprocal, square root and the comparisons bit-exactly (both sides round correctly once);
    exp2, log2 and sin within 1e-6 relative per element (two different libm implementations)."""
    print("[case] single ops", flush=True)
    from adhip import ir as IR
    rng = np.random.default_rng(17)
    n = 64 * 1024
    xa = (rng.uniform(-8.0, 8.0, n)).astype(np.float32)
    xb = (rng.uniform(-8.0, 8.0, n)).astype(np.float32)
    xp = (rng.uniform(1e-3, 100.0, n)).astype(np.float32)
    xz = xa.copy()
    xz[::7] = 0.0
    cmds = [
        IR.CreateMat(xa, [64, 1024], "a"), IR.CreateMat(xb, [64, 1024], "b"), IR.CreateMat(xp, [64, 1024], "p"),
        IR.CreateMat(xz, [64, 1024], "z"), IR.CreateMat(xa.copy(), [64, 1024], "ia"), IR.CreateMat(xa.copy(), [64, 1024], "im"),
        IR.ElwAdd(a="a", b="b", res="add"), IR.ElwMultiply(a="a", b="b", res="mul"),
        IR.ElwAddEq(s="ia", o="b"), IR.ElwMultiplyEq(s="im", o="b"),
        IR.Recip(a="a", res="rcp"), IR.Sqrt(a="p", res="sqrt"),
        IR.EqualZero(a="z", res="eq"), IR.MoreZero(a="z", res="gt"), IR.LessZero(a="z", res="lt"),
        IR.Exp2(a="a", res="exp2"), IR.Log2(a="p", res="log2"), IR.Sin(a="a", res="sin"),
    ]
    # arguments far outside the fast range of the kernels' sine (it hands over to the library routine beyond 2^15),
    # with the hand-over point itself and a few values next to multiples of pi
    big = rng.uniform(-3.0e6, 3.0e6, n).astype(np.float32)
    big[:8] = [32768.0, -32768.0, np.nextafter(np.float32(32768), np.float32(1e9)), 32767.998, 3.1415927, 6.2831855, 31415.926, 314159.27]
    cmds += [IR.CreateMat(big, [64, 1024], "big"), IR.Sin(a="big", res="sin_big")]
    keep = ["add", "mul", "ia", "im", "rcp", "sqrt", "eq", "gt", "lt", "exp2", "log2", "sin", "sin_big"]
    got = _run_ir(hip_device, cmds, keep)
    ref = _run_ir(OracleDevice(), cmds, keep)
    for k in ["add", "mul", "ia", "im", "rcp", "sqrt", "eq", "gt", "lt"]:
        assert_exact(got[k].data, ref[k].data, k)
    for k in ["exp2", "log2", "sin", "sin_big"]:
        g = got[k].data.astype(np.float64)
        r = ref[k].data.astype(np.float64)
        rel = np.abs(g - r) / np.maximum(np.abs(r), 1e-30)
        assert rel.max() <= ELW_RTOL, f"{k}: worst per-element relative error {rel.max():.3e}"


def test_repeated_execute_rebinds_payloads(hip_device):
    """A program executed again (same commands, new CreateMat contents) reuses the kept plan and buffers but must see
    the new contents, start from fresh device state, and honour a different keep list; more distinct programs than
    the context keeps must still all be right."""
    print("[case] repeated execute", flush=True)
    from adhip import ir as IR
    rng = np.random.default_rng(23)

    def prog(x, w, n_iter):
        body = IR.IRProcedure("body", [IR.ElwAddEq(s="acc", o="x"), IR.ElwAddEq(s="i", o="one"),
                                       IR.ElwAdd(a="i", b="lim", res="t"), IR.LessZero(a="t", res="c")])
        return [IR.CreateMat(x, [4, 8], "x"), IR.CreateMat(w, [8, 3], "w"), IR.CreateMat(np.zeros(32, np.float32), [4, 8], "acc"),
                IR.CreateMat(np.zeros(1, np.float32), [1], "i"), IR.CreateMat(np.ones(1, np.float32), [1], "one"),
                IR.CreateMat(np.array([-float(n_iter)], np.float32), [1], "lim"),
                IR.ElwAdd(a="i", b="lim", res="t"), IR.LessZero(a="t", res="c"),
                IR.While(conditional_var="c", block=body), IR.DotProduct(a="acc", b="w", res="y")]

    for trial in range(4):
        x = rng.standard_normal(32).astype(np.float32)
        w = rng.standard_normal(24).astype(np.float32)
        n_iter = 2 + trial          # same stream, different payload: the trip count is read on the device
        keep = ["y", "acc"] if trial != 2 else ["y"]
        out = _run_ir(hip_device, prog(x, w, n_iter), keep)
        acc = np.zeros(32, np.float32)
        for _ in range(n_iter):
            acc = acc + x
        assert_exact(out["acc"].data, acc, f"trial {trial} acc") if "acc" in keep else None
        assert_close(out["y"].data, (acc.reshape(4, 8).astype(np.float64) @ w.reshape(8, 3)).reshape(-1), RED_RTOL * math.sqrt(8), f"trial {trial} y")
        if trial == 2:
            assert hip_device.get_tensor("acc").is_none
    # more distinct programs than the context keeps, then the first one again
    for width in (4, 8, 12, 16, 20, 24, 4):
        v = rng.standard_normal(2 * width).astype(np.float32)
        out = _run_ir(hip_device, [IR.CreateMat(v, [2, width], "v"), IR.Sum(a="v", res="s")], ["s"])
        assert_close(out["s"].data, v.reshape(2, width).astype(np.float64).sum(1), RED_RTOL * math.sqrt(width), f"width {width}")


@pytest.mark.parametrize("seed,extended", [(s, False) for s in list(range(40)) + [257, 266, 290, 311]] +   # the last four: an arm reads an id an earlier arm dropped
                         [(s, True) for s in range(40)] + [(s, bool(e)) for e, s in _sweep("control")])
def test_random_control_flow_matches_oracle(seed, extended, hip_device):
    """Random programs with nested counted loops, data-dependent loops and branches (tests/fuzz_control.py):
    integer-valued tensors (which drive every predicate) bit-exact, the others within the element-wise / reduction
    tolerance.  The extended form also draws row maxima, a softmax spelled in commands (inside loops and branches, in
    place too) and maxima of integer-valued tensors."""
    print(f"[case] control fuzz seed {seed}{' extended' if extended else ''}", flush=True)
    from fuzz_control import random_control_program
    proc, keep, ints = random_control_program(seed, extended)
    ref_dev = OracleDevice()
    ref_dev.execute(proc, set(keep))
    ref = {k: ref_dev.get_tensor(k) for k in keep}
    if max(float(np.max(np.abs(ref[k].data))) for k in ints) >= 2.0 ** 22:
        pytest.skip("integer-valued tensors left the exactly representable range")
    hip_device.execute(proc, set(keep))
    for k in keep:
        got = hip_device.get_tensor(k)
        assert not got.is_none and got.dim == ref[k].dim, k
        if k in ints or k.startswith("i"):
            assert_exact(got.data, ref[k].data, k)
        else:
            assert_close(got.data, ref[k].data, 2e-5, k, scale=max(1.0, float(np.max(np.abs(ref[k].data)))))


@pytest.mark.parametrize("V,R", [(300, 64), (1, 5000), (7, 3), (2048, 1024), (5, 40000), (70000, 8)])
def test_reduction_epilogue_values(V, R, hip_device):
    """Row sums followed by element-wise consumers of the sums (one of them an in-place update of its own operand):
    wave-per-row, block-per-row and chunked shapes, so both the fused epilogue and the unfused fallback are covered."""
    print(f"[case] reduction epilogue V={V} R={R}", flush=True)
    from adhip import ir as IR
    rng = np.random.default_rng(V * 131 + R)
    x = rng.standard_normal(V * R).astype(np.float32)
    b = rng.standard_normal(V).astype(np.float32)
    cmds = [IR.CreateMat(x, [V, R], "x"), IR.CreateMat(b, [V], "b"), IR.Sum(a="x", res="s"),
            IR.CreateConstant(2.0, "two", [V]), IR.ElwMultiply(a="s", b="two", res="t"), IR.ElwAdd(a="t", b="b", res="y"),
            IR.Sin(a="y", res="z"), IR.ElwAddEq(s="b", o="s")]
    got = _run_ir(hip_device, cmds, ["s", "y", "z", "b"])
    s = x.reshape(V, R).astype(np.float64).sum(1)
    tol = RED_RTOL * math.sqrt(R)
    scale = float(np.abs(x.reshape(V, R)).sum(1).max())
    assert_close(got["s"].data, s, tol, "s", scale=scale)
    assert_close(got["y"].data, 2 * s + b, tol, "y", scale=2 * scale)
    assert_close(got["b"].data, b + s, tol, "b", scale=scale)
    # z against the device's own y: the sine of a float32 argument
    assert_close(got["z"].data, np.sin(got["y"].data.astype(np.float64)), ELW_RTOL, "z", scale=1.0)


@pytest.mark.parametrize("keep_p", [True, False])
@pytest.mark.parametrize("m,k,n", [(256, 192, 128), (130, 70, 257), (512, 64, 384), (20, 10, 12)])
def test_product_epilogue_values(m, k, n, keep_p, hip_device):
    """W += c * (A x B) with only W kept: on the matrix-core kernel the update runs on the accumulators and the product
    is never written (aligned and edge variants); the small case takes the unfused path.  A second consumer (y =
    sin(P) + bias) in the same program keeps a stored product next to its epilogue."""
    print(f"[case] product epilogue {m}x{k}x{n}", flush=True)
    from adhip import ir as IR
    rng = np.random.default_rng(m * 7 + n)
    a = rng.standard_normal(m * k).astype(np.float32)
    b = rng.standard_normal(k * n).astype(np.float32)
    w = rng.standard_normal(m * n).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    cmds = [IR.CreateMat(a, [m, k], "a"), IR.CreateMat(b, [k, n], "b"), IR.CreateMat(w, [m, n], "w"),
            IR.CreateMat(bias, [n], "bias"),
            IR.DotProduct(a="a", b="b", res="d"), IR.CreateConstant(-0.01, "c", [m, n]), IR.ElwMultiply(a="d", b="c", res="t"),
            IR.ElwAddEq(s="w", o="t"),
            IR.DotProduct(a="a", b="b", res="p"), IR.View(a="bias", target_dim=[1, n], res="b1"),
            IR.Broadcast(a="b1", dim=0, r=m, res="bb"), IR.Sin(a="p", res="sp"), IR.ElwAdd(a="sp", b="bb", res="y")]
    got = _run_ir(hip_device, cmds, ["w", "y", "p"] if keep_p else ["w", "y"])
    d = a.reshape(m, k).astype(np.float64) @ b.reshape(k, n).astype(np.float64)
    tol = RED_RTOL * math.sqrt(k)
    scale = float((np.abs(a.reshape(m, k)).astype(np.float64) @ np.abs(b.reshape(k, n)).astype(np.float64)).max())
    assert_close(got["w"].data, (w.reshape(m, n) - 0.01 * d).reshape(-1), tol, "w", scale=scale)
    if keep_p:
        assert_close(got["p"].data, d.reshape(-1), tol, "p", scale=scale)
        # y against the device's own p: the sine of a float32 argument plus one addition
        exp_y = np.sin(got["p"].data.astype(np.float64)).reshape(m, n) + bias
        assert_close(got["y"].data, exp_y.reshape(-1), 2e-6, "y", scale=1.0 + float(np.abs(bias).max()))
    else:
        # the product never reaches memory; sin amplifies its rounding error by at most 1
        exp_y = np.sin(d) + bias
        assert_close(got["y"].data, exp_y.reshape(-1), tol, "y", scale=scale)


@pytest.mark.parametrize("seed", range(24))
def test_random_epilogue_placement_matches_oracle(seed, hip_device):
    """Matrix-core products and row sums whose element-wise consumers sit at random distances behind them, with
    in-place updates in between (tests/fuzz_control.py::random_epilogue_program): whatever is or is not fused into
    the producer's kernel, the values must be the oracle's."""
    print(f"[case] epilogue fuzz seed {seed}", flush=True)
    from fuzz_control import random_epilogue_program
    proc, keep = random_epilogue_program(seed)
    ref_dev = OracleDevice()
    ref_dev.execute(proc, set(keep))
    hip_device.execute(proc, set(keep))
    tol = RED_RTOL * math.sqrt(ref_dev.max_terms)   # 64 terms per product or row sum
    for k in keep:
        got, ref = hip_device.get_tensor(k), ref_dev.get_tensor(k)
        assert not got.is_none and got.dim == ref.dim, k
        assert_close(got.data, ref.data, tol, k, scale=max(1.0, float(np.max(np.abs(ref.data)))))


def test_graph_replay_matches_direct_launches(hip_device, monkeypatch):
    """A resident program whose launches are replayed as a hipGraph from the third run on: every replay, with uploads
    and read-backs (eager work and synchronisations) between them, must give exactly what direct launches give, also
    for a counted loop whose body is replayed once per iteration."""
    print("[case] graph replay", flush=True)
    from adhip import HipDevice

    def runs(dev, builder, n):
        wl = builder(dev)
        proc, deps = wl.finish()
        prog = dev.compile(proc, deps)
        out = []
        for _ in range(n):
            prog.upload()
            prog.run()
            prog.readback()
            out.append({k: np.array(dev.get_tensor(v.id).data, copy=True) for k, v in wl.outputs.items()})
        assert "launch" in prog.describe()
        prog.close()
        return out

    builders = [lambda d: W.readme_mlp(d, seed=3), lambda d: W.mlp_train(d, 32, (16, 24, 16, 8), 3)]
    for builder in builders:
        with_graphs = runs(hip_device, builder, 6)
        monkeypatch.setenv("ADHIP_GRAPHS", "0")
        direct = runs(HipDevice(0), builder, 2)
        monkeypatch.delenv("ADHIP_GRAPHS")
        for i, got in enumerate(with_graphs):
            for k, v in got.items():
                assert_exact(v, direct[0][k], f"run {i} {k}")
        for k, v in direct[1].items():
            assert_exact(v, direct[0][k], f"direct rerun {k}")


def test_enqueue_and_sync(hip_device):
    """Runs queued back to back without waiting in between behave like the same number of waited-for runs: an in-place
    update (x += 1 followed by a row sum) accumulates once per queued run."""
    print("[case] enqueue / sync", flush=True)
    from adhip import ir as IR
    x0 = np.arange(12, dtype=np.float32)
    cmds = [IR.CreateMat(x0, [3, 4], "x"), IR.CreateConstant(1.0, "one", [3, 4]), IR.ElwAddEq(s="x", o="one"),
            IR.Sum(a="x", res="s"), IR.EX()]
    prog = hip_device.compile(IR.IRProcedure("main", cmds), {"x", "s"})
    prog.upload()
    prog.run()
    prog.readback()
    assert_exact(hip_device.get_tensor("x").data, x0 + 1, "one waited-for run")
    for _ in range(4):
        prog.enqueue()
    prog.sync()
    prog.readback()
    # the top-level CreateMat is an upload, not a kernel: it is not repeated by a run
    assert_exact(hip_device.get_tensor("x").data, x0 + 5, "four queued runs after one waited-for run")
    assert_exact(hip_device.get_tensor("s").data, (x0 + 5).reshape(3, 4).sum(1), "row sums of the last run")
    prog.close()


@pytest.mark.parametrize("seed", range(28))
def test_grouped_products_match_oracle(seed, hip_device):
    """Independent same-shape matrix products that share one grouped launch (tests/fuzz_control.py::
    random_grouped_products_program): offsets into packed weights, transposed operands, element-wise work between
    two levels of products, and products that overwrite what others of their launch still read."""
    print(f"[case] grouped products seed {seed}", flush=True)
    from fuzz_control import random_grouped_products_program
    from adhip.device import lower_describe
    proc, keep = random_grouped_products_program(seed)
    if os.environ.get("ADHIP_GROUP_DOTS", "1") != "0":
        assert "launch dots_" in lower_describe(proc, set(keep))
    ref_dev = OracleDevice()
    ref_dev.execute(proc, set(keep))
    hip_device.execute(proc, set(keep))
    got = {k: hip_device.get_tensor(k) for k in keep}
    tol = RED_RTOL * math.sqrt(ref_dev.max_terms)
    for k in keep:
        ref = ref_dev.get_tensor(k)
        assert not got[k].is_none and got[k].dim == ref.dim, k
        assert_close(got[k].data, ref.data, tol, k, scale=max(1.0, float(np.max(np.abs(ref.data)))))


@pytest.mark.parametrize("seed", range(30))
def test_layered_launches_match_oracle(seed, hip_device):
    """The same chain of reductions and element-wise passes on many tensors (tests/fuzz_control.py::
    random_layered_program): chains whose kernels are the same code run as block layers of shared launches, chains that
    update their input in place or feed the next chain keep their place."""
    print(f"[case] layered launches seed {seed}", flush=True)
    from fuzz_control import random_layered_program
    proc, keep = random_layered_program(seed)
    ref_dev = OracleDevice()
    ref_dev.execute(proc, set(keep))
    hip_device.execute(proc, set(keep))
    tol = RED_RTOL * math.sqrt(ref_dev.max_terms)
    for k in keep:
        got, ref = hip_device.get_tensor(k), ref_dev.get_tensor(k)
        assert not got.is_none and got.dim == ref.dim, k
        assert_close(got.data, ref.data, tol, k, scale=max(1.0, float(np.max(np.abs(ref.data)))))


@pytest.mark.parametrize("k_value", [-1.0, 1.0, 0.0])
def test_branch_arm_reads_id_that_an_earlier_arm_dropped(k_value, hip_device):
    """tests/programs.py::branch_reads_id_dropped_by_earlier_arm on the device, every path of the branch, bit-exact
    (small integers and halves only)."""
    print(f"[case] branch arm reads dropped id, k = {k_value}", flush=True)
    from programs import branch_reads_id_dropped_by_earlier_arm
    proc, keep, expect = branch_reads_id_dropped_by_earlier_arm(k_value)
    hip_device.execute(proc, set(keep))
    for k in keep:
        assert_exact(hip_device.get_tensor(k).data, expect[k], k)


def test_reduction_epilogue_with_split_row_index(hip_device):
    """tests/programs.py::reduction_epilogue_with_split_row_index on the device, bit-exact (small integers)."""
    print("[case] reduction epilogue with split row index", flush=True)
    from programs import reduction_epilogue_with_split_row_index
    proc, keep, expect = reduction_epilogue_with_split_row_index()
    hip_device.execute(proc, set(keep))
    assert_exact(hip_device.get_tensor("y").data, expect["y"].reshape(-1), "y")


@pytest.mark.parametrize("shape,perm", [([70000, 16, 16], [0, 2, 1]), ([300, 300, 16, 16], [0, 1, 3, 2]), ([200000, 24], [1, 0])])
def test_transposing_copy_with_many_batches(shape, perm, hip_device):
    """Dense copies of permuted tensors with more than 65535 batches or tiles (the width of grid dimensions y and z),
    bit-exact against numpy; the second operand of the addition keeps the copy from being the kept value itself."""
    print(f"[case] transposing copy {shape} {perm}", flush=True)
    from adhip import ir as IR
    rng = np.random.default_rng(3)
    a = rng.standard_normal(shape, dtype=np.float32)
    out_shape = [shape[i] for i in perm]
    b = rng.standard_normal(out_shape, dtype=np.float32)
    cmds = [IR.CreateMat(a.reshape(-1), shape, "a"), IR.Permute(a="a", p=perm, res="at"), IR.Contigious(a="at", res="y"),
            IR.CreateMat(b.reshape(-1), out_shape, "b"), IR.ElwAdd(a="at", b="b", res="z")]
    got = _run_ir(hip_device, cmds, ["y", "z"])
    assert got["y"].dim == out_shape
    assert_exact(got["y"].data, a.transpose(perm).reshape(-1), "y")
    assert_exact(got["z"].data, (a.transpose(perm) + b).reshape(-1), "z")


def test_if_with_more_arms_than_one_predicate_batch(hip_device):
    """An If with 70 conditions of which only the 67th holds: the host reads the predicates 64 at a time and must
    still find it (and must not run the else block)."""
    print("[case] If with 70 arms", flush=True)
    from adhip import ir as IR
    cmds = [IR.CreateMat(np.zeros(4, dtype=np.float32), [4], "x")]
    arms = []
    for i in range(70):
        cmds.append(IR.CreateMat(np.array([1.0 if i in (66, 68) else 0.0], dtype=np.float32), [1], f"p{i}"))
        arms.append((f"p{i}", IR.IRProcedure(f"arm{i}", [IR.CreateConstant(float(i), "k", [4]), IR.ElwAddEq(s="x", o="k")])))
    cmds.append(IR.If(conditions=arms, else_proc=IR.IRProcedure("else", [IR.CreateConstant(-1.0, "k", [4]), IR.ElwAddEq(s="x", o="k")])))
    got = _run_ir(hip_device, cmds, ["x"])
    assert_exact(got["x"].data, np.full(4, 66.0, dtype=np.float32), "x")


@pytest.mark.parametrize("V,R", [(7, 5), (64, 256), (300, 1000), (33, 4096), (4, 70000), (2048, 64), (3, 1)])
def test_max_rows_and_columns(V, R, hip_device):
    """The Max reduction over rows (contiguous) and over columns (strided operand) of the same matrix, with NaN,
    infinities and ties placed in it: bit-exact against the oracle and against numpy's fmax."""
    print(f"[case] max {V}x{R}", flush=True)
    from adhip import ir as IR
    rng = np.random.default_rng(V * 31 + R)
    x = rng.standard_normal((V, R)).astype(np.float32)
    x[0, R // 2] = np.inf
    if R > 1:
        x[V - 1, 0] = np.nan
        x[V // 2, :] = -np.inf
    if V > 3 and R > 1:
        x[1, :] = np.nan       # a row that is NaN throughout: its maximum is NaN (and so is every column's only if all of it is)
    cmds = [IR.CreateMat(x.reshape(-1), [V, R], "x"), IR.Max(a="x", res="rows"),
            IR.Permute(a="x", p=[1, 0], res="xt"), IR.Max(a="xt", res="cols")]
    got = _run_ir(hip_device, cmds, ["rows", "cols"])
    ref_dev = OracleDevice()
    ref_dev.execute(IR.IRProcedure("main", cmds + [IR.EX()]), {"rows", "cols"})
    assert got["rows"].dim == [V] and got["cols"].dim == [R]
    for k in ("rows", "cols"):
        assert_exact(got[k].data, ref_dev.get_tensor(k).data, k + " vs oracle")
    assert_exact(got["rows"].data, np.fmax.reduce(x, axis=1), "rows vs numpy")
    assert_exact(got["cols"].data, np.fmax.reduce(x, axis=0), "cols vs numpy")


@pytest.mark.parametrize("shape,dim", [((6, 10), 1), ((6, 10), 0), ((3, 5, 7), 1), ((40, 300), -1)])
def test_max_forward_backward_and_stable_softmax(shape, dim, hip_device):
    """Tensor.max(dim) forward and backward and the shifted softmax, device against oracle, and the softmax against
    float64 at arguments up to +-100 (exp alone overflows at 88)."""
    print(f"[case] max/softmax {shape} dim {dim}", flush=True)
    from adhip import autodiff
    rng = np.random.default_rng(sum(shape) + dim)
    xn = (rng.standard_normal(shape) * 30).astype(np.float32)
    xn.reshape(-1)[0] = 100.0
    xn.reshape(-1)[1] = -100.0
    wn = rng.standard_normal(shape).astype(np.float32)

    def build(dev):
        autodiff.set_device(dev)
        x = autodiff.tensor(xn, list(shape))
        w = autodiff.tensor(wn, list(shape))
        m = x.max(dim)
        s = x.softmax(dim)
        L = (s * w)
        for _ in shape:
            L = L.sum(0)
        t = m
        for _ in m.dim():
            t = t.sum(0)
        total = L + t
        total.forward()
        total.backward()
        for v in (m.val(), s.val(), x.grad()):
            v.keep()
        autodiff.execute()
        return {"m": m.val().get(), "s": s.val().get(), "dx": x.grad().get()}

    got, ref = build(hip_device), build(OracleDevice())
    assert_exact(got["m"].data, ref["m"].data, "max")
    n = shape[dim]
    compare_outputs(got, ref, {"m": ("exact",)}, ("close", RED_RTOL * math.sqrt(n)))
    z = xn.astype(np.float64)
    e = np.exp(z - z.max(dim, keepdims=True))
    s64 = e / e.sum(dim, keepdims=True)
    assert np.isfinite(got["s"].data).all()
    assert_close(got["s"].data, s64.reshape(-1), RED_RTOL * math.sqrt(n), "softmax vs float64")
    # d/dx of sum(softmax * w) + sum(max): softmax part s * (w - sum(s * w)) along dim, max part one-hot (no ties here)
    sw = (s64 * wn).sum(dim, keepdims=True)
    dmax = (z == z.max(dim, keepdims=True)).astype(np.float64)
    assert_close(got["dx"].data, (s64 * (wn - sw) + dmax).reshape(-1), 4 * RED_RTOL * math.sqrt(n), "dx vs float64")


@pytest.mark.parametrize("case", ["transposed_plus_dense", "batched_3d", "two_transposed", "concat_piece", "ragged_edges"])
def test_tiled_kernels_with_operands_read_against_the_grain(case, hip_device):
    """Element-wise passes over a permuted operand large enough for the tiled kernel, which fetches the operand's
    64x64 tiles through LDS instead of making a dense transposed copy first: plain and batched transposes, two such
    operands at once, an operand behind a concat piece, and sizes that are no multiple of the tile.  Bit-exact against
    numpy (data movement plus one exactly rounded operation per element)."""
    print(f"[case] tiled element-wise kernel: {case}", flush=True)
    from adhip import ir as IR
    from adhip.device import lower_describe
    rng = np.random.default_rng(len(case))
    f = lambda *sh: rng.standard_normal(sh, dtype=np.float32)  # noqa: E731
    if case == "transposed_plus_dense":
        a, b = f(520, 704), f(704, 520)
        cmds = [IR.CreateMat(a.reshape(-1), [520, 704], "a"), IR.CreateMat(b.reshape(-1), [704, 520], "b"),
                IR.Permute(a="a", p=[1, 0], res="at"), IR.ElwAdd(a="at", b="b", res="y")]
        want = a.T + b
    elif case == "batched_3d":
        a, b = f(5, 300, 260), f(5, 260, 300)
        cmds = [IR.CreateMat(a.reshape(-1), [5, 300, 260], "a"), IR.CreateMat(b.reshape(-1), [5, 260, 300], "b"),
                IR.Permute(a="a", p=[0, 2, 1], res="at"), IR.ElwMultiply(a="at", b="b", res="y")]
        want = a.transpose(0, 2, 1) * b
    elif case == "two_transposed":
        a, c, b = f(640, 512), f(640, 512), f(512, 640)
        cmds = [IR.CreateMat(a.reshape(-1), [640, 512], "a"), IR.CreateMat(c.reshape(-1), [640, 512], "c"),
                IR.CreateMat(b.reshape(-1), [512, 640], "b"), IR.Permute(a="a", p=[1, 0], res="at"),
                IR.Permute(a="c", p=[1, 0], res="ct"), IR.ElwMultiply(a="at", b="ct", res="m"), IR.ElwAdd(a="m", b="b", res="y")]
        want = a.T * c.T + b
    elif case == "concat_piece":
        a, b, w = f(300, 1000), f(1000, 52), f(352)
        cmds = [IR.CreateMat(a.reshape(-1), [300, 1000], "a"), IR.CreateMat(b.reshape(-1), [1000, 52], "b"),
                IR.CreateMat(w, [352], "w"), IR.Permute(a="a", p=[1, 0], res="at"), IR.Concat(a="at", b="b", dim=1, res="cc"),
                IR.View(a="w", target_dim=[1, 352], res="w1"), IR.Broadcast(a="w1", dim=0, r=1000, res="wb"),
                IR.ElwMultiply(a="cc", b="wb", res="y")]
        want = np.concatenate([a.T, b], axis=1) * w
    else:
        a, b = f(333, 997), f(997, 332)
        cmds = [IR.CreateMat(a.reshape(-1), [333, 997], "a"), IR.CreateMat(b.reshape(-1), [997, 332], "b"),
                IR.Index(a="a", index=0, dim=0, res="row0"),   # an unrelated view, to have more than one alias around
                IR.Permute(a="a", p=[1, 0], res="at"), IR.View(a="at", target_dim=[997, 333], res="at2")]
        # drop the last column of the transposed operand so that the width is a multiple of 4 but not of 64
        sl = []
        for i in range(332):
            sl.append(IR.Index(a="at2", index=i, dim=1, res=f"col{i}"))
            sl.append(IR.View(a=f"col{i}", target_dim=[997, 1], res=f"colv{i}"))
            sl.append(IR.Concat(a=(f"acc{i - 1}" if i else f"colv{i}"), b=f"colv{i}", dim=1, res=f"acc{i}") if i else
                      IR.View(a=f"colv{i}", target_dim=[997, 1], res=f"acc{i}"))
        cmds += sl + [IR.ElwAdd(a="acc331", b="b", res="y")]
        want = a.T[:, :332] + b
    proc = IR.IRProcedure("main", cmds + [IR.EX()])
    assert "[elw_tiled]" in lower_describe(proc, {"y"}) and "[transpose]" not in lower_describe(proc, {"y"})
    got = _run_ir(hip_device, cmds, ["y"])
    assert got["y"].dim == list(want.shape)
    assert_exact(got["y"].data, want.reshape(-1), "y")


@pytest.mark.gpu
@pytest.mark.parametrize("case", ["flat_ragged", "broadcast_3d", "two_outputs_in_place", "whole_bands"])
def test_large_flat_kernels_in_banded_order(case, hip_device):
    """Element-wise kernels of a million float4 and more hand their blocks out band by band instead of front to
    back (16 wavefronts of a block on 16 rows of 32 KiB).  Every element must still be computed exactly once: sizes
    that are no multiple of a band, an index that is decomposed into three coordinates after the reordering, an
    in-place update next to a second output.  Bit-exact against numpy (one exactly rounded operation per element)."""
    print(f"[case] banded element-wise kernel: {case}", flush=True)
    from adhip import ir as IR
    rng = np.random.default_rng(len(case))
    f = lambda *sh: rng.standard_normal(sh, dtype=np.float32)  # noqa: E731
    if case == "flat_ragged":
        a, b = f(1025, 4100), f(1025, 4100)
        cmds = [IR.CreateMat(a.reshape(-1), [1025, 4100], "a"), IR.CreateMat(b.reshape(-1), [1025, 4100], "b"),
                IR.ElwAdd(a="a", b="b", res="y")]
        want = {"y": a + b}
    elif case == "broadcast_3d":
        a, r, c = f(37, 300, 512), f(37, 1, 512), f(300, 1)
        cmds = [IR.CreateMat(a.reshape(-1), [37, 300, 512], "a"), IR.CreateMat(r.reshape(-1), [37, 1, 512], "r"),
                IR.CreateMat(c.reshape(-1), [300, 1], "c"),
                IR.Broadcast(a="r", dim=1, r=300, res="rb"), IR.Broadcast(a="c", dim=1, r=512, res="cb1"),
                IR.View(a="cb1", target_dim=[1, 300, 512], res="cb2"), IR.Broadcast(a="cb2", dim=0, r=37, res="cb"),
                IR.ElwMultiply(a="a", b="rb", res="m"), IR.ElwAdd(a="m", b="cb", res="y")]
        want = {"y": a * r + c.reshape(1, 300, 1)}
    elif case == "two_outputs_in_place":
        a, b = f(3000, 1400), f(3000, 1400)
        cmds = [IR.CreateMat(a.reshape(-1), [3000, 1400], "a"), IR.CreateMat(b.reshape(-1), [3000, 1400], "b"),
                IR.ElwMultiply(a="a", b="b", res="p"), IR.ElwAddEq(s="a", o="b")]
        want = {"p": a * b, "a": a + b}
    else:
        a = f(2048, 2048)
        cmds = [IR.CreateMat(a.reshape(-1), [2048, 2048], "a"), IR.ElwMultiply(a="a", b="a", res="y")]
        want = {"y": a * a}
    proc = IR.IRProcedure("main", cmds + [IR.EX()])
    from adhip.device import lower_describe
    plan = lower_describe(proc, set(want))
    assert "block=1024" in plan, plan
    got = _run_ir(hip_device, cmds, sorted(want))
    for k, w in want.items():
        assert got[k].dim == list(w.shape), k
        assert_exact(got[k].data, w.reshape(-1), k)


def _row_rider_program(case, rng):
    from adhip import ir as IR
    f = lambda *sh: rng.standard_normal(sh, dtype=np.float32)  # noqa: E731
    R, C = (520, 384) if case != "ragged" else (77, 1028)
    x = f(R, C)
    cmds = [IR.CreateMat(x.reshape(-1), [R, C], "x"), IR.CreateConstant(2.0, "two", [R, C]), IR.CreateConstant(1.0, "one", [R, C])]
    x64 = x.astype(np.float64)
    if case in ("independent_later", "ragged"):
        # the sum comes first in the program, the pass that can carry it later
        cmds += [IR.ElwMultiply(a="x", b="x", res="xx"), IR.Sum(a="xx", res="s"),
                 IR.ElwMultiply(a="x", b="two", res="t"), IR.ElwAdd(a="t", b="one", res="y")]
        want = {"s": (x64 * x64).sum(1), "y": 2 * x64 + 1}
        fused = True
    elif case == "independent_earlier":
        cmds += [IR.ElwMultiply(a="x", b="two", res="t"), IR.ElwAdd(a="t", b="one", res="y"),
                 IR.ElwMultiply(a="x", b="x", res="xx"), IR.Sum(a="xx", res="s")]
        want = {"s": (x64 * x64).sum(1), "y": 2 * x64 + 1}
        fused = True
    elif case == "sums_of_the_pass_itself":
        # the summed value is what the pass stores; a second row sum and a column sum ride along as well
        cmds += [IR.ElwMultiply(a="x", b="two", res="t"), IR.ElwAdd(a="t", b="one", res="y"), IR.Sum(a="y", res="s"),
                 IR.ElwMultiply(a="x", b="x", res="xx"), IR.Sum(a="xx", res="s2"),
                 IR.Permute(a="x", p=[1, 0], res="xt"), IR.Sum(a="xt", res="c")]
        want = {"s": (2 * x64 + 1).sum(1), "s2": (x64 * x64).sum(1), "c": x64.sum(0), "y": 2 * x64 + 1}
        fused = True
    elif case == "dependent":
        # the pass needs the sum: y = x * s[:, None]
        cmds += [IR.ElwMultiply(a="x", b="x", res="xx"), IR.Sum(a="xx", res="s"), IR.View(a="s", target_dim=[R, 1], res="sv"),
                 IR.Broadcast(a="sv", dim=1, r=C, res="sb"), IR.ElwMultiply(a="x", b="sb", res="y")]
        s_ = (x64 * x64).sum(1)
        want = {"s": s_, "y": x64 * s_[:, None]}
        fused = False
    else:  # in_place_between: something between the sum and the pass reads the buffer the pass overwrites
        cmds += [IR.ElwMultiply(a="x", b="x", res="xx"), IR.Sum(a="xx", res="s"),
                 IR.ElwAdd(a="x", b="one", res="z"),           # reads the old x
                 IR.ElwMultiplyEq(s="x", o="two")]             # x *= 2 in place: may not move in front of z
        want = {"s": (x64 * x64).sum(1), "z": x64 + 1, "x": 2 * x64}
        fused = None
    return cmds, want, fused


@pytest.mark.gpu
@pytest.mark.parametrize("case", ["independent_later", "independent_earlier", "sums_of_the_pass_itself", "dependent", "in_place_between", "ragged"])
def test_row_sums_riding_with_elementwise_pass(case, hip_device):
    """A plain row sum is produced by an element-wise pass over the same [rows, cols] space that loads its operand
    anyway (one read of x for both), wherever the two stand in the program -- unless the pass needs the sum, or moving
    it would overtake a reader of a buffer it overwrites.  Checked against float64."""
    print(f"[case] row sums riding along: {case}", flush=True)
    from adhip import ir as IR
    from adhip.device import lower_describe
    cmds, want, fused = _row_rider_program(case, np.random.default_rng(len(case)))
    plan = lower_describe(IR.IRProcedure("main", cmds + [IR.EX()]), set(want))
    if fused is not None:
        assert ("_rs0 [" in plan) == fused, plan
    got = _run_ir(hip_device, cmds, sorted(want))
    for k, w in want.items():
        assert got[k].dim == list(w.shape), k
        tol = RED_RTOL * math.sqrt(1028) if k in ("s", "s2", "c") else 2 * ELW_RTOL  # sums of at most 1028 terms
        assert_close(got[k].data, w.reshape(-1), tol, k)


def _latch_loop_program(case, rng):
    """x [rows, cols] shrinks by a factor per iteration until a predicate computed from it turns 0.
    Returns (commands, ids to keep, whether the body's last kernel is expected to latch the loop flag)."""
    from adhip import ir as IR
    rows, cols = 40, 64
    x = (rng.random((rows, cols), dtype=np.float32) + 1.0)          # in [1, 2)
    top = [IR.CreateMat(x.reshape(-1), [rows, cols], "x"), IR.CreateMat(np.zeros(1, np.float32), [1], "n"),
           IR.CreateConstant(0.5, "half", [rows, cols]), IR.CreateConstant(1.0, "one1", [1]),
           IR.CreateConstant(-40.0, "mthr", [1])]

    def predicate(prefix):
        # cond = (sum of all elements - 40 > 0)
        return [IR.Sum(a="x", res=prefix + "s"), IR.View(a=prefix + "s", target_dim=[1, rows], res=prefix + "sv"),
                IR.Sum(a=prefix + "sv", res=prefix + "t"), IR.ElwAdd(a=prefix + "t", b="mthr", res=prefix + "d"),
                IR.MoreZero(a=prefix + "d", res="cond")]
    body = [IR.ElwMultiplyEq(s="x", o="half"), IR.ElwAddEq(s="n", o="one1")]
    if case == "predicate_last":
        body += predicate("b")
        latched = True
    elif case == "kernel_after_predicate":
        # the counter update comes after the predicate's kernel in the iteration
        body = [IR.ElwMultiplyEq(s="x", o="half")] + predicate("b") + [IR.Contigious(a="x", res="copy"), IR.ElwAddEq(s="n", o="one1")]
        latched = None
    else:  # predicate_from_elementwise: cond = (n - 5 < 0) * (n - 100 < 0), a one-element kernel of its own (the product
        # of two comparisons keeps it from being the counted-loop shape)
        top += [IR.CreateConstant(-5.0, "m5", [1]), IR.CreateConstant(-100.0, "m100", [1])]

        def small(prefix):
            return [IR.ElwAdd(a="n", b="m5", res=prefix + "d"), IR.LessZero(a=prefix + "d", res=prefix + "l"),
                    IR.ElwAdd(a="n", b="m100", res=prefix + "e"), IR.LessZero(a=prefix + "e", res=prefix + "m"),
                    IR.ElwMultiply(a=prefix + "l", b=prefix + "m", res="cond")]
        body += small("b")
        latched = True
    cmds = top + (predicate("a") if case != "predicate_from_elementwise" else small("a"))
    cmds.append(IR.While(conditional_var="cond", block=IR.IRProcedure("body", body)))
    return cmds, ["x", "n", "cond"], latched


@pytest.mark.gpu
@pytest.mark.parametrize("case", ["predicate_last", "kernel_after_predicate", "predicate_from_elementwise"])
def test_loop_flag_latched_by_the_body(case, hip_device):
    """A device-predicated loop whose body ends with the kernel that produces the predicate lets that kernel keep the
    loop flag; a body in which something still runs after the predicate's kernel keeps the separate flag kernel.
    Either way the loop must stop after the same iteration as on the oracle."""
    print(f"[case] loop flag: {case}", flush=True)
    from adhip import ir as IR
    from adhip.device import lower_describe
    cmds, keep, latched = _latch_loop_program(case, np.random.default_rng(3))
    plan = lower_describe(IR.IRProcedure("main", cmds + [IR.EX()]), set(keep))
    assert "device-predicated" in plan, plan
    if latched is not None:
        assert ("latched by the body's last kernel" in plan) == latched, plan
    got = _run_ir(hip_device, cmds, keep)
    oracle = OracleDevice()
    ref = _run_ir(oracle, cmds, keep)
    assert float(ref["n"].data[0]) >= 3.0   # the loop really iterates
    for k in keep:
        assert got[k].dim == ref[k].dim, k
        assert_close(got[k].data, ref[k].data, 4 * ELW_RTOL, k)


@pytest.mark.gpu
@pytest.mark.parametrize("seed", [501, 502, 503, 504])
def test_small_programs_one_launch_per_kernel_and_merged_agree(seed, hip_device, monkeypatch):
    """Programs on tiny tensors run their single-block kernels as the phases of one launch; with ADHIP_MERGE_SMALL=0
    every kernel is a launch of its own.  Both must give the oracle's result (data-flow programs and programs with
    loops and branches; the seeds are used nowhere else, so that no kept plan of the other kind is reused)."""
    print(f"[case] merged and unmerged small programs, seed {seed}", flush=True)
    from adhip.device import lower_describe
    from fuzz_control import random_control_program
    from fuzz_programs import random_program
    proc, keep, ints = random_control_program(seed)
    merged_plan = lower_describe(proc, set(keep))
    monkeypatch.setenv("ADHIP_MERGE_SMALL", "0")
    assert "[merged]" in merged_plan and "[merged]" not in lower_describe(proc, set(keep))
    oracle = OracleDevice()
    oracle.execute(proc, set(keep))
    hip_device.execute(proc, set(keep))           # one launch per kernel
    for k in keep:
        got, ref = hip_device.get_tensor(k), oracle.get_tensor(k)
        assert got.dim == ref.dim, k
        if k in ints or k.startswith("i"):
            assert_exact(got.data, ref.data, f"unmerged {k}")
        else:
            assert_close(got.data, ref.data, 2e-5, f"unmerged {k}", scale=max(1.0, float(np.max(np.abs(ref.data)))))
    got = random_program(hip_device, seed)         # one launch per kernel
    ref = random_program(OracleDevice(), seed)
    monkeypatch.delenv("ADHIP_MERGE_SMALL")
    again = random_program(hip_device, seed + 1000)  # merged, another program
    ref2 = random_program(OracleDevice(), seed + 1000)
    for out, want in ((got, ref), (again, ref2)):
        for k, rv in want.items():
            assert out[k].dim == rv.dim, k
            assert_close(out[k].data, rv.data, 2e-4, k)


TIGHT_CASES = ([("models", 1, s) for s in range(8)] + [("models", 16, s) for s in range(4)] + [("models", 48, 0)] +
               [("programs", 16, s) for s in range(3)] + [("programs", 48, 1)] + [("control", 1, s) for s in range(6)])


@pytest.mark.parametrize("shift", [1, 3])
@pytest.mark.parametrize("generator,scale,seed", TIGHT_CASES)
def test_tightened_lowering_matches_oracle(generator, scale, seed, shift, hip_device, monkeypatch):
    """What a program is lowered to after kernels of it spilled vector registers -- every kernel-size bound halved
    `shift` times, no epilogues, no sums riding along -- is a path no known program takes on its own, so it is forced
    here (ADHIP_TIGHTEN) and held against the oracle like the ordinary lowering."""
    print(f"[case] tightened x{shift}: {generator} scale {scale} seed {seed}", flush=True)
    monkeypatch.setenv("ADHIP_TIGHTEN", str(shift))
    if generator == "control":
        from fuzz_control import random_control_program
        proc, keep, ints = random_control_program(seed, True)
        oracle = OracleDevice()
        oracle.execute(proc, set(keep))
        hip_device.execute(proc, set(keep))
        for k in keep:
            got, ref = hip_device.get_tensor(k), oracle.get_tensor(k)
            if k in ints or k.startswith("i"):
                assert_exact(got.data, ref.data, k)
            else:
                assert_close(got.data, ref.data, 2e-5, k, scale=max(1.0, float(np.max(np.abs(ref.data)))))
        return
    if generator == "models":
        from fuzz_models import random_model_program
        got = random_model_program(hip_device, seed, scale)
        oracle = OracleDevice()
        ref = random_model_program(oracle, seed, scale)
    else:
        from fuzz_programs import random_program
        got = random_program(hip_device, seed, scale=scale)
        oracle = OracleDevice()
        ref = random_program(oracle, seed, scale=scale)
    tol = RED_RTOL * math.sqrt(oracle.max_terms) * 2
    finite = [np.asarray(v.data)[np.isfinite(v.data)] for v in ref.values()]
    largest = max((float(np.max(np.abs(f))) for f in finite if f.size), default=1.0)
    for k, rv in ref.items():
        r = np.asarray(rv.data, np.float64)
        g = np.asarray(got[k].data, np.float64)
        m = np.isfinite(r)
        assert (np.isfinite(g) == m).all(), k
        own = float(np.max(np.abs(r[m]))) if m.any() else 0.0
        floor = max(own, 1e-2 * largest)
        assert (np.abs(g - r)[m] <= tol * np.maximum(np.abs(r[m]), floor)).all(), \
            f"{generator} scale {scale} seed {seed} {k}: {float(np.abs(g - r)[m].max()):.3e} > {tol * floor:.3e}"


@pytest.mark.parametrize("blocks,rows,k,n", [(3, 128, 256, 192), (8, 64, 520, 100), (2, 200, 64, 64)])
def test_product_of_concatenated_row_blocks(blocks, rows, k, n, hip_device):
    """concat([x_1^T, ..., x_b^T], 0) . B runs as one grouped launch of b products whose results are concatenated
    (tests/test_library_cpu.py holds the plan); values against float64."""
    print(f"[case] product of {blocks} concatenated row blocks {rows}x{k} . {k}x{n}", flush=True)
    from test_library_cpu import _row_concat_product
    proc, keep, want = _row_concat_product(blocks, rows, k, n, seed=blocks + rows)
    hip_device.execute(proc, keep)
    got = hip_device.get_tensor("y")
    assert got.dim == [blocks * rows, n]
    assert_close(got.data, want.reshape(-1), RED_RTOL * math.sqrt(k), "y", scale=float(np.abs(want).max()))
