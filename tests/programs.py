"""Programs shared by the oracle tests (CPU) and the parity tests (GPU).

Each `kat_*` function is a transcription of one of the reference's own end-to-end tests
(src/tests/*.rs): it builds the same graph through the same user-facing calls, executes it on
the device it is given and returns {name: ValueData}.  `GOLDEN` holds the values those tests
assert (exact, or after `.round(4)`), copied as data.
"""
from __future__ import annotations

import numpy as np

from adhip import autodiff, nn
from adhip.core import concat, constant, dot


# ---- golden vectors asserted by the reference's tests: tests/golden/reference_kats.json ------------
import json as _json
import os as _os

with open(_os.path.join(_os.path.dirname(_os.path.abspath(__file__)), "golden", "reference_kats.json")) as _f:
    _KATS_JSON = _json.load(_f)["tests"]
GOLDEN = {name: {k: (v["dim"], v["data"]) for k, v in t["expected"].items()} for name, t in _KATS_JSON.items()}
ROUNDED = {name for name, t in _KATS_JSON.items() if t["rounded"]}
# ct.x_grad[3] = -353566.88 sits where cos(2x+3) ~ 0 (the reference's file calls the test "not the
# most stable", src/tests/ct.rs:2); its last digit depends on the sin() of the runtime that produced
# it.  That one element is compared to 4e-6 relative instead of digit-for-digit.
ILL_CONDITIONED = {("ct", "x_grad"): {3: 4e-6}}


def kat_nn(dev):
    autodiff.set_device(dev)
    autodiff.eager_dep_opt()
    l1_w = autodiff.tensor([0.03, 0.02, 0.01, 0.04, 0.05, 0.063, 0.01, 0.10, 0.07, 0.02, 0.01, 0.08,
                            0.05, 0.03, 0.06], [5, 3])
    l1_b = autodiff.tensor([0.03, 0.01, 0.032], [3])
    l2_w = autodiff.tensor([0.022, 0.016, 0.007, 0.093, 0.013, 0.09], [3, 2])
    net = nn.Sequential()
    net.insert(nn.LinearWithWeights(l1_w, l1_b))
    net.insert(nn.Sigmoid())
    net.insert(nn.LinearWithWeights(l2_w, None))
    opt = nn.SGD(net.params(), 0.1)
    x = autodiff.tensor([0.01, 0.02, 0.037, 0.04, 0.05, 0.063, 0.07, 0.08, 0.09, 0.013], [2, 5])
    box = {}

    def body(_):
        y = net.f(x)
        opt.zero_grad()
        autodiff.add_heading("Forward")
        y.forward()
        autodiff.add_heading("Backward")
        y.backward()
        autodiff.add_heading("Stepping")
        opt.step()
        box["res"] = y

    autodiff.ir_for(range(0, 10), body)
    res = box["res"]
    res.val().keep()
    l1_w.val().keep()
    l1_b.val().keep()
    l2_w.val().keep()
    autodiff.execute()
    return {"y": res.val().get(), "l1_w": l1_w.val().get(), "l1_b": l1_b.val().get(),
            "l2_w": l2_w.val().get()}


def kat_grd(dev):
    autodiff.set_device(dev)
    a = autodiff.tensor([3.0, 2.0, 1.0, 3.0], [2, 2])
    b = autodiff.tensor([2.0, 5.0, 2.0, 1.0], [2, 2])
    l = a * b
    l.forward()
    l.backward()
    a += a.grad()
    l = a * b
    l.forward()
    l.backward()
    autodiff.execute()
    return {"a": a.val().get(), "a_grad": a.grad().get()}


def kat_eq(dev):
    autodiff.set_device(dev)
    x = autodiff.tensor([0.0, 1.0, 3.0, 2.0, 1.0, 3.0], [6])
    res = 3.0 * (x * (x.equal(constant(3.0, x.dim())))).pow2()
    y = res.sum(0)
    y.forward()
    y.backward()
    all_no = autodiff.tensor([0.0, 1.0, 1.0], [3]).all()
    all_no.forward()
    all_yes = autodiff.tensor([1.0, 1.0, 1.0], [3]).all()
    all_yes.forward()
    res.val().keep()
    all_no.val().keep()
    all_yes.val().keep()
    y.val().keep()
    autodiff.execute()
    return {"res": res.val().get(), "x_grad": x.grad().get(), "all_no": all_no.val().get(),
            "all_yes": all_yes.val().get(), "y": y.val().get()}


def kat_if_ctrl(dev):
    autodiff.set_device(dev)
    x = autodiff.scalar(1.0)
    y = autodiff.scalar(3.0)

    def blk():
        nonlocal y
        y += 4.0
        y.forward()

    autodiff.ir_if(lambda: x, blk)
    y += 3.0
    y.forward()
    x_two = autodiff.scalar(0.0)
    autodiff.ir_if(lambda: x_two, blk)
    autodiff.execute()
    return {"y": y.val().get()}


def kat_if_else_ctrl(dev):
    autodiff.set_device(dev)
    x = autodiff.scalar(1.0)
    y = autodiff.scalar(3.0)
    y_two = autodiff.scalar(3.0)

    def add_to(t, v):
        def f():
            t.__iadd__(v)
            t.forward()
        return f

    autodiff.ir_if_else(lambda: x, add_to(y, 4.0), add_to(y_two, 5.0))
    autodiff.ir_if_else(lambda: x - 1.0, add_to(y, 9.0), add_to(y_two, 10.0))
    autodiff.execute()
    return {"y": y.val().get(), "y_two": y_two.val().get()}


def kat_for_ctrl(dev):
    autodiff.set_device(dev)
    y = autodiff.scalar(10.0)

    def body(i):
        nonlocal y
        y += i
        y.forward()

    autodiff.ir_for(range(-3, 5), body)
    autodiff.execute()
    return {"y": y.val().get()}


def kat_evrty_ctrl(dev):
    autodiff.set_device(dev)
    y = autodiff.scalar(3.0)
    y_two = autodiff.scalar(3.0)

    def body(i):
        def neg_branch():
            y.__imul__(i)
            y.forward()

        def else_branch():
            def pos_branch():
                y_two.__imul__(i)
                y_two.forward()
            autodiff.ir_if(lambda: i.more_than(autodiff.scalar(0.0)), pos_branch)

        autodiff.ir_if_else(lambda: i.less_than(autodiff.scalar(0.0)), neg_branch, else_branch)

    autodiff.ir_for(range(-3, 5), body)
    autodiff.execute()
    return {"y": y.val().get(), "y_two": y_two.val().get()}


def kat_ct(dev):
    autodiff.set_device(dev)
    x = autodiff.tensor([1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0, 8.0], [2, 4])
    y = autodiff.tensor([7.0, 2.0, 6.0, 4.0, 9.0, 2.0, 6.0, 4.0], [2, 4])
    t = (2.0 * x + 3.0).cos()
    t2 = ((t * y) + 3.0 * (t + x)).sqrt()
    res = t2 / t
    res.forward()
    res.backward()
    res.val().keep()
    autodiff.execute()
    return {"res": res.val().get(), "x_grad": x.grad().get(), "y_grad": y.grad().get()}


def kat_rmsnorm(dev):
    autodiff.set_device(dev)
    x = autodiff.tensor([1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0, 8.0], [2, 4])
    res = nn.RMS(4).f(x)
    res.forward()
    res.val().keep()
    autodiff.execute()
    return {"res": res.val().get()}


def kat_layernorm(dev):
    autodiff.set_device(dev)
    x = autodiff.tensor([1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0, 9.0], [2, 4])
    res = nn.LayerNorm(4).f(x)
    res.forward()
    res.val().keep()
    autodiff.execute()
    return {"res": res.val().get()}


def kat_everything(dev):
    autodiff.set_device(dev)
    x = autodiff.tensor([1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0, 8.0], [2, 4])
    y = autodiff.tensor([7.0, 2.0, 6.0, 4.0, 9.0, 2.0, 6.0, 4.0], [2, 4])
    z = autodiff.tensor([7.0, 2.0], [2, 1])
    v = autodiff.tensor([1.0, 2.0, 4.0], [3, 1])
    t1 = dot(x, y.t())
    t2 = t1.sum(0).repeat(lambda n, _: n, 3, 0)
    t3 = dot(t2, z)
    result = concat([t3, 3.0 * v.pow2()], 1)
    result.forward()
    result.r(range(0, 2), 0).backward()
    result.val().keep()
    autodiff.execute()
    return {"result": result.val().get(), "x_grad": x.grad().get(), "y_grad": y.grad().get(),
            "z_grad": z.grad().get(), "v_grad": v.grad().get()}


KATS = {
    "nn": kat_nn, "grd": kat_grd, "eq": kat_eq, "if_ctrl": kat_if_ctrl,
    "if_else_ctrl": kat_if_else_ctrl, "for_ctrl": kat_for_ctrl, "evrty_ctrl": kat_evrty_ctrl,
    "ct": kat_ct, "rmsnorm": kat_rmsnorm, "layernorm": kat_layernorm, "everything": kat_everything,
}


def check_golden(name, out):
    """Assert `out` against the reference's asserted values the way the reference does:
    exact equality, after `.round(4)` for the tests that round."""
    for key, (dim, data) in GOLDEN[name].items():
        vd = out[key]
        assert not vd.is_none, f"{name}.{key} is none"
        assert vd.dim == dim, f"{name}.{key} dim {vd.dim} != {dim}"
        got = vd.round(4).data if name in ROUNDED else vd.data
        exp = np.asarray(data, dtype=np.float32)
        if name in ROUNDED:
            exp = (np.round(exp.astype(np.float64) * 1e4) / 1e4).astype(np.float32)
        got = np.asarray(got, dtype=np.float32).copy()
        for idx, rtol in ILL_CONDITIONED.get((name, key), {}).items():
            assert abs(float(got[idx]) - float(exp[idx])) <= rtol * abs(float(exp[idx])), \
                f"{name}.{key}[{idx}]: {got[idx]} vs {exp[idx]}"
            got[idx] = exp[idx]
        assert np.array_equal(got, exp), f"{name}.{key}: {got} != {exp}"


def predicated_loop_program(dev):
    """A data-dependent while loop (its predicate is a product of two comparisons, so it is not the
    counted `ir_for` shape) with an if/else and a nested if in the body.
    i = 0..6: i < 2 -> y += 10; else { if i > 3 -> z *= 2; y += 1 }.  Result: y = 25, z = 8, i = 7."""
    autodiff.set_device(dev)
    i = autodiff.scalar(0.0)
    y = autodiff.scalar(0.0)
    z = autodiff.scalar(1.0)
    pred = i.less_than(constant(7.0, [1])) * i.less_than(constant(100.0, [1]))

    def body():
        nonlocal i

        def then():
            y.__iadd__(10.0)
            y.forward()

        def other():
            def inner():
                z.__imul__(2.0)
                z.forward()
            autodiff.ir_if(lambda: i.more_than(autodiff.scalar(3.0)), inner)
            y.__iadd__(1.0)
            y.forward()

        autodiff.ir_if_else(lambda: i.less_than(autodiff.scalar(2.0)), then, other)
        i += 1.0

    autodiff.ir_while(pred, body)
    autodiff.execute()
    return {"y": y.val().get(), "z": z.val().get(), "i": i.val().get()}


def branch_reads_id_dropped_by_earlier_arm(k_value: float):
    """`f` is defined before a branch, redefined in the first arm, read in the second arm (which also updates it in
    place inside a loop) and redefined after the branch, so it is dead once the branch is over: the first arm's
    definition needs no memory, but the second arm must still find the value from before the branch.  Returns
    (procedure, keep list, expected values) for a predicate input `k_value` (< 0: first arm, > 0: second arm, 0:
    neither)."""
    import numpy as np
    from adhip import ir as IR

    def mat(name, values, shape):
        return IR.CreateMat(np.asarray(values, dtype=np.float32), list(shape), name)

    def block(cmds):
        return IR.IRProcedure("block", cmds)

    f0 = np.array([1.0, 2.0, 3.0, 4.0], dtype=np.float32)
    y0 = np.array([0.5, -1.0, 2.0, 8.0], dtype=np.float32)
    top = [mat("f", f0, [4]), mat("y", y0, [4]), mat("g", [0, 0, 0, 0], [4]), mat("k", [k_value], [1]), mat("w", [1.0], [1]),
           IR.LessZero(a="k", res="p"), IR.MoreZero(a="k", res="q")]
    arm1 = [IR.CreateConstant(0.5, "c", [4]), IR.ElwMultiply(a="y", b="c", res="f"), IR.ElwAdd(a="f", b="y", res="g")]
    body = [IR.ElwAddEq(s="f", o="y"), IR.CreateConstant(0.0, "z", [1]), IR.ElwMultiplyEq(s="w", o="z")]
    arm2 = [IR.While(conditional_var="w", block=block(body)), IR.ElwAdd(a="f", b="f", res="g")]
    tail = [IR.CreateConstant(3.0, "c3", [4]), IR.ElwMultiply(a="y", b="c3", res="f")]
    proc = IR.IRProcedure("main", top + [IR.If(conditions=[("p", block(arm1)), ("q", block(arm2))], else_proc=None)] + tail + [IR.EX()])
    if k_value < 0:
        g = 0.5 * y0 + y0
    elif k_value > 0:
        g = 2.0 * (f0 + y0)
    else:
        g = np.zeros(4, dtype=np.float32)
    return proc, ["f", "g"], {"f": 3.0 * y0, "g": g}


def reduction_epilogue_with_split_row_index():
    """y = a.permute(0, 2, 1).sum(-1) + v broadcast over the first dim, a [2,3,4], v [4]: the reduction walks a
    permuted operand, so its row index is split into two pieces inside the loop, and the element-wise consumer that
    runs as the reduction's epilogue needs one of the pieces again for v.  Returns (procedure, keep, expected)."""
    import numpy as np
    from adhip import ir as IR
    rng = np.random.default_rng(11)
    a = rng.integers(-4, 5, (2, 3, 4)).astype(np.float32)
    v = rng.integers(-4, 5, 4).astype(np.float32)
    cmds = [IR.CreateMat(a.reshape(-1), [2, 3, 4], "a"), IR.CreateMat(v, [4], "v"),
            IR.Permute(a="a", p=[0, 2, 1], res="t"), IR.View(a="t", target_dim=[8, 3], res="tv"), IR.Sum(a="tv", res="s"),
            IR.View(a="v", target_dim=[1, 4], res="vv"), IR.Broadcast(a="vv", dim=0, r=2, res="vb"),
            IR.View(a="vb", target_dim=[8], res="vf"), IR.ElwAdd(a="s", b="vf", res="y"), IR.EX()]
    expect = (a.transpose(0, 2, 1).sum(-1) + v[None, :]).reshape(-1)
    return IR.IRProcedure("main", cmds), ["y"], {"y": expect.astype(np.float32)}
