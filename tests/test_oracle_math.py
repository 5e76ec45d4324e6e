"""Pins the oracle's arithmetic and data movement against what the mathematics fixes, independently
of the formulas the oracle itself uses."""
import itertools
import math

import numpy as np
import pytest

from adhip import ir as IR
from oracle.interp import OracleDevice, ref_dot, ref_reduce_max, ref_reduce_sum, ref_unary


# ---- reductions and matmul ----------------------------------------------------------------

@pytest.mark.parametrize("vec,red", [(1, 1), (3, 6), (5, 768), (7, 1000), (2, 4096), (64, 33)])
def test_tree_sum_matches_float64_and_is_exact_on_integers(vec, red):
    rng = np.random.default_rng(vec * 1000 + red)
    a = rng.standard_normal((vec, red)).astype(np.float32)
    got = ref_reduce_sum(a)
    ref = a.astype(np.float64).sum(1)
    scale = np.abs(a.astype(np.float64)).sum(1)
    assert np.all(np.abs(got - ref) <= 1e-5 * math.sqrt(red) * np.maximum(scale, 1e-30))
    # every element is counted exactly once: integers sum exactly, also for non-power-of-two sizes
    ints = rng.integers(-8, 9, size=(vec, red)).astype(np.float32)
    assert np.array_equal(ref_reduce_sum(ints), ints.sum(1, dtype=np.float64).astype(np.float32))
    assert np.array_equal(ref_reduce_sum(np.ones((vec, red), np.float32)), np.full(vec, red, np.float32))


def test_tree_sum_reads_strided_input():
    a = np.arange(24, dtype=np.float32).reshape(4, 6)
    assert np.array_equal(ref_reduce_sum(a.T), a.sum(0))


def test_row_max_by_brute_force():
    """`Max` against plain loops with explicit comparisons (no numpy reduction): the largest element of every row;
    a NaN is passed over unless the whole row is NaN; -0.0 and +0.0 compare equal (either may come back); rows of
    -inf stay -inf; position of the maximum does not matter."""
    rng = np.random.default_rng(5)
    a = rng.standard_normal((9, 37)).astype(np.float32)
    a[1, 5] = np.nan
    a[2, :] = np.nan
    a[3, :] = -np.inf
    a[4, 7] = np.inf
    a[5, :] = -0.0
    a[5, 3] = 0.0
    a[6, 0] = 1e30            # first position
    a[7, 36] = 1e30           # last position
    got = ref_reduce_max(a)
    for i in range(a.shape[0]):
        best = None
        for j in range(a.shape[1]):
            v = float(a[i, j])
            if v != v:
                continue
            if best is None or v > best:
                best = v
        if best is None:
            assert got[i] != got[i], f"row {i}: all NaN must give NaN"
        else:
            assert float(got[i]) == best, (i, got[i], best)
    assert np.array_equal(ref_reduce_max(a[:1, :1]), a[:1, 0])
    # strided input (a transposed view)
    b = np.arange(24, dtype=np.float32).reshape(4, 6)
    assert np.array_equal(ref_reduce_max(b.T), b.max(0))


def test_max_command_and_softmax_through_the_oracle():
    """`Tensor.max(dim)` on every dim of a 3-D tensor against loops, its backward (equal shares among ties), and the
    shifted softmax against float64 at arguments where exp alone overflows."""
    from adhip import autodiff
    dev = OracleDevice()
    autodiff.set_device(dev)
    rng = np.random.default_rng(9)
    xn = rng.integers(-3, 4, size=(3, 4, 5)).astype(np.float32)
    x = autodiff.tensor(xn, [3, 4, 5])
    outs = []
    for d in range(3):
        m = x.max(d)
        m.forward()
        m.val().keep()
        outs.append(m)
    total = outs[2].sum(0).sum(0)
    total.forward()
    total.backward()
    x.grad().keep()
    s = (x * 40.0).softmax(-1)
    s.forward()
    s.val().keep()
    autodiff.execute()
    for d in range(3):
        got = outs[d].val().get().numpy()
        exp = np.empty([n for i, n in enumerate(xn.shape) if i != d], dtype=np.float32)
        for idx in itertools.product(*[range(n) for n in exp.shape]):
            full = list(idx)
            full.insert(d, slice(None))
            exp[idx] = max(float(v) for v in xn[tuple(full)])
        assert np.array_equal(got, exp), d
    g = x.grad().get().numpy()
    for i in range(3):
        for j in range(4):
            row = xn[i, j]
            ties = [k for k in range(5) if row[k] == row.max()]
            for k in range(5):
                assert abs(g[i, j, k] - (1.0 / len(ties) if k in ties else 0.0)) < 1e-6
    z = xn.astype(np.float64) * 40.0
    e = np.exp(z - z.max(-1, keepdims=True))
    ref = e / e.sum(-1, keepdims=True)
    got = s.val().get().numpy()
    assert np.isfinite(got).all() and np.abs(got - ref).max() < 2e-6


@pytest.mark.parametrize("m,k,n", [(1, 1, 1), (2, 5, 3), (17, 33, 9), (64, 128, 32)])
def test_dot_matches_float64_and_is_exact_on_integers(m, k, n):
    rng = np.random.default_rng(m + 10 * k + 100 * n)
    a = rng.standard_normal((m, k)).astype(np.float32)
    b = rng.standard_normal((k, n)).astype(np.float32)
    ref = a.astype(np.float64) @ b.astype(np.float64)
    bound = 1e-5 * math.sqrt(k) * (np.abs(a.astype(np.float64)) @ np.abs(b.astype(np.float64)))
    assert np.all(np.abs(ref_dot(a, b) - ref) <= bound + 1e-30)
    ai = rng.integers(-4, 5, size=(m, k)).astype(np.float32)
    bi = rng.integers(-4, 5, size=(k, n)).astype(np.float32)
    assert np.array_equal(ref_dot(ai, bi), (ai.astype(np.int64) @ bi.astype(np.int64)).astype(np.float32))
    # transposed operands through strides: (A^T)^T . B
    assert np.array_equal(ref_dot(np.ascontiguousarray(ai.T).T, bi), ref_dot(ai, bi))
    # a wrong operand order or a transposed operand would fail this unless the matrices commute
    if m == n and m > 1:
        assert not np.array_equal(ref_dot(ai, bi), ref_dot(bi.T.copy(), ai.T.copy()).T) or np.array_equal(ai @ bi, (bi.T @ ai.T).T)


def test_dot_accumulates_in_ascending_k_in_float32():
    # 2^24 + 1 + 1: sequential float32 accumulation loses both ones, any pairwise order keeps them
    a = np.array([[16777216.0, 1.0, 1.0]], dtype=np.float32)
    b = np.ones((3, 1), dtype=np.float32)
    assert ref_dot(a, b)[0, 0] == np.float32(16777216.0)


# ---- unary kernels --------------------------------------------------------------------------

def test_unary_kernels_special_values():
    x = np.array([-4.0, -1.0, -0.0, 0.0, 0.25, 1.0, 3.0, 1024.0], dtype=np.float32)
    assert np.array_equal(ref_unary(IR.T_EQUAL_ZERO, x), (x == 0).astype(np.float32))
    assert np.array_equal(ref_unary(IR.T_MORE_ZERO, x), (x > 0).astype(np.float32))
    assert np.array_equal(ref_unary(IR.T_LESS_ZERO, x), (x < 0).astype(np.float32))
    # sqrt takes |x| (reference kernels/unary.rs:11), unlike numpy/torch which give NaN for negatives
    assert np.array_equal(ref_unary(IR.T_SQRT, x), np.sqrt(np.abs(x)))
    nz = x[x != 0]
    assert np.array_equal(ref_unary(IR.T_RECIP, nz), (np.float32(1.0) / nz))
    ints = np.arange(-10, 11, dtype=np.float32)
    assert np.array_equal(ref_unary(IR.T_EXP2, ints), np.ldexp(np.float32(1.0), ints.astype(np.int32)))
    pows = np.ldexp(np.float32(1.0), np.arange(-10, 11)).astype(np.float32)
    assert np.array_equal(ref_unary(IR.T_LOG2, pows), np.arange(-10, 11, dtype=np.float32))
    assert ref_unary(IR.T_SIN, np.zeros(1, np.float32))[0] == 0.0
    s = ref_unary(IR.T_SIN, np.array([math.pi / 6, math.pi / 2], dtype=np.float32))
    assert abs(s[0] - 0.5) < 1e-6 and abs(s[1] - 1.0) < 1e-6


# ---- data movement against brute-force index arithmetic -------------------------------------

def _brute(cmds, bufs):
    """Evaluate a chain of data commands by pushing each output coordinate backwards to a source
    element, the way the reference builds its index expressions (helper/shape.rs:51-76), in pure
    Python: no reshape / transpose / take / concatenate."""
    shapes = {k: list(v.shape) for k, v in bufs.items()}
    defs = {}
    for c in cmds:
        if c[0] == "view":
            _, a, dims, res = c
            shapes[res] = list(dims)
        elif c[0] == "index":
            _, a, idx, dim, res = c
            shapes[res] = shapes[a][:dim] + shapes[a][dim + 1:]
        elif c[0] == "permute":
            _, a, p, res = c
            shapes[res] = [shapes[a][i] for i in p]
        elif c[0] == "broadcast":
            _, a, dim, r, res = c
            shapes[res] = list(shapes[a])
            shapes[res][dim] = r
        elif c[0] == "concat":
            _, a, b, dim, res = c
            shapes[res] = list(shapes[a])
            shapes[res][dim] += shapes[b][dim]
        defs[c[-1]] = c

    def lin(coord, shape):
        g = 0
        for c, s in zip(coord, shape):
            g = g * s + c
        return g

    def unlin(g, shape):
        out = []
        for s in reversed(shape):
            out.append(g % s)
            g //= s
        return list(reversed(out))

    def fetch(id, coord):
        if id in bufs:
            return bufs[id].reshape(-1)[lin(coord, shapes[id])]
        c = defs[id]
        if c[0] == "view":
            return fetch(c[1], unlin(lin(coord, shapes[id]), shapes[c[1]]))
        if c[0] == "index":
            return fetch(c[1], coord[:c[3]] + [c[2]] + coord[c[3]:])
        if c[0] == "permute":
            src = [0] * len(coord)
            for i, p in enumerate(c[2]):
                src[p] = coord[i]
            return fetch(c[1], src)
        if c[0] == "broadcast":
            src = list(coord)
            src[c[2]] = 0
            return fetch(c[1], src)
        if c[0] == "concat":
            split = shapes[c[1]][c[3]]
            if coord[c[3]] < split:
                return fetch(c[1], coord)
            src = list(coord)
            src[c[3]] -= split
            return fetch(c[2], src)
        raise AssertionError

    last = cmds[-1][-1]
    out = np.empty(shapes[last], dtype=np.float32)
    for coord in itertools.product(*[range(s) for s in shapes[last]]):
        out[coord] = fetch(last, list(coord))
    return out


def _to_ir(cmds):
    out = []
    for c in cmds:
        if c[0] == "view":
            out.append(IR.View(a=c[1], target_dim=list(c[2]), res=c[3]))
        elif c[0] == "index":
            out.append(IR.Index(a=c[1], index=c[2], dim=c[3], res=c[4]))
        elif c[0] == "permute":
            out.append(IR.Permute(a=c[1], p=list(c[2]), res=c[3]))
        elif c[0] == "broadcast":
            out.append(IR.Broadcast(a=c[1], dim=c[2], r=c[3], res=c[4]))
        elif c[0] == "concat":
            out.append(IR.Concat(a=c[1], b=c[2], dim=c[3], res=c[4]))
    return out


CHAINS = [
    # non-involutive permutation (the reference's own back-mapping is only right for swaps)
    [("permute", "x", [1, 2, 0], "p")],
    [("permute", "x", [2, 0, 1], "p"), ("view", "p", [4, 6], "v"), ("permute", "v", [1, 0], "t")],
    [("index", "x", 1, 1, "i"), ("view", "i", [2, 1, 4], "u"), ("broadcast", "u", 1, 3, "b")],
    [("permute", "x", [0, 2, 1], "p"), ("concat", "p", "z", 2, "c"), ("index", "c", 2, 1, "i")],
    [("concat", "x", "x", 0, "c"), ("view", "c", [6, 8], "v"), ("permute", "v", [1, 0], "t"), ("index", "t", 5, 0, "i")],
    [("view", "x", [6, 4], "v"), ("index", "v", 3, 0, "i"), ("view", "i", [1, 4], "u"), ("broadcast", "u", 0, 5, "b"),
     ("permute", "b", [1, 0], "t")],
]


@pytest.mark.parametrize("chain", range(len(CHAINS)))
def test_oracle_data_movement_matches_brute_force(chain):
    rng = np.random.default_rng(chain)
    x = rng.standard_normal((2, 3, 4)).astype(np.float32)
    z = rng.standard_normal((2, 4, 2)).astype(np.float32)
    cmds = CHAINS[chain]
    expect = _brute(cmds, {"x": x, "z": z})
    last = cmds[-1][-1]
    proc = IR.IRProcedure("main", [IR.CreateMat(x.reshape(-1), [2, 3, 4], "x"), IR.CreateMat(z.reshape(-1), [2, 4, 2], "z")]
                          + _to_ir(cmds) + [IR.Contigious(a=last, res="out"), IR.EX()])
    dev = OracleDevice()
    dev.execute(proc, {"out"})
    got = dev.get_tensor("out")
    assert got.dim == list(expect.shape)
    assert np.array_equal(got.data.reshape(expect.shape), expect)


# ---- execution model --------------------------------------------------------------------------

def test_views_are_resolved_when_used_not_when_made():
    one = np.ones(4, np.float32)
    proc = IR.IRProcedure("main", [
        IR.CreateMat(np.arange(4, dtype=np.float32), [2, 2], "a"), IR.CreateMat(one, [2, 2], "o"),
        IR.Permute(a="a", p=[1, 0], res="t"), IR.ElwAddEq(s="a", o="o"), IR.Contigious(a="t", res="u"), IR.EX()])
    dev = OracleDevice()
    dev.execute(proc, {"u"})
    assert np.array_equal(dev.get_tensor("u").data, np.array([1, 3, 2, 4], np.float32))


def test_control_flow_semantics():
    body = IR.IRProcedure("b", [IR.CreateConstant(-1.0, "m", [1]), IR.ElwAddEq(s="c", o="m"),
                                IR.CreateConstant(2.0, "two", [1]), IR.ElwMultiplyEq(s="y", o="two")])
    skipped = IR.IRProcedure("s", [IR.CreateConstant(100.0, "h", [1]), IR.ElwAddEq(s="y", o="h")])
    taken = IR.IRProcedure("t", [IR.CreateConstant(0.5, "q", [1]), IR.ElwAddEq(s="y", o="q")])
    proc = IR.IRProcedure("main", [
        IR.CreateMat(np.array([3.0], np.float32), [1], "c"), IR.CreateMat(np.array([1.0], np.float32), [1], "y"),
        IR.CreateMat(np.array([2.0], np.float32), [1], "nt"), IR.CreateMat(np.array([1.0], np.float32), [1], "yes"),
        IR.While(conditional_var="c", block=body),          # three iterations: y = 8
        IR.If(conditions=[("nt", skipped), ("yes", taken)], else_proc=skipped),  # 2.0 != 1.0, second arm runs
        IR.EX(),
        IR.ElwAddEq(s="y", o="yes"),                        # never reached
    ])
    dev = OracleDevice()
    dev.execute(proc, {"y", "c", "zz"})
    assert dev.get_tensor("y").data[0] == 8.5
    assert dev.get_tensor("c").data[0] == 0.0
    assert dev.get_tensor("zz").is_none


def test_reference_softmax_formula_on_a_square_matrix():
    """The reference's softmax is `x.exp() / x.exp().sum(dim)` (src/nn/activations/softmax.rs:28-30): the sum loses
    `dim`, and the division broadcasts it back by the trailing-dim rule, so on a square matrix element (i, j) is divided
    by the sum of row j.  The caller side here normalises along `dim` instead (with the maximum subtracted first).
    Both formulas spelled out on one 3x3 matrix: they differ, each matches its own closed form, and only the second
    has rows that add up to 1."""
    from adhip import autodiff
    x = np.array([[0.0, 1.0, 2.0], [1.0, 1.0, 1.0], [3.0, 0.0, -1.0]], dtype=np.float32)
    dev = OracleDevice()
    autodiff.set_device(dev)
    t = autodiff.tensor(x.reshape(-1), [3, 3])
    ours = t.softmax(1)
    reference = t.exp() / t.exp().sum(1)      # the reference's composition, through the same operators
    for v in (ours, reference):
        v.forward()
        v.val().keep()
    autodiff.execute()
    e = np.exp(x.astype(np.float64))
    got_ours = ours.val().get().numpy()
    got_ref = reference.val().get().numpy()
    np.testing.assert_allclose(got_ours, e / e.sum(1, keepdims=True), rtol=1e-6)
    np.testing.assert_allclose(got_ref, e / e.sum(1)[None, :], rtol=1e-6)       # divided by the sum of row j
    np.testing.assert_allclose(got_ours.sum(1), 1.0, rtol=1e-6)
    assert np.abs(got_ref.sum(1) - 1.0).max() > 0.1
    assert np.abs(got_ours - got_ref).max() > 0.05
