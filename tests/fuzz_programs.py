"""Random programs for differential testing of the device against the oracle: a seeded generator that
combines tensors through the caller-side API (element-wise ops, unary functions, comparisons, sums,
permutes, views, slices, concats, matmuls, in-place updates) and then runs forward and backward."""
import numpy as np

from adhip import autodiff
from adhip.core import concat, constant, dot


def random_program(dev, seed: int, n_ops: int = 24, scale: int = 1):
    """`scale` multiplies the two basic extents (4 and 6) of the leaf shapes: at 1 every kernel is a few threads, at 16
    and beyond the 128-bit element-wise forms, sums riding along with element-wise passes, chunked reductions and the
    matrix-core products (with extents that fit no tile) come into play.  Leaf values shrink with the scale so that
    sums over the longer dims stay in the range the small programs have."""
    rng = np.random.default_rng(seed)
    autodiff.set_device(dev)
    p, q = 4 * scale, 6 * scale
    shapes = [[p, q], [q], [p, 1], [2, q // 2, p], [q, p], [q // 2, p], [1], [8, p, q]]
    amp = 1.5 / np.sqrt(scale)
    limit = 4096 * scale * scale
    pool = []
    leaves = []
    for sh in shapes:
        data = rng.uniform(-amp, amp, size=int(np.prod(sh))).astype(np.float32)
        t = autodiff.tensor(data, sh)
        pool.append(t)
        leaves.append(t)

    def pick(pred=None):
        cands = [t for t in pool if pred is None or pred(t)]
        return cands[rng.integers(len(cands))] if cands else None

    def broadcastable(a, b):
        da, db = a.dim(), b.dim()
        if da == db:
            return True
        for i in range(1, min(len(da), len(db)) + 1):
            if da[-i] != db[-i] and da[-i] != 1 and db[-i] != 1:
                return False
        return True

    for _ in range(n_ops):
        kind = rng.integers(12)
        a = pick()
        out = None
        try:
            if kind == 0:
                b = pick(lambda t: broadcastable(a, t))
                out = a + b
            elif kind == 1:
                b = pick(lambda t: broadcastable(a, t))
                out = a * b
            elif kind == 2:
                out = a - float(rng.uniform(-1, 1))
            elif kind == 3:
                f = rng.integers(5)
                if f == 0:
                    out = a.sin()
                elif f == 1:
                    out = (a * 0.5).exp2()
                elif f == 2:
                    out = (a * a + 1.0).recip()
                elif f == 3:
                    out = (a * a + 0.5).sqrt()
                else:
                    out = (a * a + 1.0).log2()
            elif kind == 4 and len(a.dim()) >= 1:
                out = a.sum(int(rng.integers(len(a.dim()))))
            elif kind == 5 and len(a.dim()) >= 2:
                out = a.permute([int(x) for x in rng.permutation(len(a.dim()))])
            elif kind == 6:
                n = int(np.prod(a.dim()))
                divs = [d for d in range(1, int(n ** 0.5) + 1) if n % d == 0]
                divs = sorted(divs + [n // d for d in divs if d * d != n])
                d0 = divs[rng.integers(len(divs))]
                out = a.view([d0, n // d0])
            elif kind == 7 and len(a.dim()) >= 1:
                dim = int(rng.integers(len(a.dim())))
                if a.dim()[dim] >= 2:
                    lo = int(rng.integers(a.dim()[dim] - 1))
                    hi = int(rng.integers(lo + 1, a.dim()[dim] + 1))
                    out = a.r(range(lo, hi), dim)
            elif kind == 8:
                b = pick(lambda t: len(t.dim()) == len(a.dim()) and len(a.dim()) >= 1)
                if b is not None:
                    for dim in range(len(a.dim())):
                        if all(a.dim()[k] == b.dim()[k] for k in range(len(a.dim())) if k != dim):
                            out = concat([a, b], dim)
                            break
            elif kind == 9 and len(a.dim()) == 2:
                b = pick(lambda t: len(t.dim()) == 2 and t.dim()[0] == a.dim()[1])
                if b is not None:
                    out = dot(a, b)
            elif kind == 10:
                out = a * a.more_than(constant(0.1, a.dim())) + a.less_than(constant(-0.2, a.dim()))
            elif kind == 11 and len(a.dim()) == 2:
                out = a.t().contigious() if rng.integers(2) else a.t()
        except (AssertionError, RuntimeError):
            out = None
        if out is not None and int(np.prod(out.dim())) <= limit and int(np.prod(out.dim())) > 0:
            pool.append(out)

    # a scalar target that touches several recent values, then forward and backward
    target = None
    for t in pool[-5:]:
        s = t
        for _ in list(s.dim()):
            s = s.sum(0)
        target = s if target is None else target + s
    target.forward()
    target.backward()
    target.val().keep()
    outs = {"target": target.val()}
    for i, t in enumerate(pool[len(shapes):]):
        v = t.val()
        if v is not None:
            v.keep()
            outs[f"v{i}"] = v
    for i, t in enumerate(leaves):
        try:
            outs[f"g{i}"] = t.grad()
        except RuntimeError:
            pass
    autodiff.execute()
    return {k: v.get() for k, v in outs.items()}
