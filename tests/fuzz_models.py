"""Random programs out of the building blocks of models, for differential testing: row maxima, softmax, mean and
variance, LayerNorm and RMS, Linear with its in-place bias, tensor `*=` / `-=`, Attention and AttentionMasked (with
and without the probabilities kept for somebody else), Concats of many distinct values -- glued together by
element-wise operations, sums and products, then forward and backward.

Every operation is applied twice: to the caller-side graph (adhip.core, which emits the IR both the device and the
oracle execute) and to a float64 `torch` shadow written with torch's own functions (`torch.softmax`, `amax`, `var`,
`layer_norm`, ...), which shares no code with the front end.  `random_model_program(dev, seed, scale)` returns the
device's (or oracle's) kept values; `shadow_model_program(seed, scale)` the float64 answers for the same names."""
import math

import numpy as np

from adhip import autodiff, nn
from adhip.core import concat, dot


class _Pair:
    """A caller-side tensor and its float64 shadow (None when no shadow is kept)."""

    def __init__(self, t, s):
        self.t, self.s = t, s

    def dim(self):
        return list(self.t.dim()) if self.t is not None else list(self.s.shape)


def _build(dev, seed, scale, n_ops, shadow, kinds=None):
    torch = None
    if shadow:
        import torch
    rng = np.random.default_rng(seed)
    if dev is not None:
        autodiff.set_device(dev)
    p, q = 4 * scale, 6 * scale
    amp = 1.5
    limit = 8192 * scale * scale

    def leaf(shape, lo=-amp, hi=amp, grad=True):
        data = rng.uniform(lo, hi, size=int(np.prod(shape))).astype(np.float32)
        t = autodiff.tensor(data, list(shape)) if dev is not None else None
        s = None
        if shadow:
            s = torch.tensor(data.astype(np.float64).reshape(shape), requires_grad=grad)
        return _Pair(t, s)

    shapes = [[q, p], [q, p], [p, p], [p, q], [p], [q, q], [q], [p, 1], [q, p], [p, q]]
    leaves = [leaf(sh) for sh in shapes]
    pool = list(leaves)

    def pick(pred=None):
        cands = [x for x in pool if pred is None or pred(x)]
        return cands[int(rng.integers(len(cands)))] if cands else None

    def is2d(x):
        return len(x.dim()) == 2

    def apply(ft, fs, *xs):
        """ft on the caller-side tensors, fs on the shadows"""
        t = ft(*[x.t for x in xs]) if dev is not None else None
        s = fs(*[x.s for x in xs]) if shadow else None
        if s is not None and s.dim() == 0:
            s = s.reshape(1)   # the caller side has no rank 0: a vector's reduction has shape [1]
        return _Pair(t, s)

    extra_leaves = []
    for step in range(n_ops):
        kind = int(rng.integers(14))
        if kinds is not None:
            kind = kinds[int(rng.integers(len(kinds)))]
        a = pick()
        out = None
        if kind == 0:
            b = pick(lambda x: x.dim() == a.dim())
            out = apply(lambda u, v: u + v, lambda u, v: u + v, a, b) if rng.integers(2) else apply(lambda u, v: u * v, lambda u, v: u * v, a, b)
        elif kind == 1:
            f = int(rng.integers(3))
            if f == 0:
                out = apply(lambda u: u.sin(), lambda u: torch.sin(u), a)
            elif f == 1:
                out = apply(lambda u: u.sigmoid(), lambda u: torch.sigmoid(u), a)
            else:
                out = apply(lambda u: (u * u + 1.0).sqrt(), lambda u: torch.sqrt(u * u + 1.0), a)
        elif kind == 2 and len(a.dim()) >= 1:
            d = int(rng.integers(len(a.dim())))
            if a.dim()[d] >= 1:
                out = apply(lambda u: u.max(d), lambda u: torch.amax(u, dim=d), a)
        elif kind == 3 and len(a.dim()) >= 1:
            d = int(rng.integers(len(a.dim())))
            out = apply(lambda u: u.softmax(d), lambda u: torch.softmax(u, dim=d), a)
        elif kind == 4 and len(a.dim()) >= 1:
            d = int(rng.integers(len(a.dim())))
            if a.dim()[d] >= 2:
                if rng.integers(2):
                    out = apply(lambda u: u.mean(d), lambda u: torch.mean(u, dim=d), a)
                elif len(a.dim()) >= 2:   # (the caller-side composition of var needs a dim to put back)
                    c = int(rng.integers(2))
                    out = apply(lambda u: u.var(d, c), lambda u: torch.var(u, dim=d, correction=c), a)
        elif kind == 5 and is2d(a) and a.dim()[1] >= 4:
            n = a.dim()[1]
            scale_leaf = leaf([n], 0.5, 1.5)
            extra_leaves.append(scale_leaf)
            if rng.integers(2):
                bias_leaf = leaf([n])
                extra_leaves.append(bias_leaf)

                def ln_t(u, g, b):
                    m = nn.LayerNorm.__new__(nn.LayerNorm)
                    m.scale, m.bias = g, b
                    return m.f(u)
                out = apply(ln_t, lambda u, g, b: torch.nn.functional.layer_norm(u, (n,), g, b, eps=1e-9), a, scale_leaf, bias_leaf)
            else:
                def rms_t(u, g):
                    m = nn.RMS.__new__(nn.RMS)
                    m.scale = g
                    return m.f(u)
                out = apply(rms_t, lambda u, g: g * (u / torch.sqrt(torch.mean(u * u, dim=-1, keepdim=True) + 1e-9)), a, scale_leaf)
        elif kind == 6 and is2d(a):
            w = pick(lambda x: is2d(x) and x.dim()[0] == a.dim()[1])
            if w is not None:
                k, n = w.dim()
                b = leaf([n])
                extra_leaves.append(b)

                def lin_t(u, ww, bb):
                    return nn.LinearWithWeights(ww, bb).f(u) * (1.0 / math.sqrt(k))   # res = dot; res += bias
                out = apply(lin_t, lambda u, ww, bb: (u @ ww + bb) * (1.0 / math.sqrt(k)), a, w, b)
        elif kind == 7:
            # tensor `*=`, `-=`, `+=` on a fresh value.  The factor of `*=` is a constant of the backward pass: the
            # caller side's MultiplyNode reads its left operand's value when it propagates, and after an in-place
            # update that id holds the updated contents (so does the reference's, src/graph/ops/ops.rs: `*=` is meant
            # for parameter updates, not for differentiated values).
            m = leaf(a.dim(), 0.5, 1.5, grad=False)
            c = pick(lambda x: x.dim() == a.dim())

            def inplace_t(u, v, w):
                r = u + 0.25
                r *= v
                r -= w
                r += 0.5
                return r
            out = apply(inplace_t, lambda u, v, w: (u + 0.25) * v - w + 0.5, a, m, c)
        elif kind in (8, 9) and is2d(a):
            # attention over (Q [s, d], K [s2, d], V [s2, dv]); kind 9 multiplies the scaled scores by a mask first
            s1, d = a.dim()
            K = pick(lambda x: is2d(x) and x.dim()[1] == d)
            V = pick(lambda x: K is not None and is2d(x) and x.dim()[0] == K.dim()[0]) if K is not None else None
            if K is not None and V is not None:
                s2 = K.dim()[0]
                keep_p = int(rng.integers(3)) == 0
                if int(rng.integers(2)):
                    # inference: no gradient flows back through the attention, so nothing but the product reads the
                    # probabilities and the fused kernel applies (head widths permitting)
                    a, K, V = (apply(lambda u: u.detach(), lambda u: u.detach(), x) for x in (a, K, V))
                if kind == 9:
                    mask = leaf([s1, s2], 0.25, 1.25, grad=False)

                    def att_t(Q, Kk, Vv, M):
                        return nn.AttentionMasked(Q, Kk, Vv, d, M)
                    out = apply(att_t, lambda Q, Kk, Vv, M: torch.softmax(Q @ Kk.T / math.sqrt(d) * M, dim=-1) @ Vv, a, K, V, mask)
                elif keep_p:
                    # the probabilities are somebody else's operand too: they have to exist in memory
                    P = apply(lambda Q, Kk: (dot(Q, Kk.t()) / math.sqrt(float(d))).softmax(-1),
                              lambda Q, Kk: torch.softmax(Q @ Kk.T / math.sqrt(d), dim=-1), a, K)
                    pool.append(P)
                    out = apply(lambda Pp, Vv: dot(Pp, Vv), lambda Pp, Vv: Pp @ Vv, P, V)
                else:
                    out = apply(lambda Q, Kk, Vv: nn.Attention(Q, Kk, Vv, d), lambda Q, Kk, Vv: torch.softmax(Q @ Kk.T / math.sqrt(d), dim=-1) @ Vv, a, K, V)
        elif kind == 10 and len(a.dim()) >= 1:
            # a Concat of many distinct values: k different functions of values shaped like a
            k = int(rng.integers(3, 13))
            dim = int(rng.integers(len(a.dim())))
            parts = []
            for j in range(k):
                b = pick(lambda x: x.dim() == a.dim())
                c = float(rng.uniform(0.5, 1.5))
                parts.append(apply(lambda u, cc=c: u * cc, lambda u, cc=c: u * cc, b))
            if int(np.prod(a.dim())) * k <= limit:
                out = apply(lambda *us: concat(list(us), dim), lambda *us: torch.cat(list(us), dim=dim), *parts)
        elif kind == 11 and is2d(a):
            b = pick(lambda x: is2d(x) and x.dim()[0] == a.dim()[1])
            if b is not None:
                k = a.dim()[1]
                out = apply(lambda u, v: dot(u, v) * (1.0 / math.sqrt(k)), lambda u, v: (u @ v) * (1.0 / math.sqrt(k)), a, b)
        elif kind == 12 and len(a.dim()) >= 1:
            d = int(rng.integers(len(a.dim())))
            out = apply(lambda u: u.sum(d) * (1.0 / math.sqrt(a.dim()[d])), lambda u: torch.sum(u, dim=d) * (1.0 / math.sqrt(a.dim()[d])), a)
        elif kind == 13 and is2d(a):
            out = apply(lambda u: u.t(), lambda u: u.T, a)
        if out is not None and 0 < int(np.prod(out.dim())) <= limit:
            pool.append(out)

    # a scalar target that touches several recent values, then forward and backward
    recent = pool[-6:]

    def total_t(*us):
        target = None
        for u in us:
            s = u
            for _ in list(s.dim()):
                s = s.sum(0)
            target = s if target is None else target + s
        return target

    def total_s(*us):
        return sum(u.sum() for u in us).reshape(1)
    target = apply(total_t, total_s, *recent)
    all_leaves = leaves + extra_leaves
    return target, pool[len(leaves):], all_leaves


def random_model_program(dev, seed: int, scale: int = 1, n_ops: int = 18, kinds=None):
    """`kinds` restricts the operations drawn (see the numbered branches of `_build`)."""
    target, values, leaves = _build(dev, seed, scale, n_ops, shadow=False, kinds=kinds)
    target.t.forward()
    target.t.backward()
    target.t.val().keep()
    outs = {"target": target.t.val()}
    for i, x in enumerate(values):
        v = x.t.val()
        if v is not None:
            v.keep()
            outs[f"v{i}"] = v
    for i, x in enumerate(leaves):
        try:
            outs[f"g{i}"] = x.t.grad()
        except RuntimeError:
            pass
    autodiff.execute()
    return {k: v.get() for k, v in outs.items()}


def shadow_model_program(seed: int, scale: int = 1, n_ops: int = 18, kinds=None):
    """name -> float64 numpy array of what `random_model_program` keeps (gradients only of leaves the target reaches)."""
    import torch
    target, values, leaves = _build(None, seed, scale, n_ops, shadow=True, kinds=kinds)
    target.s.backward()
    outs = {"target": target.s.detach().numpy()}
    for i, x in enumerate(values):
        outs[f"v{i}"] = x.s.detach().numpy()
    for i, x in enumerate(leaves):
        if x.s.requires_grad and x.s.grad is not None:
            outs[f"g{i}"] = x.s.grad.numpy()
    return outs
