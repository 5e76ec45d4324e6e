"""Random IR programs with nested control flow, written directly as commands (not through the graph front end), for
differential testing of the device against the oracle.

What they stress: ids redefined inside loops and branches, in-place updates next to reads of the old value, views
taken before a loop and used inside it (late binding), sums and matmuls inside loop bodies, values that are only
conditionally rewritten, counted loops, data-dependent loops and branches.

Two families of tensors keep the comparison meaningful:
  * integer-valued ones (names k*): only additions, negations and multiplications by small integers, so every
    device computes them exactly; all predicates are derived from these, so both sides take the same path;
  * real-valued ones (names f*): contractive arithmetic (scaled sums, sines, exp2 of bounded arguments), compared
    with a tolerance.
Every id is created at the top level before any control flow, blocks only redefine existing ids, so no path reads an
undefined id."""
import numpy as np

from adhip import ir as IR

SHAPES = [[4, 6], [6, 4], [6], [4], [1]]


class _Gen:
    def __init__(self, seed, extended=False):
        self.extended = extended   # also draw row maxima, a softmax spelled in commands and a maximum of integers
        self.rng = np.random.default_rng(seed)
        self.n = 0
        self.counters = 0
        self.ints = {}    # id -> shape
        self.reals = {}
        self.top = []
        self.early_views = []   # [6,4] views of [4,6] tensors, defined before the first control command

    def fresh(self, prefix):
        self.n += 1
        return f"{prefix}{self.n}"

    def pick(self, pool, shape=None):
        c = [i for i, s in pool.items() if shape is None or s == shape]
        return c[int(self.rng.integers(len(c)))] if c else None

    def const(self, out, value, shape):
        cid = self.fresh("c")
        out.append(IR.CreateConstant(float(value), cid, list(shape)))
        return cid

    # ---- one straight-line command group appended to `out`
    def compute(self, out, depth):
        rng = self.rng
        kind = int(rng.integers(13 if self.extended else 10))
        if kind == 10:     # real: the largest element of every row of a [4,6], written to a [4]
            a = self.pick(self.reals, [4])
            b = self.pick(self.reals, [4, 6])
            out.append(IR.Max(a=b, res=a))
        elif kind == 11:   # real: softmax over the rows of a [4,6] spelled in commands (in place when a == b)
            a = self.pick(self.reals, [4, 6])
            b = self.pick(self.reals, [4, 6])
            m, mv, mb, n, d, e1, e, sm, r, rv, rb = (self.fresh("t") for _ in range(11))
            out += [IR.Max(a=b, res=m), IR.View(a=m, target_dim=[4, 1], res=mv), IR.Broadcast(a=mv, dim=1, r=6, res=mb),
                    IR.ElwMultiply(a=mb, b=self.const(out, -1.0, [4, 6]), res=n), IR.ElwAdd(a=b, b=n, res=d),
                    IR.ElwMultiply(a=d, b=self.const(out, 1.4426950408889634, [4, 6]), res=e1), IR.Exp2(a=e1, res=e),
                    IR.Sum(a=e, res=sm), IR.Recip(a=sm, res=r), IR.View(a=r, target_dim=[4, 1], res=rv),
                    IR.Broadcast(a=rv, dim=1, r=6, res=rb), IR.ElwMultiply(a=e, b=rb, res=a)]
        elif kind == 12:   # int: scalar k[1] = the largest element of a [4] (exact)
            a = self.pick(self.ints, [1])
            b = self.pick(self.ints, [4])
            v = self.fresh("t")
            out += [IR.View(a=b, target_dim=[1, 4], res=v), IR.Max(a=v, res=a)]
        elif kind == 0:    # real: a = 0.5 * (b + c)
            a = self.pick(self.reals)
            sh = self.reals[a]
            b, c = self.pick(self.reals, sh), self.pick(self.reals, sh)
            t = self.fresh("t")
            out += [IR.ElwAdd(a=b, b=c, res=t), IR.ElwMultiply(a=t, b=self.const(out, 0.5, sh), res=a)]
        elif kind == 1:    # real: a = sin(b) * c  (in place when a == b)
            a = self.pick(self.reals)
            sh = self.reals[a]
            b, c = self.pick(self.reals, sh), self.pick(self.reals, sh)
            t = self.fresh("t")
            out += [IR.Sin(a=b, res=t), IR.ElwMultiply(a=t, b=c, res=a)]
        elif kind == 2:    # real, in place: a += 0.25 * b ; a *= 0.5
            a = self.pick(self.reals)
            sh = self.reals[a]
            b = self.pick(self.reals, sh)
            t = self.fresh("t")
            out += [IR.ElwMultiply(a=b, b=self.const(out, 0.25, sh), res=t), IR.ElwAddEq(s=a, o=t),
                    IR.ElwMultiplyEq(s=a, o=self.const(out, 0.5, sh))]
        elif kind == 3:    # real: row sums of a [4,6] spread back over another [4,6] through broadcast
            a = self.pick(self.reals, [4, 6])
            b = self.pick(self.reals, [4, 6])
            s, v, w, t = self.fresh("t"), self.fresh("t"), self.fresh("t"), self.fresh("t")
            out += [IR.Sum(a=b, res=s), IR.View(a=s, target_dim=[4, 1], res=v), IR.Broadcast(a=v, dim=1, r=6, res=w),
                    IR.ElwMultiply(a=w, b=self.const(out, 1.0 / 8.0, [4, 6]), res=t), IR.ElwAdd(a=t, b=a, res=a),
                    IR.ElwMultiplyEq(s=a, o=self.const(out, 0.5, [4, 6]))]
        elif kind == 4:    # real: column sums via permute, written to a [6]
            a = self.pick(self.reals, [6])
            b = self.pick(self.reals, [4, 6])
            p, s = self.fresh("t"), self.fresh("t")
            out += [IR.Permute(a=b, p=[1, 0], res=p), IR.Sum(a=p, res=s),
                    IR.ElwMultiply(a=s, b=self.const(out, 0.25, [6]), res=a)]
        elif kind == 5:    # real: [4,6] x [6,4] -> [4,4] -> row sums -> [4]
            a = self.pick(self.reals, [4])
            x, y = self.pick(self.reals, [4, 6]), self.pick(self.reals, [6, 4])
            d, s = self.fresh("t"), self.fresh("t")
            out += [IR.DotProduct(a=x, b=y, res=d), IR.Sum(a=d, res=s),
                    IR.ElwMultiply(a=s, b=self.const(out, 1.0 / 32.0, [4]), res=a)]
        elif kind == 6:    # real: transposed copy between the two matrix shapes (out[i] = in[p[i]]), through a fresh
            a = self.pick(self.reals, [6, 4])   # view or through one that was taken before any control flow
            if self.early_views and rng.integers(2):
                p = self.early_views[int(rng.integers(len(self.early_views)))]
                out += [IR.ElwMultiply(a=p, b=self.const(out, 0.5, [6, 4]), res=a)]
            else:
                b = self.pick(self.reals, [4, 6])
                p = self.fresh("t")
                out += [IR.Permute(a=b, p=[1, 0], res=p), IR.Contigious(a=p, res=a)]
        elif kind == 7:    # int: a = b + c or a = -b or a += small
            a = self.pick(self.ints)
            sh = self.ints[a]
            r = int(rng.integers(3))
            if r == 0:
                out.append(IR.ElwAdd(a=self.pick(self.ints, sh), b=self.pick(self.ints, sh), res=a))
            elif r == 1:
                out.append(IR.ElwMultiply(a=self.pick(self.ints, sh), b=self.const(out, -1.0, sh), res=a))
            else:
                out.append(IR.ElwAddEq(s=a, o=self.const(out, float(rng.integers(-3, 4)), sh)))
        elif kind == 8:    # int: scalar k[1] = sum of a [4] (through a [1,4] view)
            a = self.pick(self.ints, [1])
            b = self.pick(self.ints, [4])
            v, s = self.fresh("t"), self.fresh("t")
            out += [IR.View(a=b, target_dim=[1, 4], res=v), IR.Sum(a=v, res=s), IR.ElwAdd(a=s, b=a, res=a)]
        else:              # int: a [4] += broadcast of a scalar
            a = self.pick(self.ints, [4])
            b = self.pick(self.ints, [1])
            w = self.fresh("t")
            out += [IR.Broadcast(a=b, dim=0, r=4, res=w), IR.ElwAddEq(s=a, o=w)]

    def predicate(self, out):
        """A [1] predicate (0/1) from an integer-valued scalar: k > c, k < c or k == c."""
        k = self.pick(self.ints, [1])
        t, p = self.fresh("t"), self.fresh("p")
        out.append(IR.ElwAdd(a=k, b=self.const(out, -float(self.rng.integers(-4, 5)), [1]), res=t))
        cmp = [IR.MoreZero, IR.LessZero, IR.EqualZero][int(self.rng.integers(3))]
        out.append(cmp(a=t, res=p))
        return p

    def block(self, out, depth, n_cmds):
        for _ in range(n_cmds):
            r = int(self.rng.integers(10))
            if depth < 2 and r == 0:
                self.loop(out, depth, counted=True)
            elif depth < 2 and r == 1:
                self.loop(out, depth, counted=False)
            elif depth < 3 and r == 2:
                self.branch(out, depth)
            else:
                self.compute(out, depth)

    def loop(self, out, depth, counted):
        """Trip count 0..3.  Counted: the `x += 1; t = x + (-n); c = t < 0` shape of the front end's for-loop.
        Otherwise the predicate is the product of that comparison and a data-dependent one."""
        self.counters += 1
        i, t, c = f"i{self.counters}", f"it{self.counters}", f"ic{self.counters}"
        n = int(self.rng.integers(0, 4))
        self.top.append(IR.CreateMat(np.zeros(1, np.float32), [1], i))
        body = []
        self.block(body, depth + 1, int(self.rng.integers(1, 4)))

        def head(dst):
            dst.append(IR.ElwAdd(a=i, b=self.const(dst, -float(n), [1]), res=t))
            dst.append(IR.LessZero(a=t, res=c))
        out.append(IR.ElwMultiplyEq(s=i, o=self.const(out, 0.0, [1])))   # the counter restarts each time the loop is met
        head(out)
        cond = c
        body.append(IR.ElwAddEq(s=i, o=self.const(body, 1.0, [1])))
        head(body)
        if not counted:
            cond = f"iw{self.counters}"
            k = self.pick(self.ints, [1])
            lim = float(self.rng.integers(0, 12))

            def data_pred(dst):
                tt, pp = self.fresh("t"), self.fresh("p")
                dst.append(IR.ElwAdd(a=k, b=self.const(dst, -lim, [1]), res=tt))
                dst.append(IR.LessZero(a=tt, res=pp))
                dst.append(IR.ElwMultiply(a=c, b=pp, res=cond))
            data_pred(out)
            data_pred(body)
        out.append(IR.While(conditional_var=cond, block=IR.IRProcedure(f"loop{self.counters}", body)))

    def branch(self, out, depth):
        arms = []
        for _ in range(int(self.rng.integers(1, 3))):
            p = self.predicate(out)
            body = []
            self.block(body, depth + 1, int(self.rng.integers(1, 3)))
            arms.append((p, IR.IRProcedure(self.fresh("arm"), body)))
        else_proc = None
        if self.rng.integers(2):
            body = []
            self.block(body, depth + 1, int(self.rng.integers(1, 3)))
            else_proc = IR.IRProcedure(self.fresh("else"), body)
        out.append(IR.If(conditions=arms, else_proc=else_proc))


def random_control_program(seed: int, extended: bool = False):
    """Returns (procedure, keep list, names of the integer-valued ids).  `extended` adds row maxima, a softmax spelled in
    commands and integer maxima to the operations drawn (the plain form keeps the programs of its seeds as they were)."""
    g = _Gen(seed, extended)
    rng = g.rng
    for sh in SHAPES:
        for _ in range(2):
            rid = g.fresh("f")
            g.reals[rid] = sh
            g.top.append(IR.CreateMat(rng.uniform(-1.0, 1.0, int(np.prod(sh))).astype(np.float32), list(sh), rid))
    for sh in ([4], [4], [1], [1], [1]):
        kid = g.fresh("k")
        g.ints[kid] = sh
        g.top.append(IR.CreateMat(rng.integers(-3, 4, int(np.prod(sh))).astype(np.float32), list(sh), kid))
    # views taken before any control flow; blocks read them after their sources changed (views bind late)
    for rid in [i for i, sh in g.reals.items() if sh == [4, 6]]:
        v = g.fresh("v")
        g.top.append(IR.Permute(a=rid, p=[1, 0], res=v))
        g.early_views.append(v)
    main = []
    g.block(main, 0, int(rng.integers(6, 12)))
    keep = sorted(list(g.reals) + list(g.ints) + [f"i{j + 1}" for j in range(g.counters)])
    proc = IR.IRProcedure("main", g.top + main + [IR.EX()])
    return proc, keep, sorted(g.ints)


def random_epilogue_program(seed: int):
    """Straight-line programs around 64x64 matrix products (large enough for the matrix-core kernel) and row sums,
    with element-wise consumers placed at random distances after their producer and in-place updates of the same
    tensors in between: the cases in which a consumer may or may not be moved up into its producer's kernel.
    Returns (procedure, keep list)."""
    rng = np.random.default_rng(seed)
    n = 64
    cmds, mats, vecs = [], [], []
    for i in range(4):
        cmds.append(IR.CreateMat((rng.standard_normal(n * n) / 8).astype(np.float32), [n, n], f"m{i}"))
        mats.append(f"m{i}")
    for i in range(2):
        cmds.append(IR.CreateMat(rng.standard_normal(n).astype(np.float32), [n], f"v{i}"))
        vecs.append(f"v{i}")
    cnt = [0]

    def fresh(p):
        cnt[0] += 1
        return f"{p}{cnt[0]}"

    def const(v, shape):
        c = fresh("c")
        cmds.append(IR.CreateConstant(float(v), c, list(shape)))
        return c

    pending = []   # (kind, producer id) whose consumer has not been emitted yet
    for _ in range(int(rng.integers(8, 14))):
        r = int(rng.integers(9))
        pick = lambda pool: pool[int(rng.integers(len(pool)))]  # noqa: E731
        if r == 0:      # product
            d = fresh("d")
            a, b = pick(mats), pick(mats)
            if rng.integers(2):
                t = fresh("t")
                cmds.append(IR.Permute(a=b, p=[1, 0], res=t))
                b = t
            cmds.append(IR.DotProduct(a=a, b=b, res=d))
            pending.append(("mat", d))
        elif r == 1:    # row sums
            s = fresh("s")
            cmds.append(IR.Sum(a=pick(mats), res=s))
            pending.append(("vec", s))
        elif r in (2, 7, 8) and pending:   # consumer of an earlier producer: in-place update of a tensor or a new value
            kind, p = pending.pop(int(rng.integers(len(pending))))
            pool, shape = (mats, [n, n]) if kind == "mat" else (vecs, [n])
            t = fresh("t")
            cmds.append(IR.ElwMultiply(a=p, b=const(-0.125, shape), res=t))
            if rng.integers(2):
                cmds.append(IR.ElwAddEq(s=pick(pool), o=t))
            else:
                y = fresh("y")
                cmds += [IR.ElwAdd(a=t, b=pick(pool), res=y), IR.Sin(a=y, res=pick(pool))]
        elif r == 3:    # in-place scaling of a matrix (a write between producers and consumers)
            cmds.append(IR.ElwMultiplyEq(s=pick(mats), o=const(0.5, [n, n])))
        elif r == 4:    # matrix = matrix + matrix^T
            t = fresh("t")
            cmds += [IR.Permute(a=pick(mats), p=[1, 0], res=t), IR.ElwAdd(a=pick(mats), b=t, res=pick(mats))]
        elif r == 5:    # vector broadcast over a matrix, in place
            t, w = fresh("t"), fresh("t")
            cmds += [IR.View(a=pick(vecs), target_dim=[1, n], res=t), IR.Broadcast(a=t, dim=0, r=n, res=w),
                     IR.ElwAddEq(s=pick(mats), o=w)]
        else:           # vector update
            cmds.append(IR.ElwAddEq(s=pick(vecs), o=pick(vecs)))
            cmds.append(IR.ElwMultiplyEq(s=vecs[0], o=const(0.5, [n])))
    keep = mats + vecs + [p for _, p in pending]
    return IR.IRProcedure("main", cmds + [IR.EX()]), keep


def random_grouped_products_program(seed: int):
    """Many independent matrix products of one shape, the way multi-head attention issues them: per-head weights
    that are slices of one packed tensor (so the operands differ only by an offset), element-wise work between two
    levels of products, transposed operands, sums over the heads, and a rotation `w[h] = x . w[h+1]` in which every
    product overwrites a matrix that another product of the same level still reads.  Sizes are large enough for the
    matrix-core kernel, with aligned and unaligned variants and two with an inner dimension long enough to be cut
    into ranges.  Returns (procedure, keep list)."""
    rng = np.random.default_rng(1000 + seed)
    heads = int(rng.integers(2, 21))
    M, N, K = [(64, 64, 64), (128, 64, 96), (72, 80, 66), (96, 32, 160), (64, 128, 64), (64, 64, 512), (72, 40, 530)][seed % 7]
    cmds, keep = [], []

    def mat(name, shape, scale=1.0):
        cmds.append(IR.CreateMat((rng.standard_normal(int(np.prod(shape))) * scale).astype(np.float32), list(shape), name))
        return name

    x = mat("x", [M, K])
    packing = int(rng.integers(3))
    w = []
    if packing == 0:      # [heads, K, N]: dense slices at an offset
        mat("wp", [heads, K, N], K ** -0.5)
        for h in range(heads):
            cmds.append(IR.Index(a="wp", index=h, dim=0, res=f"w{h}"))
            w.append(f"w{h}")
    elif packing == 1:    # [K, heads, N]: strided slices at an offset
        mat("wp", [K, heads, N], K ** -0.5)
        for h in range(heads):
            cmds.append(IR.Index(a="wp", index=h, dim=1, res=f"w{h}"))
            w.append(f"w{h}")
    else:                 # separate matrices
        for h in range(heads):
            w.append(mat(f"w{h}", [K, N], K ** -0.5))
    # level 1: s[h] = x . w[h]
    s = []
    for h in range(heads):
        cmds.append(IR.DotProduct(a=x, b=w[h], res=f"s{h}"))
        s.append(f"s{h}")
        if rng.integers(3) == 0:
            keep.append(f"s{h}")
    second = int(rng.integers(3))
    if second == 0:
        # level 2 behind element-wise work: g[h] = sin(s[h])^T . x, then the sum over the heads
        for h in range(heads):
            cmds += [IR.Sin(a=s[h], res=f"u{h}"), IR.Permute(a=f"u{h}", p=[1, 0], res=f"ut{h}"),
                     IR.DotProduct(a=f"ut{h}", b=x, res=f"g{h}")]
        cmds.append(IR.CreateConstant(0.0, "acc", [N, K]))
        for h in range(heads):
            cmds.append(IR.ElwAddEq(s="acc", o=f"g{h}"))
        keep += ["acc", f"g{heads - 1}"]
    elif second == 1:
        # level 2 on transposed weights: dx = sum over h of s[h] . w[h]^T
        cmds.append(IR.CreateConstant(0.0, "dx", [M, K]))
        for h in range(heads):
            cmds += [IR.Permute(a=w[h], p=[1, 0], res=f"wt{h}"), IR.DotProduct(a=s[h], b=f"wt{h}", res=f"d{h}"),
                     IR.ElwAddEq(s="dx", o=f"d{h}")]
        keep += ["dx", "d0"]
    else:
        keep.append(s[0])
    if M == N == K:
        # rotation over square matrices: every product reads the old contents of the matrix the next one overwrites
        r = [mat(f"r{h}", [K, K], K ** -0.5) for h in range(heads)]
        for h in range(heads - 1):
            cmds.append(IR.DotProduct(a=x, b=r[h + 1], res=r[h]))
        cmds.append(IR.DotProduct(a=x, b=r[0], res=r[heads - 1]))   # ... and one that depends on a new value
        keep += r
    return IR.IRProcedure("main", cmds + [IR.EX()]), sorted(set(keep))


def random_layered_program(seed: int):
    """The same short chain of reductions and element-wise passes applied to many tensors of one shape, one tensor
    after the other, as a model with several heads or several same-sized layers does: the kernels of the chains are
    the same code on other buffers, which the device may run as block layers of shared launches.  Chains read
    slices of packed tensors and separate tensors, some results feed an accumulation across the chains, and some
    chains update their input in place (those must keep their place in the order).  Returns (procedure, keep)."""
    rng = np.random.default_rng(5000 + seed)
    heads = int(rng.integers(2, 24))
    R, C = [(64, 128), (33, 20), (256, 64), (128, 256), (7, 300)][seed % 5]
    cmds, keep = [], []
    packed = bool(rng.integers(2))
    if packed:
        cmds.append(IR.CreateMat(rng.uniform(-1, 1, heads * R * C).astype(np.float32), [heads, R, C], "xp"))
    xs = []
    for h in range(heads):
        if packed:
            cmds.append(IR.Index(a="xp", index=h, dim=0, res=f"x{h}"))
        else:
            cmds.append(IR.CreateMat(rng.uniform(-1, 1, R * C).astype(np.float32), [R, C], f"x{h}"))
        xs.append(f"x{h}")
    cmds.append(IR.CreateMat(rng.uniform(-1, 1, R * C).astype(np.float32), [R, C], "shared"))
    cmds.append(IR.CreateConstant(0.0, "acc", [R, C]))
    chain = int(rng.integers(3))
    for h in range(heads):
        x = xs[h]
        if chain == 0:
            # softmax-like: e = exp2(x); n = rowsum(e); p = e * (1/n broadcast over the columns)
            cmds += [IR.Exp2(a=x, res=f"e{h}"), IR.Sum(a=f"e{h}", res=f"n{h}"), IR.Recip(a=f"n{h}", res=f"i{h}"),
                     IR.View(a=f"i{h}", target_dim=[R, 1], res=f"iv{h}"), IR.Broadcast(a=f"iv{h}", dim=1, r=C, res=f"ib{h}"),
                     IR.ElwMultiply(a=f"e{h}", b=f"ib{h}", res=f"p{h}")]
        elif chain == 1:
            # column statistics: m = colsum(x * shared); p = sin(x) + m broadcast over the rows
            cmds += [IR.ElwMultiply(a=x, b="shared", res=f"t{h}"), IR.Permute(a=f"t{h}", p=[1, 0], res=f"tt{h}"),
                     IR.Sum(a=f"tt{h}", res=f"n{h}"), IR.View(a=f"n{h}", target_dim=[1, C], res=f"nv{h}"),
                     IR.Broadcast(a=f"nv{h}", dim=0, r=R, res=f"nb{h}"), IR.Sin(a=x, res=f"s{h}"),
                     IR.ElwAdd(a=f"s{h}", b=f"nb{h}", res=f"p{h}")]
        else:
            # two reductions in a row: n = rowsum(x * x); total = sum(n); p = x / total  (positive terms: a total that
            # cancels to almost nothing would carry the rounding of the whole sum)
            cmds += [IR.ElwMultiply(a=x, b=x, res=f"q{h}"), IR.Sum(a=f"q{h}", res=f"n{h}"), IR.View(a=f"n{h}", target_dim=[1, R], res=f"nr{h}"),
                     IR.Sum(a=f"nr{h}", res=f"gs{h}"), IR.Recip(a=f"gs{h}", res=f"g{h}"), IR.View(a=f"g{h}", target_dim=[1, 1], res=f"gv{h}"),
                     IR.Broadcast(a=f"gv{h}", dim=0, r=R, res=f"gb0{h}"), IR.Broadcast(a=f"gb0{h}", dim=1, r=C, res=f"gb{h}"),
                     IR.ElwMultiply(a=x, b=f"gb{h}", res=f"p{h}")]
        r = int(rng.integers(5))
        if r == 0 and not packed:
            cmds.append(IR.ElwAddEq(s=x, o=f"p{h}"))          # in-place update of this chain's input
            keep.append(x)
        elif r == 1:
            cmds.append(IR.ElwAddEq(s="acc", o=f"p{h}"))      # accumulation across the chains
        elif r == 2 and h + 1 < heads and not packed:
            cmds.append(IR.ElwAddEq(s=xs[h + 1], o=f"p{h}"))  # the next chain depends on this one
        elif r == 3:
            keep.append(f"n{h}")
        keep.append(f"p{h}")
    keep.append("acc")
    return IR.IRProcedure("main", cmds + [IR.EX()]), sorted(set(keep))
