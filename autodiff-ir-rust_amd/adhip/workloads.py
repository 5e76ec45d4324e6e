"""The five synthetic workloads the backend is measured and parity-tested on, written against the
caller-side API exactly as a user of the reference would write them.  Sizes are parameters: the
benchmark uses the full sizes, the parity tests the same programs at sizes a CPU oracle finishes
in seconds.

Every builder takes the device, installs it with `autodiff.set_device`, builds the graph, and
returns a `Workload` whose `.run()` executes it and whose `.outputs` maps names to `Value`s to
`get()` afterwards.  Inputs come from `numpy.random.default_rng(seed)`, float32.
"""
from __future__ import annotations

from typing import Callable, Dict, Optional

import numpy as np

from . import autodiff, nn
from .core import STATE, Tensor, Value, concat, constant


class Workload:
    def __init__(self, name: str, outputs: Dict[str, Value], inputs: Dict[str, np.ndarray],
                 algorithmic_bytes: Optional[float] = None, flops: Optional[float] = None,
                 unfused_bytes: Optional[float] = None):
        self.name = name
        self.outputs = outputs
        self.inputs = inputs
        # bytes one run has to move when every tensor the caller can observe is read or written exactly once and
        # nothing else touches memory (the figure throughput is quoted on)
        self.algorithmic_bytes = algorithmic_bytes
        # the same workload priced pass by pass (forward and backward as separate sweeps over the inputs): not a
        # bandwidth when divided by the time of a fused run, kept as a named secondary figure only
        self.unfused_bytes = unfused_bytes
        self.flops = flops

    def finish(self):
        """Append EX (what `autodiff.execute()` does first) and return (procedure, keep list)
        without running anything; used to compile a resident program."""
        from . import ir as IR
        if not STATE.irb.proc.main or not isinstance(STATE.irb.proc.main[-1], IR.EX):
            STATE.irb.add_cmd(IR.EX())
        return STATE.irb.proc, set(STATE.dep_tracker)

    def run(self):
        autodiff.execute()
        return self.get()

    def get(self):
        return {k: v.get() for k, v in self.outputs.items()}


def _uniform(rng, shape, lo=-1.0, hi=1.0):
    return rng.uniform(lo, hi, size=shape).astype(np.float32)


# ---- config 1: README MLP ---------------------------------------------------------------

def readme_mlp(dev, seed: int = 0) -> Workload:
    """x [2,5]; Linear(5,3, no bias) -> sigmoid -> Linear(3,2, bias); forward, backward of
    sum(output) (seed of ones), one SGD step with lr 0.1."""
    autodiff.set_device(dev)
    rng = np.random.default_rng(seed)
    w1 = _uniform(rng, (5, 3))
    w2 = _uniform(rng, (3, 2))
    b2 = _uniform(rng, (2,))
    xs = np.array([1, 2, 3, 4, 5, 6, 7, 8, 3.2, 6.3], dtype=np.float32)
    x = autodiff.tensor(xs, [2, 5])
    W1 = autodiff.tensor(w1, [5, 3])
    W2 = autodiff.tensor(w2, [3, 2])
    B2 = autodiff.tensor(b2, [2])
    net = nn.Sequential()
    net.insert(nn.LinearWithWeights(W1, None))
    net.insert(nn.Sigmoid())
    net.insert(nn.LinearWithWeights(W2, B2))
    opt = nn.SGD(net.params(), 0.1)
    y = net.f(x)
    y.forward()
    y.backward()
    grads = {"dW1": W1.grad(), "dW2": W2.grad(), "db2": B2.grad(), "dx": x.grad()}
    for g in grads.values():
        g.keep()
    y.val().keep()
    opt.step()
    outs = {"y": y.val(), "W1": W1.val(), "W2": W2.val(), "b2": B2.val()}
    outs.update(grads)
    return Workload("readme_mlp", outs, {"x": xs, "W1": w1, "W2": w2, "b2": b2})


# ---- config 2: fused element-wise + broadcast -------------------------------------------

def fused_elw(dev, rows: int = 8192, cols: int = 8192, seed: int = 0, backward: bool = True) -> Workload:
    """y = sigmoid(a*b + c + bias) - 0.5*exp(a) + sin(b)*cos(c), bias [cols] broadcast over rows;
    L = y.sum(0).sum(0); backward of L to a, b, c, bias."""
    autodiff.set_device(dev)
    rng = np.random.default_rng(seed)
    an, bn, cn = (_uniform(rng, (rows, cols)) for _ in range(3))
    biasn = _uniform(rng, (cols,))
    a = autodiff.tensor(an, [rows, cols])
    b = autodiff.tensor(bn, [rows, cols])
    c = autodiff.tensor(cn, [rows, cols])
    bias = autodiff.tensor(biasn, [cols])
    y = (a * b + c + bias).sigmoid() - 0.5 * a.exp() + b.sin() * c.cos()
    L = y.sum(0).sum(0)
    L.forward()
    y.val().keep()
    L.val().keep()
    outs = {"y": y.val(), "L": L.val()}
    n = rows * cols
    unfused = 4.0 * (4 * n + cols)          # forward on its own: read a,b,c,bias; write y
    fused = unfused + 4.0                   # ... and L
    if backward:
        L.backward()
        outs.update({"da": a.grad(), "db": b.grad(), "dc": c.grad(), "dbias": bias.grad()})
        unfused += 4.0 * (6 * n + 2 * cols)  # backward on its own: read a,b,c,bias again; write da,db,dc,dbias
        fused += 4.0 * (3 * n + cols)        # one pass: the inputs are read once, da,db,dc,dbias written
    return Workload("fused_elw", outs, {"a": an, "b": bn, "c": cn, "bias": biasn}, algorithmic_bytes=fused,
                    unfused_bytes=unfused)


# ---- config 3: reductions ---------------------------------------------------------------

def reductions(dev, rows: int = 16384, cols: int = 4096, seed: int = 0, backward: bool = True) -> Workload:
    """s0 = x.powf(2).sum(1); s1 = x.sum(0); s2 = (x*x).sum(1).sum(0); backward of each to x."""
    autodiff.set_device(dev)
    rng = np.random.default_rng(seed)
    xn = rng.standard_normal((rows, cols), dtype=np.float32)
    x = autodiff.tensor(xn, [rows, cols])
    s0 = x.powf(2.0).sum(1)
    s1 = x.sum(0)
    s2 = (x * x).sum(1).sum(0)
    outs = {}
    for name, s in (("s0", s0), ("s1", s1), ("s2", s2)):
        s.forward()
        s.val().keep()
        outs[name] = s.val()
    n = rows * cols
    small = 4.0 * (rows + cols + 1)
    unfused = 3 * 4.0 * n + small           # three reductions, x read once by each
    fused = 4.0 * n + small                 # one pass over x yields all three sums (s2 is the sum of s0)
    if backward:
        s0.backward()
        s1.backward()
        s2.backward()
        outs["dx"] = x.grad()
        unfused += 2 * 4.0 * n              # read x, write dx
        fused += 4.0 * n                    # as lowered: the one pass over x also writes dx (row and column sums ride along)
    return Workload("reductions", outs, {"x": xn}, algorithmic_bytes=fused, unfused_bytes=unfused)


# ---- config 4: dense MLP training -------------------------------------------------------

def mlp_train(dev, batch: int = 4096, dims=(4096, 4096, 4096, 1024), iters: int = 10, lr: float = 0.01,
              seed: int = 0) -> Workload:
    """Linear(d0,d1)+sigmoid, Linear(d1,d2)+sigmoid, Linear(d2,d3), all with bias; Xavier-uniform
    weights, biases U(-0.05,0.05); loss = mean((y-t)^2) composed from IR ops; forward + backward +
    SGD for `iters` iterations inside an IR for-loop."""
    autodiff.set_device(dev)
    autodiff.eager_dep_opt()  # read back only what is kept explicitly, as the reference's nn test does
    rng = np.random.default_rng(seed)
    xn = rng.standard_normal((batch, dims[0]), dtype=np.float32)
    tn = _uniform(rng, (batch, dims[-1]), 0.0, 1.0)
    inputs = {"x": xn, "t": tn}
    x = autodiff.tensor(xn, [batch, dims[0]])
    t = autodiff.tensor(tn, [batch, dims[-1]])
    net = nn.Sequential()
    weights = []
    for li in range(len(dims) - 1):
        fan_in, fan_out = dims[li], dims[li + 1]
        bound = np.sqrt(6.0 / (fan_in + fan_out))
        wn = _uniform(rng, (fan_in, fan_out), -bound, bound)
        bn = _uniform(rng, (fan_out,), -0.05, 0.05)
        inputs[f"W{li}"] = wn
        inputs[f"b{li}"] = bn
        W = autodiff.tensor(wn, [fan_in, fan_out])
        B = autodiff.tensor(bn, [fan_out])
        weights.append((W, B))
        net.insert(nn.LinearWithWeights(W, B))
        if li + 2 < len(dims):
            net.insert(nn.Sigmoid())
    opt = nn.SGD(net.params(), lr)
    scale = 1.0 / float(batch * dims[-1])
    box = {}

    def body(_):
        y = net.f(x)
        d = y - t
        loss = (d * d).sum(1).sum(0) * scale
        opt.zero_grad()
        loss.forward()
        loss.backward()
        opt.step()
        box["loss"] = loss

    autodiff.ir_for(range(0, iters), body)
    loss = box["loss"]
    loss.val().keep()
    x.grad().keep()  # keeps the first layer's dX product alive, as in the flop count of the config
    outs = {"loss": loss.val(), "dx": x.grad()}
    for li, (W, B) in enumerate(weights):
        W.val().keep()
        B.val().keep()
        outs[f"W{li}"] = W.val()
        outs[f"b{li}"] = B.val()
    flops = 0.0
    for li in range(len(dims) - 1):
        flops += 3 * 2.0 * batch * dims[li] * dims[li + 1]  # forward, dX, dW
    return Workload("mlp_train", outs, inputs, flops=flops * iters)


# ---- config 5: tensor manipulation + data-dependent loop ---------------------------------

def manip_loop(dev, nb: int = 64, n1: int = 512, n2: int = 1024, n3: int = 256, lo: int = 128, hi: int = 896,
               max_iters: int = 50, seed: int = 0, snapshot_at: Optional[int] = None) -> Workload:
    """p [nb,n1,n2], q [nb,n2,n3], w [n1+n3]; r = concat(p.permute(0,2,1), q, dim=2)[:, lo:hi, :]
    .view([nb*(hi-lo), n1+n3]) * w; while not (r.sum(1) < 1).all() and i < max_iters:
    r -= 0.01 * r.sum(1)[:, None]."""
    autodiff.set_device(dev)
    rng = np.random.default_rng(seed)
    pn = _uniform(rng, (nb, n1, n2))
    qn = _uniform(rng, (nb, n2, n3))
    wn = _uniform(rng, (n1 + n3,))
    p = autodiff.tensor(pn, [nb, n1, n2])
    q = autodiff.tensor(qn, [nb, n2, n3])
    w = autodiff.tensor(wn, [n1 + n3])
    rows, width = nb * (hi - lo), n1 + n3
    gathered = concat([p.permute([0, 2, 1]), q], 2).r(range(lo, hi), 1).view([rows, width])
    g0 = gathered.contigious()           # the gather stage on its own (bit-exact check)
    g0.forward()
    g0.val().keep()
    r = gathered * w
    i = autodiff.scalar(0.0)
    limit = float(max_iters if snapshot_at is None else snapshot_at)
    not_done = 1.0 - r.sum(1).less_than(constant(1.0, [rows])).all()
    pred = not_done * i.less_than(constant(limit, [1]))
    r.forward()

    def body():
        nonlocal r, i
        rv = r.val().to_node()
        r -= 0.01 * rv.sum(1).unsqueeze(-1)
        i += 1.0

    autodiff.ir_while(pred, body)
    r.val().keep()
    outs = {"gathered": g0.val(), "r": r.val(), "i": i.val()}
    return Workload("manip_loop", outs, {"p": pn, "q": qn, "w": wn},
                    algorithmic_bytes=4.0 * 2 * rows * width)


# ---- a transformer encoder layer (the caller-side modules of reference src/nn/transformer.rs) ----------

def encoder_layer(dev, seq: int = 64, d_model: int = 32, heads: int = 4, ff_dim: int = 64, seed: int = 0,
                  backward: bool = True) -> Workload:
    """x [seq, d_model]; y = TransformerEncoderLayer(d_model, heads, ff_dim)(x); L = (y * r).sum(0).sum(0) with a fixed
    random r; backward to x and every parameter.  Weights are N(0, 1/fan_in) and passed in explicitly (the
    reference's `randn` is unseeded), so a restatement in another framework can use the same values."""
    autodiff.set_device(dev)
    rng = np.random.default_rng(seed)
    inputs: Dict[str, np.ndarray] = {}

    def mat(name, fan_in, fan_out):
        w = (rng.standard_normal((fan_in, fan_out)) / np.sqrt(fan_in)).astype(np.float32)
        inputs[name] = w
        return autodiff.tensor(w, [fan_in, fan_out])

    def vec(name, n):
        b = (0.1 * rng.standard_normal(n)).astype(np.float32)
        inputs[name] = b
        return autodiff.tensor(b, [n])

    layer = nn.TransformerEncoderLayer(d_model, heads, ff_dim)
    d_v = d_model // heads
    named = {}
    for h in range(heads):
        for kind, group in (("wq", layer.attention.wq), ("wk", layer.attention.wk), ("wv", layer.attention.wv)):
            group[h].w = mat(f"{kind}{h}", d_model, d_v)
            named[f"{kind}{h}"] = group[h].w
    layer.attention.wo.w = mat("wo", d_model, d_model)
    named["wo"] = layer.attention.wo.w
    layer.ffwd.w_expand.w = mat("w1", d_model, ff_dim)
    layer.ffwd.w_expand.b = vec("b1", ff_dim)
    layer.ffwd.w_contract.w = mat("w2", ff_dim, d_model)
    layer.ffwd.w_contract.b = vec("b2", d_model)
    named.update({"w1": layer.ffwd.w_expand.w, "b1": layer.ffwd.w_expand.b, "w2": layer.ffwd.w_contract.w,
                  "b2": layer.ffwd.w_contract.b, "ln1_scale": layer.layer_norm_att.scale,
                  "ln2_scale": layer.layer_norm_ffwd.scale})
    xn = rng.standard_normal((seq, d_model)).astype(np.float32)
    rn = rng.standard_normal((seq, d_model)).astype(np.float32)
    inputs["x"], inputs["r"] = xn, rn
    x = autodiff.tensor(xn, [seq, d_model])
    r = autodiff.tensor(rn, [seq, d_model])
    y = layer.f(x)
    L = (y * r).sum(0).sum(0)
    L.forward()
    y.val().keep()
    L.val().keep()
    outs = {"y": y.val(), "L": L.val()}
    if backward:
        L.backward()
        outs["dx"] = x.grad()
        for name, p in named.items():
            outs["d" + name] = p.grad()
        for v in outs.values():
            v.keep()
    # matmul flops: forward 2*M*N*K per product, backward twice that
    fl = 0.0
    fl += heads * 3 * 2.0 * seq * d_model * d_v            # q, k, v projections
    fl += heads * 2 * 2.0 * seq * seq * d_v                # scores and weighted values
    fl += 2.0 * seq * d_model * d_model                     # output projection
    fl += 2 * 2.0 * seq * d_model * ff_dim                  # feed-forward
    return Workload("encoder_layer", outs, inputs, flops=fl * (3.0 if backward else 1.0))


def attention_forward(dev, seq: int = 64, d_model: int = 64, heads: int = 4, seed: int = 0, scale_x: float = 1.0) -> Workload:
    """y = MultiHeadAttention(d_model, heads)(x), forward only (inference): per-head projections, attention, the
    heads concatenated, the output projection (reference src/nn/transformer.rs:34-99).  Weights N(0, 1/fan_in), passed
    in explicitly."""
    autodiff.set_device(dev)
    rng = np.random.default_rng(seed)
    inputs: Dict[str, np.ndarray] = {}
    mha = nn.MultiHeadAttention(d_model, heads)
    d_v = d_model // heads

    def mat(name, fan_in, fan_out):
        w = (rng.standard_normal((fan_in, fan_out)) / np.sqrt(fan_in)).astype(np.float32)
        inputs[name] = w
        return autodiff.tensor(w, [fan_in, fan_out])

    for h in range(heads):
        mha.wq[h].w = mat(f"wq{h}", d_model, d_v)
        mha.wk[h].w = mat(f"wk{h}", d_model, d_v)
        mha.wv[h].w = mat(f"wv{h}", d_model, d_v)
    mha.wo.w = mat("wo", d_model, d_model)
    xn = (scale_x * rng.standard_normal((seq, d_model))).astype(np.float32)
    inputs["x"] = xn
    x = autodiff.tensor(xn, [seq, d_model])
    y = mha.f(x)
    y.forward()
    y.val().keep()
    fl = heads * 3 * 2.0 * seq * d_model * d_v + heads * 2 * 2.0 * seq * seq * d_v + 2.0 * seq * d_model * d_model
    wl = Workload("attention_forward", {"y": y.val()}, inputs, flops=fl)
    wl.attention_flops = heads * 2 * 2.0 * seq * seq * d_v
    return wl


def encoder_train(dev, seq: int = 64, d_model: int = 32, heads: int = 4, ff_dim: int = 64, iters: int = 3,
                  lr: float = 0.05, seed: int = 0) -> Workload:
    """`iters` SGD steps on one TransformerEncoderLayer inside an IR for-loop: y = layer(x); loss = mean((y - t)^2);
    zero_grad, forward, backward, step.  Every weight is updated in place while the next iteration's products read
    it, which is what a training loop over the reference's modules does (src/tests/nn.rs:10-45 for the MLP)."""
    autodiff.set_device(dev)
    autodiff.eager_dep_opt()
    rng = np.random.default_rng(seed)
    inputs: Dict[str, np.ndarray] = {}
    layer = nn.TransformerEncoderLayer(d_model, heads, ff_dim)
    d_v = d_model // heads
    named = {}

    def mat(name, fan_in, fan_out):
        w = (rng.standard_normal((fan_in, fan_out)) / np.sqrt(fan_in)).astype(np.float32)
        inputs[name] = w
        named[name] = autodiff.tensor(w, [fan_in, fan_out])
        return named[name]

    def vec(name, n):
        b = (0.1 * rng.standard_normal(n)).astype(np.float32)
        inputs[name] = b
        named[name] = autodiff.tensor(b, [n])
        return named[name]

    for h in range(heads):
        for kind, group in (("wq", layer.attention.wq), ("wk", layer.attention.wk), ("wv", layer.attention.wv)):
            group[h].w = mat(f"{kind}{h}", d_model, d_v)
    layer.attention.wo.w = mat("wo", d_model, d_model)
    layer.ffwd.w_expand.w = mat("w1", d_model, ff_dim)
    layer.ffwd.w_expand.b = vec("b1", ff_dim)
    layer.ffwd.w_contract.w = mat("w2", ff_dim, d_model)
    layer.ffwd.w_contract.b = vec("b2", d_model)
    named["ln1_scale"] = layer.layer_norm_att.scale
    named["ln2_scale"] = layer.layer_norm_ffwd.scale
    xn = rng.standard_normal((seq, d_model)).astype(np.float32)
    tn = rng.standard_normal((seq, d_model)).astype(np.float32)
    inputs["x"], inputs["t"] = xn, tn
    x = autodiff.tensor(xn, [seq, d_model])
    t = autodiff.tensor(tn, [seq, d_model])
    opt = nn.SGD(list(named.values()), lr)
    scale = 1.0 / float(seq * d_model)
    box = {}

    def body(_):
        y = layer.f(x)
        d = y - t
        loss = (d * d).sum(1).sum(0) * scale
        opt.zero_grad()
        loss.forward()
        loss.backward()
        opt.step()
        box["loss"] = loss

    autodiff.ir_for(range(0, iters), body)
    outs = {"loss": box["loss"].val()}
    for name, p in named.items():
        outs[name] = p.val()
    for v in outs.values():
        v.keep()
    return Workload("encoder_train", outs, inputs)
