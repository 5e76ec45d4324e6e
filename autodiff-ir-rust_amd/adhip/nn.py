"""The `nn` compositions the device path is exercised with: Linear, Sequential, activations,
norms and SGD (reference src/nn/{linear,sequential,module}.rs, src/nn/activations/*.rs,
src/nn/norm/*.rs, src/nn/optimizers/sgd.rs).  All of them are compositions of graph ops."""
from __future__ import annotations

from typing import List, Optional

from . import autodiff
from .core import Tensor, constant, dot


class Module:
    def params(self) -> List[Tensor]:
        return []

    def f(self, x: Tensor) -> Tensor:
        raise NotImplementedError


class Linear(Module):
    """y = x . W (+ b); W is [in, out] (linear.rs:21-28)."""

    def __init__(self, inp: int, out: int, bias: bool):
        self.w = autodiff.randn([inp, out])
        self.b = autodiff.randn([out]) if bias else None

    def params(self):
        return [self.w, self.b] if self.b is not None else [self.w]

    def f(self, x: Tensor) -> Tensor:
        res = dot(x, self.w)
        if self.b is not None:
            res += self.b
        return res


class LinearWithWeights(Linear):
    def __init__(self, w: Tensor, b: Optional[Tensor]):
        if b is not None:
            assert b.dim()[0] == w.dim()[1], "weight dim [a,b] must match bias dim [b]"
        self.w = w
        self.b = b


class Sigmoid(Module):
    def f(self, x):
        return 1.0 / (1.0 + (-x).exp())


class ReLU(Module):
    def f(self, x):
        return x * x.more_than(constant(0.0, x.dim()))


class Softmax(Module):
    def __init__(self, dim: int):
        self.dim = dim

    def f(self, x):
        return x.softmax(self.dim)


class RMS(Module):
    """norm/rms.rs:15-19 (eps 1e-9, scale of ones)."""

    def __init__(self, d_model: int):
        self.scale = autodiff.ones([d_model])

    def params(self):
        return [self.scale]

    def f(self, x):
        eps = 1e-9
        var = x.pow2().mean(-1).unsqueeze(-1) + eps
        input_norm = x / var.sqrt()
        return self.scale * input_norm


class LayerNorm(Module):
    """norm/layer.rs:16-22 (biased variance, eps 1e-9)."""

    def __init__(self, d_model: int):
        self.scale = autodiff.ones([d_model])
        self.bias = autodiff.zeros([d_model])

    def params(self):
        return [self.scale]

    def f(self, x):
        eps = 1e-9
        y = (x - x.mean(-1).unsqueeze(-1)) / (x.var(-1, 0) + eps).sqrt().unsqueeze(-1)
        return y * self.scale + self.bias


class Sequential(Module):
    def __init__(self):
        self.n: List[Module] = []

    def insert(self, func: Module) -> None:
        self.n.append(func)

    def params(self):
        out: List[Tensor] = []
        for m in self.n:
            out.extend(m.params())
        return out

    def f(self, x):
        res = x
        for layer in self.n:
            res = layer.f(res)
        return res


class SGD:
    """p -= lr * grad, emitted per parameter as mul(lr), mul(-1), `+=` (sgd.rs:9-14)."""

    def __init__(self, m: List[Tensor], lr: float):
        self.n = m
        self.lr = float(lr)

    def step(self):
        for p in self.n:
            p -= self.lr * p.grad().to_node()
            p.forward()

    def zero_grad(self):
        for p in self.n:
            p.reset_grad()


# ---- attention / transformer encoder (reference src/nn/transformer.rs) ------------------------------
# Everything works on 2-D tensors [sequence, features]: DotProduct is 2-D in the IR.  `softmax` normalises along the
# given dim with the maximum subtracted first (core.Tensor.softmax, which also says where the reference's own
# composition differs).

def Attention(Q: Tensor, K: Tensor, V: Tensor, d_model: int) -> Tensor:
    """dot(softmax(dot(Q, K^T) / sqrt(d_model), -1), V)  (transformer.rs:10-18)."""
    import math
    return dot((dot(Q, K.t()) / math.sqrt(float(d_model))).softmax(-1), V)


def AttentionMasked(Q: Tensor, K: Tensor, V: Tensor, d_model: int, mask: Tensor) -> Tensor:
    """As Attention with the scaled scores multiplied by `mask` before the softmax (transformer.rs:21-30)."""
    import math
    return dot((dot(Q, K.t()) / math.sqrt(float(d_model)) * mask).softmax(-1), V)


class MultiHeadAttention(Module):
    """Per head its own Linear(d_model, d_model / heads, no bias) for query, key and value; heads concatenated on
    the last dim, then Linear(d_model, d_model, no bias) (transformer.rs:34-99)."""

    def __init__(self, d_model: int, num_heads: int, mask: Optional[Tensor] = None):
        assert d_model % num_heads == 0, "d_model must be divisible by num heads"
        d_v = d_model // num_heads
        self.wq = [Linear(d_model, d_v, False) for _ in range(num_heads)]
        self.wk = [Linear(d_model, d_v, False) for _ in range(num_heads)]
        self.wv = [Linear(d_model, d_v, False) for _ in range(num_heads)]
        self.wo = Linear(d_model, d_model, False)
        self.num_heads = num_heads
        self.d_model = d_model
        self.mask = mask

    def params(self):
        out: List[Tensor] = []
        for group in (self.wq, self.wk, self.wv):
            for lin in group:
                out.extend(lin.params())
        out.extend(self.wo.params())
        return out

    def f(self, query: Tensor, key: Optional[Tensor] = None, value: Optional[Tensor] = None) -> Tensor:
        key = query if key is None else key
        value = query if value is None else value
        heads = []
        for i in range(self.num_heads):
            q, k, v = self.wq[i].f(query), self.wk[i].f(key), self.wv[i].f(value)
            if self.mask is not None:
                heads.append(AttentionMasked(q, k, v, self.d_model, self.mask))
            else:
                heads.append(Attention(q, k, v, self.d_model))
        from .core import concat
        return self.wo.f(concat(heads, -1))


def MaskedMultiHeadAttention(d_model: int, num_heads: int, mask: Tensor) -> MultiHeadAttention:
    return MultiHeadAttention(d_model, num_heads, mask)


class AttentionFeedforward(Module):
    """Linear(d_model, inner, bias) then Linear(inner, d_model, bias), nothing in between (transformer.rs:130-155)."""

    def __init__(self, d_model: int, inner_dim: int):
        self.w_expand = Linear(d_model, inner_dim, True)
        self.w_contract = Linear(inner_dim, d_model, True)

    def params(self):
        return self.w_expand.params() + self.w_contract.params()

    def f(self, x):
        return self.w_contract.f(self.w_expand.f(x))


class TransformerEncoderLayer(Module):
    """y = LayerNorm(x + MHA(x, x, x)); LayerNorm(y + FF(y))  (transformer.rs:158-192)."""

    def __init__(self, d_model: int, num_heads: int, ff_dim: int):
        self.attention = MultiHeadAttention(d_model, num_heads)
        self.layer_norm_att = LayerNorm(d_model)
        self.layer_norm_ffwd = LayerNorm(d_model)
        self.ffwd = AttentionFeedforward(d_model, ff_dim)

    def params(self):
        return self.attention.params() + self.ffwd.params() + self.layer_norm_att.params() + self.layer_norm_ffwd.params()

    def f(self, x):
        y = self.layer_norm_att.f(x + self.attention.f(x, x, x))
        return self.layer_norm_ffwd.f(y + self.ffwd.f(y))


class TransformerEncoder(Module):
    def __init__(self, num_layers: int, d_model: int, num_heads: int, ff_dim: int):
        self.layers = Sequential()
        for _ in range(num_layers):
            self.layers.insert(TransformerEncoderLayer(d_model, num_heads, ff_dim))

    def params(self):
        return self.layers.params()

    def f(self, x):
        return self.layers.f(x)
