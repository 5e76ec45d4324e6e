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
        return x.exp() / x.exp().sum(self.dim)


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
