"""A float64 restatement of `workloads.encoder_layer` in torch (CPU autograd), used to check the oracle and the
device on a whole encoder layer.  It restates the reference's compositions: attention with a softmax over the last
dim (the evident intent of reference src/nn/activations/softmax.rs:28-30, whose own broadcast divides by the wrong
row's sum) and its LayerNorm (biased variance, eps 1e-9, scale trainable, bias fixed at zero)."""
import math

import torch


def encoder_layer_reference(inputs, heads):
    t = {k: torch.tensor(v, dtype=torch.float64, requires_grad=True) for k, v in inputs.items()}
    x, r = t["x"], t["r"]
    seq, d_model = x.shape

    def softmax_ref(s):
        return torch.softmax(s, -1)

    def layer_norm(v, scale):
        mean = v.mean(-1, keepdim=True)
        var = ((v - mean) ** 2).sum(-1) / v.shape[-1]
        return (v - mean) / torch.sqrt(var + 1e-9).unsqueeze(-1) * scale

    ln1 = torch.ones(d_model, dtype=torch.float64, requires_grad=True)
    ln2 = torch.ones(d_model, dtype=torch.float64, requires_grad=True)
    outs = []
    for h in range(heads):
        q, k, v = x @ t[f"wq{h}"], x @ t[f"wk{h}"], x @ t[f"wv{h}"]
        outs.append(softmax_ref(q @ k.T / math.sqrt(float(d_model))) @ v)
    att = torch.cat(outs, -1) @ t["wo"]
    y1 = layer_norm(x + att, ln1)
    ff = (y1 @ t["w1"] + t["b1"]) @ t["w2"] + t["b2"]
    y = layer_norm(y1 + ff, ln2)
    L = (y * r).sum()
    L.backward()
    res = {"y": y.detach().numpy(), "L": L.detach().numpy().reshape(1), "dx": x.grad.numpy(),
           "dln1_scale": ln1.grad.numpy(), "dln2_scale": ln2.grad.numpy()}
    for name in inputs:
        if name not in ("x", "r"):
            res["d" + name] = t[name].grad.numpy()
    return res
