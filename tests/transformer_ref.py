"""Independent fp32 numpy restatement of the config 4 encoder block, written from the mathematics (LayerNorm,
scaled dot-product attention with softmax, tanh-GELU feed-forward, residual adds), not from the operator list:
it pins the graph description and the oracle's floating-point operators against a library computation."""
import re

import numpy as np


def constants_in_order(spec):
    groups = {"gamma": [], "beta": [], "w": [], "b": [], "c": []}
    for name, value in spec.consts.items():
        key = re.match(r"[a-z_]+", name).group(0)
        groups[key].append(np.asarray(value, dtype=np.float32))
    return groups


def encoder_block_fp32(spec, x, heads):
    g = constants_in_order(spec)
    w, b = g["w"], g["b"]  # q, k, v, out, ffn1, ffn2
    x = x.astype(np.float32)
    B, S, D = x.shape
    dh = D // heads

    def layer_norm(t, gamma, beta):
        mu = t.mean(axis=2, keepdims=True)
        var = ((t - mu) ** 2).mean(axis=2, keepdims=True)
        return (t - mu) / np.sqrt(var + 1e-3) * gamma + beta

    def linear(t, i):
        return t @ w[i][0] + b[i][0]

    y = layer_norm(x, g["gamma"][0], g["beta"][0]).reshape(B * S, D)
    split = lambda t: t.reshape(B, S, heads, dh).transpose(0, 2, 1, 3)  # [B, H, S, dh]
    q, k, v = split(linear(y, 0)), split(linear(y, 1)), split(linear(y, 2))
    scores = (q @ k.transpose(0, 1, 3, 2)) / np.sqrt(dh)
    scores = scores - scores.max(axis=3, keepdims=True)
    p = np.exp(scores)
    p = p / p.sum(axis=3, keepdims=True)
    ctx = (p @ v).transpose(0, 2, 1, 3).reshape(B * S, D)
    x1 = x + linear(ctx, 3).reshape(B, S, D)
    y2 = layer_norm(x1, g["gamma"][1], g["beta"][1]).reshape(B * S, D)
    h = linear(y2, 4)
    gelu = 0.5 * h * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (h + 0.044715 * h ** 3)))
    return x1 + linear(gelu, 5).reshape(B, S, D)
