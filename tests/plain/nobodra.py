"""Whole-sequence Nobodra forward, written out mechanism by mechanism with plain tensor operations.

No cache, no state carried between calls, no batching: every call recomputes one whole sequence, token loops where
the definition is a recurrence.  CPU tensors, in the dtype of the weights passed in (float64 in the tests).  Shares
nothing with the package: names of checkpoint tensors and config.json keys are read here on their own.

Notation: n tokens, width W; a layer's mixer has H heads, G key groups (head h reads group h // (H / G)), key size d,
value size e.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch


def scaled_unit_rms(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) * weight over the last dimension (eps under the root)."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * weight


def stream_norm(x: torch.Tensor, stored: torch.Tensor, eps: float) -> torch.Tensor:
    """The model's norm: the stored weight lies around zero and the factor is 1 + stored."""
    return scaled_unit_rms(x, 1.0 + stored, eps)


def swish(x: torch.Tensor) -> torch.Tensor:
    return x / (1.0 + torch.exp(-x))


def rotate_front(x: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """x [n, heads, d]: the first `dims` dims of every head rotated by the token's position, dim i paired with
    i + dims/2 and turned by the angle position * base^(-2i/dims); dims beyond pass unchanged."""
    n, half = x.shape[0], dims // 2
    rate = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=x.dtype)
    angle = torch.arange(n, dtype=x.dtype)[:, None, None] * rate
    first, second = x[..., :half], x[..., half:dims]
    return torch.cat((first * angle.cos() - second * angle.sin(), second * angle.cos() + first * angle.sin(), x[..., dims:]), -1)


def keys_as_values_attention(x, w_q, w_k, w_o, q_weight, k_weight, *, heads, groups, d, eps, scale, window=None, rot=None):
    """Grouped-query attention whose values are its keys as projected (before the per-head norm and the rotation).
    window: token i sees j with 0 <= i - j < window (None: every j <= i).  rot: (base, dims) or None."""
    n = x.shape[0]
    q = (x @ w_q.T).view(n, heads, d)
    k = (x @ w_k.T).view(n, groups, d)
    values = k
    q, k = scaled_unit_rms(q, q_weight, eps), scaled_unit_rms(k, k_weight, eps)
    if rot is not None:
        q, k = rotate_front(q, *rot), rotate_front(k, *rot)
    out = torch.zeros(n, heads, d, dtype=x.dtype)
    for h in range(heads):
        g = h // (heads // groups)
        for i in range(n):
            first = 0 if window is None else max(0, i - window + 1)
            scores = (k[first:i + 1, g] @ q[i, h]) * scale
            out[i, h] = torch.softmax(scores, 0) @ values[first:i + 1, g]
    return out.reshape(n, heads * d) @ w_o.T


def short_convolution(x: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """x [n, channels], taps [channels, t]: y[i, c] = sum_j taps[c, j] * x[i - (t - 1 - j), c], zero before the start."""
    n, t = x.shape[0], taps.shape[1]
    y = torch.zeros_like(x)
    for i in range(n):
        for j in range(t):
            source = i - (t - 1 - j)
            if source >= 0:
                y[i] += taps[:, j] * x[source]
    return y


def unit(x: torch.Tensor) -> torch.Tensor:
    return x / torch.sqrt(x.pow(2).sum(-1, keepdim=True) + 1e-6)


def gated_delta_rule(x, w, *, heads, groups, d, e, eps):
    """w: the mixer's tensors by their checkpoint names ('q', 'q.conv', 'A_log', ...).  Token by token and head by head:
    the memory M [d, e] is decayed, corrected towards the token's value along its key, and read with the query."""
    n = x.shape[0]
    q = swish(short_convolution(x @ w["q"].T, w["q.conv"])).view(n, groups, d)
    k = swish(short_convolution(x @ w["k"].T, w["k.conv"])).view(n, groups, d)
    v = swish(short_convolution(x @ w["v"].T, w["v.conv"])).view(n, heads, e)
    q, k = unit(q) / math.sqrt(d), unit(k)
    step = torch.sigmoid(x @ w["b"].T)
    decay = torch.exp(-torch.exp(w["A_log"]) * torch.nn.functional.softplus(x @ w["a"].T + w["dt_bias"]))
    gate = swish(x @ w["g"].T).view(n, heads, e)
    out = torch.zeros(n, heads, e, dtype=x.dtype)
    for h in range(heads):
        g = h // (heads // groups)
        memory = torch.zeros(d, e, dtype=x.dtype)
        for i in range(n):
            memory = decay[i, h] * memory
            correction = step[i, h] * (v[i, h] - memory.T @ k[i, g])
            memory = memory + torch.outer(k[i, g], correction)
            out[i, h] = memory.T @ q[i, g]
    out = scaled_unit_rms(out, w["norm"], eps) * gate
    return out.reshape(n, heads * e) @ w["o"].T


def routed_experts(x, router, bias, ups, downs, top, margins=None):
    """Per token: the `top` experts of largest router logit, weighted by the softmax over their logits alone; an
    expert is down(relu(up x)^2).  margins: a list that receives, per token, how far the last chosen logit lies
    above the first one left out."""
    logits = x @ router.T + bias
    out = torch.zeros_like(x)
    for i in range(x.shape[0]):
        ordered = torch.argsort(logits[i], descending=True, stable=True)
        chosen = ordered[:top]
        share = torch.softmax(logits[i, chosen], 0)
        if margins is not None:
            margins.append(float(logits[i, ordered[top - 1]] - logits[i, ordered[top]]) if top < len(ordered) else math.inf)
        for p, expert in zip(share, chosen.tolist()):
            out[i] += p * (torch.relu(ups[expert] @ x[i]).pow(2) @ downs[expert].T)
    return out


def forward(weights: dict, raw: dict, ids, margins=None) -> torch.Tensor:
    """Logits [n, vocab] of one sequence from its start; `raw` is the config.json content."""
    eps = raw["norm"]["eps"]
    x = weights["embed"][torch.as_tensor(ids)]
    for index, layer in enumerate(raw["layers"]):
        p, m = f"l{index}.", layer["mixer"]
        if layer["type"] == "attention":
            mask, rot = m.get("mask"), m.get("rot")
            mixed = keys_as_values_attention(
                x, weights[p + "mix.q"], weights[p + "mix.k"], weights[p + "mix.o"], weights[p + "mix.q.norm"], weights[p + "mix.k.norm"],
                heads=m["heads"], groups=m["kv_heads"], d=m["dim"], eps=eps, scale=m.get("scale", 1.0 / math.sqrt(m["dim"])),
                window=None if mask is None else mask["size"], rot=None if rot is None else (rot["base"], rot["dims"]))
        else:
            names = ("q", "k", "v", "q.conv", "k.conv", "v.conv", "b", "a", "A_log", "dt_bias", "g", "norm", "o")
            mixed = gated_delta_rule(x, {name: weights[p + "mix." + name] for name in names}, heads=m["heads"], groups=m["kv_heads"],
                                     d=m["dim"], e=m["vdim"], eps=eps)
        x = x + stream_norm(mixed, weights[p + "norm1"], eps)
        if layer["mlp"] is not None:
            count = layer["mlp"]["router"]["experts"]
            fed = routed_experts(x, weights[p + "mlp.router"], weights[p + "mlp.router.b"], [weights[f"{p}mlp.e{e}.up"] for e in range(count)],
                                 [weights[f"{p}mlp.e{e}.down"] for e in range(count)], layer["mlp"]["router"]["top"], margins)
            x = x + stream_norm(fed, weights[p + "norm2"], eps)
    return stream_norm(x, weights["final.norm"], eps) @ weights["head"].T


def load_model_dir(model_dir, dtype=torch.float64):
    from safetensors.torch import load_file

    model_dir = Path(model_dir)
    raw = json.loads((model_dir / "config.json").read_text())
    return raw, {name: t.to(dtype) for name, t in load_file(str(model_dir / "model.safetensors")).items()}
