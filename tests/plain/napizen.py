"""Whole-sequence Napizen forward, written out mechanism by mechanism with plain tensor operations.

No cache, no batching: every call recomputes one whole sequence, with loops over heads, tokens and experts where the
definition has them.  CPU tensors in the dtype of the weights passed in (float64 in the tests).  Shares nothing with the
package: names of checkpoint tensors and config.json keys are read here on their own, and a head's keys and values are
made for every position as the definition has them (the package never makes them).

Notation: n tokens, width W; a mixer has H heads, a head d plain and r rotated query/key dims and values of e dims, and
every position a latent row of c values.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x divided by its root mean square over the last dimension (eps under the root)."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def centred_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """(x - mean) / sqrt(mean of squared deviations + eps) * weight: a layer norm with a weight and no bias."""
    off = x - x.mean(-1, keepdim=True)
    return off / torch.sqrt(off.pow(2).mean(-1, keepdim=True) + eps) * weight


def swish(x: torch.Tensor) -> torch.Tensor:
    return x / (1.0 + torch.exp(-x))


def pair_rates(rot: dict) -> tuple[list, float]:
    """(turning rate of each pair, factor on cos and sin) for rot = {base, dims, scaling?}."""
    dims, base = rot["dims"], rot["base"]
    rates = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    s = rot.get("scaling")
    if s is None:
        return rates, 1.0

    def pair_turning(times):      # the (fractional) pair that turns `times` times over the original context
        return dims * math.log(s["original"] / (2.0 * math.pi * times)) / (2.0 * math.log(base))

    lo, hi = max(math.floor(pair_turning(s["fast"])), 0), min(math.ceil(pair_turning(s["slow"])), dims - 1)
    out = []
    for i, rate in enumerate(rates):
        blend = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(rate / s["factor"] * blend + rate * (1.0 - blend))
    return out, 0.1 * math.log(s["factor"]) + 1.0


def turn_pairs(x: torch.Tensor, rot: dict, first_position: int = 0) -> torch.Tensor:
    """x [n, ..., dims]: dims 2i and 2i + 1 of the last dimension are a pair, turned by position * rate_i."""
    rates, factor = pair_rates(rot)
    out = torch.empty_like(x)
    for token in range(x.shape[0]):
        for i, rate in enumerate(rates):
            angle = (first_position + token) * rate
            c, s = math.cos(angle) * factor, math.sin(angle) * factor
            u, v = x[token, ..., 2 * i], x[token, ..., 2 * i + 1]
            out[token, ..., 2 * i], out[token, ..., 2 * i + 1] = u * c - v * s, v * c + u * s
    return out


def latent_attention(x, w, m: dict, eps: float, weights_out: list | None = None) -> torch.Tensor:
    """The mixer on x [n, W]; w: its tensors by their short names (q, dkv, dkv.norm, uk, uv, sink, g, o); m: its config."""
    n, heads, d, r, e, c = x.shape[0], m["heads"], m["dim"], m.get("rot_dim", 0), m["vdim"], m["kv_rank"]
    q = (x @ w["q"].T).view(n, heads, d + r)
    down = x @ w["dkv"].T
    latent = unit_rms(down[:, :c], eps) * w["dkv.norm"]
    shared = down[:, c:]
    q_plain, q_turned = q[..., :d], q[..., d:]
    if r:
        q_turned, shared = turn_pairs(q_turned, m["rot"]), turn_pairs(shared, m["rot"])
    scale = m["scale"] if m.get("scale") is not None else 1.0 / math.sqrt(d + r)
    gate = torch.sigmoid(x @ w["g"].T)
    out = torch.zeros(n, heads, e, dtype=x.dtype)
    for h in range(heads):
        keys = latent @ w["uk"][h * d:(h + 1) * d].T          # [n, d]
        values = latent @ w["uv"][h * e:(h + 1) * e].T        # [n, e]
        for i in range(n):
            scores = (keys[:i + 1] @ q_plain[i, h] + shared[:i + 1] @ q_turned[i, h]) * scale
            top = max(float(scores.max()), float(w["sink"][h]))
            raised = torch.exp(scores - top)
            share = raised / (raised.sum() + math.exp(float(w["sink"][h]) - top))
            if weights_out is not None:
                weights_out.append((h, i, share))
            out[i, h] = gate[i, h] * (share @ values[:i + 1])
    return out.reshape(n, heads * e) @ w["o"].T


def gated_ff(x, gate, up, down) -> torch.Tensor:
    return (swish(x @ gate.T) * (x @ up.T)) @ down.T


def choose_experts(logits: torch.Tensor, correction: torch.Tensor, router: dict, margins: list | None = None):
    """Per token: (chosen experts, their weights).  margins: per token, how far the last chosen choice score lies
    above the best one left out, and (with groups) the last kept group above the best one dropped."""
    count, top = router["experts"], router["top"]
    chosen, shares = [], []
    for t in range(logits.shape[0]):
        score = torch.sigmoid(logits[t])
        choice = score + correction
        allowed = [True] * count
        margin = math.inf
        groups = router.get("groups")
        if groups is not None and groups["keep"] < groups["count"]:
            per = count // groups["count"]
            totals = []
            for g in range(groups["count"]):
                inside = sorted((float(choice[e]) for e in range(g * per, (g + 1) * per)), reverse=True)
                totals.append(sum(inside[:2]))
            order = sorted(range(groups["count"]), key=lambda g: (-totals[g], g))
            kept = set(order[:groups["keep"]])
            margin = totals[order[groups["keep"] - 1]] - totals[order[groups["keep"]]]
            allowed = [e // per in kept for e in range(count)]
        ranked = sorted((e for e in range(count) if allowed[e]), key=lambda e: (-float(choice[e]), e))
        picked = ranked[:top]
        if len(ranked) > top:
            margin = min(margin, float(choice[ranked[top - 1]] - choice[ranked[top]]))
        total = sum(float(score[e]) for e in picked) + 1e-20
        chosen.append(picked)
        shares.append([float(score[e]) / total * router.get("scale", 1.0) for e in picked])
        if margins is not None:
            margins.append(margin)
    return chosen, shares


def routed_ff(x, w, mlp: dict, margins: list | None = None) -> torch.Tensor:
    """w: router, correction, e<j>.gate / .up / .down."""
    chosen, shares = choose_experts(x @ w["router"].T, w["correction"], mlp["router"], margins)
    out = torch.zeros_like(x)
    for t in range(x.shape[0]):
        for e, share in zip(chosen[t], shares[t]):
            out[t] += share * gated_ff(x[t:t + 1], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"])[0]
    return out


def under(weights: dict, prefix: str) -> dict:
    return {name[len(prefix):]: t for name, t in weights.items() if name.startswith(prefix)}


def forward(weights: dict, raw: dict, ids, streams: list | None = None) -> torch.Tensor:
    """Logits [n, vocab] of the whole sequence `ids`; streams: receives the stream after every layer."""
    eps, alpha = raw["norm"]["eps"], raw.get("postln_alpha", 1.0)
    x = weights["embed"][torch.as_tensor(ids, dtype=torch.long)] * (raw.get("embedding") or {}).get("scale", 1.0)
    for index, layer in enumerate(raw["layers"]):
        w = under(weights, f"l{index}.")
        x = centred_norm(alpha * x + latent_attention(x, under(w, "mix."), layer["mixer"], eps), w["norm1"], eps)
        mlp = layer["mlp"]
        if mlp is not None:
            f = under(w, "mlp.")
            y = gated_ff(x, f["gate"], f["up"], f["down"]) if mlp["kind"] == "dense" else routed_ff(x, f, mlp)
            x = centred_norm(alpha * x + y, w["norm2"], eps)
        elif "norm2" in w:          # a layer without feed-forward whose second norm is stored all the same: nothing is added
            x = centred_norm(alpha * x, w["norm2"], eps)
        if streams is not None:
            streams.append(x.clone())
    logits = centred_norm(x, weights["final.norm"], eps) @ weights["head"].T
    cap = raw.get("logit_softcap")
    return logits if cap is None else cap * torch.tanh(logits / cap)


def load_model_dir(folder, dtype=torch.float64):
    from safetensors.torch import load_file

    folder = Path(folder)
    raw = json.loads((folder / "config.json").read_text())
    return raw, {name: t.to(dtype) for name, t in load_file(str(folder / "model.safetensors")).items()}
