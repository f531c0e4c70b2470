"""Napizen: configuration -> ModelSpec.

Every layer normalises the sum of the stream and a sublayer's output, the sublayers reading the stream itself:
h = norm1(alpha * h + mixer(h)), then h = norm2(alpha * h + feed_forward(h)) where the layer has a feed-forward, with
layer norms (mean taken off, a weight, no bias) and one alpha for the model.  The mixer is latent attention (one small row
kept per position, a rotated key part shared by the heads, neighbouring pairs rotated with stretched slow frequencies,
a sink in the softmax's denominator, a gate per head); the feed-forward is a dense gated one (silu) or routed experts of
that kind, chosen by sigmoid scores with a correction that takes part in the choice only, among the experts of the
best groups.  The embedding is scaled; the model's norm, the head and a soft cap of the logits follow the last layer.

Checkpoint tensors are named without a `.weight` ending: `embed`, `head`, `final.norm`, `l<i>.norm1`, `l<i>.mix.q`,
`l<i>.mix.dkv.norm`, `l<i>.mix.sink`, `l<i>.mlp.gate`, `l<i>.mlp.router`, `l<i>.mlp.correction`, `l<i>.mlp.e<j>.up`.
"""

from __future__ import annotations

from ..config.napizen import MAX_POSITIONS, NapizenConfig, NapizenLayer
from ..parts import PartSpec
from .nobodra import LAYER_NAMES
from .nobodra import checkpoint_name as _short_name
from .spec import ModelSpec, ScheduleEntry


def checkpoint_name(name: str) -> str:
    """The checkpoint's name of the tensor that the parts call `name`."""
    return _short_name(name).replace("dkv_norm", "dkv.norm")


def _mixer(config: NapizenConfig, layer: NapizenLayer) -> PartSpec:
    position = PartSpec("none")
    if layer.rot_dims is not None and layer.rot_dim:
        scaling = None if layer.rot_scaling is None else dict(zip(("factor", "original", "fast", "slow"), layer.rot_scaling))
        position = PartSpec("rope_interleaved", {"rotary_dim": layer.rot_dims, "theta": layer.rot_base, "scaling": scaling})
    return PartSpec("latent_attention", {
        "hidden_size": config.width, "num_heads": layer.heads, "head_dim": layer.dim, "rot_dim": layer.rot_dim, "value_dim": layer.vdim,
        "kv_rank": layer.kv_rank, "position": position, "norm_eps": config.norm_eps, "scale": layer.scale, "sink": True, "gate": True})


def _feed_forward(config: NapizenConfig, layer: NapizenLayer) -> PartSpec:
    mlp = layer.mlp
    if mlp.kind == "dense":
        return PartSpec("swiglu", {"hidden_size": config.width, "intermediate_size": mlp.ff})
    return PartSpec("routed_experts", {
        "hidden_size": config.width, "intermediate_size": mlp.ff, "num_experts": mlp.experts, "top": mlp.top, "router_bias": True,
        "bias_name": "correction", "activation": "silu_gated", "rule": "sigmoid", "groups": mlp.groups, "keep": mlp.keep,
        "weight_scale": mlp.weight_scale})


def build_spec(config: NapizenConfig) -> ModelSpec:
    norm = PartSpec("layernorm", {"size": config.width, "eps": config.norm_eps})
    layers = []
    for layer in config.layers:
        params = {"mixer": _mixer(config, layer), "mixer_norm": norm, "alpha": config.alpha, "names": LAYER_NAMES}
        if layer.mlp is not None:
            params["feed_forward"] = _feed_forward(config, layer)
            params["ff_norm"] = norm
        else:
            params["norm_without_ff"] = norm      # asked for as optional: see PostNormBlock
        layers.append(PartSpec("postnorm", params))
    return ModelSpec(
        architecture=NapizenConfig.ARCHITECTURE, vocab_size=config.vocab_size, hidden_size=config.width, layers=tuple(layers),
        schedule=tuple(ScheduleEntry(i) for i in range(len(layers))), final_norm=norm, max_positions=MAX_POSITIONS,
        eos_token_ids=(), embedding_multiplier=config.embedding_scale, embedding_name="embed", head_name="head",
        final_norm_prefix="final.norm", layer_prefix="l{index}", checkpoint_dtype="bfloat16", checkpoint_name=checkpoint_name,
        after_head=None if config.logit_softcap is None else PartSpec("soft_cap", {"cap": config.logit_softcap}))
