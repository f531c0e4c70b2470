"""Nobodra: configuration -> ModelSpec.

Every layer normalises what its sublayers give out (h += norm1(mixer(h)), h += norm2(feed_forward(h)), the
sublayers reading h itself), with RMS norms whose weights are stored around zero (1 + w).  A layer's mixer is
either sliding-window grouped-query attention whose values are its keys as projected (per-head q/k RMS norm,
rotation of the first rot.dims dims, the score scale from the configuration) or the gated delta rule; its
feed-forward, where it has one, is a set of routed experts with the square of relu between their two matrices.
The model's norm and the head follow the last layer.

Checkpoint tensors are named without a `.weight` ending: `embed`, `head`, `final.norm`, `l<i>.norm1`,
`l<i>.mix.q`, `l<i>.mix.q.norm`, `l<i>.mix.q.conv`, `l<i>.mlp.router`, `l<i>.mlp.router.b`, `l<i>.mlp.e<j>.up`;
`checkpoint_name` turns a part's own tensor name into the checkpoint's.
"""

from __future__ import annotations

import re

from ..config.nobodra import MAX_POSITIONS, NobodraConfig, NobodraLayer
from ..parts import PartSpec
from .spec import ModelSpec, ScheduleEntry

LAYER_NAMES = {"mixer": "mix", "feed_forward": "mlp", "mixer_norm": "norm1", "ff_norm": "norm2"}
_EXPERT = re.compile(r"\.experts\.(\d+)\.")


def checkpoint_name(name: str) -> str:
    """The checkpoint's name of the tensor that the parts call `name`."""
    name = name.removesuffix(".weight")
    name = _EXPERT.sub(r".e\1.", name)
    name = name.replace("_proj", "").replace("_conv", ".conv").replace("q_norm", "q.norm").replace("k_norm", "k.norm")
    return name.replace("router.bias", "router.b")


def _mixer(config: NobodraConfig, layer: NobodraLayer) -> PartSpec:
    if layer.type == "delta":
        return PartSpec("gated_delta_rule", {
            "hidden_size": config.width, "num_heads": layer.heads, "num_kv_heads": layer.kv_heads, "head_dim": layer.dim,
            "value_dim": layer.vdim, "conv_taps": layer.conv, "norm_eps": config.norm_eps})
    position = PartSpec("none") if layer.rot_dims is None else PartSpec("rope_half", {"rotary_dim": layer.rot_dims, "theta": layer.rot_base})
    return PartSpec("gqa_attention", {
        "hidden_size": config.width, "num_heads": layer.heads, "num_kv_heads": layer.kv_heads, "head_dim": layer.dim,
        "position": position, "qk_norm": True, "qk_norm_eps": config.norm_eps, "scale": layer.scale, "window": layer.window,
        "values_from_keys": True})


def build_spec(config: NobodraConfig) -> ModelSpec:
    norm = PartSpec("rmsnorm", {"size": config.width, "eps": config.norm_eps, "unit_offset": True})
    layers = []
    for layer in config.layers:
        params = {"mixer": _mixer(config, layer), "mixer_norm": norm, "names": LAYER_NAMES}
        if layer.mlp is not None:
            params["feed_forward"] = PartSpec("routed_experts", {
                "hidden_size": config.width, "intermediate_size": layer.mlp.ff, "num_experts": layer.mlp.experts, "top": layer.mlp.top,
                "router_bias": True, "activation": "relu_squared"})
            params["ff_norm"] = norm
        layers.append(PartSpec("outnorm", params))
    return ModelSpec(
        architecture=NobodraConfig.ARCHITECTURE, vocab_size=config.vocab_size, hidden_size=config.width, layers=tuple(layers),
        schedule=tuple(ScheduleEntry(i) for i in range(len(layers))), final_norm=norm, max_positions=MAX_POSITIONS,
        eos_token_ids=(), embedding_name="embed", head_name="head", final_norm_prefix="final.norm", layer_prefix="l{index}",
        checkpoint_dtype="bfloat16", checkpoint_name=checkpoint_name)
