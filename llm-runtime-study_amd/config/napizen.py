"""Typed Napizen configuration read from the keys of its config.json.

A Napizen model is a stack of layers listed in config.json, each with the kind of its mixer (`type`: "latent_attention"),
the mixer's sizes and constants (`mixer`) and its feed-forward (`mlp`: a dense gated one, routed experts, or null for a
layer without one).  Every size and constant is read from the file; what the file does not say does not exist: a mixer
without `rot.scaling` rotates plainly, a router without `groups` chooses among all its experts, a model without
`logit_softcap` leaves its logits as they are.

    {"architecture": "Napizen", "vocab": V, "width": W, "norm": {"eps": e}, "postln_alpha": a, "embedding": {"scale": s},
     "logit_softcap": c, "layers": [
        {"type": "latent_attention",
         "mixer": {"heads", "dim", "rot_dim", "vdim", "kv_rank", "scale",
                   "rot": {"base", "dims", "scaling": {"factor", "original", "fast", "slow"}}},
         "mlp": {"kind": "dense", "ff"}
              | {"kind": "moe", "expert": {"ff"}, "router": {"experts", "top", "scale", "groups": {"count", "keep"}}}
              | null}, ...]}
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

from ..errors import ConfigError
from .fields import optional, required
from .nobodra import MAX_POSITIONS, _positive, _section


def _number(raw: Mapping[str, Any], name: str, where: str, default=None) -> float:
    try:
        value = required(raw, name, (int, float)) if default is None else optional(raw, name, (int, float), default)
    except ConfigError as exc:
        raise ConfigError(f"{where}: {exc}") from None
    return float(value)


@dataclass(frozen=True)
class NapizenFeedForward:
    kind: str                       # "dense" | "moe"
    ff: int
    experts: int = 0
    top: int = 0
    weight_scale: float = 1.0
    groups: int = 0                 # 0: the router chooses among all experts
    keep: int = 0

    KINDS = ("dense", "moe")

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "NapizenFeedForward":
        kind = raw.get("kind")
        if kind not in cls.KINDS:
            raise ConfigError(f"{where}: unknown feed-forward kind {kind!r}; expected one of: {', '.join(cls.KINDS)}")
        if kind == "dense":
            return cls("dense", _positive(raw, "ff", where))
        router = _section(raw, "router", where)
        experts, top = _positive(router, "experts", where), _positive(router, "top", where)
        if top > experts:
            raise ConfigError(f"{where}: top {top} exceeds the {experts} experts")
        scale = _number(router, "scale", where, 1.0)
        if not scale > 0:
            raise ConfigError(f"{where}: router.scale must be positive, got {scale}")
        groups = keep = 0
        if router.get("groups") is not None:
            section = _section(router, "groups", where)
            groups, keep = _positive(section, "count", where), _positive(section, "keep", where)
            if experts % groups or keep > groups or keep * (experts // groups) < top:
                raise ConfigError(f"{where}: {experts} experts in {groups} groups of which {keep} are kept cannot give {top} choices")
        return cls("moe", _positive(_section(raw, "expert", where), "ff", where), experts, top, scale, groups, keep)

    def to_json_dict(self) -> dict:
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        router: dict = {"experts": self.experts, "top": self.top, "scale": self.weight_scale}
        if self.groups:
            router["groups"] = {"count": self.groups, "keep": self.keep}
        return {"kind": "moe", "expert": {"ff": self.ff}, "router": router}


@dataclass(frozen=True)
class NapizenLayer:
    type: str                       # "latent_attention"
    heads: int
    dim: int                        # plain (unrotated) query/key dims of a head
    rot_dim: int                    # rotated ones
    vdim: int
    kv_rank: int
    scale: float | None
    rot_base: float | None
    rot_dims: int | None
    rot_scaling: tuple | None       # (factor, original, fast, slow)
    mlp: NapizenFeedForward | None

    TYPES = ("latent_attention",)

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], index: int) -> "NapizenLayer":
        where = f"layer {index}"
        if not isinstance(raw, dict):
            raise ConfigError(f"{where} must be an object")
        kind = raw.get("type")
        if kind not in cls.TYPES:
            raise ConfigError(f"{where}: unknown type {kind!r}; expected one of: {', '.join(cls.TYPES)}")
        mixer = _section(raw, "mixer", where)
        mlp = raw.get("mlp")
        if mlp is not None and not isinstance(mlp, dict):
            raise ConfigError(f"{where}: `mlp` must be an object or null")
        rot_dim = required(mixer, "rot_dim", int) if "rot_dim" in mixer else 0
        if rot_dim < 0 or rot_dim % 2:
            raise ConfigError(f"{where}: rot_dim must be even and not negative, got {rot_dim}")
        scale = None
        if mixer.get("scale") is not None:
            scale = _number(mixer, "scale", where)
            if not scale > 0:
                raise ConfigError(f"{where}: scale must be positive, got {scale}")
        rot_base = rot_dims = rot_scaling = None
        if mixer.get("rot") is not None:
            rot = _section(mixer, "rot", where)
            rot_dims, rot_base = _positive(rot, "dims", where), _number(rot, "base", where)
            if rot_dims != rot_dim:
                raise ConfigError(f"{where}: the rotation covers a head's whole rotated part, so rot.dims must equal rot_dim, got {rot_dims} and {rot_dim}")
            if rot_base <= 0 or rot_base == 1:
                raise ConfigError(f"{where}: rot.base must be positive and not 1, got {rot_base}")
            if rot.get("scaling") is not None:
                scaling = _section(rot, "scaling", where)
                rot_scaling = tuple(_number(scaling, name, where) for name in ("factor", "original", "fast", "slow"))
                if min(rot_scaling) <= 0:
                    raise ConfigError(f"{where}: rot.scaling factor, original, fast and slow must be positive, got {rot_scaling}")
        elif rot_dim:
            raise ConfigError(f"{where}: a rotated part of {rot_dim} dims needs `rot`")
        return cls(type=kind, heads=_positive(mixer, "heads", where), dim=_positive(mixer, "dim", where), rot_dim=rot_dim,
                   vdim=_positive(mixer, "vdim", where), kv_rank=_positive(mixer, "kv_rank", where), scale=scale, rot_base=rot_base,
                   rot_dims=rot_dims, rot_scaling=rot_scaling, mlp=None if mlp is None else NapizenFeedForward.from_dict(mlp, where))

    def to_json_dict(self) -> dict:
        mixer: dict = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "kv_rank": self.kv_rank}
        if self.scale is not None:
            mixer["scale"] = self.scale
        if self.rot_dims is not None:
            mixer["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
            if self.rot_scaling is not None:
                mixer["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), self.rot_scaling))
        return {"type": self.type, "mixer": mixer, "mlp": None if self.mlp is None else self.mlp.to_json_dict()}


@dataclass(frozen=True)
class NapizenConfig:
    vocab_size: int
    width: int
    norm_eps: float
    alpha: float                     # the stream's factor in a layer's sums, norm(alpha * h + sublayer(h))
    embedding_scale: float
    logit_softcap: float | None
    layers: tuple
    eos_token_ids: tuple = ()        # the design names no end-of-sequence token: generation runs to its length limit
    model_type: str = "napizen"

    ARCHITECTURE = "Napizen"

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "NapizenConfig":
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("layers must be a non-empty list")
        eps = _number(_section(raw, "norm", "config.json"), "eps", "config.json")
        if eps <= 0:
            raise ConfigError(f"norm.eps must be positive, got {eps}")
        embedding = raw.get("embedding") if raw.get("embedding") is not None else {}
        if not isinstance(embedding, dict):
            raise ConfigError("config.json: `embedding` must be an object")
        cap = None
        if raw.get("logit_softcap") is not None:
            cap = _number(raw, "logit_softcap", "config.json")
            if not cap > 0:
                raise ConfigError(f"logit_softcap must be positive, got {cap}")
        return cls(vocab_size=_positive(raw, "vocab", "config.json"), width=_positive(raw, "width", "config.json"), norm_eps=eps,
                   alpha=_number(raw, "postln_alpha", "config.json", 1.0), embedding_scale=_number(embedding, "scale", "config.json", 1.0),
                   logit_softcap=cap, layers=tuple(NapizenLayer.from_dict(layer, index) for index, layer in enumerate(layers)))

    def validate_context_length(self, max_seq_len: int) -> None:
        if not 0 < max_seq_len <= MAX_POSITIONS:
            raise ConfigError(f"max_seq_len must be within 1..{MAX_POSITIONS}, got {max_seq_len}")

    def to_json_dict(self) -> dict:
        out = {"architecture": self.ARCHITECTURE, "vocab": self.vocab_size, "width": self.width, "norm": {"eps": self.norm_eps},
               "postln_alpha": self.alpha, "embedding": {"scale": self.embedding_scale},
               "layers": [layer.to_json_dict() for layer in self.layers]}
        if self.logit_softcap is not None:
            out["logit_softcap"] = self.logit_softcap
        return out
