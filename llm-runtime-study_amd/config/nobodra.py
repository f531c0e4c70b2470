"""Typed Nobodra configuration read from the keys of its config.json.

A Nobodra model is a stack of layers that may all differ: config.json lists them, each with the kind of its mixer
(`type`: "attention" or "delta"), the mixer's sizes and constants (`mixer`) and its feed-forward (`mlp`, or null
for a layer without one).  Nothing is assumed that the file does not say: a mixer without `mask` sees the whole
context, one without `rot` is not rotated, one without `scale` scores with 1 / sqrt(dim).

    {"architecture": "Nobodra", "vocab": V, "width": W, "norm": {"eps": e}, "layers": [
        {"type": "attention", "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", "mask": {"size"}, "rot": {"base", "dims"}},
         "mlp": {"kind": "moe", "expert": {"ff"}, "router": {"experts", "top"}} | null},
        {"type": "delta", "mixer": {"heads", "kv_heads", "dim", "vdim", "conv"}, "mlp": ...}, ...]}
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

from ..errors import ConfigError
from .fields import optional, required

MAX_POSITIONS = 1 << 24        # positions are turned into float32 angles: exact up to here


def _section(raw: Mapping[str, Any], name: str, where: str) -> Mapping[str, Any]:
    value = raw.get(name)
    if not isinstance(value, dict):
        raise ConfigError(f"{where}: `{name}` must be an object")
    return value


def _positive(raw: Mapping[str, Any], name: str, where: str) -> int:
    try:
        value = required(raw, name, int)
    except ConfigError as exc:
        raise ConfigError(f"{where}: {exc}") from None
    if value <= 0:
        raise ConfigError(f"{where}: {name} must be positive, got {value}")
    return value


@dataclass(frozen=True)
class NobodraExperts:
    ff: int
    experts: int
    top: int

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "NobodraExperts":
        if raw.get("kind") != "moe":
            raise ConfigError(f"{where}: unknown feed-forward kind {raw.get('kind')!r}; expected 'moe'")
        router = _section(raw, "router", where)
        made = cls(_positive(_section(raw, "expert", where), "ff", where), _positive(router, "experts", where), _positive(router, "top", where))
        if made.top > made.experts:
            raise ConfigError(f"{where}: top {made.top} exceeds the {made.experts} experts")
        return made

    def to_json_dict(self) -> dict:
        return {"kind": "moe", "expert": {"ff": self.ff}, "router": {"experts": self.experts, "top": self.top}}


@dataclass(frozen=True)
class NobodraLayer:
    type: str                       # "attention" | "delta"
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    mlp: NobodraExperts | None
    # attention
    scale: float | None = None
    window: int | None = None
    rot_base: float | None = None
    rot_dims: int | None = None
    # delta
    conv: int | None = None

    TYPES = ("attention", "delta")

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], index: int) -> "NobodraLayer":
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
        common = dict(type=kind, heads=_positive(mixer, "heads", where), kv_heads=_positive(mixer, "kv_heads", where),
                      dim=_positive(mixer, "dim", where), vdim=_positive(mixer, "vdim", where),
                      mlp=None if mlp is None else NobodraExperts.from_dict(mlp, where))
        if common["heads"] % common["kv_heads"]:
            raise ConfigError(f"{where}: heads must be a multiple of kv_heads, got {common['heads']} and {common['kv_heads']}")
        if kind == "delta":
            return cls(conv=_positive(mixer, "conv", where), **common)
        if common["vdim"] != common["dim"]:
            raise ConfigError(f"{where}: an attention layer's values are its keys, so vdim must equal dim, got {common['vdim']} and {common['dim']}")
        scale = optional(mixer, "scale", (int, float), None)
        if scale is not None and not scale > 0:
            raise ConfigError(f"{where}: scale must be positive, got {scale}")
        window = rot_base = rot_dims = None
        if mixer.get("mask") is not None:
            window = _positive(_section(mixer, "mask", where), "size", where)
        if mixer.get("rot") is not None:
            rot = _section(mixer, "rot", where)
            rot_dims, rot_base = _positive(rot, "dims", where), float(required(rot, "base", (int, float)))
            if rot_dims % 2 or rot_dims > common["dim"] or rot_base <= 0:
                raise ConfigError(f"{where}: rot.dims must be even and at most dim, rot.base positive, got {rot_dims} and {rot_base}")
        return cls(scale=None if scale is None else float(scale), window=window, rot_base=rot_base, rot_dims=rot_dims, **common)

    def to_json_dict(self) -> dict:
        mixer: dict = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim}
        if self.type == "delta":
            mixer["conv"] = self.conv
        else:
            if self.scale is not None:
                mixer["scale"] = self.scale
            if self.window is not None:
                mixer["mask"] = {"size": self.window}
            if self.rot_dims is not None:
                mixer["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
        return {"type": self.type, "mixer": mixer, "mlp": None if self.mlp is None else self.mlp.to_json_dict()}


@dataclass(frozen=True)
class NobodraConfig:
    vocab_size: int
    width: int
    norm_eps: float
    layers: tuple
    eos_token_ids: tuple = ()        # the design names no end-of-sequence token: generation runs to its length limit
    model_type: str = "nobodra"

    ARCHITECTURE = "Nobodra"

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "NobodraConfig":
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("layers must be a non-empty list")
        eps = float(required(_section(raw, "norm", "config.json"), "eps", (int, float)))
        if eps <= 0:
            raise ConfigError(f"norm.eps must be positive, got {eps}")
        return cls(vocab_size=_positive(raw, "vocab", "config.json"), width=_positive(raw, "width", "config.json"), norm_eps=eps,
                   layers=tuple(NobodraLayer.from_dict(layer, index) for index, layer in enumerate(layers)))

    def validate_context_length(self, max_seq_len: int) -> None:
        if not 0 < max_seq_len <= MAX_POSITIONS:
            raise ConfigError(f"max_seq_len must be within 1..{MAX_POSITIONS}, got {max_seq_len}")

    def to_json_dict(self) -> dict:
        return {"architecture": self.ARCHITECTURE, "vocab": self.vocab_size, "width": self.width, "norm": {"eps": self.norm_eps},
                "layers": [layer.to_json_dict() for layer in self.layers]}
