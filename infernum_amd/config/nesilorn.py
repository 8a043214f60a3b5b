"""Configuration of the Nesilorn decoder, read from its own config.json keys.

The file names its design in ``architecture`` and describes every layer by itself:
  vocab, width, embedding.scale, norm.eps,
  layers[i].type   the mixer ("latent_attention"),
  layers[i].mixer  {heads, dim, rot_dim, vdim, kv_rank, scale, rot: {base, dims}, mask: {size}},
  layers[i].mlp    null | {kind: "dense", ff} | {kind: "moe", expert: {ff, limit}, router: {experts, top}}.
Layers may differ in every size.  Constants that the design fixes (the experts' sigmoid slope, the tanh form of
GELU) are in the model's spec builder, not here.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple

from .base import ConfigError, KeyReader

NESILORN_MODEL_TYPE = "Nesilorn"
MIXER_TYPES = ("latent_attention",)
MLP_KINDS = ("dense", "moe")


def _need(r: Optional[KeyReader], where: str, key: str) -> KeyReader:
    if r is None:
        raise ConfigError(f"{where}: required key '{key}' is missing")
    return r


@dataclass(frozen=True)
class LatentMixerConfig:
    heads: int
    dim: int                    # plain (unrotated) query/key values a head
    rot_dim: int                # rotated query/key values a head; the key's are shared by all heads
    vdim: int
    kv_rank: int
    scale: float
    rot_base: float
    rot_dims: int               # how many of the rot_dim values are rotated (the first ones)
    window: Optional[int]       # a query sees itself and the window - 1 tokens before it; None: all

    @staticmethod
    def from_reader(r: KeyReader) -> "LatentMixerConfig":
        rot = _need(r.obj("rot"), r.where, "rot")
        mask = r.obj("mask")
        m = LatentMixerConfig(
            heads=r.integer("heads", minimum=1), dim=r.integer("dim", minimum=1),
            rot_dim=r.integer("rot_dim", minimum=0), vdim=r.integer("vdim", minimum=1),
            kv_rank=r.integer("kv_rank", minimum=1), scale=r.number("scale", positive=True),
            rot_base=rot.number("base", positive=True), rot_dims=rot.integer("dims", minimum=0),
            window=mask.integer("size", None, minimum=1) if mask is not None else None)
        if m.rot_dims > m.rot_dim or m.rot_dims % 2:
            raise ConfigError(f"{r.where}: rot.dims must be even and at most rot_dim {m.rot_dim}, got {m.rot_dims}")
        return m

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "kv_rank": self.kv_rank,
               "scale": self.scale, "rot": {"base": self.rot_base, "dims": self.rot_dims}}
        if self.window is not None:
            out["mask"] = {"size": self.window}
        return out


@dataclass(frozen=True)
class MlpConfig:
    kind: str                   # "dense" | "moe"
    ff: int                     # of the dense layer, or of one expert
    experts: int = 0
    top: int = 0
    limit: float = 0.0

    @staticmethod
    def from_reader(r: KeyReader) -> "MlpConfig":
        kind = r.string("kind", choices=MLP_KINDS)
        if kind == "dense":
            return MlpConfig("dense", r.integer("ff", minimum=1))
        ex, ro = _need(r.obj("expert"), r.where, "expert"), _need(r.obj("router"), r.where, "router")
        m = MlpConfig("moe", ex.integer("ff", minimum=1), ro.integer("experts", minimum=1), ro.integer("top", minimum=1),
                      ex.number("limit", positive=True))
        if m.top > m.experts:
            raise ConfigError(f"{r.where}: router.top {m.top} is more than router.experts {m.experts}")
        return m

    def to_dict(self) -> dict:
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        return {"kind": "moe", "expert": {"ff": self.ff, "limit": self.limit},
                "router": {"experts": self.experts, "top": self.top}}


@dataclass(frozen=True)
class NesilornLayerConfig:
    type: str
    mixer: LatentMixerConfig
    mlp: Optional[MlpConfig]


@dataclass(frozen=True)
class NesilornConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    layers: Tuple[NesilornLayerConfig, ...]
    model_type: str = NESILORN_MODEL_TYPE

    # what the generation entry points ask of every configuration
    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    bos_token_id = None
    eos_token_id = None

    @staticmethod
    def from_dict(raw: Mapping[str, Any], where: str = "config.json") -> "NesilornConfig":
        r = KeyReader(raw, where)
        emb, norm = r.obj("embedding"), _need(r.obj("norm"), where, "norm")
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError(f"{where}: 'layers' must be a list with at least one layer")
        layers = []
        for i, entry in enumerate(listed):
            lr = KeyReader(entry, f"{where}:layers[{i}]")
            kind = lr.string("type", choices=MIXER_TYPES)
            mixer = LatentMixerConfig.from_reader(_need(lr.obj("mixer"), lr.where, "mixer"))
            mlp = lr.obj("mlp")
            layers.append(NesilornLayerConfig(kind, mixer, MlpConfig.from_reader(mlp) if mlp is not None else None))
        return NesilornConfig(
            vocab=r.integer("vocab", minimum=1), width=r.integer("width", minimum=1),
            embedding_scale=emb.number("scale", 1.0) if emb is not None else 1.0,
            norm_eps=norm.number("eps", positive=True), layers=tuple(layers))

    def to_dict(self) -> dict:
        return {"architecture": self.model_type, "vocab": self.vocab, "width": self.width,
                "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
                "layers": [{"type": l.type, "mixer": l.mixer.to_dict(), "mlp": l.mlp.to_dict() if l.mlp else None}
                           for l in self.layers]}
