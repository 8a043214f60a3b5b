"""Configuration of the Rogizen decoder, read from its own config.json keys.

The file names its design in ``architecture`` and describes every layer by itself:
  vocab, width, embedding.scale, norm.eps, logit_softcap,
  loop             null | {start, stop, times}: layers start .. stop-1 run ``times`` times in a row,
  layers[i].type   the mixer: "attention" | "mamba2",
  layers[i].mixer  attention: {heads, kv_heads, dim, vdim, conv, scale, rot: {base, dims, scaling: {factor, original,
                   fast, slow}}, mask: {size}};  mamba2: {heads, vdim, state, groups, norm_groups, conv},
  layers[i].mlp    null | {kind: "dense", ff}.
Layers may differ in every size.  What a file does not mention is not there: no ``loop``, no repetition and no
re-entry matrix; no ``mask``, all earlier keys; no ``rot.scaling``, the plain frequencies; no ``logit_softcap``, the
logits as the head leaves them.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple, Union

from .base import ConfigError, KeyReader

ROGIZEN_MODEL_TYPE = "Rogizen"
MIXER_TYPES = ("attention", "mamba2")
MLP_KINDS = ("dense",)


def _need(r: Optional[KeyReader], where: str, key: str) -> KeyReader:
    if r is None:
        raise ConfigError(f"{where}: required key '{key}' is missing")
    return r


@dataclass(frozen=True)
class RotScaling:
    factor: float
    original: float
    fast: float
    slow: float

    def to_dict(self) -> dict:
        return {"factor": self.factor, "original": self.original, "fast": self.fast, "slow": self.slow}


@dataclass(frozen=True)
class ConvAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int                   # taps of the convolution on queries and keys
    scale: float
    rot_base: Optional[float]   # None: the file has no 'rot' at all
    rot_dims: int               # how many of a head's first values are rotated
    rot_scaling: Optional[RotScaling]
    chunk: Optional[int]        # a query sees the keys of its own chunk of so many positions; None: all earlier keys

    @staticmethod
    def from_reader(r: KeyReader) -> "ConvAttentionConfig":
        rot, mask = r.obj("rot"), r.obj("mask")
        sc = rot.obj("scaling") if rot is not None else None
        m = ConvAttentionConfig(
            heads=r.integer("heads", minimum=1), kv_heads=r.integer("kv_heads", minimum=1),
            dim=r.integer("dim", minimum=1), vdim=r.integer("vdim", minimum=1), conv=r.integer("conv", minimum=1),
            scale=r.number("scale", positive=True),
            rot_base=rot.number("base", positive=True) if rot is not None else None,
            rot_dims=rot.integer("dims", minimum=0) if rot is not None else 0,
            rot_scaling=RotScaling(sc.number("factor", positive=True), sc.number("original", positive=True),
                                   sc.number("fast", positive=True), sc.number("slow", positive=True)) if sc is not None else None,
            chunk=mask.integer("size", None, minimum=1) if mask is not None else None)
        if m.heads % m.kv_heads:
            raise ConfigError(f"{r.where}: heads {m.heads} is not a multiple of kv_heads {m.kv_heads}")
        if m.vdim != m.dim:
            raise ConfigError(f"{r.where}: the values are the keys, so vdim {m.vdim} must equal dim {m.dim}")
        if m.rot_dims > m.dim or m.rot_dims % 2:
            raise ConfigError(f"{r.where}: rot.dims must be even and at most dim {m.dim}, got {m.rot_dims}")
        return m

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv,
               "scale": self.scale}
        if self.rot_base is not None:
            out["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
        if self.rot_scaling is not None:
            out["rot"]["scaling"] = self.rot_scaling.to_dict()
        if self.chunk is not None:
            out["mask"] = {"size": self.chunk}
        return out


@dataclass(frozen=True)
class Mamba2Config:
    heads: int
    vdim: int                   # values a head
    state: int
    groups: int
    norm_groups: int
    conv: int

    @staticmethod
    def from_reader(r: KeyReader) -> "Mamba2Config":
        m = Mamba2Config(heads=r.integer("heads", minimum=1), vdim=r.integer("vdim", minimum=1),
                         state=r.integer("state", minimum=1), groups=r.integer("groups", minimum=1),
                         norm_groups=r.integer("norm_groups", minimum=1), conv=r.integer("conv", minimum=1))
        if m.heads % m.groups:
            raise ConfigError(f"{r.where}: heads {m.heads} is not a multiple of groups {m.groups}")
        if (m.heads * m.vdim) % m.norm_groups:
            raise ConfigError(f"{r.where}: norm_groups {m.norm_groups} does not divide heads * vdim {m.heads * m.vdim}")
        return m

    def to_dict(self) -> dict:
        return {"heads": self.heads, "vdim": self.vdim, "state": self.state, "groups": self.groups,
                "norm_groups": self.norm_groups, "conv": self.conv}


@dataclass(frozen=True)
class MlpConfig:
    kind: str
    ff: int

    def to_dict(self) -> dict:
        return {"kind": self.kind, "ff": self.ff}


@dataclass(frozen=True)
class RogizenLayerConfig:
    type: str
    mixer: Union[ConvAttentionConfig, Mamba2Config]
    mlp: Optional[MlpConfig]


@dataclass(frozen=True)
class LoopConfig:
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class RogizenConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    layers: Tuple[RogizenLayerConfig, ...]
    loop: Optional[LoopConfig] = None
    logit_softcap: Optional[float] = None
    model_type: str = ROGIZEN_MODEL_TYPE

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

    def layer_runs(self) -> Tuple[Tuple[int, bool], ...]:
        """(layer, whether a pass of the loop starts with this run) in the order the layers run."""
        n = len(self.layers)
        if self.loop is None:
            return tuple((i, False) for i in range(n))
        a, b = self.loop.start, self.loop.stop
        runs = [(i, False) for i in range(a)]
        for _ in range(self.loop.times):
            runs += [(i, i == a) for i in range(a, b)]
        return tuple(runs + [(i, False) for i in range(b, n)])

    @staticmethod
    def from_dict(raw: Mapping[str, Any], where: str = "config.json") -> "RogizenConfig":
        r = KeyReader(raw, where)
        emb, norm = r.obj("embedding"), _need(r.obj("norm"), where, "norm")
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError(f"{where}: 'layers' must be a list with at least one layer")
        layers = []
        for i, entry in enumerate(listed):
            lr = KeyReader(entry, f"{where}:layers[{i}]")
            kind = lr.string("type", choices=MIXER_TYPES)
            mr = _need(lr.obj("mixer"), lr.where, "mixer")
            mixer = ConvAttentionConfig.from_reader(mr) if kind == "attention" else Mamba2Config.from_reader(mr)
            mlp = lr.obj("mlp")
            layers.append(RogizenLayerConfig(kind, mixer, MlpConfig(mlp.string("kind", choices=MLP_KINDS),
                                                                  mlp.integer("ff", minimum=1)) if mlp is not None else None))
        loop, lp = None, r.obj("loop")
        if lp is not None:
            loop = LoopConfig(lp.integer("start", minimum=0), lp.integer("stop", minimum=0), lp.integer("times", minimum=0))
            if not loop.start <= loop.stop <= len(layers):
                raise ConfigError(f"{where}: loop {loop.start} .. {loop.stop} does not lie within the {len(layers)} layers")
        cap = r.number("logit_softcap", None)
        if cap is not None and cap <= 0:
            raise ConfigError(f"{where}: logit_softcap must be positive, got {cap}")
        return RogizenConfig(
            vocab=r.integer("vocab", minimum=1), width=r.integer("width", minimum=1),
            embedding_scale=emb.number("scale", 1.0) if emb is not None else 1.0,
            norm_eps=norm.number("eps", positive=True), layers=tuple(layers), loop=loop, logit_softcap=cap)

    def to_dict(self) -> dict:
        out = {"architecture": self.model_type, "vocab": self.vocab, "width": self.width,
               "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
               "layers": [{"type": l.type, "mixer": l.mixer.to_dict(), "mlp": l.mlp.to_dict() if l.mlp else None}
                          for l in self.layers]}
        if self.loop is not None:
            out["loop"] = {"start": self.loop.start, "stop": self.loop.stop, "times": self.loop.times}
        if self.logit_softcap is not None:
            out["logit_softcap"] = self.logit_softcap
        return out
