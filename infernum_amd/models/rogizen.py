"""The Rogizen decoder as a ModelSpec: pre-norm layers whose mixer is a state-space recurrence (``mamba2``) or an
attention with convolved queries and keys whose values are its keys (``conv_attention``), a gated feed-forward or
none, a stretch of layers that runs several times with the same weights (every pass with a cache and state of its
own, entered through a matrix over [stream ; embedding output]), and capped logits.  Tensor names: ``embed``,
``loop.in``, ``final.norm``, ``head``, ``l<i>.norm1|norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``.
"""
from __future__ import annotations

from ..config.registry import register_architecture
from ..config.rogizen import ROGIZEN_MODEL_TYPE, RogizenConfig
from ..parts.base import LayerSpec, ModelSpec, PartSpec, ScheduleEntry


def rogizen_model_spec(cfg: RogizenConfig, init_std: float = 0.05) -> ModelSpec:
    W = cfg.width

    def norm(prefix: str) -> PartSpec:
        return PartSpec("rmsnorm", {"size": W, "eps": cfg.norm_eps, "init": ("uniform", 0.8, 1.2), "name": ""}, prefix)

    loops = cfg.loop is not None and cfg.loop.times > 0 and cfg.loop.stop > cfg.loop.start
    layers = []
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}.", layer.mixer
        if layer.type == "attention":
            position = {"kind": "none"}
            if m.rot_dims > 0:
                scaling = dict(m.rot_scaling.to_dict(), rope_type="yarn") if m.rot_scaling is not None else None
                position = {"kind": "rope", "params": {"head_dim": m.dim, "theta": m.rot_base, "rotary_dim": m.rot_dims,
                                                       "scaling": scaling, "pairing": "neighbours"}}
            mixer = PartSpec("conv_attention", {
                "hidden_size": W, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
                "conv_taps": m.conv, "norm_eps": cfg.norm_eps, "position": position, "chunk": m.chunk, "scale": m.scale,
                "init_std": init_std}, p + "mix.")
        else:
            mixer = PartSpec("mamba2", {
                "hidden_size": W, "num_heads": m.heads, "head_dim": m.vdim, "state_size": m.state, "groups": m.groups,
                "norm_groups": m.norm_groups, "conv_taps": m.conv, "norm_eps": cfg.norm_eps, "init_std": init_std},
                p + "mix.")
        ff = None
        if layer.mlp is not None:
            ff = PartSpec("swiglu", {"hidden_size": W, "intermediate_size": layer.mlp.ff, "init_std": init_std,
                                     "names": ("gate", "up", "down")}, p + "mlp.")
        extra = {}
        if loops and i == cfg.loop.start:           # every pass of the loop enters through this layer
            extra["stream_in"] = ("stream_in", PartSpec("concat_linear", {"hidden_size": W, "name": "in",
                                                                          "init_std": (2 * W) ** -0.5}, "loop."))
        layers.append(LayerSpec(block="prenorm", mixer=mixer, feed_forward=ff, mixer_norm=norm(p + "norm1"),
                                feed_forward_norm=norm(p + "norm2") if ff is not None else None, extra=extra))
    return ModelSpec(
        vocab_size=cfg.vocab, hidden_size=W,
        embedding=PartSpec("token", {"vocab_size": cfg.vocab, "hidden_size": W, "scale": cfg.embedding_scale,
                                     "name": "", "init_std": 1.0 / max(cfg.embedding_scale, 1e-3),
                                     "keep_output": loops}, "embed"),
        layers=layers, schedule=[ScheduleEntry(i) for i, _ in cfg.layer_runs()],
        final_norm=norm("final.norm"),
        head=PartSpec("linear", {"vocab_size": cfg.vocab, "hidden_size": W, "name": "", "softcap": cfg.logit_softcap,
                                 "init_std": W ** -0.5}, "head"),
    )


register_architecture(ROGIZEN_MODEL_TYPE, RogizenConfig, rogizen_model_spec)
