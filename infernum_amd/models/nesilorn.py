"""The Nesilorn decoder as a ModelSpec: latent attention with a window and an output gate, a dense or a routed
feed-forward (or none), each behind a norm that sits on the branch's output, a scaled embedding and a head tied
to the unscaled table.  Tensor names: ``embed``, ``final.norm``, ``l<i>.norm1|norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``.
"""
from __future__ import annotations

from ..config.nesilorn import NESILORN_MODEL_TYPE, NesilornConfig
from ..config.registry import register_architecture
from ..parts.base import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

EXPERT_SIGMOID_SLOPE = 1.702        # y = g sigmoid(1.702 g) (u + 1): fixed by the design


def nesilorn_model_spec(cfg: NesilornConfig, norm_init: tuple = ("normal", 0.2), init_std: float = 0.05) -> ModelSpec:
    W = cfg.width

    def norm(prefix: str) -> PartSpec:
        return PartSpec("rmsnorm", {"size": W, "eps": cfg.norm_eps, "init": norm_init, "unit_offset": True, "name": ""},
                        prefix)

    layers = []
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}.", layer.mixer
        position = {"kind": "none"}
        if m.rot_dims > 0:
            position = {"kind": "rope", "params": {"head_dim": m.rot_dim + m.kv_rank, "theta": m.rot_base,
                                                   "rotary_dim": m.rot_dims}}
        mixer = PartSpec(layer.type, {
            "hidden_size": W, "num_heads": m.heads, "head_dim": m.dim, "rot_dim": m.rot_dim, "value_dim": m.vdim,
            "rank": m.kv_rank, "norm_eps": cfg.norm_eps, "scale": m.scale, "position": position, "window": m.window,
            "gate": True, "init_std": init_std,
        }, p + "mix.")
        ff = None
        if layer.mlp is not None and layer.mlp.kind == "dense":
            ff = PartSpec("dense", {"hidden_size": W, "intermediate_size": layer.mlp.ff, "activation": "gelu_tanh",
                                    "names": ("up", "down"), "init_std": init_std}, p + "mlp.")
        elif layer.mlp is not None:
            ff = PartSpec("routed_experts", {
                "hidden_size": W, "intermediate_size": layer.mlp.ff, "num_experts": layer.mlp.experts,
                "top": layer.mlp.top, "limit": layer.mlp.limit, "alpha": EXPERT_SIGMOID_SLOPE, "router_bias": True,
                "init_std": init_std}, p + "mlp.")
        layers.append(LayerSpec(block="branchnorm", mixer=mixer, feed_forward=ff, mixer_norm=norm(p + "norm1"),
                                feed_forward_norm=norm(p + "norm2") if ff is not None else None))
    return ModelSpec(
        vocab_size=cfg.vocab, hidden_size=W,
        embedding=PartSpec("token", {"vocab_size": cfg.vocab, "hidden_size": W, "scale": cfg.embedding_scale,
                                     "name": "", "init_std": 1.0}, "embed"),
        layers=layers, schedule=[ScheduleEntry(i) for i in range(len(layers))],
        final_norm=norm("final.norm"),
        head=PartSpec("linear", {"vocab_size": cfg.vocab, "hidden_size": W, "fallback": "embed", "tied": True},
                      "head."),
    )


register_architecture(NESILORN_MODEL_TYPE, NesilornConfig, nesilorn_model_spec)
