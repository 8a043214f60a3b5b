"""Small Nesilorn configurations for the tests, and a helper that writes their model folders from the plain
implementation's random weights.

N1: three layers that differ in every size: a dense, a routed and a missing feed-forward; two windows (two cache
    groups); latent head sizes 32 and 48 (multiples of 16: the matrix-core attention kernels in bfloat16).
N2: sizes that no fast kernel takes (latent head size 26, width 100, odd vocabulary); one expert of three; all of
    two experts; a window of one token (a query sees itself alone) and a layer without a mask; a scale of 1.
N4: see below.
N3: twenty heads on the one cached head (more than one tile of sixteen heads); plain query size equal to the
    latent's; rotated part partly rotated (rot.dims below rot_dim); four experts, three chosen, of sizes that
    send portions of 64 tokens and more to the grouped product and shorter ones to the tiles.
"""
import json
import os

import plain_nesilorn as PN


def _mixer(heads, dim, rot_dim, vdim, kv_rank, window, base=10000.0, dims=None, scale=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
         "scale": scale if scale is not None else (dim + rot_dim) ** -0.5,
         "rot": {"base": base, "dims": rot_dim if dims is None else dims}}
    if window is not None:
        m["mask"] = {"size": window}
    return m


def _moe(ff, experts, top, limit):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}


def _layer(mixer, mlp):
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp}


N1 = {"architecture": "Nesilorn", "vocab": 200, "width": 64, "embedding": {"scale": 0.75}, "norm": {"eps": 1e-5},
      "layers": [
          _layer(_mixer(3, 16, 8, 24, 24, 20), {"kind": "dense", "ff": 96}),
          _layer(_mixer(4, 8, 16, 8, 32, 37, base=500.0), _moe(24, 5, 2, 1.5)),
          _layer(_mixer(3, 16, 8, 24, 24, 20), None),
      ]}
N2 = {"architecture": "Nesilorn", "vocab": 333, "width": 100, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-6},
      "layers": [
          _layer(_mixer(5, 12, 6, 10, 20, 1), _moe(20, 3, 1, 0.5)),
          _layer(_mixer(2, 20, 6, 30, 20, None, base=77.0), _moe(36, 2, 2, 3.0)),
          _layer(_mixer(5, 12, 6, 10, 20, 300), {"kind": "dense", "ff": 50}),
      ]}
N3 = {"architecture": "Nesilorn", "vocab": 256, "width": 128, "embedding": {"scale": 2.5}, "norm": {"eps": 3e-6},
      "layers": [
          _layer(_mixer(20, 64, 32, 16, 64, 48, base=1000000.0, dims=16), _moe(64, 4, 3, 2.0)),
          _layer(_mixer(20, 64, 32, 16, 64, 48, base=1000000.0, dims=16), {"kind": "dense", "ff": 200}),
      ]}
# N4: no routed layer (nothing hangs on a close call of a router, so bfloat16 is held to its tolerance at every
#     place); head sizes 80 and 32 for the matrix-core attention kernels; windows at and across page borders.
N4 = {"architecture": "Nesilorn", "vocab": 300, "width": 96, "embedding": {"scale": 0.625}, "norm": {"eps": 2e-6},
      "layers": [
          _layer(_mixer(6, 16, 16, 16, 64, 32), {"kind": "dense", "ff": 160}),
          _layer(_mixer(18, 8, 8, 8, 24, 17, base=3000.0), None),
          _layer(_mixer(6, 16, 16, 16, 64, 32), {"kind": "dense", "ff": 72}),
      ]}
RAW = {"N1": N1, "N2": N2, "N3": N3, "N4": N4}
SEED = {"N1": 5, "N2": 6, "N3": 7, "N4": 8}


def write_model(name_or_cfg, out_dir: str, seed=None, weights=None):
    """Writes config.json and model.safetensors (bfloat16 values, stored as fp32 or bf16 alike exact); returns
    (configuration dict, weights dict) as the plain implementation reads them."""
    import torch
    from infernum_amd.weights.safetensors_io import write_safetensors
    cfg = RAW[name_or_cfg] if isinstance(name_or_cfg, str) else name_or_cfg
    seed = (SEED[name_or_cfg] if isinstance(name_or_cfg, str) else 0) if seed is None else seed
    w = weights if weights is not None else PN.random_weights(cfg, seed)
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_safetensors(os.path.join(out_dir, "model.safetensors"),
                      ((n, t.to(torch.bfloat16).contiguous()) for n, t in sorted(w.items())))
    return cfg, w
