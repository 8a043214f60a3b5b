"""Small Rogizen configurations for the tests, and a helper that writes their model folders from the plain
implementation's random weights.

R1: an attention layer with a feed-forward, then two recurrent layers (one bare, one with a feed-forward) that run
    three times; chunks of 20 positions (no multiple of the page); half of a head rotated, with scaled frequencies;
    head size 16 and 32 for the matrix-core attention kernels; capped logits.
R2: sizes that no fast kernel takes (head size 26, width 100, odd vocabulary); as many key/value heads as heads; the
    whole head rotated, plain frequencies; no mask; two taps; one norm part, as many groups as heads; no loop, no
    cap, embedding scale 1.
R3: a loop of one layer that runs twice, entered at layer 0; twenty heads over one key/value head; chunks of one
    page; a convolution of one tap (nothing carried); a recurrent layer with a state of 64 x 64 a head.
R4: the loop is the whole model and runs once; chunks of 37; no rotation at all; chunks of 1 (a query sees itself
    alone); five taps.
R5: recurrent layers only (no pages at all), the second twice; heads of 32 and 16 values and states of 48 and 16
    (sizes the chunked recurrence takes); no feed-forward anywhere.
R6: attention layers only, one tap (no state slot at all), the first three times; no mask in one, chunks of 32 in
    the other; a vocabulary larger than the width by far.
"""
import json
import os

import plain_rogizen as PR


def _attn(heads, kv_heads, dim, conv, chunk=None, rot=None, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "conv": conv,
         "scale": scale if scale is not None else dim ** -0.5}
    if rot is not None:
        m["rot"] = rot
    if chunk is not None:
        m["mask"] = {"size": chunk}
    return m


def _ssm(heads, vdim, state, groups, norm_groups, conv):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "norm_groups": norm_groups, "conv": conv}


def _layer(kind, mixer, ff=None):
    return {"type": kind, "mixer": mixer, "mlp": {"kind": "dense", "ff": ff} if ff else None}


R1 = {"architecture": "Rogizen", "vocab": 200, "width": 64, "embedding": {"scale": 3.0}, "norm": {"eps": 1e-5},
      "logit_softcap": 8.0, "loop": {"start": 1, "stop": 3, "times": 3},
      "layers": [
          _layer("attention", _attn(4, 2, 16, 3, chunk=20, rot={"base": 300.0, "dims": 8, "scaling": {
              "factor": 4.0, "original": 64, "fast": 8.0, "slow": 2.0}}), ff=96),
          _layer("mamba2", _ssm(3, 16, 8, 1, 3, 4)),
          _layer("mamba2", _ssm(4, 8, 16, 2, 2, 2), ff=40),
          _layer("attention", _attn(3, 1, 32, 2, chunk=48, rot={"base": 10000.0, "dims": 32}), None),
      ]}
R2 = {"architecture": "Rogizen", "vocab": 333, "width": 100, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-6},
      "layers": [
          _layer("mamba2", _ssm(4, 10, 5, 4, 1, 2), ff=50),
          _layer("attention", _attn(5, 5, 26, 2, rot={"base": 77.0, "dims": 26}, scale=0.3), ff=60),
          _layer("mamba2", _ssm(4, 10, 5, 4, 1, 2)),
      ]}
R3 = {"architecture": "Rogizen", "vocab": 256, "width": 128, "embedding": {"scale": 11.3}, "norm": {"eps": 3e-6},
      "logit_softcap": 25.0, "loop": {"start": 0, "stop": 1, "times": 2},
      "layers": [
          _layer("mamba2", _ssm(2, 64, 64, 2, 1, 4), ff=200),
          _layer("attention", _attn(20, 1, 32, 1, chunk=16, rot={"base": 1000000.0, "dims": 16, "scaling": {
              "factor": 16.0, "original": 32, "fast": 4.0, "slow": 0.5}}, scale=0.25), ff=72),
      ]}
R4 = {"architecture": "Rogizen", "vocab": 300, "width": 96, "embedding": {"scale": 0.625}, "norm": {"eps": 2e-6},
      "logit_softcap": 2.5, "loop": {"start": 0, "stop": 3, "times": 1},
      "layers": [
          _layer("attention", _attn(6, 3, 48, 5, chunk=37, rot={"base": 10000.0, "dims": 0}), None),
          _layer("mamba2", _ssm(6, 16, 12, 3, 6, 3), ff=160),
          _layer("attention", _attn(2, 2, 16, 3, chunk=1), ff=72),
      ]}
R5 = {"architecture": "Rogizen", "vocab": 150, "width": 80, "embedding": {"scale": 8.9}, "norm": {"eps": 1e-6},
      "logit_softcap": 20.0, "loop": {"start": 1, "stop": 2, "times": 2},
      "layers": [
          _layer("mamba2", _ssm(2, 32, 48, 1, 2, 3)),
          _layer("mamba2", _ssm(4, 16, 16, 2, 1, 4)),
      ]}
R6 = {"architecture": "Rogizen", "vocab": 1100, "width": 48, "embedding": {"scale": 6.9}, "norm": {"eps": 1e-5},
      "logit_softcap": 15.0, "loop": {"start": 0, "stop": 1, "times": 3},
      "layers": [
          _layer("attention", _attn(3, 3, 16, 1, rot={"base": 500.0, "dims": 4}), ff=64),
          _layer("attention", _attn(4, 2, 32, 1, chunk=32, rot={"base": 40000.0, "dims": 8, "scaling": {
              "factor": 6.0, "original": 128, "fast": 16.0, "slow": 1.5}}, scale=0.2), None),
      ]}
RAW = {"R1": R1, "R2": R2, "R3": R3, "R4": R4, "R5": R5, "R6": R6}
SEED = {"R1": 5, "R2": 6, "R3": 7, "R4": 15, "R5": 9, "R6": 10}


def write_model(name_or_cfg, out_dir: str, seed=None, weights=None):
    """Writes config.json and model.safetensors (bfloat16 values); returns (configuration dict, weights dict) as
    the plain implementation reads them."""
    import torch
    from infernum_amd.weights.safetensors_io import write_safetensors
    cfg = RAW[name_or_cfg] if isinstance(name_or_cfg, str) else name_or_cfg
    seed = (SEED[name_or_cfg] if isinstance(name_or_cfg, str) else 0) if seed is None else seed
    w = weights if weights is not None else PR.random_weights(cfg, seed)
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_safetensors(os.path.join(out_dir, "model.safetensors"),
                      ((n, t.to(torch.bfloat16).contiguous()) for n, t in sorted(w.items())))
    return cfg, w
