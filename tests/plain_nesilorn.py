"""A plain, slow Nesilorn decoder: whole sequences, no cache, one function per mechanism.

It shares no code with infernum_amd: the configuration is a plain dict (the
parsed config.json), the weights a dict name -> CPU tensor.  Everything is
computed in ``dtype`` (float64 by default) on the CPU; with ``round_to`` the
places where the engine keeps bfloat16 (inputs of matrix products, stored
activations, the cache) are rounded so, which gives a model of rounding alone.

Notation: W width, T tokens of one sequence, positions 0 .. T-1.
  layer:    x <- x + N1(mixer(x));  x <- x + N2(ff(x))        (the norm sits on the branch, not in front)
  N(y)      = y / sqrt(mean(y^2) + eps) * (1 + w)
  mixer:    latent attention, see ``latent_attention``
  ff:       dense  D gelu_tanh(U x), or routed experts, see ``routed_experts``
  logits    = E N_final(x)   with E the embedding table (unscaled);  x_0 = E[token] * s
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import torch


def _r(x: torch.Tensor, round_to: Optional[torch.dtype]) -> torch.Tensor:
    return x if round_to is None else x.to(round_to).to(x.dtype)


def unit_rms(y: torch.Tensor, eps: float) -> torch.Tensor:
    return y / torch.sqrt((y * y).mean(dim=-1, keepdim=True) + eps)


def offset_norm(y: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """Weight stored around zero: unit_rms(y) * (1 + w)."""
    return unit_rms(y, eps) * (1.0 + w)


def plain_weight_norm(y: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return unit_rms(y, eps) * w


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rotate_half_split(v: torch.Tensor, positions: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """v [T, ..., n]: the first ``dims`` values of the last axis are rotated, value i with value i + dims/2, by
    the angle p * base^(-2i/dims); the rest pass."""
    half = dims // 2
    i = torch.arange(half, dtype=torch.float64)
    f = torch.as_tensor(float(base), dtype=torch.float64) ** (-2.0 * i / dims)
    a = positions.to(torch.float64)[:, None] * f[None, :]                       # [T, half]
    shape = [v.shape[0]] + [1] * (v.dim() - 2) + [half]
    cs, sn = torch.cos(a).to(v.dtype).reshape(shape), torch.sin(a).to(v.dtype).reshape(shape)
    u, w = v[..., :half], v[..., half:dims]
    return torch.cat([u * cs - w * sn, w * cs + u * sn, v[..., dims:]], dim=-1)


def visible(T: int, window: Optional[int]) -> torch.Tensor:
    """[T, T] bool: query i sees key j when 0 <= i - j (< window)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if window:
        ok &= (i - j) < window
    return ok


def latent_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float,
                     round_to: Optional[torch.dtype] = None, positions: Optional[torch.Tensor] = None) -> torch.Tensor:
    """h [T, W] -> [T, W].  ``w``: the mixer's tensors by their local names (q, dkv, dkv.norm, uk, uv, g, o).
    Keys and values are formed head by head from the latent, the direct way."""
    T = h.shape[0]
    H, dn, dr, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T) if positions is None else positions
    hr = _r(h, round_to)
    q = _r(hr @ w["q"].t(), round_to).view(T, H, dn + dr)
    low = _r(hr @ w["dkv"].t(), round_to)
    c = _r(plain_weight_norm(low[:, :rank], w["dkv.norm"], eps), round_to)          # [T, rank]
    k_rot = low[:, rank:rank + dr]                                                  # [T, dr], one for all heads
    rot = m["rot"]
    q_rot = _r(rotate_half_split(q[..., dn:], pos, rot["base"], rot["dims"]), round_to)
    k_rot = _r(rotate_half_split(k_rot, pos, rot["base"], rot["dims"]), round_to)
    k_plain = _r(c @ w["uk"].t(), round_to).view(T, H, dn)
    v = _r(c @ w["uv"].t(), round_to).view(T, H, dv)
    s = torch.einsum("ihd,jhd->hij", q[..., :dn], k_plain) + torch.einsum("ihd,jd->hij", q_rot, k_rot)
    s = s * m["scale"]
    window = (m.get("mask") or {}).get("size")
    s = s.masked_fill(~visible(T, window)[None], float("-inf"))
    p = torch.softmax(s, dim=-1)
    o = torch.einsum("hij,jhd->ihd", p, v).reshape(T, H * dv)
    gate = torch.sigmoid(_r(hr @ w["g"].t(), round_to))
    o = _r(_r(o, round_to) * gate, round_to)
    return _r(o @ w["o"].t(), round_to)


def dense_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], round_to: Optional[torch.dtype] = None) -> torch.Tensor:
    hr = _r(h, round_to)
    return _r(_r(gelu_tanh(_r(hr @ w["up"].t(), round_to)), round_to) @ w["down"].t(), round_to)


def route(h: torch.Tensor, w_router: torch.Tensor, bias: torch.Tensor, top: int):
    """-> chosen experts [T, top] and their weights: softmax over the chosen logits only."""
    z = h @ w_router.t() + bias
    val, idx = torch.topk(z, top, dim=-1)
    return idx, torch.softmax(val, dim=-1)


def expert(h: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor, limit: float,
           round_to: Optional[torch.dtype] = None) -> torch.Tensor:
    g = torch.clamp(_r(h @ gate.t(), round_to), max=limit)
    u = torch.clamp(_r(h @ up.t(), round_to), min=-limit, max=limit)
    y = _r(g * torch.sigmoid(1.702 * g) * (u + 1.0), round_to)
    return _r(y @ down.t(), round_to)


def routed_experts(h: torch.Tensor, w: Dict[str, torch.Tensor], mlp: dict,
                   round_to: Optional[torch.dtype] = None, margins: Optional[List[torch.Tensor]] = None) -> torch.Tensor:
    """``margins`` collects, per token, by how much the last chosen logit beats the first that is not chosen."""
    hr = _r(h, round_to)
    E, top, limit = mlp["router"]["experts"], mlp["router"]["top"], mlp["expert"]["limit"]
    idx, wt = route(hr, w["router"], w["router.b"], top)
    if margins is not None and top < E:
        z = (hr @ w["router"].t() + w["router.b"]).sort(dim=-1, descending=True).values
        margins.append(z[:, top - 1] - z[:, top])
    out = torch.zeros_like(h)
    for e in range(E):
        rows, slot = (idx == e).nonzero(as_tuple=True)
        if rows.numel() == 0:
            continue
        y = expert(hr[rows], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"], limit, round_to)
        out.index_add_(0, rows, y * wt[rows, slot][:, None])
    return _r(out, round_to)


def _local(weights: Dict[str, torch.Tensor], prefix: str, dtype) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v.to(dtype) for k, v in weights.items() if k.startswith(prefix)}


def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens: Sequence[int], dtype=torch.float64,
            round_to: Optional[torch.dtype] = None, layers_out: Optional[List[torch.Tensor]] = None,
            margins: Optional[List[torch.Tensor]] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence; ``layers_out`` collects the residual stream after every layer,
    ``margins`` the routers' margins (see ``routed_experts``) of every routed layer."""
    eps = cfg["norm"]["eps"]
    E = weights["embed"].to(dtype)
    x = E[torch.as_tensor(list(tokens), dtype=torch.long)] * cfg["embedding"]["scale"]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        if layer["type"] != "latent_attention":
            raise ValueError(f"unknown mixer {layer['type']!r}")
        a = latent_attention(x, _local(weights, p + "mix.", dtype), layer["mixer"], eps, round_to)
        x = x + offset_norm(a, weights[p + "norm1"].to(dtype), eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            wl = _local(weights, p + "mlp.", dtype)
            f = dense_ff(x, wl, round_to) if mlp["kind"] == "dense" else routed_experts(x, wl, mlp, round_to, margins)
            x = x + offset_norm(f, weights[p + "norm2"].to(dtype), eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    f = _r(offset_norm(x, weights["final.norm"].to(dtype), eps), round_to)
    return f @ E.t()


# ---------------------------------------------------------------- random models for the tests
def random_weights(cfg: dict, seed: int, std: float = 0.08) -> Dict[str, torch.Tensor]:
    """Weights of a configuration drawn from a seed, at values that bfloat16 holds exactly."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def mat(*shape, s=None):
        s = s if s is not None else 1.0 / math.sqrt(shape[-1])
        return (torch.randn(*shape, generator=g) * s).to(torch.bfloat16).to(torch.float32)

    out = {"embed": mat(cfg["vocab"], W, s=1.0), "final.norm": mat(W, s=0.2)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        H, dn, dr, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
        out[p + "norm1"] = mat(W, s=0.2)
        out[p + "mix.q"] = mat(H * (dn + dr), W)
        out[p + "mix.dkv"] = mat(rank + dr, W)
        out[p + "mix.dkv.norm"] = (1.0 + mat(rank, s=0.2)).to(torch.bfloat16).to(torch.float32)
        out[p + "mix.uk"] = mat(H * dn, rank)
        out[p + "mix.uv"] = mat(H * dv, rank)
        out[p + "mix.g"] = mat(H * dv, W)
        out[p + "mix.o"] = mat(W, H * dv)
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        out[p + "norm2"] = mat(W, s=0.2)
        if mlp["kind"] == "dense":
            out[p + "mlp.up"] = mat(mlp["ff"], W)
            out[p + "mlp.down"] = mat(W, mlp["ff"])
        else:
            E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
            out[p + "mlp.router"] = mat(E, W, s=2.0 / math.sqrt(W))
            out[p + "mlp.router.b"] = mat(E, s=0.5)
            for e in range(E):
                out[p + f"mlp.e{e}.gate"] = mat(ff, W, s=2.0 / math.sqrt(W))
                out[p + f"mlp.e{e}.up"] = mat(ff, W, s=2.0 / math.sqrt(W))
                out[p + f"mlp.e{e}.down"] = mat(W, ff)
    return out
