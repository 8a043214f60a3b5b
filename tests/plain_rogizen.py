"""A plain, slow Rogizen decoder: whole sequences, no cache, one function per mechanism.

It shares no code with infernum_amd: the configuration is a plain dict (the parsed config.json), the weights a
dict name -> CPU tensor.  Everything is computed in ``dtype`` (float64 by default) on the CPU; with ``round_to``
the places where the engine keeps bfloat16 (inputs and results of matrix products, the convolutions and their
activations, the cache) are rounded so, which gives a model of rounding alone.

Notation: W width, T tokens of one sequence, positions p = 0 .. T-1, x the residual stream.
  layer      x <- x + mixer(N1(x));  x <- x + ff(N2(x)) when the layer has a feed-forward
  N(y)       = y / sqrt(mean(y^2) + eps) * w
  loop       layers a .. b-1 run n times with the same weights; every pass starts with x <- L [x ; e],
             e the scaled embedding rows
  mixers     ``conv_attention`` and ``mamba2``; ff: D (silu(G y) * (U y))
  logits     = c tanh(E N_final(x) / c)
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


def _r(x: torch.Tensor, round_to: Optional[torch.dtype]) -> torch.Tensor:
    return x if round_to is None else x.to(round_to).to(x.dtype)


def unit_rms(y: torch.Tensor, eps: float) -> torch.Tensor:
    return y / torch.sqrt((y * y).mean(dim=-1, keepdim=True) + eps)


def weighted_norm(y: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return unit_rms(y, eps) * w


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def causal_conv(u: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """u [T, C], w [C, taps]: y[t] = sum_j w[:, j] u[t - (taps-1) + j], with zeros before the first token."""
    T, C = u.shape
    taps = w.shape[1]
    y = torch.zeros_like(u)
    for j in range(taps):
        lag = taps - 1 - j                      # tap j meets the input lag tokens back
        if lag < T:
            y[lag:] += w[:, j] * u[:T - lag]
    return y if bias is None else y + bias


def rotary_frequencies(rot: dict) -> (torch.Tensor, float):
    """The angular frequency of every rotated pair, and the factor on both cosine and sine."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    f = [base ** (-2.0 * i / dims) for i in range(half)]
    sc = rot.get("scaling")
    if not sc:
        return torch.tensor(f, dtype=torch.float64), 1.0
    factor, original = float(sc["factor"]), float(sc["original"])

    def turn_dim(turns: float) -> float:
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(turn_dim(float(sc["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(sc["slow"]))), dims - 1)
    out = []
    for i in range(half):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f[i] / factor * ramp + f[i] * (1.0 - ramp))
    return torch.tensor(out, dtype=torch.float64), 0.1 * math.log(factor) + 1.0


def rotate_neighbours(v: torch.Tensor, positions: torch.Tensor, rot: dict) -> torch.Tensor:
    """v [T, heads, n]: of the first rot.dims values, value 2i is paired with value 2i+1."""
    dims = int(rot["dims"])
    if dims == 0:
        return v
    f, mag = rotary_frequencies(rot)
    a = positions.to(torch.float64)[:, None] * f[None, :]
    cs = (torch.cos(a) * mag).to(v.dtype)[:, None, :]
    sn = (torch.sin(a) * mag).to(v.dtype)[:, None, :]
    out = v.clone()
    e, o = v[..., 0:dims:2], v[..., 1:dims:2]
    out[..., 0:dims:2] = e * cs - o * sn
    out[..., 1:dims:2] = o * cs + e * sn
    return out


def chunk_visible(T: int, size: Optional[int]) -> torch.Tensor:
    """[T, T] bool: query i sees key j <= i of its own chunk of ``size`` positions (all j <= i without one)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if size:
        ok &= (i // size) == (j // size)
    return ok


def conv_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float,
                   round_to: Optional[torch.dtype] = None) -> torch.Tensor:
    """h [T, W] -> [T, W].  Queries and keys: projection with bias, short convolution, norm per head, rotation;
    the values are the keys as the convolution left them."""
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    pos = torch.arange(T)
    hr = _r(h, round_to)
    q = _r(hr @ w["q"].t() + w["q.b"], round_to)
    k = _r(hr @ w["k"].t() + w["k.b"], round_to)
    q = _r(causal_conv(q, w["q.conv"]), round_to).view(T, H, d)
    k = _r(causal_conv(k, w["k.conv"]), round_to).view(T, G, d)
    v = k
    rot = m.get("rot") or {"dims": 0, "base": 10000.0}
    q = rotate_neighbours(weighted_norm(q, w["q.norm"], eps), pos, rot)
    k = rotate_neighbours(weighted_norm(k, w["k.norm"], eps), pos, rot)
    q, k = _r(q, round_to), _r(k, round_to)
    mask = chunk_visible(T, (m.get("mask") or {}).get("size"))
    out = torch.zeros(T, H, d, dtype=h.dtype)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].t()) * float(m["scale"])
        s = s.masked_fill(~mask, float("-inf"))
        out[:, hd] = torch.softmax(s, dim=-1) @ v[:, g]
    out = _r(out.reshape(T, H * d), round_to)
    return _r(out @ w["o"].t() + w["o.b"], round_to)


def mamba2(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float,
           round_to: Optional[torch.dtype] = None) -> torch.Tensor:
    """h [T, W] -> [T, W].  Per head a state S [N, P] with S_t = exp(-exp(a) dt_t) S_(t-1) + dt_t B_t x_t^T and
    y_t = S_t^T C_t + D x_t; gate silu(z) before a norm in equal parts."""
    T = h.shape[0]
    nh, P, N, G, parts = m["heads"], m["vdim"], m["state"], m["groups"], m["norm_groups"]
    inner = nh * P
    hr = _r(h, round_to)
    proj = _r(hr @ w["in"].t(), round_to)
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = _r(silu(_r(causal_conv(xbc, w["conv"], w["conv.b"]), round_to)), round_to)
    x = xbc[:, :inner].view(T, nh, P)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + w["dt_bias"])                                     # [T, nh]
    decay = torch.exp(-torch.exp(w["A_log"])[None, :] * dt)              # [T, nh]
    y = torch.zeros(T, nh, P, dtype=h.dtype)
    per = nh // G
    S = torch.zeros(nh, N, P, dtype=h.dtype)                             # all heads side by side, token after token
    for t in range(T):
        Bh, Ch = B[t].repeat_interleave(per, dim=0), C[t].repeat_interleave(per, dim=0)      # [nh, N]
        S = decay[t][:, None, None] * S + dt[t][:, None, None] * Bh[:, :, None] * x[t][:, None, :]
        y[t] = (S * Ch[:, :, None]).sum(dim=1) + w["D"][:, None] * x[t]
    y = y.reshape(T, inner) * silu(z)
    y = unit_rms(y.view(T, parts, inner // parts), eps).reshape(T, inner) * w["norm"]
    return _r(_r(y, round_to) @ w["o"].t(), round_to)


def gated_feed_forward(y: torch.Tensor, w: Dict[str, torch.Tensor], round_to: Optional[torch.dtype] = None) -> torch.Tensor:
    yr = _r(y, round_to)
    a = _r(silu(yr @ w["gate"].t()) * (yr @ w["up"].t()), round_to)
    return _r(a @ w["down"].t(), round_to)


def _sub(weights: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def layer_runs(cfg: dict) -> List[tuple]:
    """(layer, starts a pass) in the order the layers run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    runs = [(i, False) for i in range(a)]
    for _ in range(times):
        runs += [(i, i == a) for i in range(a, b)]
    return runs + [(i, False) for i in range(b, n)]


def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens, dtype: torch.dtype = torch.float64,
            round_to: Optional[torch.dtype] = None, streams: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence.  ``streams``, when given, receives the residual stream after every
    layer run."""
    wt = {k: (v.to(dtype) if v.dtype.is_floating_point else v) for k, v in weights.items()}
    eps = float(cfg["norm"]["eps"])
    ids = torch.as_tensor(tokens, dtype=torch.long)
    e = wt["embed"][ids] * float((cfg.get("embedding") or {}).get("scale", 1.0))
    x = e.clone()
    for i, starts in layer_runs(cfg):
        L = cfg["layers"][i]
        if starts:
            x = _r(torch.cat([_r(x, round_to), _r(e, round_to)], dim=-1), round_to) @ wt["loop.in"].t()
        mix = {"attention": conv_attention, "mamba2": mamba2}[L["type"]]
        x = x + mix(weighted_norm(x, wt[f"l{i}.norm1"], eps), _sub(wt, f"l{i}.mix."), L["mixer"], eps, round_to)
        if L.get("mlp") is not None:
            x = x + gated_feed_forward(weighted_norm(x, wt[f"l{i}.norm2"], eps), _sub(wt, f"l{i}.mlp."), round_to)
        if streams is not None:
            streams.append(x.clone())
    y = _r(weighted_norm(x, wt["final.norm"], eps), round_to)
    logits = y @ wt["head"].t()
    cap = cfg.get("logit_softcap")
    if cap:
        logits = float(cap) * torch.tanh(logits / float(cap))
    return logits


# ------------------------------------------------------------------ random models


def tensor_shapes(cfg: dict) -> Dict[str, tuple]:
    W, V = cfg["width"], cfg["vocab"]
    out = {"embed": (V, W), "final.norm": (W,), "head": (V, W)}
    if cfg.get("loop"):
        out["loop.in"] = (W, 2 * W)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        out[p + "norm1"] = (W,)
        if L["type"] == "mamba2":
            inner, gn = m["heads"] * m["vdim"], m["groups"] * m["state"]
            out.update({p + "mix.in": (2 * inner + 2 * gn + m["heads"], W), p + "mix.conv": (inner + 2 * gn, m["conv"]),
                        p + "mix.conv.b": (inner + 2 * gn,), p + "mix.dt_bias": (m["heads"],),
                        p + "mix.A_log": (m["heads"],), p + "mix.D": (m["heads"],), p + "mix.norm": (inner,),
                        p + "mix.o": (W, inner)})
        else:
            nq, nk = m["heads"] * m["dim"], m["kv_heads"] * m["dim"]
            out.update({p + "mix.q": (nq, W), p + "mix.q.b": (nq,), p + "mix.k": (nk, W), p + "mix.k.b": (nk,),
                        p + "mix.q.norm": (m["dim"],), p + "mix.k.norm": (m["dim"],), p + "mix.q.conv": (nq, m["conv"]),
                        p + "mix.k.conv": (nk, m["conv"]), p + "mix.o": (W, m["heads"] * m["vdim"]), p + "mix.o.b": (W,)})
        if L.get("mlp") is not None:
            ff = L["mlp"]["ff"]
            out.update({p + "norm2": (W,), p + "mlp.gate": (ff, W), p + "mlp.up": (ff, W), p + "mlp.down": (W, ff)})
    return out


def random_weights(cfg: dict, seed: int = 0, store: torch.dtype = torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Weights of a size that keeps the stream of order one through every layer; rounded to ``store``."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.rsplit(".", 1)[-1]
        if name.endswith("norm") or name.endswith("norm1") or name.endswith("norm2"):
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif last == "A_log":
            t = torch.log(0.5 + 3.0 * torch.rand(shape, generator=g))
        elif last == "dt_bias":
            t = -2.0 + 2.0 * torch.rand(shape, generator=g)
        elif last == "D":
            t = 0.5 + torch.rand(shape, generator=g)
        elif last == "b":
            t = 0.3 * torch.randn(shape, generator=g)
        elif last == "conv":
            t = torch.randn(shape, generator=g) / math.sqrt(shape[1])
        elif name == "embed":
            t = torch.randn(shape, generator=g) / max(float((cfg.get("embedding") or {}).get("scale", 1.0)), 1e-3)
        elif name == "loop.in":
            t = torch.randn(shape, generator=g) / math.sqrt(shape[1] / 2)
        else:
            t = torch.randn(shape, generator=g) / math.sqrt(shape[-1])
        out[name] = t.to(store)
    return out
