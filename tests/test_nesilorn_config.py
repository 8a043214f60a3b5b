"""Nesilorn on the CPU: the configuration's keys and errors, the model spec's parts and tensor names, and the
plain implementation against itself (the direct form of latent attention against the folded one)."""
import copy

import pytest
import torch

import nesilorn_models as NM
import plain_nesilorn as PN
from infernum_amd import models  # noqa: F401  (registers the architectures)
from infernum_amd.config import ConfigError, NesilornConfig, config_from_dict, model_spec_for
from infernum_amd.weights.random_init import _cpu_model


@pytest.mark.parametrize("name", ["N1", "N2", "N3"])
def test_configuration_round_trip_and_tensor_names(name):
    raw = NM.RAW[name]
    cfg = config_from_dict(raw)
    assert isinstance(cfg, NesilornConfig) and cfg.to_dict() == raw
    assert (cfg.vocab_size, cfg.hidden_size, cfg.num_hidden_layers) == (raw["vocab"], raw["width"], len(raw["layers"]))
    model = _cpu_model(cfg, torch.float32)
    expected = model.expected_weights()
    plain = PN.random_weights(raw, 0)
    file_names = {n for n, ws in expected.items() if ws.write_when_random}
    assert file_names == set(plain)
    assert all(tuple(expected[n].shape) == tuple(plain[n].shape) for n in plain)
    assert expected["head.weight"].fallback == "embed"
    spec = model_spec_for(cfg)
    for ls, layer in zip(spec.layers, raw["layers"]):
        assert ls.block == "branchnorm" and ls.mixer.kind == "latent_attention"
        assert (ls.feed_forward is None) == (layer["mlp"] is None) == (ls.feed_forward_norm is None)
        if layer["mlp"] is not None:
            assert ls.feed_forward.kind == {"dense": "dense", "moe": "routed_experts"}[layer["mlp"]["kind"]]
    # layers with different windows land in different cache groups, equal ones share one
    windows = {(m.cache_spec().kind, m.cache_spec().window) for m in (b.mixer for b in model.blocks)}
    assert len(windows) == len({(l["mixer"].get("mask") or {}).get("size") for l in raw["layers"]})


def _broken(path, value):
    raw = copy.deepcopy(NM.N1)
    node = raw
    for k in path[:-1]:
        node = node[k]
    if value is None:
        del node[path[-1]]
    else:
        node[path[-1]] = value
    return raw


@pytest.mark.parametrize("path,value", [
    (("width",), None), (("norm",), None), (("layers",), []), (("layers", 0, "type"), "convolution"),
    (("layers", 0, "mixer", "heads"), 0), (("layers", 0, "mixer", "rot", "dims"), 10), (("layers", 0, "mixer", "rot", "dims"), 3),
    (("layers", 1, "mlp", "kind"), "sparse"), (("layers", 1, "mlp", "router", "top"), 6), (("layers", 1, "mlp", "expert", "limit"), 0.0),
    (("layers", 0, "mixer", "scale"), -1.0), (("layers", 0, "mixer", "mask", "size"), 0),
])
def test_configuration_errors_name_the_key(path, value):
    with pytest.raises(ConfigError) as e:
        config_from_dict(_broken(path, value))
    assert str(path[-1]) in str(e.value) or "layers" in str(e.value)


def test_an_unknown_design_is_refused():
    with pytest.raises(ConfigError):
        config_from_dict({"architecture": "Nesilorn2"})


def test_plain_latent_attention_direct_against_folded():
    """The plain implementation forms keys and values head by head; folding the key's up projection into the query
    and applying the value's after the mix over latents must give the same: the identity the engine rests on."""
    m = NM._mixer(3, 16, 8, 24, 24, 11)
    w = {k[len("l0.mix."):]: v.double() for k, v in
         PN.random_weights({"vocab": 4, "width": 48, "layers": [{"mixer": m, "mlp": None}]}, 2).items() if k.startswith("l0.mix.")}
    T, H, dn, dr, dv, rank = 40, 3, 16, 8, 24, 24
    h = torch.randn(T, 48, generator=torch.Generator().manual_seed(1), dtype=torch.float64)
    want = PN.latent_attention(h, w, m, 1e-5)
    pos = torch.arange(T)
    q = (h @ w["q"].t()).view(T, H, dn + dr)
    low = h @ w["dkv"].t()
    c = PN.plain_weight_norm(low[:, :rank], w["dkv.norm"], 1e-5)
    kr = PN.rotate_half_split(low[:, rank:], pos, m["rot"]["base"], m["rot"]["dims"])
    qr = PN.rotate_half_split(q[..., dn:], pos, m["rot"]["base"], m["rot"]["dims"])
    qa = torch.einsum("thd,hdr->thr", q[..., :dn], w["uk"].view(H, dn, rank))
    s = (torch.einsum("ihr,jr->hij", qa, c) + torch.einsum("ihd,jd->hij", qr, kr)) * m["scale"]
    s = s.masked_fill(~PN.visible(T, 11)[None], float("-inf"))
    mix = torch.einsum("hij,jr->ihr", torch.softmax(s, -1), c)
    o = torch.einsum("ihr,hvr->ihv", mix, w["uv"].view(H, dv, rank)).reshape(T, H * dv)
    got = (o * torch.sigmoid(h @ w["g"].t())) @ w["o"].t()
    assert (got - want).abs().max().item() <= 1e-10


def test_plain_window_and_first_tokens():
    v = PN.visible(6, 3)
    assert v[0].tolist() == [True, False, False, False, False, False]
    assert v[4].tolist() == [False, False, True, True, True, False]
    assert PN.visible(4, None)[3].tolist() == [True] * 4
    assert PN.visible(3, 1).int().tolist() == [[1, 0, 0], [0, 1, 0], [0, 0, 1]]
