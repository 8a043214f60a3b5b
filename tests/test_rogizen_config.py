"""The Rogizen configuration reader and model spec on the CPU, and pins of the plain implementation."""
import math

import pytest
import torch

import plain_rogizen as PR
import rogizen_models as RM
from infernum_amd import models  # noqa: F401  (registers the architectures)
from infernum_amd.config.base import ConfigError
from infernum_amd.config.registry import config_from_dict, model_spec_for
from infernum_amd.config.rogizen import RogizenConfig
from infernum_amd.models.model import DecoderModel
from infernum_amd.parts.base import Runtime
from infernum_amd.parts.rope import rope_inverse_frequencies, rope_magnitude


@pytest.mark.parametrize("name", list(RM.RAW))
def test_reads_every_key_and_writes_it_back(name):
    raw = RM.RAW[name]
    cfg = config_from_dict(raw)
    assert isinstance(cfg, RogizenConfig)
    assert cfg.to_dict() == {k: v for k, v in raw.items()}
    assert [i for i, _ in cfg.layer_runs()] == [i for i, _ in PR.layer_runs(raw)]
    assert [s for _, s in cfg.layer_runs()] == [s for _, s in PR.layer_runs(raw)]


@pytest.mark.parametrize("name", list(RM.RAW))
def test_the_spec_wants_the_tensors_of_the_file(name):
    raw = RM.RAW[name]
    model = DecoderModel(model_spec_for(config_from_dict(raw)), Runtime(torch.device("cpu"), torch.float32))
    want = {k: tuple(v.shape) for k, v in model.expected_weights().items()}
    assert want == PR.tensor_shapes(raw)
    assert len(model.spec.schedule) == len(PR.layer_runs(raw))
    # every run of a looped layer has a cache and a state of its own
    assert all(e.cache_of is None for e in model.spec.schedule)
    needs = model.cache_needs()
    for (layer, _), (cs, ss) in zip(PR.layer_runs(raw), needs):
        L = raw["layers"][layer]
        if L["type"] == "mamba2":
            m = L["mixer"]
            conv = (m["conv"] - 1) * (m["heads"] * m["vdim"] + 2 * m["groups"] * m["state"])
            assert cs is None and ss.shape == (conv + m["heads"] * m["state"] * m["vdim"],)
        else:
            m = L["mixer"]
            size = (m.get("mask") or {}).get("size")
            assert (cs.kind, cs.window) == (("chunk", size) if size else ("full", 0))
            assert (ss is None) == (m["conv"] == 1)


def test_what_a_file_does_not_mention_is_not_there():
    raw = dict(RM.R2)
    cfg = config_from_dict(raw)
    assert cfg.loop is None and cfg.logit_softcap is None
    spec = model_spec_for(cfg)
    assert "loop.in" not in DecoderModel(spec, Runtime(torch.device("cpu"), torch.float32)).expected_weights()
    assert not any(l.extra for l in spec.layers)


@pytest.mark.parametrize("change,match", [
    (lambda c: c["layers"][0]["mixer"].update(vdim=8), "vdim"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "kv_heads"),
    (lambda c: c["layers"][1]["mixer"].update(groups=2), "groups"),
    (lambda c: c["layers"][1]["mixer"].update(norm_groups=5), "norm_groups"),
    (lambda c: c["loop"].update(stop=9), "loop"),
    (lambda c: c["layers"][0].update(type="conv"), "type"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "rot.dims"),
    (lambda c: c.update(logit_softcap=-1.0), "logit_softcap"),
])
def test_refuses_what_does_not_fit(change, match):
    import copy
    raw = copy.deepcopy(RM.R1)
    change(raw)
    with pytest.raises(ConfigError, match=match):
        config_from_dict(raw)


def test_scaled_frequencies_against_the_plain_table():
    for rot in ({"base": 300.0, "dims": 8, "scaling": {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 2.0}},
                {"base": 1e6, "dims": 64, "scaling": {"factor": 16.0, "original": 4096, "fast": 32.0, "slow": 1.0}},
                {"base": 10000.0, "dims": 2, "scaling": {"factor": 2.0, "original": 8, "fast": 1.0, "slow": 1.0}}):
        sc = dict(rot["scaling"], rope_type="yarn")
        want, mag = PR.rotary_frequencies(rot)
        got = rope_inverse_frequencies(rot["dims"], rot["base"], sc)
        assert torch.allclose(got, want, rtol=1e-15, atol=0)
        assert rope_magnitude(sc) == mag == 0.1 * math.log(rot["scaling"]["factor"]) + 1.0
    # the fastest pairs keep their frequency, the slowest are divided by the factor
    f, _ = PR.rotary_frequencies({"base": 1e4, "dims": 64, "scaling": {"factor": 8.0, "original": 1024, "fast": 32.0, "slow": 1.0}})
    plain, _ = PR.rotary_frequencies({"base": 1e4, "dims": 64})
    assert f[0] == plain[0] and abs(f[-1] * 8.0 / plain[-1] - 1.0) < 1e-12


# ------------------------------------------------------------------------ pins of the plain implementation
def test_plain_convolution_token_by_token():
    g = torch.Generator().manual_seed(1)
    u, w, b = torch.randn(9, 5, generator=g).double(), torch.randn(5, 4, generator=g).double(), torch.randn(5, generator=g).double()
    y = PR.causal_conv(u, w, b)
    for t in range(9):
        want = b.clone()
        for j in range(4):
            if t - 3 + j >= 0:
                want += w[:, j] * u[t - 3 + j]
        assert torch.allclose(y[t], want, atol=1e-12)
    assert torch.equal(PR.causal_conv(u, w)[:4], PR.causal_conv(u[:4], w))          # causal


def test_plain_chunks():
    m = PR.chunk_visible(10, 4)
    assert m[3].tolist() == [True] * 4 + [False] * 6
    assert m[4].tolist() == [False] * 4 + [True] + [False] * 5
    assert m[9].tolist() == [False] * 8 + [True] * 2
    assert torch.equal(PR.chunk_visible(6, None), torch.tril(torch.ones(6, 6, dtype=torch.bool)))


def test_plain_recurrence_is_causal_and_forgets_at_its_own_rate():
    cfg = RM.R1
    w = {k: v.double() for k, v in PR.random_weights(cfg, 3).items()}
    m = cfg["layers"][1]["mixer"]
    sub = {k[len("l1.mix."):]: v for k, v in w.items() if k.startswith("l1.mix.")}
    h = torch.randn(30, cfg["width"], generator=torch.Generator().manual_seed(2)).double()
    full = PR.mamba2(h, sub, m, 1e-5)
    assert torch.allclose(full[:11], PR.mamba2(h[:11], sub, m, 1e-5), atol=1e-12)
    h2 = h.clone()
    h2[0] += 1.0
    assert (PR.mamba2(h2, sub, m, 1e-5)[-1] - full[-1]).abs().max() > 0                 # the state reaches back


def test_rotation_keeps_lengths_but_for_the_factor():
    rot = {"base": 50.0, "dims": 6, "scaling": {"factor": 4.0, "original": 16, "fast": 4.0, "slow": 1.0}}
    v = torch.randn(5, 2, 10, generator=torch.Generator().manual_seed(0)).double()
    out = PR.rotate_neighbours(v, torch.arange(5), rot)
    mag = 0.1 * math.log(4.0) + 1.0
    assert torch.allclose(out[..., :6].norm(dim=-1), v[..., :6].norm(dim=-1) * mag, rtol=1e-12)
    assert torch.equal(out[..., 6:], v[..., 6:])
    assert torch.allclose(out[0, :, :6], v[0, :, :6] * mag, rtol=1e-12)                 # position 0: no turn
