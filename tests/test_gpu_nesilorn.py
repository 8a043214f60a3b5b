"""The Nesilorn decoder on the GPU against the plain implementation (plain_nesilorn.py): each mechanism alone, then
the engine on small models of other sizes than any real one: whole prompts, the tail decoded token by token,
portions down to two tokens, mixed batches over pools so small that pages are used again (freed pages hold
NaN), keys at the windows' edges, and greedy generation through the runtime and its scheduler."""
import math

import pytest
import torch

import nesilorn_models as NM
import plain_nesilorn as PN
import trace_tools as TT
from part_harness import DEV, TOL as PART_TOL, Steps, build, dense, rel_err, runtime

pytestmark = pytest.mark.gpu
BOTH = pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
# largest |difference| of a logit as a fraction of the RMS of the plain logits (see test_gpu_engine.py)
TOL = {"float32": 2e-5, "bfloat16": 6e-2}
LENGTHS = {"N1": (1, 7, 45, 83, 130), "N2": (3, 61, 33, 97), "N3": (9, 70, 121), "N4": (2, 17, 33, 64, 150)}
MIXED = {"N1": (70, 131, 64, 150, 33, 97, 66, 81), "N2": (150, 165, 120, 190, 147), "N3": (129, 65, 90, 47, 72, 99),
         "N4": (70, 131, 64, 150, 33, 97, 66, 81)}
PAGE = {"N1": 16, "N2": 4, "N3": 8, "N4": 16}
NAMES = ["N1", "N2", "N3", "N4"]
# In bfloat16 a router's close call may fall the other way than in the plain model (its input is the rounded
# stream), and the token then takes another expert, which changes that place and, through attention, the places
# after it: places from a request's first such call on (a margin below this in the plain model) are held to be
# finite only.  The 32-bit path is held at every place, N4 (no router) in both types, and the routed layer alone
# in test_routed_experts.
CLOSE_CALL = 0.1
# bfloat16 tolerance per configuration: one and a half times what rounding alone costs the plain model (every
# stored activation rounded to bfloat16) at the places that are sure of their experts, and at least TOL's.  The
# norms on the branches bring every branch to unit size, rounding included, so the routed configurations sit
# above the 6e-2 of the Llama ones.
BF16_TOL = {}


def _x(n, h, dtype, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(n, h, generator=g) * scale
    return x.to(torch.bfloat16).float() if dtype == "bfloat16" else x


# ------------------------------------------------------------------------------------ mechanisms alone
@BOTH
@pytest.mark.parametrize("H", [64, 100, 4100])
def test_norm_on_the_branch(dtype, H):
    """h += unit_rms(delta) * (1 + w); the rounded stream comes back for the next sublayer; partial sums are added
    in the order of their index; a delta near zero shows where eps stands."""
    from infernum_amd.kernels.api import SplitSum
    rt = runtime(dtype)
    w0 = (torch.randn(H, generator=torch.Generator().manual_seed(3)) * 0.2).to(torch.bfloat16).float()
    norm, _ = build("norm", "rmsnorm", {"size": H, "eps": 1e-5, "unit_offset": True, "name": ""}, rt, {"": w0})
    h, delta = _x(7, H, "float32", 1), _x(7, H, dtype, 2, 3.0)
    delta[3] = 0.0
    delta[3, 1] = 2.0 ** -10
    hd, x = h.to(DEV).clone(), torch.empty((7, H), dtype=rt.dtype, device=DEV)
    norm.add_normed(hd, delta.to(DEV).to(rt.dtype), x)
    want = h.double() + PN.offset_norm(delta.double(), w0.double(), 1e-5)
    assert rel_err(hd, want) <= 2e-6
    assert rel_err(x, want) <= PART_TOL[dtype]
    parts = torch.stack([delta * 0.25, delta * 0.5, delta * 0.25]).to(DEV)
    hd2 = h.to(DEV).clone()
    norm.add_normed(hd2, SplitSum(parts.contiguous()), None)
    assert rel_err(hd2, want) <= 2e-6


@BOTH
def test_embedding_scale_and_the_tied_head(dtype):
    rt = runtime(dtype)
    emb, w = build("embedding", "token", {"vocab_size": 50, "hidden_size": 24, "scale": 0.3, "name": ""}, rt)
    from infernum_amd.parts.base import StepContext
    ids = torch.tensor([4, 49, 0, 4], dtype=torch.int32, device=DEV)
    z = torch.zeros(1, dtype=torch.int32, device=DEV)
    ctx = StepContext(4, 1, 0, ids, ids, ids, z, z, z, [], [], z)
    h = emb.forward(ctx)
    assert h.dtype == torch.float32
    assert rel_err(h, w[""][[4, 49, 0, 4]] * 0.3) <= 1e-6
    assert torch.equal(emb.table.cpu().double(), w[""])             # the table itself stays unscaled for the head


@BOTH
@pytest.mark.parametrize("H,I,n", [(64, 96, 5), (100, 50, 70), (256, 1024, 200)])
def test_dense_feed_forward(dtype, H, I, n):
    rt = runtime(dtype)
    ff, w = build("feed_forward", "dense", {"hidden_size": H, "intermediate_size": I, "names": ("up", "down")}, rt)
    x = _x(n, H, dtype, 4)
    got = dense(ff.forward(x.to(DEV).to(rt.dtype), None), rt)
    assert rel_err(got, PN.dense_ff(x.double(), w)) <= PART_TOL[dtype]


def test_gelu_tanh_values():
    from infernum_amd.kernels import api as K
    z = torch.linspace(-9, 9, 1001)
    got = K.activation(z.to(DEV), "gelu_tanh", torch.empty(1001, device=DEV))
    assert (got.cpu().double() - PN.gelu_tanh(z.double())).abs().max().item() <= 2e-6


@pytest.mark.parametrize("E,top,n", [(5, 2, 33), (3, 1, 7), (2, 2, 9), (64, 6, 300), (1, 1, 4)])
def test_router_choice_and_weights(E, top, n):
    from infernum_amd.kernels import api as K
    g = torch.Generator().manual_seed(E * 7 + top)
    z, b = torch.randn(n, E, generator=g) * 2, torch.randn(E, generator=g)
    ids, wt = K.router_topk(z.to(DEV), b.to(DEV), top)
    val, idx = torch.topk(z.double() + b.double(), top, dim=-1)
    assert torch.equal(ids.cpu().long(), idx)
    assert (wt.cpu().double() - torch.softmax(val, -1)).abs().max().item() <= 1e-6
    assert (wt.sum(-1).cpu() - 1).abs().max().item() <= 1e-6


@BOTH
@pytest.mark.parametrize("H,I,E,top,limit,n", [(64, 24, 5, 2, 1.5, 40), (100, 20, 3, 1, 0.5, 9), (96, 36, 2, 2, 3.0, 70),
                                               (128, 64, 16, 4, 2.0, 260), (64, 16, 8, 3, 1.0, 1),
                                               (192, 128, 4, 2, 1.5, 300), (192, 128, 4, 2, 1.5, 95)])
def test_routed_experts(dtype, H, I, E, top, limit, n):
    """Against the plain experts, with inputs large enough that the limit cuts gate and up values on both sides;
    a router whose bias alone decides (weights zero) shows the bias; every expert gets tokens, some none."""
    rt = runtime(dtype)
    ff, w = build("feed_forward", "routed_experts", {"hidden_size": H, "intermediate_size": I, "num_experts": E,
                                                     "top": top, "limit": limit}, rt, seed=E)
    x = _x(n, H, dtype, 5, 2.0)
    mlp = {"router": {"experts": E, "top": top}, "expert": {"limit": limit}}
    y = ff.forward(x.to(DEV).to(rt.dtype), None)
    assert y.parts.shape == (top, n, H) and y.parts.dtype == torch.float32
    want = PN.routed_experts(x.double(), w, mlp)
    got = y.parts.sum(0)
    # a close call of the router would change a token's experts: leave those rows out (none at these seeds in fp32)
    z = x.double() @ w["router"].t() + w["router.b"]
    srt = z.sort(-1, descending=True).values
    safe = torch.ones(n, dtype=torch.bool) if top == E else (srt[:, top - 1] - srt[:, top]) > 1e-2
    assert safe.float().mean() > 0.8
    assert rel_err(got[safe.to(DEV)], want[safe]) <= PART_TOL[dtype]
    g_all = torch.stack([x.double() @ w[f"e{e}.gate"].t() for e in range(E)])
    assert (g_all > limit).any() and (g_all.abs() < limit).any()


@pytest.mark.parametrize("counts,N,Kd", [((0, 1, 128, 129, 0, 300, 7), 200, 128), ((5,), 256, 64), ((130, 0, 0, 126), 520, 192)])
def test_grouped_product(counts, N, Kd):
    """Rows in groups of unequal size (empty ones, one row, a tile's 128 and one more), each group with a matrix of
    its own; rows behind the last group stay as they were."""
    from infernum_amd.kernels import api as K
    g = torch.Generator().manual_seed(len(counts) + N)
    rows = sum(counts) + 3
    x = (torch.randn(rows, Kd, generator=g)).to(torch.bfloat16)
    w = (torch.randn(len(counts), N, Kd, generator=g) / Kd ** 0.5).to(torch.bfloat16)
    at = torch.tensor([0] + list(torch.tensor(counts).cumsum(0)), dtype=torch.int32)
    out = torch.full((rows, N), 7.0, dtype=torch.bfloat16, device=DEV)
    K.gemm_mfma_grouped(x.to(DEV), w.to(DEV), at.to(DEV), out)
    for i, n in enumerate(counts):
        lo = int(at[i])
        want = x[lo:lo + n].double() @ w[i].double().t()
        if n:
            assert rel_err(out[lo:lo + n], want) <= PART_TOL["bfloat16"], i
    assert torch.equal(out[sum(counts):].cpu(), torch.full((3, N), 7.0, dtype=torch.bfloat16))


def _mixer_params(m, W, eps):
    pos = {"kind": "rope", "params": {"head_dim": m["rot_dim"] + m["kv_rank"], "theta": m["rot"]["base"],
                                      "rotary_dim": m["rot"]["dims"]}}
    return {"hidden_size": W, "num_heads": m["heads"], "head_dim": m["dim"], "rot_dim": m["rot_dim"],
            "value_dim": m["vdim"], "rank": m["kv_rank"], "norm_eps": eps, "scale": m["scale"], "position": pos,
            "window": (m.get("mask") or {}).get("size")}


def _run_mixer(mixer, steps, x, cuts, rt):
    """Feeds x [T, W] of one request through the mixer in the portions ``cuts``."""
    out, p = [], 0
    for n in cuts:
        ctx, packed = steps.begin([("a", n)])
        out.append(dense(mixer.forward(x[p:p + n].to(DEV).to(rt.dtype), ctx, steps.views[0]), rt).float().cpu())
        steps.end(packed)
        p += n
    assert p == x.shape[0]
    return torch.cat(out)


@BOTH
@pytest.mark.parametrize("m,W,T", [
    (NM._mixer(3, 16, 8, 24, 24, 20), 64, 75),                       # head size 32, window inside the prompt
    (NM._mixer(5, 12, 6, 10, 20, None, base=77.0), 100, 50),          # head size 26: the plain kernels; no window
    (NM._mixer(20, 64, 32, 16, 64, 48, base=1e6, dims=16), 128, 130),  # twenty heads, part of the rotated part rotated
    (NM._mixer(2, 8, 8, 8, 8, 1), 32, 12),                            # a window of one token
])
def test_latent_attention_alone(dtype, m, W, T):
    """The mixer over a paged cache against the direct form (keys and values made head by head from the latent):
    the whole sequence at once, and in portions with single tokens between them."""
    rt = runtime(dtype)
    mixer, w = build("mixer", "latent_attention", _mixer_params(m, W, 1e-5), rt, seed=T)
    x = _x(T, W, dtype, 8)
    want = PN.latent_attention(x.double(), w, m, 1e-5)
    for cuts in ([T], [T - 9, 1, 1, 2, 1, 3, 1]):
        steps = Steps([(mixer.cache_spec(), None)], rt, page_size=4, num_pages=64, poison=True)
        got = _run_mixer(mixer, steps, x, cuts, rt)
        assert rel_err(got, want) <= PART_TOL[dtype], cuts


def _standing_out(dtype, window, T, star):
    """A mixer (two heads, pages of 4) and inputs in which token ``star``'s shared rotated key part is large and
    every later query points at it: wherever that key is visible it takes nearly all the weight."""
    rt = runtime(dtype)
    W = 32
    m = NM._mixer(2, 8, 8, 8, 16, window, base=1e8)                  # slow rotation: the alignment survives the distance
    tensors = PN.random_weights({"vocab": 4, "width": W, "layers": [{"mixer": m, "mlp": None}]}, 1)
    w = {k[len("l0.mix."):]: v for k, v in tensors.items() if k.startswith("l0.mix.")}
    # both heads' rotated query rows are the rotated key rows of the down projection: q_rot(x) = r(x)
    for h in range(2):
        w["q"][h * 16 + 8:h * 16 + 16] = w["dkv"][16:24]
    mixer, w = build("mixer", "latent_attention", _mixer_params(m, W, 1e-5), rt, tensors=w)
    x = _x(T, W, dtype, 3, 0.3)
    # later queries lean towards the star's rotated key part, by a step u that leaves their latents as they are:
    # (latent rows of the down projection) u = 0, (rotated key rows) u = 8 r(x_star)
    A = w["dkv"].double()
    u = torch.linalg.pinv(A) @ torch.cat([torch.zeros(16, dtype=torch.float64), 8.0 * (A[16:] @ x[star].double())])
    x[star + 1:] = x[star + 1:] + u.float()
    x[star] = x[star] * 24.0
    if dtype == "bfloat16":
        x = x.to(torch.bfloat16).float()
    return rt, mixer, w, m, x


@BOTH
@pytest.mark.parametrize("window", [5, 16, 17, 21])
def test_a_key_that_stands_out_at_the_windows_edge(dtype, window):
    """The rows just inside the window of the key that stands out (distance window - 1) follow it, the rows just
    outside (distance window) must not see it.  Whole, and with the edge rows decoded one by one across pages of 4."""
    T, star = 64, 9
    rt, mixer, w, m, x = _standing_out(dtype, window, T, star)
    want = PN.latent_attention(x.double(), w, m, 1e-5)
    without = PN.latent_attention(x.double(), w, dict(m, mask={"size": window - 1}), 1e-5)
    inside, outside = star + window - 1, star + window
    assert (want[inside] - without[inside]).abs().max() > 10 * PART_TOL["bfloat16"] * want.pow(2).mean().sqrt()   # it shows
    for cuts in ([T], [star + window - 3] + [1] * 6 + [T - star - window - 3]):
        steps = Steps([(mixer.cache_spec(), None)], rt, page_size=4, num_pages=32, poison=True)
        got = _run_mixer(mixer, steps, x, cuts, rt)
        assert rel_err(got[[inside, outside]], want[[inside, outside]]) <= PART_TOL[dtype], cuts
        assert rel_err(got, want) <= PART_TOL[dtype], cuts


@BOTH
def test_a_far_key_among_hundreds(dtype):
    """Without a window, a key 600 places back that stands out must still be seen: in a prompt, in the portion
    after it, and by tokens decoded one by one."""
    T, star = 640, 3
    rt, mixer, w, m, x = _standing_out(dtype, None, T, star)
    want = PN.latent_attention(x.double(), w, m, 1e-5)
    without = PN.latent_attention(x.double(), w, dict(m, mask={"size": T - 40}), 1e-5)
    assert (want[T - 1] - without[T - 1]).abs().max() > 10 * PART_TOL["bfloat16"] * want.pow(2).mean().sqrt()
    for cuts in ([T], [300, T - 300 - 5] + [1] * 5):
        steps = Steps([(mixer.cache_spec(), None)], rt, page_size=4, num_pages=192, poison=True)
        got = _run_mixer(mixer, steps, x, cuts, rt)
        assert rel_err(got[-8:], want[-8:]) <= PART_TOL[dtype], cuts
        # scores of some tens under the key that stands out: bfloat16 rounds them by a tenth, which the rows
        # where it competes with near keys show in their weights
        assert rel_err(got, want) <= PART_TOL[dtype] * (2 if dtype == "bfloat16" else 1), cuts


# ------------------------------------------------------------------------------------ the engine
@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name in NAMES:
        d = str(tmp_path_factory.mktemp(name))
        cfg, w = NM.write_model(name, d)
        reqs = TT.make_requests(cfg["vocab"], LENGTHS[name], seed=11)
        mreqs = TT.make_requests(cfg["vocab"], MIXED[name], seed=23)
        out[name] = (d, cfg, w, reqs, {r: _plain(cfg, w, t) for r, t in reqs.items()},
                     mreqs, {r: _plain(cfg, w, t) for r, t in mreqs.items()})
        cost = 0.0
        for group, refs in ((reqs, out[name][4]), (mreqs, out[name][6])):
            for r, t in group.items():
                if refs[r].sure:
                    rounded = PN.forward(cfg, w, t, dtype=torch.float32, round_to=torch.bfloat16).double()
                    d = (rounded - refs[r].logits)[:refs[r].sure].abs().max().item()
                    cost = max(cost, d / refs[r].logits.pow(2).mean().sqrt().item())
        BF16_TOL[name] = max(TOL["bfloat16"], 1.5 * cost)
        print(f"{name}: rounding alone costs {cost:.2e} of the logits' RMS")
    return out


class _Ref:
    """Plain logits of a request and the number of its places before a router's first close call."""

    def __init__(self, logits, sure):
        self.logits, self.sure = logits, sure


def _plain(cfg, w, toks):
    margins = []
    logits = PN.forward(cfg, w, toks, margins=margins)
    close = torch.zeros(len(toks), dtype=torch.bool)
    for m in margins:
        close |= m < CLOSE_CALL
    return _Ref(logits, int(close.nonzero()[0]) if close.any() else len(toks))


def _engine(model_dir, dtype, page_size, num_pages, **kw):
    from infernum_amd import CacheConfig, Engine
    return Engine.from_pretrained(model_dir, dtype=dtype, **kw,
                                  cache_config=CacheConfig(page_size=page_size, num_pages=num_pages,
                                                           num_state_slots=8, poison_freed_pages=True))


def _check(got, ref, dtype, what, name=None):
    tol = BF16_TOL.get(name, TOL[dtype]) if dtype == "bfloat16" else TOL[dtype]
    if not isinstance(next(iter(ref.values())), _Ref):
        ref = {r: _Ref(t, t.shape[0]) for r, t in ref.items()}
    assert len(got) == sum(v.logits.shape[0] for v in ref.values()) and all(torch.isfinite(t).all() for t in got.values())
    if dtype == "bfloat16":
        got = {(r, p): t for (r, p), t in got.items() if p < ref[r].sure}
        assert len(got) >= 10, "too few places are sure of their experts"
    ref = {r: v.logits for r, v in ref.items()}
    worst, rms, where = TT.error_against(got, ref, every_place=dtype != "bfloat16")
    print(f"{what}: max|diff| = {worst:.3e}, rms of logits = {rms:.3e}, ratio {worst / rms:.2e} at {where}")
    assert worst == worst, f"{what}: NaN in the logits at {where}"
    assert worst <= tol * rms, f"{what}: max|diff| {worst:.3e} > {tol} * rms {rms:.3e} at {where}"


@BOTH
@pytest.mark.parametrize("name", NAMES)
def test_layers_one_by_one(models, name, dtype):
    """The residual stream after every layer (the engine cut after k layers is a model of its own here: the
    same files, a configuration with the first k layers)."""
    import json
    import os
    import shutil
    d, cfg, w, reqs, *_ = models[name]
    toks = reqs["r2"]
    layers, margins = [], []
    PN.forward(cfg, w, toks, layers_out=layers, margins=margins)
    routed = [i for i, l in enumerate(cfg["layers"]) if l["mlp"] is not None and l["mlp"]["kind"] == "moe"
              and l["mlp"]["router"]["top"] < l["mlp"]["router"]["experts"]]
    sure = torch.ones(len(toks), dtype=torch.bool)
    for k in range(1, len(cfg["layers"]) + 1):
        sub = dict(cfg, layers=cfg["layers"][:k])
        sd = d + f"_first{k}"
        NM.write_model(sub, sd, weights={n: t for n, t in w.items() if not n.startswith("l") or int(n[1:n.index(".")]) < k})
        eng = _engine(sd, dtype, PAGE[name], 64)
        from infernum_amd.engine import StepEntry
        logits = eng.step([StepEntry("a", toks, list(range(len(toks))))]).cpu().double()
        E = w["embed"].double()
        want = PN.offset_norm(layers[k - 1], w["final.norm"].double(), cfg["norm"]["eps"]) @ E.t()
        if dtype == "bfloat16" and k - 1 in routed:
            close = margins[routed.index(k - 1)] < CLOSE_CALL
            sure &= ~(torch.cumsum(close.int(), 0) > 0)               # from a close call on, the places after it too
        err = (logits - want)[sure].abs().max().item() / want.pow(2).mean().sqrt().item()
        print(f"{name} {dtype} after layer {k}: {err:.2e} over {int(sure.sum())} places")
        assert err <= (BF16_TOL[name] if dtype == "bfloat16" else TOL[dtype])
        shutil.rmtree(sd, ignore_errors=True)


@BOTH
@pytest.mark.parametrize("name", NAMES)
@pytest.mark.parametrize("how", ["whole", "tail", "portions"])
def test_one_request_at_a_time(models, name, dtype, how):
    d, cfg, w, reqs, ref, *_ = models[name]
    eng = _engine(d, dtype, PAGE[name], 64)
    steps = {"whole": TT.trace_whole, "tail": lambda r: TT.trace_tail_one_by_one(r, 40), "portions": TT.trace_portions}[how](reqs)
    got = TT.run_steps(eng, steps)
    _check(got, ref, dtype, f"{name} {dtype} {how}", name)
    eng.cache.check()
    assert all(eng.cache.free_pages(g) == 64 for g in range(len(eng.cache.groups)))
    if eng.program is not None:
        eng.program.check_guards()
        assert eng.program.num_python_ops == 0             # every part wrote its own launches


@BOTH
@pytest.mark.parametrize("name", NAMES)
def test_mixed_batches_with_pages_used_again(models, name, dtype):
    d, cfg, w, _, _, reqs, ref = models[name]
    prompt_len = {r: max(2, len(t) - 20 - 7 * i) for i, (r, t) in enumerate(reqs.items())}
    steps, max_tokens = TT.trace_mixed(reqs, prompt_len, seed=5)
    ps = PAGE[name]
    eng = _engine(d, dtype, ps, max_tokens // ps)
    assert sum(-(-len(t) // 64) * 64 for t in reqs.values()) > max_tokens   # the pool cannot hold them all: pages come back
    got = TT.run_steps(eng, steps)
    _check(got, ref, dtype, f"{name} {dtype} mixed", name)
    eng.cache.check()
    if dtype == "float32":
        # the same rows from a batch and alone, bit for bit in the 32-bit path
        alone = TT.run_steps(_engine(d, dtype, ps, 64), TT.trace_whole(reqs))
        assert all(torch.equal(got[k], alone[k]) for k in got)


@BOTH
def test_long_decoding_past_every_window(models, dtype):
    """A short prompt, then 150 tokens one by one: every window passes over decoded tokens and the window groups
    give pages back on the way; decode steps are replayed from graphs after the first two."""
    d, cfg, w, *_ = models["N1"]
    toks = TT.make_requests(cfg["vocab"], (160,), seed=3)["r0"]
    ref = {"r0": _plain(cfg, w, toks)}
    eng = _engine(d, dtype, 16, 12)
    got = TT.run_steps(eng, TT.trace_tail_one_by_one({"r0": toks}, 150))
    _check(got, ref, dtype, f"N1 {dtype} long decoding", "N1")
    assert eng.graph_replays > 100


def test_greedy_generation_through_the_scheduler(models):
    """Runtime.generate_batch (scheduler, portions, the sampler's argmax) against the plain model's greedy tokens,
    in 32-bit; prompts of unequal length, more requests than run at once."""
    from infernum_amd import BatchConfig, GenerateOptions, Runtime
    d, cfg, w, *_ = models["N1"]
    prompts = list(TT.make_requests(cfg["vocab"], (5, 31, 2, 18, 9), seed=9).values())
    rt = Runtime.from_pretrained(d, dtype="float32", batch_config=BatchConfig(block_size=16, num_blocks=24,
                                                                              max_batch_size=3, max_prefill_tokens=8,
                                                                              max_tokens_per_step=16, step_token_multiple=1))
    outs = rt.generate_batch(prompts, GenerateOptions(max_new_tokens=12))
    for p, got in zip(prompts, outs):
        toks = list(p)
        for _ in range(12):
            toks.append(int(PN.forward(cfg, w, toks)[-1].argmax()))
        assert list(got) == toks[len(p):], (p, got, toks[len(p):])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_and_generate_programs(models, tmp_path, dtype):
    """bin/trace_run and bin/generate as a user starts them, on a Nesilorn folder: the model class comes from
    config.json; steps on standard input, logits in files; generated tokens on standard output."""
    import json
    import os
    import subprocess
    import sys
    import numpy as np
    d, cfg, w, _, _, reqs, ref = models["N4"]
    prompt_len = {r: max(2, len(t) - 12) for r, t in reqs.items()}
    steps, max_tokens = TT.trace_mixed(reqs, prompt_len, seed=4)
    out = tmp_path / "out"
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", d, "--dtype", dtype,
                           "--out", str(out), "--max-tokens", str(max_tokens)],
                          input="".join(json.dumps(s) + "\n" for s in steps), text=True, capture_output=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    assert proc.stdout.split("\n")[:-1] == [f"done {s['step']}" for s in steps]
    pos, got = {}, {}
    for s in steps:
        n_want = sum(len(e["want"]) for e in s["entries"])
        arr = np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(n_want, cfg["vocab"])
        row = 0
        for e in s["entries"]:
            base = pos.get(e["id"], 0)
            for k in e["want"]:
                got[(e["id"], base + k)] = torch.from_numpy(arr[row].copy())
                row += 1
            pos[e["id"]] = base + len(e["tokens"])
    _check(got, ref, dtype, f"trace_run N4 {dtype} mixed", "N4")
    if dtype == "float32":
        prompt = reqs["r4"][:9]
        gen = subprocess.run([sys.executable, os.path.join(root, "bin", "generate"), "-m", d, "--prompt-ids",
                              ",".join(map(str, prompt)), "-n", "6", "--greedy", "--dtype", "float32"],
                             text=True, capture_output=True, timeout=600)
        assert gen.returncode == 0, gen.stderr[-3000:]
        toks = list(prompt)
        for _ in range(6):
            toks.append(int(PN.forward(cfg, w, toks)[-1].argmax()))
        assert " " + " ".join(map(str, toks[9:])) + "\n" in gen.stdout, gen.stdout[-2000:]
