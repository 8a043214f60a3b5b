"""The Rogizen decoder on the GPU against the plain implementation (plain_rogizen.py): each mechanism alone, then
the engine on small models of other sizes than any real one: whole prompts, the tail decoded token by token,
portions down to two tokens, mixed batches over pools so small that pages and state slots are used again (freed
pages hold NaN), keys at the chunks' edges, a state that reaches hundreds of tokens back, and greedy generation
through the runtime and its scheduler."""
import math

import pytest
import torch

import plain_rogizen as PR
import rogizen_models as RM
import trace_tools as TT
from part_harness import DEV, TOL as PART_TOL, Steps, build, dense, rel_err, runtime

pytestmark = pytest.mark.gpu
BOTH = pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
# largest |difference| of a logit as a fraction of the RMS of the plain logits (see test_gpu_engine.py)
TOL = {"float32": 2e-5, "bfloat16": 6e-2}
LENGTHS = {"R1": (1, 7, 45, 83, 130), "R2": (3, 61, 33, 97), "R3": (9, 70, 121), "R4": (2, 17, 38, 64, 150),
           "R5": (1, 64, 65, 200), "R6": (5, 63, 129)}
MIXED = {"R1": (70, 131, 64, 150, 33, 97, 66, 81), "R2": (150, 165, 120, 190, 147), "R3": (129, 65, 90, 47, 72, 99),
         "R4": (70, 131, 64, 150, 33, 97, 66, 81), "R5": (150, 100, 64, 190, 129, 77), "R6": (70, 131, 64, 150, 33, 97)}
PAGE = {"R1": 16, "R2": 4, "R3": 8, "R4": 16, "R5": 16, "R6": 8}
NAMES = ["R1", "R2", "R3", "R4", "R5", "R6"]
# tolerance per configuration: three times what rounding alone costs the plain model (computed in 32-bit; for
# bfloat16 with every stored activation rounded to bfloat16 besides), and at least TOL's.  The recurrent layers'
# norm over a few values that nearly cancel, and states carried over a hundred tokens, make some places sensitive.
MEASURED_TOL = {}


def _x(n, h, dtype, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(n, h, generator=g) * scale
    return x.to(torch.bfloat16).float() if dtype == "bfloat16" else x


def _measured(dtype, want, plain):
    """The tolerance of a comparison whose plain result is sensitive to rounding (a norm over a few values that
    nearly cancel, a state that holds one large value for hundreds of tokens): three times what rounding alone
    costs the plain form (``plain(torch.float32, None)`` in 32-bit, ``plain(torch.float32, torch.bfloat16)`` with
    every stored activation rounded to bfloat16), and at least the parts' usual tolerance."""
    got = plain(torch.float32, torch.bfloat16 if dtype == "bfloat16" else None)
    return max(PART_TOL[dtype], 3.0 * rel_err(got.to(torch.bfloat16) if dtype == "bfloat16" else got, want))


def _ctx(lengths, slots=None):
    """Step rows of requests with ``lengths`` new tokens each, as the kernels read them."""
    starts = [0]
    for n in lengths:
        starts.append(starts[-1] + n)
    seq = [s for s, n in enumerate(lengths) for _ in range(n)]
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)                     # noqa: E731
    return i32(seq), i32(starts), i32(slots if slots is not None else list(range(len(lengths))))


# ------------------------------------------------------------------------------------ kernels alone
@BOTH
@pytest.mark.parametrize("C,taps", [(5, 1), (70, 2), (300, 4), (64, 7), (2056, 4)])
@pytest.mark.parametrize("tap_major", [False, True])
@pytest.mark.parametrize("lens1,lens2", [((1, 9, 2), (3, 1, 6)), ((40, 30, 2), (3, 70, 65))])
def test_convolution_with_its_state(dtype, C, taps, tap_major, lens1, lens2):
    """Three requests of unequal length beside each other, fed in two steps: the second step's first rows read the
    first step's last taps-1 inputs from the slots (slots not in the order of the requests), a request shorter than
    the taps reads zeros and its own rows; biases on both sides; the input a column range of wider rows (at a
    16-byte border when the channels come in eights: the kernel of eight channels a thread, and from 64 rows on
    the one that takes four rows a thread); weights stored channel by channel or tap by tap."""
    from infernum_amd.kernels import api as K
    rt = runtime(dtype)
    g = torch.Generator().manual_seed(C + taps)
    w, b_in, b_out = torch.randn(C, taps, generator=g), torch.randn(C, generator=g), torch.randn(C, generator=g)
    lens3 = (1, 1, 1)                       # a last step of single tokens: the kernel that moves the state as it goes
    us = [_x(a + b + 1, C, dtype, 20 + i) for i, (a, b) in enumerate(zip(lens1, lens2))]
    want = [PR.silu(PR.causal_conv(u.double() + b_in.double(), w.double(), b_out.double())) for u in us]
    state = torch.zeros(8, max((taps - 1) * C, 1) + 3, device=DEV)[:, :max((taps - 1) * C, 1)]
    slots = [5, 0, 2]
    got = [[], [], []]
    w_dev = (w.t().contiguous() if tap_major else w).to(DEV)
    done = [0, 0, 0]
    for step, lens in enumerate((lens1, lens2, lens3)):
        rows = torch.cat([u[done[i]:done[i] + lens[i]] for i, u in enumerate(us)])
        done = [d + n for d, n in zip(done, lens)]
        wide = torch.full((rows.shape[0], C + 16), 7.0)
        wide[:, 8:8 + C] = rows
        u_dev = wide.to(DEV).to(rt.dtype)[:, 8:8 + C]
        seq, starts, sl = _ctx(lens, slots)
        out = torch.empty((rows.shape[0], C), dtype=rt.dtype, device=DEV)
        kw = dict(bias_in=b_in.to(DEV), bias_out=b_out.to(DEV), activation="silu", tap_major=tap_major)
        if step == 2 and taps > 1:
            twin, out2 = state.clone(), torch.empty_like(out)
            K.causal_conv(u_dev, w_dev, twin, seq, starts, sl, out2, **kw)
            K.conv_state_update(u_dev, taps, twin, starts, sl, bias_in=b_in.to(DEV))
            K.causal_conv_single(u_dev, w_dev, state, seq, sl, out, **kw)
            assert torch.equal(out, out2) and torch.equal(state, twin)          # the same bits both ways
        else:
            K.causal_conv(u_dev, w_dev, state, seq, starts, sl, out, **kw)
            if taps > 1:
                K.conv_state_update(u_dev, taps, state, starts, sl, bias_in=b_in.to(DEV))
        p = 0
        for i, n in enumerate(lens):
            got[i].append(out[p:p + n].float().cpu())
            p += n
    for i in range(3):
        assert rel_err(torch.cat(got[i]).to(rt.dtype), want[i]) <= PART_TOL[dtype], i


@BOTH
@pytest.mark.parametrize("nh,nkv,d,rot,pairing,scaled", [(4, 2, 16, 8, "neighbours", True), (5, 5, 26, 26, "neighbours", False),
                                                         (3, 1, 32, 0, "neighbours", False), (2, 1, 80, 16, "half", False),
                                                         (20, 1, 32, 16, "neighbours", True), (16, 4, 128, 64, "neighbours", True),
                                                         (3, 3, 48, 48, "neighbours", False), (2, 2, 64, 0, "neighbours", False),
                                                         (1, 1, 256, 6, "neighbours", False)])
def test_norm_and_rotation_of_queries_and_keys(dtype, nh, nkv, d, rot, pairing, scaled):
    """Queries against the plain norm and rotation at positions up to some thousands; keys in their pages, and the
    values there are the keys as they came in."""
    from infernum_amd.kernels import api as K
    from infernum_amd.parts.rope import rope_inverse_frequencies, rope_magnitude
    rt = runtime(dtype)
    N, ps, pages = 11, 4, 6
    rd = {"base": 300.0, "dims": rot}
    if scaled:
        rd["scaling"] = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 2.0}
    sc = dict(rd["scaling"], rope_type="yarn") if scaled else None
    x = _x(N, (nh + nkv) * d, dtype, nh + d)
    g = torch.Generator().manual_seed(1)
    qn, kn = torch.rand(d, generator=g) + 0.5, torch.rand(d, generator=g) + 0.5
    pos = torch.tensor([0, 1, 2, 3, 63, 64, 65, 700, 701, 4095, 5000], dtype=torch.int32)
    slots = torch.tensor([3, 0, 23, 9, 10, 11, 12, 4, 17, 5, 20], dtype=torch.int32)
    k_pages = torch.zeros(pages, nkv, ps, d, dtype=rt.dtype, device=DEV)
    v_pages = torch.zeros(pages, nkv, d, ps, dtype=rt.dtype, device=DEV)
    q = torch.empty(N, nh * d, dtype=rt.dtype, device=DEV)
    freq = rope_inverse_frequencies(rot, rd["base"], sc).to(DEV) if rot else None
    assert pairing == "neighbours" or not scaled
    K.qk_prepare(x.to(DEV).to(rt.dtype), q, nh, nkv, d, pos.to(DEV), qn.to(DEV), kn.to(DEV), 1e-5, freq, rot, pairing,
                 rope_magnitude(sc), slots.to(DEV), k_pages, v_pages, values_are_keys=True)
    xq, xk = x[:, :nh * d].double().view(N, nh, d), x[:, nh * d:].double().view(N, nkv, d)
    if pairing == "neighbours":
        turn = lambda v: PR.rotate_neighbours(v, pos.long(), rd)                      # noqa: E731
    else:                                   # value i with value i + rot/2, the plain frequencies
        def turn(v):
            f = rd["base"] ** (-torch.arange(rot // 2, dtype=torch.float64) * 2 / rot)
            a = pos.double()[:, None, None] * f
            lo, hi = v[..., :rot // 2], v[..., rot // 2:rot]
            return torch.cat([lo * a.cos() - hi * a.sin(), hi * a.cos() + lo * a.sin(), v[..., rot:]], -1)
    assert rel_err(q.view(N, nh, d), turn(PR.weighted_norm(xq, qn.double(), 1e-5))) <= PART_TOL[dtype]
    wk = turn(PR.weighted_norm(xk, kn.double(), 1e-5))
    for t in range(N):
        page, off = int(slots[t]) // ps, int(slots[t]) % ps
        assert rel_err(k_pages[page, :, off], wk[t]) <= PART_TOL[dtype]
        assert torch.equal(v_pages[page, :, :, off].float().cpu(), x[t, nh * d:].view(nkv, d))


def _plain_recurrence(x, Bm, Cm, dt_raw, dt_bias, a_log, skip, S0):
    """x [T, nh, P], Bm and Cm [T, G, N], dt_raw [T, nh], S0 [nh, N, P], all float64: (y [T, nh, P], S after T)."""
    T, nh, P = x.shape
    per = nh // Bm.shape[1]
    dt = PR.softplus(dt_raw + dt_bias)
    decay = torch.exp(-torch.exp(a_log)[None, :] * dt)
    S, y = S0.clone(), torch.zeros(T, nh, P, dtype=torch.float64)
    for t in range(T):
        Bh, Ch = Bm[t].repeat_interleave(per, 0), Cm[t].repeat_interleave(per, 0)
        S = decay[t][:, None, None] * S + dt[t][:, None, None] * Bh[:, :, None] * x[t][:, None, :]
        y[t] = (S * Ch[:, :, None]).sum(1) + skip[:, None] * x[t]
    return y, S


@pytest.mark.parametrize("nh,P,Ns,G", [(4, 32, 48, 2), (2, 16, 16, 1), (3, 64, 128, 3), (8, 32, 80, 2), (1, 16, 112, 1)])
@pytest.mark.parametrize("kernel", ["token_by_token", "chunks"])
def test_recurrence_over_requests_of_unequal_length(nh, P, Ns, G, kernel):
    """Requests of 1, 63, 64, 65, 130 and 200 tokens in one step, each from a state that is not zero, in slots out of
    order: outputs and the states left behind, against the plain recurrence.  Both kernels: token after token, and
    matrix products over chunks of 64 (a chunk's last row, the first of the next, a partial last chunk, a single
    token).  One head forgets slowly, so that the state a chunk hands on carries weight."""
    from infernum_amd.kernels import api as K
    lens, slots = (1, 63, 64, 65, 130, 200), [4, 0, 6, 1, 3, 5]
    T, cd = sum(lens), nh * P + 2 * G * Ns
    g = torch.Generator().manual_seed(nh * 100 + Ns)
    xbc = (torch.randn(T, cd, generator=g) * 0.7).to(torch.bfloat16)
    dt_raw = torch.randn(T, nh + 3, generator=g).to(torch.bfloat16)[:, :nh]
    dt_bias, a_log, skip = torch.rand(nh, generator=g) - 1.0, torch.rand(nh, generator=g) * 2 - 1.0, torch.rand(nh, generator=g) + 0.5
    a_log[0] = -6.0
    state0 = torch.randn(7, nh * Ns * P + 5, generator=g)
    state = state0.to(DEV)[:, 2:2 + nh * Ns * P]
    assert K.ssd_chunked_takes(torch.bfloat16, nh, P, Ns, G, cd)
    seq, starts, sl = _ctx(lens, slots)
    y = torch.full((T, nh * P), 7.0, device=DEV)
    run = K.ssd_chunked if kernel == "chunks" else K.ssd_scan
    run(xbc.to(DEV), dt_raw.to(DEV), dt_bias.to(DEV), a_log.to(DEV), skip.to(DEV), state, y, starts, sl, nh, P, Ns, G)
    p = 0
    for n, slot in zip(lens, slots):
        rows = xbc[p:p + n].double()
        want, S = _plain_recurrence(rows[:, :nh * P].view(n, nh, P), rows[:, nh * P:nh * P + G * Ns].view(n, G, Ns),
                                    rows[:, nh * P + G * Ns:].view(n, G, Ns), dt_raw[p:p + n].double(), dt_bias.double(),
                                    a_log.double(), skip.double(), state0[slot, 2:2 + nh * Ns * P].double().view(nh, Ns, P))
        assert rel_err(y[p:p + n], want.view(n, -1)) <= 2e-5, (n, slot)
        assert rel_err(state[slot], S.view(-1)) <= 2e-5, (n, slot)
        p += n
    assert torch.equal(state[2].cpu(), state0[2, 2:2 + nh * Ns * P])           # a slot of no request stays


def test_sizes_the_chunked_recurrence_leaves_to_the_other_kernel():
    from infernum_amd.kernels import api as K
    assert not K.ssd_chunked_takes(torch.float32, 2, 32, 16, 1, 96)           # 32-bit steps go token after token
    assert not K.ssd_chunked_takes(torch.bfloat16, 4, 10, 32, 2, 168)          # a head of 10 values
    assert not K.ssd_chunked_takes(torch.bfloat16, 4, 16, 5, 4, 104)           # a state of 5
    assert not K.ssd_chunked_takes(torch.bfloat16, 1, 16, 256, 1, 528)         # a state past 128


@BOTH
@pytest.mark.parametrize("inner,parts,n", [(48, 3, 5), (40, 1, 70), (128, 2, 3), (96, 6, 33), (2048, 8, 4)])
def test_gate_then_norm_in_parts(dtype, inner, parts, n):
    """unit_rms(y silu(z)) w over equal parts of the row: the gate comes before the norm (the other order gives
    other numbers, which the test holds apart); a part near zero shows where eps stands."""
    from infernum_amd.kernels import api as K
    rt = runtime(dtype)
    y, z = _x(n, inner, "float32", 1, 2.0), _x(n, inner + 5, dtype, 2, 2.0)
    y[0, :inner // parts] = 2.0 ** -12
    w = torch.rand(inner, generator=torch.Generator().manual_seed(3)) + 0.5
    out = torch.empty(n, inner, dtype=rt.dtype, device=DEV)
    K.gated_group_norm(y.to(DEV), z.to(DEV).to(rt.dtype)[:, :inner], w.to(DEV), parts, 1e-5, out)
    zz = z[:, :inner].double()
    want = PR.unit_rms((y.double() * PR.silu(zz)).view(n, parts, -1), 1e-5).reshape(n, inner) * w.double()
    assert rel_err(out, want) <= PART_TOL[dtype]
    other = PR.unit_rms(y.double().view(n, parts, -1), 1e-5).reshape(n, inner) * w.double() * PR.silu(zz)
    assert rel_err(out, other) > 10 * PART_TOL[dtype]


def test_capped_logits():
    from infernum_amd.kernels import api as K
    z = torch.linspace(-200, 200, 4002).view(3, -1).contiguous()
    for cap in (2.5, 30.0):
        got = K.softcap(z.to(DEV).clone(), cap)
        assert (got.cpu().double() - cap * torch.tanh(z.double() / cap)).abs().max().item() <= 4e-6 * cap
        assert got.abs().max().item() <= cap


@BOTH
def test_entering_a_pass_through_the_matrix(dtype):
    """h <- L [h ; e] with what the layer before left unadded: the delta is added first, the sums are fp32."""
    from infernum_amd.parts.base import StepContext
    from infernum_amd.parts.embedding import EMBEDDING_OUTPUT
    rt = runtime(dtype)
    W, n = 40, 9
    part, w = build("stream_in", "concat_linear", {"hidden_size": W, "name": "in"}, rt)
    h, delta, e = _x(n, W, "float32", 1), _x(n, W, dtype, 2), _x(n, W, dtype, 3)
    z = torch.zeros(1, dtype=torch.int32, device=DEV)
    ctx = StepContext(n, 1, 0, z, z, z, z, z, z, [], [], z)
    ctx.extras[EMBEDDING_OUTPUT] = e.to(DEV).to(rt.dtype)
    hd = h.to(DEV).clone()
    part.forward(hd, delta.to(DEV).to(rt.dtype), ctx)
    assert hd.dtype == torch.float32
    s = h.double() + delta.double()
    if dtype == "bfloat16":
        s = s.to(torch.bfloat16).double()
    assert rel_err(hd, torch.cat([s, e.double()], -1) @ w["in"].t()) <= (2e-5 if dtype == "float32" else 4e-3)


# ------------------------------------------------------------------------------------ the mixers alone
def _run_mixer(mixer, steps, x, cuts, rt, request="a"):
    """Feeds x [T, W] of one request through the mixer in the portions ``cuts``."""
    out, p = [], 0
    for n in cuts:
        ctx, packed = steps.begin([(request, n)])
        out.append(dense(mixer.forward(x[p:p + n].to(DEV).to(rt.dtype), ctx, steps.views[0]), rt).float().cpu())
        steps.end(packed)
        p += n
    assert p == x.shape[0]
    return torch.cat(out)


def _ssm_params(m, W, eps):
    return {"hidden_size": W, "num_heads": m["heads"], "head_dim": m["vdim"], "state_size": m["state"],
            "groups": m["groups"], "norm_groups": m["norm_groups"], "conv_taps": m["conv"], "norm_eps": eps}


def _attn_params(m, W, eps):
    position = {"kind": "none"}
    rot = m.get("rot")
    if rot and rot["dims"]:
        sc = dict(rot["scaling"], rope_type="yarn") if rot.get("scaling") else None
        position = {"kind": "rope", "params": {"head_dim": m["dim"], "theta": rot["base"], "rotary_dim": rot["dims"],
                                               "scaling": sc, "pairing": "neighbours"}}
    return {"hidden_size": W, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"], "head_dim": m["dim"],
            "conv_taps": m["conv"], "norm_eps": eps, "position": position, "chunk": (m.get("mask") or {}).get("size"),
            "scale": m["scale"]}


@BOTH
@pytest.mark.parametrize("m,W,T", [
    (RM._ssm(3, 16, 8, 1, 3, 4), 64, 75),
    (RM._ssm(4, 10, 5, 4, 1, 2), 100, 50),            # as many groups as heads, one norm part, odd sizes
    (RM._ssm(2, 64, 64, 2, 1, 4), 128, 40),           # a state of 64 x 64 a head
    (RM._ssm(6, 16, 12, 3, 6, 1), 96, 33),            # one tap: no convolution state
    (RM._ssm(1, 200, 3, 1, 4, 3), 32, 20),            # one head, wider than a wave; a state of three
    (RM._ssm(8, 32, 128, 2, 2, 4), 256, 70),          # a state of 128
])
def test_state_space_mixer_alone(dtype, m, W, T):
    """Against the plain recurrence: whole, token by token, and in portions with single tokens between them; the
    slot starts at zero although the pool was filled with other numbers before."""
    rt = runtime(dtype)
    mixer, w = build("mixer", "mamba2", _ssm_params(m, W, 1e-5), rt, seed=T)
    x = _x(T, W, dtype, 13)
    want = PR.mamba2(x.double(), w, m, 1e-5)
    tol = _measured(dtype, want, lambda dt, rnd: PR.mamba2(x.to(dt), {k: v.to(dt) for k, v in w.items()}, m, 1e-5, rnd))
    for cuts in ([T], [1] * T, [T - 14, 1, 1, 2, 1, 3, 6]):
        steps = Steps([(None, mixer.state_spec())], rt, slots=3)
        for pool in steps.cache.state:
            pool.fill_(3.0)                                     # what an earlier request left in the slots
        got = _run_mixer(mixer, steps, x, cuts, rt)
        assert rel_err(got.to(rt.dtype), want) <= tol, cuts[:3]


@BOTH
def test_a_state_that_reaches_hundreds_of_tokens_back(dtype):
    """One head forgets slowly (decay near one) and token 3's input is large: 600 tokens later the output still
    carries it, in a prompt, in the portion after it, and in tokens decoded one by one; the other head forgets at
    once and shows nothing."""
    rt = runtime(dtype)
    m, W, T = RM._ssm(2, 16, 8, 1, 2, 3), 32, 640
    mixer, w = build("mixer", "mamba2", _ssm_params(m, W, 1e-5), rt, seed=2)
    tensors = {k: v.clone() for k, v in w.items()}
    tensors["A_log"] = torch.tensor([-9.0, 2.0], dtype=torch.float64)
    tensors["dt_bias"] = torch.tensor([-1.0, 1.0], dtype=torch.float64)
    mixer, w = build("mixer", "mamba2", _ssm_params(m, W, 1e-5), rt, tensors=tensors)
    x = _x(T, W, dtype, 5, 0.5)
    x[3] *= 8.0
    if dtype == "bfloat16":
        x = x.to(torch.bfloat16).float()
    want = PR.mamba2(x.double(), w, m, 1e-5)
    x0 = x.clone()
    x0[3] = 0.0
    tol = _measured(dtype, want, lambda dt, rnd: PR.mamba2(x.to(dt), {k: v.to(dt) for k, v in w.items()}, m, 1e-5, rnd))
    shows = (want[-8:] - PR.mamba2(x0.double(), w, m, 1e-5)[-8:]).abs().max() / want.pow(2).mean().sqrt()
    assert shows > 10 * tol, (shows, tol)
    for cuts in ([T], [300, T - 305] + [1] * 5):
        steps = Steps([(None, mixer.state_spec())], rt, slots=2)
        got = _run_mixer(mixer, steps, x, cuts, rt)
        assert rel_err(got.to(rt.dtype), want) <= tol, cuts[:2]


@BOTH
@pytest.mark.parametrize("m,W,T", [
    (RM._attn(4, 2, 16, 3, chunk=20, rot={"base": 300.0, "dims": 8, "scaling": {"factor": 4.0, "original": 64, "fast": 8.0,
                                                                             "slow": 2.0}}), 64, 75),
    (RM._attn(5, 5, 26, 2, rot={"base": 77.0, "dims": 26}, scale=0.3), 100, 50),       # the plain kernels; no mask
    (RM._attn(20, 1, 32, 1, chunk=16, rot={"base": 1e6, "dims": 16}, scale=0.25), 128, 130),   # one tap: no state
    (RM._attn(2, 2, 16, 5, chunk=1), 32, 12),                                          # a query sees itself alone
    (RM._attn(3, 1, 64, 4, chunk=37, rot={"base": 1e4, "dims": 64}), 48, 90),
])
def test_attention_with_convolved_queries_and_keys_alone(dtype, m, W, T):
    """The mixer over a paged cache and a state slot against the plain form: whole, and in portions with single
    tokens between them that cut pages, chunks and the convolution's reach."""
    rt = runtime(dtype)
    mixer, w = build("mixer", "conv_attention", _attn_params(m, W, 1e-5), rt, seed=T)
    x = _x(T, W, dtype, 8)
    want = PR.conv_attention(x.double(), w, m, 1e-5)
    for cuts in ([T], [T - 9, 1, 1, 2, 1, 3, 1], [1] * 6 + [T - 6]):
        steps = Steps([(mixer.cache_spec(), mixer.state_spec())], rt, page_size=4, num_pages=64, poison=True)
        got = _run_mixer(mixer, steps, x, cuts, rt)
        assert rel_err(got.to(rt.dtype), want) <= PART_TOL[dtype], cuts[:3]


def _standing_out(dtype, chunk, T, star, taps=3):
    """A mixer (two heads over one key head of 16, pages of 4) and inputs in which every query after token ``star``
    points at that token's key: wherever the key is visible it takes nearly all the weight, and the output is its
    value.  The keys come from a projection that does not see the direction u; the queries see u alone and answer
    it with the star's key, on top of a bias."""
    rt = runtime(dtype)
    W, d = 32, 16
    m = RM._attn(2, 1, d, taps, chunk=chunk, scale=2.0)
    cfg = {"vocab": 4, "width": W, "layers": [{"type": "attention", "mixer": m, "mlp": None}]}
    w = {k[len("l0.mix."):]: v.double() for k, v in PR.random_weights(cfg, 1).items() if k.startswith("l0.mix.")}
    g = torch.Generator().manual_seed(4)
    u = torch.randn(W, generator=g).double()
    u /= u.norm()
    w["k"] = w["k"] - (w["k"] @ u)[:, None] * u[None, :]
    w["k"] = w["k"].to(torch.bfloat16).double()
    x = _x(T, W, dtype, 3, 1.0).double()
    x = x - (x @ u)[:, None] * u[None, :]
    k = PR.causal_conv(x @ w["k"].t() + w["k.b"], w["k.conv"])
    target = PR.weighted_norm(k[star].view(1, d), w["k.norm"], 1e-5)[0]
    w["q"] = torch.cat([torch.outer(target, u)] * 2).to(torch.bfloat16).double()
    # a bias gives the rows that do not see u a query of ordinary size (a query near zero would be divided by
    # the root of eps, and 32-bit rounding of the product with it)
    w["q.b"] = (0.3 * torch.randn(2 * d, generator=g)).to(torch.bfloat16).double()
    w["q.conv"] = torch.zeros(2 * d, taps, dtype=torch.float64)
    w["q.conv"][:, -1] = 1.0
    w["q.norm"] = torch.ones(d, dtype=torch.float64)
    x[star + 1:] += u
    x = x.float()
    if dtype == "bfloat16":
        x = x.to(torch.bfloat16).float()
    mixer, w = build("mixer", "conv_attention", _attn_params(m, W, 1e-5), rt, tensors=w)
    return rt, mixer, w, m, x


@BOTH
@pytest.mark.parametrize("chunk,where", [(5, "first"), (16, "first"), (17, "first"), (21, "first"), (16, "last"), (21, "last"),
                                         (8, "middle")])
def test_a_key_that_stands_out_at_the_chunks_edge(dtype, chunk, where):
    """The key that stands out is the first, the last or a middle place of the second chunk.  The chunk's last row
    follows it (but for the chunk's own last key, which only that row and none after it sees); the next chunk's first
    row, one place on, must not.  Whole, and with the rows around the edge decoded one by one across pages of 4."""
    T = 3 * chunk + 7
    star = {"first": chunk, "last": 2 * chunk - 1, "middle": chunk + chunk // 2}[where]
    rt, mixer, w, m, x = _standing_out(dtype, chunk, T, star)
    want = PR.conv_attention(x.double(), w, m, 1e-5)
    inside, outside = 2 * chunk - 1, 2 * chunk
    rms = want.pow(2).mean().sqrt()
    # scores of some tens: bfloat16 rounds them by a tenth, which the rows where the key competes with others show
    tol = _measured(dtype, want, lambda dt, rnd: PR.conv_attention(x.to(dt), {k: v.to(dt) for k, v in w.items()}, m, 1e-5, rnd))
    for wrong in (chunk + 1, chunk - 1):          # a mask one place off shows at the edge rows
        other = PR.conv_attention(x.double(), w, dict(m, mask={"size": wrong}), 1e-5)
        assert (want[[inside, outside]] - other[[inside, outside]]).abs().max() > 5 * tol * rms
    edge = 2 * chunk
    for cuts in ([T], [edge - 3] + [1] * 6 + [T - edge - 3], [1] * T):
        steps = Steps([(mixer.cache_spec(), mixer.state_spec())], rt, page_size=4, num_pages=32, poison=True)
        got = _run_mixer(mixer, steps, x, cuts, rt)
        assert rel_err(got.to(rt.dtype), want) <= tol, cuts[:2]


@BOTH
def test_a_far_key_among_hundreds(dtype):
    """Without a mask, a key 600 places back that stands out must still be seen: in a prompt, in the portion after
    it, and by tokens decoded one by one; with chunks of 512 the same key is seen up to place 511 and not after."""
    T, star = 640, 3
    for chunk in (None, 512):
        rt, mixer, w, m, x = _standing_out(dtype, chunk, T, star)
        want = PR.conv_attention(x.double(), w, m, 1e-5)
        without = PR.conv_attention(x.double(), w, dict(m, mask={"size": 500}), 1e-5)
        row = T - 1 if chunk is None else 511
        tol = _measured(dtype, want, lambda dt, rnd: PR.conv_attention(x.to(dt), {k: v.to(dt) for k, v in w.items()}, m, 1e-5, rnd))
        assert (want[row] - without[row]).abs().max() > 5 * tol * want.pow(2).mean().sqrt()
        for cuts in ([T], [300, 209, 1, 1, 1, 1, 1, T - 514]):
            steps = Steps([(mixer.cache_spec(), mixer.state_spec())], rt, page_size=4, num_pages=192, poison=True)
            got = _run_mixer(mixer, steps, x, cuts, rt)
            assert rel_err(got.to(rt.dtype), want) <= tol, cuts[:2]


# ------------------------------------------------------------------------------------ the engine
@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name in NAMES:
        d = str(tmp_path_factory.mktemp(name))
        cfg, w = RM.write_model(name, d)
        reqs = TT.make_requests(cfg["vocab"], LENGTHS[name], seed=11)
        mreqs = TT.make_requests(cfg["vocab"], MIXED[name], seed=23)
        ref = {r: PR.forward(cfg, w, t) for r, t in reqs.items()}
        mref = {r: PR.forward(cfg, w, t) for r, t in mreqs.items()}
        for dtype, rnd in (("float32", None), ("bfloat16", torch.bfloat16)):
            cost = 0.0
            for group, refs in ((reqs, ref), (mreqs, mref)):
                for r, t in group.items():
                    rounded = PR.forward(cfg, w, t, dtype=torch.float32, round_to=rnd).double()
                    cost = max(cost, (rounded - refs[r]).abs().max().item() / refs[r].pow(2).mean().sqrt().item())
            MEASURED_TOL[name, dtype] = max(TOL[dtype], 3.0 * cost)
            print(f"{name}: {dtype} rounding alone costs {cost:.2e} of the logits' RMS")
        out[name] = (d, cfg, w, reqs, ref, mreqs, mref)
    return out


def _engine(model_dir, dtype, page_size, num_pages, slots=8, **kw):
    from infernum_amd import CacheConfig, Engine
    return Engine.from_pretrained(model_dir, dtype=dtype, **kw,
                                  cache_config=CacheConfig(page_size=page_size, num_pages=num_pages,
                                                           num_state_slots=slots, poison_freed_pages=True))


def _check(got, ref, dtype, what, name=None):
    tol = MEASURED_TOL.get((name, dtype), TOL[dtype])
    assert len(got) == sum(v.shape[0] for v in ref.values()) and all(torch.isfinite(t).all() for t in got.values())
    worst, rms, where = TT.error_against(got, ref)
    print(f"{what}: max|diff| = {worst:.3e}, rms of logits = {rms:.3e}, ratio {worst / rms:.2e} at {where}")
    assert worst == worst, f"{what}: NaN in the logits at {where}"
    assert worst <= tol * rms, f"{what}: max|diff| {worst:.3e} > {tol} * rms {rms:.3e} at {where}"


def _first_layers(cfg, k):
    """The model of the first k layers: a loop that reaches past them ends there, one that starts past them is gone."""
    sub = dict(cfg, layers=cfg["layers"][:k])
    loop = cfg.get("loop")
    if loop:
        if loop["start"] >= k:
            sub.pop("loop")
        else:
            sub["loop"] = dict(loop, stop=min(loop["stop"], k))
    return sub


@BOTH
@pytest.mark.parametrize("name", NAMES)
def test_layers_one_by_one(models, name, dtype):
    """The logits of the models made of the first k layers (the same tensors), k = 1, 2, ...: a layer that differs
    shows at its own k."""
    import shutil
    from infernum_amd.engine import StepEntry
    d, cfg, w, reqs, *_ = models[name]
    toks = reqs["r2"]
    for k in range(1, len(cfg["layers"]) + 1):
        sub, sd = _first_layers(cfg, k), d + f"_first{k}"
        keep = {n: t for n, t in w.items() if not (n[0] == "l" and n[1].isdigit()) or int(n[1:n.index(".")]) < k}
        if "loop" not in sub:
            keep.pop("loop.in", None)
        RM.write_model(sub, sd, weights=keep)
        eng = _engine(sd, dtype, PAGE[name], 64)
        logits = eng.step([StepEntry("a", toks, list(range(len(toks))))]).cpu().double()
        want = PR.forward(sub, keep, toks)
        err = (logits - want).abs().max().item() / want.pow(2).mean().sqrt().item()
        print(f"{name} {dtype} first {k} layers: {err:.2e}")
        assert err <= MEASURED_TOL[name, dtype]
        shutil.rmtree(sd, ignore_errors=True)


@BOTH
@pytest.mark.parametrize("name", NAMES)
@pytest.mark.parametrize("how", ["whole", "tail", "portions", "one_by_one"])
def test_one_request_at_a_time(models, name, dtype, how):
    d, cfg, w, reqs, ref, *_ = models[name]
    eng = _engine(d, dtype, PAGE[name], 64)
    steps = {"whole": TT.trace_whole, "tail": lambda r: TT.trace_tail_one_by_one(r, 40), "portions": TT.trace_portions,
             "one_by_one": lambda r: TT.trace_tail_one_by_one(r, 10 ** 6)}[how](reqs)
    got = TT.run_steps(eng, steps)
    _check(got, ref, dtype, f"{name} {dtype} {how}", name)
    eng.cache.check()
    assert all(eng.cache.free_pages(g) == 64 for g in range(len(eng.cache.groups)))
    if eng.program is not None:
        eng.program.check_guards()
        assert eng.program.num_python_ops == 0             # every part wrote its own launches


@BOTH
@pytest.mark.parametrize("name", NAMES)
def test_mixed_batches_with_pages_and_slots_used_again(models, name, dtype):
    d, cfg, w, _, _, reqs, ref = models[name]
    prompt_len = {r: max(2, len(t) - 20 - 7 * i) for i, (r, t) in enumerate(reqs.items())}
    steps, max_tokens = TT.trace_mixed(reqs, prompt_len, seed=5)
    ps = PAGE[name]
    eng = _engine(d, dtype, ps, max_tokens // ps, slots=4)          # four slots for up to four live of more requests
    assert sum(-(-len(t) // 64) * 64 for t in reqs.values()) > max_tokens   # the pool cannot hold them all: pages come back
    assert len(reqs) > 4
    got = TT.run_steps(eng, steps)
    _check(got, ref, dtype, f"{name} {dtype} mixed", name)
    eng.cache.check()
    if dtype == "float32":
        # the same rows from a batch and alone, bit for bit in the 32-bit path
        alone = TT.run_steps(_engine(d, dtype, ps, 64), TT.trace_whole(reqs))
        assert all(torch.equal(got[k], alone[k]) for k in got)


@BOTH
def test_long_decoding_past_every_chunk(models, dtype):
    """A short prompt, then 150 tokens one by one: chunks end and begin under decoded tokens and the chunk groups
    give pages back on the way; decode steps are replayed from graphs after the first two."""
    d, cfg, w, *_ = models["R1"]
    toks = TT.make_requests(cfg["vocab"], (160,), seed=3)["r0"]
    ref = {"r0": PR.forward(cfg, w, toks)}
    eng = _engine(d, dtype, 16, 12)
    got = TT.run_steps(eng, TT.trace_tail_one_by_one({"r0": toks}, 150))
    _check(got, ref, dtype, f"R1 {dtype} long decoding", "R1")
    assert eng.graph_replays > 100


def test_greedy_generation_through_the_scheduler(models):
    """Runtime.generate_batch (scheduler, portions, the sampler's argmax) against the plain model's greedy tokens,
    in 32-bit; prompts of unequal length, more requests than run at once."""
    from infernum_amd import BatchConfig, GenerateOptions, Runtime
    d, cfg, w, *_ = models["R1"]
    prompts = list(TT.make_requests(cfg["vocab"], (5, 31, 2, 18, 9), seed=9).values())
    rt = Runtime.from_pretrained(d, dtype="float32", batch_config=BatchConfig(block_size=16, num_blocks=24,
                                                                              max_batch_size=3, max_prefill_tokens=8,
                                                                              max_tokens_per_step=16, step_token_multiple=1))
    outs = rt.generate_batch(prompts, GenerateOptions(max_new_tokens=12))
    for p, got in zip(prompts, outs):
        toks = list(p)
        for _ in range(12):
            toks.append(int(PR.forward(cfg, w, toks)[-1].argmax()))
        assert list(got) == toks[len(p):], (p, got, toks[len(p):])


@BOTH
def test_trace_run_and_generate_programs(models, tmp_path, dtype):
    """bin/trace_run and bin/generate as a user starts them, on a Rogizen folder: the model class comes from
    config.json; steps on standard input, logits in files; generated tokens on standard output."""
    import json
    import os
    import subprocess
    import sys
    import numpy as np
    d, cfg, w, _, _, reqs, ref = models["R3"]
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
    _check(got, ref, dtype, f"trace_run R3 {dtype} mixed", "R3")
    if dtype == "float32":
        prompt = reqs["r4"][:9]
        gen = subprocess.run([sys.executable, os.path.join(root, "bin", "generate"), "-m", d, "--prompt-ids",
                              ",".join(map(str, prompt)), "-n", "6", "--greedy", "--dtype", "float32"],
                             text=True, capture_output=True, timeout=600)
        assert gen.returncode == 0, gen.stderr[-3000:]
        toks = list(prompt)
        for _ in range(6):
            toks.append(int(PR.forward(cfg, w, toks)[-1].argmax()))
        assert " " + " ".join(map(str, toks[9:])) + "\n" in gen.stdout, gen.stdout[-2000:]
