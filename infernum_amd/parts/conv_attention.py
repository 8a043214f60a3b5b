"""Attention whose queries and keys pass a short causal convolution, and whose values are its keys.

q = Wq x + bq and k = Wk x + bk (heads consecutive within a row); every channel of both then runs through a
convolution over the request's last ``conv_taps`` tokens, y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the
request's start.  What leaves the convolution is, for a key head, already the value of that head: there is no value
projection.  Queries and keys then get an RMS norm per head (one weight of the head's size for all query heads, one
for all key heads) and the position encoding's rotation; scores, mask (all keys, a window, or chunks), softmax and
the grouping of query heads over key/value heads are the attention mixer's own, and so are its kernels.  The output
projection has a bias.

Between steps the mixer keeps two things per request: pages of keys and values like any attention, and the last
``conv_taps - 1`` projected rows (with their bias, fp32) in a state slot, so that a prompt cut anywhere goes on as if
it had not been cut.
"""
from __future__ import annotations

from typing import Any, Dict, Mapping, Optional

import torch

from ..kernels import api as K
from .attention import Attention
from .base import CacheView, Runtime, StateSpec, StepContext, WeightSpec, register_part
from .linear import emit_linear, linear, prepare_weights


class ConvAttention(Attention):
    graph_safe = True

    def __init__(self, rt: Runtime, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, conv_taps: int,
                 norm_eps: float, position: Optional[Mapping[str, Any]] = None, window: Optional[int] = None,
                 chunk: Optional[int] = None, scale: Optional[float] = None, qk_norm: bool = True,
                 init_std: float = 0.02, kernels: str = "auto"):
        super().__init__(rt, hidden_size, num_heads, num_kv_heads, head_dim, position=position, window=window,
                         scale=scale, kernels=kernels, init_std=init_std, chunk=chunk)
        self.taps = int(conv_taps)
        if self.taps < 1:
            raise ValueError(f"a convolution needs at least one tap, got {conv_taps}")
        self.norm_eps, self.qk_norm = float(norm_eps), bool(qk_norm)
        self.channels = (self.nh + self.nkv) * self.d
        self.w_qk: Optional[torch.Tensor] = None

    # ---- what it needs ---------------------------------------------------
    def state_spec(self) -> Optional[StateSpec]:
        return StateSpec(((self.taps - 1) * self.channels,)) if self.taps > 1 else None

    def weights(self) -> Dict[str, WeightSpec]:
        nh, nkv, d, H, taps = self.nh, self.nkv, self.d, self.hidden_size, self.taps
        init, small = ("normal", self.init_std), dict(follows_compute_dtype=False)
        out = {
            "q": WeightSpec((nh * d, H), init), "q.b": WeightSpec((nh * d,), ("normal", 0.1), **small),
            "k": WeightSpec((nkv * d, H), init), "k.b": WeightSpec((nkv * d,), ("normal", 0.1), **small),
            "q.conv": WeightSpec((nh * d, taps), ("normal", taps ** -0.5), **small),
            "k.conv": WeightSpec((nkv * d, taps), ("normal", taps ** -0.5), **small),
            "o": WeightSpec((H, nh * d), init), "o.b": WeightSpec((H,), ("normal", 0.1), **small),
        }
        if self.qk_norm:
            out["q.norm"] = WeightSpec((d,), ("uniform", 0.8, 1.2), **small)
            out["k.norm"] = WeightSpec((d,), ("uniform", 0.8, 1.2), **small)
        return out

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        f32 = lambda name: tensors[name].to(torch.float32).contiguous()            # noqa: E731
        self.w_qk = torch.cat([tensors["q"], tensors["k"]], dim=0).contiguous()
        self.w_o = tensors["o"].contiguous()
        self.b_qk = torch.cat([f32("q.b"), f32("k.b")]).contiguous()
        self.b_o = f32("o.b")
        self.w_conv = torch.cat([f32("q.conv"), f32("k.conv")], dim=0).t().contiguous()      # tap by tap: [taps, channels]
        self.q_norm = f32("q.norm") if self.qk_norm else None
        self.k_norm = f32("k.norm") if self.qk_norm else None
        prepare_weights(self.rt, [(self.w_qk, None, False), (self.w_o, None, False)])

    def _state(self, cache: CacheView) -> torch.Tensor:
        if self.taps > 1:
            if cache.state is None:
                raise K.KernelError("conv_attention needs a state slot for its convolution")
            return cache.state
        return torch.zeros((1, 1), dtype=torch.float32, device=self.rt.device)      # one tap: nothing is carried

    # ---- one step --------------------------------------------------------
    def forward(self, x: torch.Tensor, ctx: StepContext, cache: CacheView):
        nh, nkv, d, pos = self.nh, self.nkv, self.d, self.position
        if cache.k_pages is None or not cache.writable:
            raise K.KernelError("conv_attention needs pages of its own")
        g, n, dev = cache.group, x.shape[0], x.device
        state = self._state(cache)
        u = linear(x, self.w_qk, kernels=self.rt.kernels)
        y = torch.empty_like(u)
        if self.taps > 1 and ctx.num_decode == ctx.num_seqs:            # every request brings one token
            K.causal_conv_single(u, self.w_conv, state, ctx.token_seq, ctx.state_slots, y, bias_in=self.b_qk, tap_major=True)
        else:
            K.causal_conv(u, self.w_conv, state, ctx.token_seq, ctx.seq_starts, ctx.state_slots, y, bias_in=self.b_qk,
                          tap_major=True)
            if self.taps > 1:
                K.conv_state_update(u, self.taps, state, ctx.seq_starts, ctx.state_slots, bias_in=self.b_qk)
        q = torch.empty((n, nh * d), dtype=self.rt.dtype, device=dev)
        K.qk_prepare(y, q, nh, nkv, d, ctx.positions, self.q_norm, self.k_norm, self.norm_eps, pos.inv_freq,
                     pos.rotary_dim if pos.inv_freq is not None else 0, pos.pairing, pos.magnitude, ctx.slots[g],
                     cache.k_pages, cache.v_pages, values_are_keys=True)
        out = torch.empty((n, nh * d), dtype=self.rt.dtype, device=dev)
        self.attend(q, out, ctx, cache)
        return K.add_bias(linear(out, self.w_o, kernels=self.rt.kernels), self.b_o)

    def native(self, program, view: CacheView) -> None:
        if type(self).forward is not ConvAttention.forward:
            return super(Attention, self).native(program, view)
        from ..engine.program import ALWAYS, STREAM, Guard
        if view is None or view.k_pages is None or not view.writable:
            raise K.KernelError("conv_attention needs pages of its own")
        nh, nkv, d, rt, pos, C, taps = self.nh, self.nkv, self.d, self.rt, self.position, self.channels, self.taps
        act, N, T = program.act_code, program.N, program.T
        state = self._state(view)
        stride = int(state.stride(0))
        k, v, g = view.k_pages, view.v_pages, view.group
        program.keep(self.w_qk, self.w_o, self.b_qk, self.b_o, self.w_conv, self.q_norm, self.k_norm, state, pos.inv_freq)
        u = emit_linear(program, program.x, N, self.w_qk, rt.dtype, None, False, "conv_attention.u", "conv_attention.qk").tensor()
        y = program.buffer("conv_attention.y", T * C * program.act_bytes)
        portions = Guard.between(program.NP, 1) if taps > 1 else ALWAYS
        program.op("core", "ia_causal_conv", [u, act, C, self.b_qk, self.w_conv, None, 0, y, act, C, state, stride,
                                              program.token_seq, program.seq_starts, program.state_slots, N, C, taps, 1,
                                              STREAM], portions)
        if taps > 1:
            program.op("core", "ia_conv_state_update", [u, act, C, self.b_qk, state, stride, program.seq_starts,
                                                        program.state_slots, program.B, C, taps, STREAM], portions)
            program.op("core", "ia_causal_conv_single", [u, act, C, self.b_qk, self.w_conv, None, 0, y, act, C, state, stride,
                                                         program.token_seq, program.state_slots, N, C, taps, 1, STREAM],
                       ~portions)
        q = program.buffer("attention.q", T * nh * d * program.act_bytes)
        rot = pos.rotary_dim if pos.inv_freq is not None else 0
        program.op("core", "ia_qk_prepare",
                   [y, act, C, q, nh * d, self.q_norm, self.k_norm, float(self.norm_eps), program.positions,
                    program.slots(g), pos.inv_freq if rot else None,
                    int(bool(rot) and pos.inv_freq.dtype == torch.float64), rot, K.PAIRINGS[pos.pairing],
                    float(pos.magnitude), k, v, N, nh, nkv, d, int(k.shape[2]), int(k.shape[0]), 1, STREAM])
        out = self.emit_attend(program, view, q, nh * d, ALWAYS)
        o = emit_linear(program, out, N, self.w_o, rt.dtype, None, False, "conv_attention.out", "conv_attention.o")
        program.op("core", "ia_add_bias", [o.tensor(), act, self.b_o, N, self.hidden_size, STREAM])
        program.pending = o


register_part("mixer", "conv_attention", ConvAttention)
