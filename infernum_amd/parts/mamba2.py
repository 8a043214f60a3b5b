"""A selective state-space mixer (the Mamba-2 form: one decay per head and token).

One input projection makes, side by side in a row, the gate z (inner = heads x head_dim values), then x (inner), B and
C (groups x state values each) and one raw step size per head.  x, B and C together pass a short causal convolution per
channel (with a bias) and silu.  Per head h, which reads the B and C of group h // (heads / groups), with
dt = softplus(raw + dt_bias_h) and a state S of [state, head_dim] that starts at zero:

    S_t = exp(-exp(A_log_h) dt_t) S_(t-1) + dt_t B_t x_t^T,        y_t = S_t^T C_t + D_h x_t.

The heads' y, concatenated, are multiplied by silu(z), divided by their root mean square in ``norm_groups`` equal parts
(the gate comes before the norm), multiplied by a weight, and projected back to the model's width.

Between steps a request keeps, in one state slot of fp32 values: the last ``conv_taps - 1`` inputs of the convolution,
then S of every head.  Step sizes, decays, the state and the gated norm are fp32 whatever the activations' type.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import api as K
from .base import CacheView, Mixer, Runtime, StateSpec, StepContext, WeightSpec, register_part
from .linear import emit_linear, linear, prepare_weights


class Mamba2Mixer(Mixer):
    graph_safe = True

    def __init__(self, rt: Runtime, hidden_size: int, num_heads: int, head_dim: int, state_size: int, groups: int,
                 norm_groups: int, conv_taps: int, norm_eps: float, init_std: float = 0.02):
        super().__init__(rt)
        self.hidden_size, self.nh, self.P, self.Ns = int(hidden_size), int(num_heads), int(head_dim), int(state_size)
        self.G, self.norm_groups, self.taps, self.norm_eps = int(groups), int(norm_groups), int(conv_taps), float(norm_eps)
        self.init_std = init_std
        self.inner = self.nh * self.P
        if self.nh % self.G:
            raise ValueError(f"{self.nh} heads are not a multiple of {self.G} groups")
        if self.inner % self.norm_groups:
            raise ValueError(f"the norm's {self.norm_groups} parts do not divide the {self.inner} inner values")
        if self.taps < 1:
            raise ValueError(f"a convolution needs at least one tap, got {conv_taps}")
        self.conv_dim = self.inner + 2 * self.G * self.Ns
        self.row = 2 * self.inner + 2 * self.G * self.Ns + self.nh
        self.conv_floats = (self.taps - 1) * self.conv_dim

    # ---- what it needs ---------------------------------------------------
    def state_spec(self) -> StateSpec:
        return StateSpec((self.conv_floats + self.nh * self.Ns * self.P,))

    def weights(self) -> Dict[str, WeightSpec]:
        H, small = self.hidden_size, dict(follows_compute_dtype=False)
        return {
            "in": WeightSpec((self.row, H), ("normal", self.init_std)),
            "conv": WeightSpec((self.conv_dim, self.taps), ("normal", self.taps ** -0.5), **small),
            "conv.b": WeightSpec((self.conv_dim,), ("normal", 0.1), **small),
            "dt_bias": WeightSpec((self.nh,), ("uniform", -2.0, 0.0), **small),
            "A_log": WeightSpec((self.nh,), ("uniform", -0.7, 1.2), **small),
            "D": WeightSpec((self.nh,), ("uniform", 0.5, 1.5), **small),
            "norm": WeightSpec((self.inner,), ("uniform", 0.8, 1.2), **small),
            "o": WeightSpec((H, self.inner), ("normal", self.init_std)),
        }

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        f32 = lambda name: tensors[name].to(torch.float32).contiguous()            # noqa: E731
        self.w_in, self.w_o = tensors["in"].contiguous(), tensors["o"].contiguous()
        self.w_conv, self.b_conv = f32("conv").t().contiguous(), f32("conv.b")        # tap by tap: [taps, channels]
        self.dt_bias, self.a_log, self.skip, self.w_norm = f32("dt_bias"), f32("A_log"), f32("D"), f32("norm")
        prepare_weights(self.rt, [(self.w_in, None, False), (self.w_o, None, True)])

    def _states(self, cache: CacheView):
        """The slot's two parts as the kernels take them: (the convolution's inputs, the heads' S), both views of the
        slots' rows with the slot's stride."""
        if cache is None or cache.state is None:
            raise K.KernelError("mamba2 needs a state slot")
        return cache.state, cache.state[:, self.conv_floats:]

    def _chunked(self, xbc: torch.Tensor, portion_tokens: int) -> bool:
        """Steps that bring enough tokens of prompts run the recurrence as matrix products over chunks (where
        there is a kernel for the sizes); the others, decode steps among them, token after token from registers."""
        return portion_tokens >= K.SSD_CHUNKED_FROM and K.ssd_chunked_takes(xbc.dtype, self.nh, self.P, self.Ns, self.G,
                                                                           int(xbc.stride(0)))

    # ---- one step --------------------------------------------------------
    def forward(self, x: torch.Tensor, ctx: StepContext, cache: CacheView):
        n, dev, inner, cd = x.shape[0], x.device, self.inner, self.conv_dim
        conv_state, ssm_state = self._states(cache)
        proj = linear(x, self.w_in, kernels=self.rt.kernels)                     # [n, z | x B C | dt]
        u = proj[:, inner:inner + cd]
        xbc = torch.empty((n, cd), dtype=self.rt.dtype, device=dev)
        if self.taps > 1 and ctx.num_decode == ctx.num_seqs:            # every request brings one token
            K.causal_conv_single(u, self.w_conv, conv_state, ctx.token_seq, ctx.state_slots, xbc, bias_out=self.b_conv,
                                 activation="silu", tap_major=True)
        else:
            K.causal_conv(u, self.w_conv, conv_state, ctx.token_seq, ctx.seq_starts, ctx.state_slots, xbc,
                          bias_out=self.b_conv, activation="silu", tap_major=True)
            if self.taps > 1:
                K.conv_state_update(u, self.taps, conv_state, ctx.seq_starts, ctx.state_slots)
        y = torch.empty((n, inner), dtype=torch.float32, device=dev)
        scan = K.ssd_chunked if self._chunked(xbc, ctx.num_tokens - ctx.num_decode) else K.ssd_scan
        scan(xbc, proj[:, inner + cd:], self.dt_bias, self.a_log, self.skip, ssm_state, y, ctx.seq_starts,
             ctx.state_slots, self.nh, self.P, self.Ns, self.G)
        gated = torch.empty((n, inner), dtype=self.rt.dtype, device=dev)
        K.gated_group_norm(y, proj[:, :inner], self.w_norm, self.norm_groups, self.norm_eps, gated)
        return linear(gated, self.w_o, keep_split=True, kernels=self.rt.kernels)

    def native(self, program, view: CacheView) -> None:
        if type(self).forward is not Mamba2Mixer.forward:
            return super().native(program, view)
        from ..engine.program import ALWAYS, STREAM, Guard
        rt, inner, cd, row, taps = self.rt, self.inner, self.conv_dim, self.row, self.taps
        act, ab, N, T = program.act_code, program.act_bytes, program.N, program.T
        state, _ = self._states(view)
        stride = int(state.stride(0))
        ssm = state[:, self.conv_floats:]
        program.keep(state, ssm, self.w_conv, self.b_conv, self.dt_bias, self.a_log, self.skip, self.w_norm)
        proj = emit_linear(program, program.x, N, self.w_in, rt.dtype, None, False, "mamba2.proj", "mamba2.in").tensor()
        u, dt, xbc = proj.at(inner * ab), proj.at((inner + cd) * ab), program.buffer("mamba2.xbc", T * cd * ab)
        portions = Guard.between(program.NP, 1) if taps > 1 else ALWAYS
        program.op("core", "ia_causal_conv", [u, act, row, None, self.w_conv, self.b_conv, 1, xbc, act, cd, state, stride,
                                              program.token_seq, program.seq_starts, program.state_slots, N, cd, taps, 1,
                                              STREAM], portions)
        if taps > 1:
            program.op("core", "ia_conv_state_update", [u, act, row, None, state, stride, program.seq_starts,
                                                        program.state_slots, program.B, cd, taps, STREAM], portions)
            program.op("core", "ia_causal_conv_single", [u, act, row, None, self.w_conv, self.b_conv, 1, xbc, act, cd, state,
                                                         stride, program.token_seq, program.state_slots, N, cd, taps, 1,
                                                         STREAM], ~portions)
        y = program.buffer("mamba2.y", T * inner * 4)
        args = [xbc, act, cd, dt, row, self.dt_bias, self.a_log, self.skip, ssm, stride, y, program.seq_starts,
                program.state_slots, program.B, self.nh, self.P, self.Ns, self.G, STREAM]
        if K.ssd_chunked_takes(rt.dtype, self.nh, self.P, self.Ns, self.G, cd):
            long = Guard.between(program.NPT, K.SSD_CHUNKED_FROM)
            program.op("core", "ia_ssd_chunked", args, long)
            program.op("core", "ia_ssd_scan", args, ~long)
        else:
            program.op("core", "ia_ssd_scan", args)
        gated = program.buffer("mamba2.gated", T * inner * ab)
        program.op("core", "ia_gated_group_norm", [y, proj, act, row, self.w_norm, gated, N, inner, self.norm_groups,
                                                   float(self.norm_eps), STREAM])
        program.pending = emit_linear(program, gated, N, self.w_o, rt.dtype, None, True, "mamba2.out", "mamba2.o")


register_part("mixer", "mamba2", Mamba2Mixer)
