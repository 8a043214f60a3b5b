"""SwiGLU feed-forward: down( silu(x Wg^T) * (x Wu^T) ), no bias, exact SiLU.

infernum-llama/src/graph_builder.rs:498-507; infernum-cuda/kernels/silu.cu:36-40.
Gate and up are one [2I, H] matrix, so one product makes both.

``dense``: down( act(x Wu^T) ) without a gate; ``activation`` names the function
(``gelu_tanh``), ``names`` the two tensors' local names.
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence

import torch

from ..kernels import api as K
from .base import FeedForward, Runtime, StepContext, WeightSpec, register_part
from .linear import emit_linear, linear, prepare_weights


class SwiGLUFeedForward(FeedForward):
    graph_safe = True
    def __init__(self, rt: Runtime, hidden_size: int, intermediate_size: int, init_std: float = 0.02,
                 names: Sequence[str] = ("gate_proj.weight", "up_proj.weight", "down_proj.weight")):
        """``names``: the local tensor names of the gate, up and down matrices."""
        super().__init__(rt)
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.init_std, self.names = init_std, tuple(names)
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def weights(self) -> Dict[str, WeightSpec]:
        H, I = self.hidden_size, self.intermediate_size
        init = ("normal", self.init_std)
        gate, up, down = self.names
        return {gate: WeightSpec((I, H), init), up: WeightSpec((I, H), init), down: WeightSpec((H, I), init)}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        gate, up, down = self.names
        self.w_gate_up = torch.cat([tensors[gate], tensors[up]], dim=0).contiguous()
        self.w_down = tensors[down].contiguous()
        prepare_weights(self.rt, [(self.w_gate_up, "swiglu", False), (self.w_down, None, True)])

    def forward(self, x: torch.Tensor, ctx: Optional[StepContext] = None):
        act = linear(x, self.w_gate_up, epilogue="swiglu", kernels=self.rt.kernels)
        return linear(act, self.w_down, keep_split=True, kernels=self.rt.kernels)

    def native(self, program, view=None) -> None:
        if type(self).forward is not SwiGLUFeedForward.forward:
            return super().native(program, view)
        dt = self.rt.dtype
        act = emit_linear(program, program.x, program.N, self.w_gate_up, dt, "swiglu", False, "swiglu.act", "swiglu.gate_up")
        program.pending = emit_linear(program, act.tensor(), program.N, self.w_down, dt, None, True, "swiglu.out",
                                      "swiglu.down")


register_part("feed_forward", "swiglu", SwiGLUFeedForward)


class DenseFeedForward(FeedForward):
    """down( act(up x) ): two matrices and an activation between them."""
    graph_safe = True

    def __init__(self, rt: Runtime, hidden_size: int, intermediate_size: int, activation: str = "gelu_tanh",
                 names: Sequence[str] = ("up_proj.weight", "down_proj.weight"), init_std: float = 0.02):
        super().__init__(rt)
        if activation not in K.ACTIVATIONS:
            raise ValueError(f"activation {activation!r}: one of {sorted(K.ACTIVATIONS)}")
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.activation, self.names, self.init_std = activation, tuple(names), init_std
        self.w_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def weights(self) -> Dict[str, WeightSpec]:
        H, I = self.hidden_size, self.intermediate_size
        init = ("normal", self.init_std)
        return {self.names[0]: WeightSpec((I, H), init), self.names[1]: WeightSpec((H, I), init)}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.w_up = tensors[self.names[0]].contiguous()
        self.w_down = tensors[self.names[1]].contiguous()
        prepare_weights(self.rt, [(self.w_up, None, False), (self.w_down, None, True)])

    def forward(self, x: torch.Tensor, ctx: Optional[StepContext] = None):
        act = K.activation(linear(x, self.w_up, kernels=self.rt.kernels), self.activation)
        return linear(act, self.w_down, keep_split=True, kernels=self.rt.kernels)

    def native(self, program, view=None) -> None:
        if type(self).forward is not DenseFeedForward.forward:
            return super().native(program, view)
        from ..engine.program import STREAM
        dt = self.rt.dtype
        up = emit_linear(program, program.x, program.N, self.w_up, dt, None, False, "dense.act", "dense.up").tensor()
        program.op("core", "ia_activation", [up, up, program.act_code, program.N * self.intermediate_size,
                                             K.ACTIVATIONS[self.activation], STREAM])
        program.pending = emit_linear(program, up, program.N, self.w_down, dt, None, True, "dense.out", "dense.down")


register_part("feed_forward", "dense", DenseFeedForward)
