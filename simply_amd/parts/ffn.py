"""Dense gated feed-forward: down(act(gate(x)) * up(x))  (simply/model_lib.py:643-730 with
use_gated_activation_in_ffn=True, ffn_use_bias=False; `act` by its name in the registry, as
simply/model_lib.py:723 looks `ffn_activation` up)."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..registry import ACTIVATIONS, FEED_FORWARDS
from .base import FeedForward, ParamSpec, PendingNorm, as_product_weight, project

# activation name -> its code in the gated product's epilogue (simply/model_lib.py:93-104 registers these three)
ACTIVATIONS.register("gelu_tanh", ops.ACT_GELU_TANH)
ACTIVATIONS.register("silu", ops.ACT_SILU)
ACTIVATIONS.register("squared_relu", ops.ACT_SQUARED_RELU)


@FEED_FORWARDS.register("gated_dense")
class GatedDense(FeedForward):
    accepts_pending = True
    defers_sum = True

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "gelu_tanh"):
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.activation = activation
        self.activation_code = int(ACTIVATIONS.get(activation))   # an unknown name is refused with the known ones
        self.gate_proj = self.up_proj = self.down_proj = self.gate_up = None

    def param_specs(self):
        D, F = self.hidden_size, self.intermediate_size
        return {"gate_proj": ParamSpec((F, D)), "up_proj": ParamSpec((F, D)), "down_proj": ParamSpec((D, F))}

    def load(self, tensors):
        gate, up = tensors["gate_proj"], tensors["up_proj"]
        if gate.dtype == torch.bfloat16 and gate.is_cuda:
            # one tiled weight for both factors, their tiles in turn: the fused kernels stream it once
            from ..kernels.packing import pack_gate_up

            self.gate_up, self.gate_proj, self.up_proj = pack_gate_up(gate, up), None, None
        else:
            self.gate_up, self.gate_proj, self.up_proj = None, gate, up
        self.down_proj = as_product_weight(tensors["down_proj"])

    def forward(self, x: torch.Tensor, ctx=None, defer_sum=False) -> torch.Tensor:
        # gelu(x.Wg^T) * (x.Wu^T), one kernel
        if self.gate_up is not None:
            z = project(x, self.gate_up, activation=self.activation_code)
        else:
            if isinstance(x, PendingNorm):
                x = x.materialize()
            z = ops.gemm(x, self.gate_proj, w2=self.up_proj, activation=self.activation_code)
        return ops.gemm(z, self.down_proj, defer_sum=defer_sum)
