"""Dense SwiGLU feed-forward: down(silu(gate(x)) * up(x)), no biases.

infer/src/model/qwen3/prefill.rs:291-337.  gate and up are kept as one [2I, H] matrix
(gate rows first, as the reference's optional fusion does, weights.rs:111-121) so a step
runs one product for both.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import Part, WeightDecl, register
from .linear import Linear


@register("feed_forward", "swiglu")
class SwiGLU(Part):
    """params: hidden_size, intermediate_size."""

    graph_safe = True  # launches depend on shapes only, never on the values of a step

    @classmethod
    def declare_weights(cls, params):
        h, i = params["hidden_size"], params["intermediate_size"]
        return {"gate": WeightDecl((i, h)), "up": WeightDecl((i, h)), "down": WeightDecl((h, i))}

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.inter = int(params["intermediate_size"])
        gate, up = tensors["gate"], tensors["up"]
        if gate.dtype != up.dtype:
            raise ValueError("gate and up projections must be stored in one type")
        # bfloat16: rows interleaved in blocks of 16 (16 gate rows, the 16 matching up rows, ...), so
        # that one tile of the decode kernel holds both halves of 16 outputs and applies the activation
        # itself.  Otherwise gate rows first, then up rows.
        self.block = 16 if (gate.dtype == torch.bfloat16 and self.inter % 16 == 0) else 0
        if self.block:
            h = gate.shape[1]
            fused = torch.stack([gate.view(-1, 16, h), up.view(-1, 16, h)], dim=1).reshape(2 * self.inter, h)
        else:
            fused = torch.cat([gate, up], dim=0)
        self.gate_up = Linear(fused.contiguous(), rt.weight_tiles)
        self.down = Linear(tensors["down"], rt.weight_tiles)

    def products(self):
        if self.gate_up.weight.dtype != torch.bfloat16:
            return []
        return [("gate_up", self.gate_up.out_features, self.gate_up.in_features, bool(self.block), None),
                ("down", self.down.out_features, self.down.in_features, False, "norm")]

    def forward(self, x):
        """x [T, H] -> [T, H], or a float32 stack [S, T, H] to be added in order (see Linear)."""
        if self.block:
            act = ops.gate_up_act(x, self.gate_up.weight, self.gate_up.tiles)   # one product with the activation, or two kernels
        else:
            gu = self.gate_up(x)
            act = ops.silu_mul(gu[:, : self.inter], gu[:, self.inter:])
        return self.down(act, partials_ok=True)
