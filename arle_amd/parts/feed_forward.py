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
        self.gate_up = Linear(torch.cat([gate, up], dim=0).contiguous())
        self.down = Linear(tensors["down"])

    def forward(self, x):
        gu = self.gate_up(x)
        act = ops.silu_mul(gu[:, : self.inter], gu[:, self.inter:])
        return self.down(act)
