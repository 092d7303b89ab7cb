"""RMSNorm: x / sqrt(mean(x^2) + eps) * w with the plain weight w (not 1 + w).

crates/cuda-kernels/csrc/misc/norm.cu:8,59,221-359; the residual add fused in as at :462-.
The weight keeps the type the checkpoint stores it in (bfloat16 or float32).
"""
from __future__ import annotations

from ..kernels import ops
from .base import Part, WeightDecl, register


@register("norm", "rmsnorm")
class RMSNorm(Part):
    """params: width, eps."""

    graph_safe = True  # launches depend on shapes only, never on the values of a step

    @classmethod
    def declare_weights(cls, params):
        return {"weight": WeightDecl((params["width"],), init="ones")}

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.weight = tensors["weight"]
        self.eps = float(params["eps"])
        self.width = int(params["width"])

    def forward(self, x, rows=None):
        return ops.rmsnorm(x, self.weight, self.eps, self.rt.act_dtype, rows=rows)

    def add_norm(self, residual, delta, rows=None):
        """residual (float32) += delta, then the norm of it; delta None: just the norm."""
        if delta is None:
            return ops.rmsnorm(residual, self.weight, self.eps, self.rt.act_dtype, rows=rows)
        return ops.add_rmsnorm(residual, delta, self.weight, self.eps, self.rt.act_dtype, rows=rows)
