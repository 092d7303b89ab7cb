"""Position encodings applied to queries and keys.

`rope_neox`: half-split rotary encoding over the first `rotary_dim` dims of a head
(all of them for Qwen3): inv_freq_i = theta^(-2i/rotary_dim), angle = pos * inv_freq_i,
pairs (i, i + rotary_dim/2).  infer/src/weight_loader.rs:955-989 builds the same table
(and then narrows it to bf16, which this engine does not: angles, cos and sin stay
32-bit); rotation as crates/cuda-kernels/csrc/attention/prefill_attention_paged_prep.cu:60-76.
`none`: no position encoding.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import Part, register


def rope_table(rotary_dim: int, theta: float, positions: int):
    """(cos, sin), each float32 [positions, rotary_dim/2] on the CPU: angle(pos, i) = pos * theta^(-2i/rotary_dim).

    float32 throughout, as the reference computes it on the host (infer/src/weight_loader.rs:963-981).
    """
    half = rotary_dim // 2
    base = torch.tensor(float(theta), dtype=torch.float32)
    exponent = torch.arange(half, dtype=torch.float32) * 2.0 / float(rotary_dim)
    inv_freq = 1.0 / torch.pow(base, exponent)
    angle = torch.arange(positions, dtype=torch.float32)[:, None] * inv_freq[None, :]
    return torch.cos(angle).contiguous(), torch.sin(angle).contiguous()


@register("position", "rope_neox")
class RopeNeox(Part):
    """params: head_dim, rotary_dim (default head_dim), theta, max_positions."""

    fusable = True  # the q/k preparation kernel applies this encoding itself

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.head_dim = int(params["head_dim"])
        self.rotary_dim = int(params.get("rotary_dim", self.head_dim))
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError("rotary_dim must be even and in 1..head_dim")
        self.theta = float(params["theta"])
        self.cos, self.sin = self._table(int(params["max_positions"]))

    # layers with the same encoding share one table: (device, rotary_dim, theta, positions) -> (cos, sin)
    _shared: dict = {}

    def _table(self, positions: int):
        key = (str(self.rt.device), self.rotary_dim, self.theta, positions)
        if key not in RopeNeox._shared:
            RopeNeox._shared[key] = self._make_table(positions)
        return RopeNeox._shared[key]

    def _make_table(self, positions: int):
        cos, sin = rope_table(self.rotary_dim, self.theta, positions)
        return cos.to(self.rt.device), sin.to(self.rt.device)

    def ensure_positions(self, n: int) -> None:
        """Grow the table if a request runs past what it was sized for."""
        if n > self.cos.shape[0]:
            self.cos, self.sin = self._table(max(n, 2 * self.cos.shape[0]))

    def prepare(self, max_positions: int) -> None:
        self.ensure_positions(max_positions)

    def fused_rotary(self):
        return self.cos, self.sin, self.rotary_dim

    def apply(self, q, k, positions, num_q_heads, num_kv_heads):
        ops.qk_prep(q, k, k, num_q_heads=num_q_heads, num_kv_heads=num_kv_heads,
                    head_dim=self.head_dim, eps=0.0, cos=self.cos, sin=self.sin,
                    rotary_dim=self.rotary_dim, positions=positions)


@register("position", "none")
class NoPosition(Part):
    fusable = True  # nothing to apply
    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)

    def ensure_positions(self, n: int) -> None:
        pass

    def fused_rotary(self):
        return None, None, 0

    def apply(self, q, k, positions, num_q_heads, num_kv_heads):
        pass
