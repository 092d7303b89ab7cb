"""Arrangements of a mixer, a feed-forward and norms in one layer.

`pre_norm`: h += mixer(norm(h)); h += ffn(norm(h))  (infer/src/model/qwen3/prefill.rs:618-776).
The residual stream is float32.  A block receives the residual and the delta its
predecessor has not added yet, so that every add is fused into the norm that follows it
(the reference's fused_add_rms_norm chain, infer/src/model/qwen3/batch_decode.rs:2411-2456).
"""
from __future__ import annotations

from .base import register


@register("block", "pre_norm")
class PreNormBlock:
    """norm roles: "mixer_in", "ffn_in"."""

    norm_roles = ("mixer_in", "ffn_in")

    def __init__(self, mixer, feed_forward, norms: dict):
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norms = norms
        self.norm_mixer = norms["mixer_in"]
        self.norm_ffn = norms["ffn_in"]

    def forward(self, residual, delta, batch, cache_view):
        a = self.norm_mixer.add_norm(residual, delta)
        m = self.mixer.forward(a, batch, cache_view)
        b = self.norm_ffn.add_norm(residual, m)
        return residual, self.feed_forward.forward(b)
