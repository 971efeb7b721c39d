"""Arrangements of a layer's parts."""

from __future__ import annotations

from tokamak_amd.config.registry import register_part
from tokamak_amd.parts.base import Block


class PreNormBlock(Block):
    """x = x + mixer(norm(x)); x = x + feed_forward(norm(x))
    (reference: src/tokamak/model/transformer.py:107-108).

    The residual stream ``resid`` is float32.  Each sub-layer's output is left
    ``pending`` and added by the next norm's fused kernel, so the sum is formed
    in float32 and the stream is written once per sub-layer.  An optional
    ``position`` part prepares the step's position data for the mixer.
    """

    roles = ("mixer_norm", "mixer", "feed_forward_norm", "feed_forward")
    optional = ("position",)

    def __init__(self, parts) -> None:
        super().__init__(parts)
        self.mixer_norm = parts["mixer_norm"]
        self.feed_forward_norm = parts["feed_forward_norm"]
        self.feed_forward = parts["feed_forward"]
        self.position = parts.get("position")

    def forward(self, resid, pending, batch, store, writes_cache):
        position = None if self.position is None else self.position.prepare(batch)
        h = self.mixer_norm.forward(resid, pending)
        pending = self.mixer.forward(h, batch, store, writes_cache, position)
        h = self.feed_forward_norm.forward(resid, pending)
        return self.feed_forward.forward(h, batch)


register_part("block", "pre_norm", PreNormBlock)
