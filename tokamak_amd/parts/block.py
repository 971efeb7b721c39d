"""Arrangements of a layer's parts."""

from __future__ import annotations

from tokamak_amd.config.registry import register_part
from tokamak_amd.kernels.linear import Added, StreamSink
from tokamak_amd.parts.base import Block


class PreNormBlock(Block):
    """x = x + mixer(norm(x)); x = x + feed_forward(norm(x))
    (reference: src/tokamak/model/transformer.py:107-108).

    The residual stream ``resid`` is float32.  Each sub-layer's output is left
    ``pending`` and added by the next norm's fused kernel, so the sum is formed
    in float32 and the stream is written once per sub-layer.  Parts that can
    (``fuses_residual``) are offered the stream itself, so that in a decode step
    of few rows their last product adds into it and the next product finishes
    the norm, with no kernel in between.  An optional ``position`` part prepares
    the step's position data for the mixer.
    """

    roles = ("mixer_norm", "mixer", "feed_forward_norm", "feed_forward")
    optional = ("position",)
    fuses_residual = True
    replays_parts = True

    def __init__(self, parts) -> None:
        super().__init__(parts)
        self.mixer_norm = parts["mixer_norm"]
        self.feed_forward_norm = parts["feed_forward_norm"]
        self.feed_forward = parts["feed_forward"]
        self.position = parts.get("position")
        self.entry_norm = self.mixer_norm

    def forward(self, resid, pending, batch, store, writes_cache, then=None):
        position = None if self.position is None else self.position.prepare(batch)
        h = _normed(self.mixer_norm, resid, pending, self.mixer)
        into = _sink(self.mixer, self.feed_forward_norm, resid)
        pending = self.mixer.forward(h, batch, store, writes_cache, position, **into)
        h = _normed(self.feed_forward_norm, resid, pending, self.feed_forward)
        into = _sink(self.feed_forward, then, resid)
        return self.feed_forward.forward(h, batch, **into)


def _normed(norm, resid, pending, consumer):
    """norm(resid + pending) for ``consumer``; left for the consumer to finish if both know how."""
    if norm.fuses_residual:
        return norm.forward(resid, pending, defer=consumer.fuses_residual)
    return norm.forward(resid, None if isinstance(pending, Added) else pending)


def _sink(producer, next_norm, resid) -> dict:
    """The keyword with which ``producer`` is offered the stream, if it can use it."""
    if not producer.fuses_residual:
        return {}
    if next_norm is not None and next_norm.fuses_residual:
        return {"add_into": next_norm.sink(resid)}
    return {"add_into": StreamSink(resid, None)}


register_part("block", "pre_norm", PreNormBlock)
