"""Captured decode steps.

A step in which every request brings exactly one token has a fixed shape once
the batch size, the block-table width and what the parts' planners say of the step
(for attention: how the context is split) are fixed.
Such a step is recorded once into a HIP graph and replayed: one launch instead
of several hundred.  The graph reads its descriptor from a static device
buffer that is refilled (one host-to-device copy) before every replay; nothing
in it allocates, clears memory or calls a library.

The step that meets a new shape runs eagerly, once, and is recorded afterwards
without being executed again: a part that advances per-request state sees every
token exactly once, whether its step was the recorded one or a replay.
"""

from __future__ import annotations

import gc

import torch

from tokamak_amd.engine.batch import PackedBatch, batch_from_device


def pow2_at_least(n: int, floor: int) -> int:
    v = floor
    while v < n:
        v *= 2
    return v


class DecodeGraph:
    """One recorded decode shape.

    The descriptor travels through two pinned host buffers used in turn, each
    with an event that marks the end of its last copy: a caller may queue
    several replays without synchronising, and the host never rewrites a buffer
    whose copy has not run yet.
    """

    def __init__(self, model, storage, packed: PackedBatch, device, feed=None) -> None:
        self.size = int(packed.buf.size)
        self._host = [torch.empty(self.size, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        self._copied = [torch.cuda.Event(), torch.cuda.Event()]
        self._turn = 0
        self.dev = torch.empty(self.size, dtype=torch.int32, device=device)
        self.batch = batch_from_device(packed, self.dev)
        self._load(packed, feed)
        # this step itself, eagerly: code objects are loaded and the allocator is warm
        # before the recording starts; the recording executes nothing
        self.first_logits = model.forward(self.batch, storage)
        torch.cuda.synchronize(device)
        self.batch.memo.clear()
        # what the recording holds: the most that is live at once while it is recorded (its
        # private pool keeps that much), measured from here on
        torch.cuda.reset_peak_memory_stats(device)
        before = torch.cuda.memory_allocated(device)
        self.graph = torch.cuda.CUDAGraph()
        # No garbage collection while the stream is being recorded: a collection that starts in
        # the middle of the step (any allocation may start one) can free cyclic garbage that
        # owns GPU objects of its own, an older runner's recorded steps say, and destroying
        # those is not allowed during a recording: the HIP runtime then ends the process.
        # (torch collects once before the recording starts; what the step itself drops goes
        # by reference count as always.)
        collecting = gc.isenabled()
        gc.disable()
        try:
            with torch.cuda.graph(self.graph):
                self.logits = model.forward(self.batch, storage)
        finally:
            if collecting:
                gc.enable()
        self.bytes = max(0, torch.cuda.max_memory_allocated(device) - before) + self.size * 4
        self.replays = 0

    def _load(self, packed: PackedBatch, feed=None) -> None:
        """The descriptor to the device; then ``feed(batch)`` puts in the token ids that are
        still on the GPU (outside the recording: how many there are changes from step to step)."""
        if packed.buf.size != self.size:
            raise ValueError("descriptor does not have the shape this graph was captured for")
        turn = self._turn
        self._turn = 1 - turn
        self._copied[turn].synchronize()       # the copy that last read this buffer has run
        self._host[turn].numpy()[:] = packed.buf
        self.dev.copy_(self._host[turn], non_blocking=True)
        self._copied[turn].record()
        self.batch.num_feed = packed.num_feed
        if feed is not None:
            feed(self.batch)

    def run(self, packed: PackedBatch, feed=None) -> torch.Tensor:
        """Replay with a new descriptor; the returned logits live in the graph's
        own memory and are overwritten by the next replay."""
        self._load(packed, feed)
        self.graph.replay()
        self.replays += 1
        return self.logits
