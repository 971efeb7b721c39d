"""Captured decode steps.

A step in which every request brings exactly one token has a fixed shape once
the batch size, the block-table width and the split of the context are fixed.
Such a step is recorded once into a HIP graph and replayed: one launch instead
of several hundred.  The graph reads its descriptor from a static device
buffer that is refilled (one host-to-device copy) before every replay; nothing
in it allocates, clears memory or calls a library.
"""

from __future__ import annotations

import torch

from tokamak_amd.engine.batch import PackedBatch, batch_from_device


def pow2_at_least(n: int, floor: int) -> int:
    v = floor
    while v < n:
        v *= 2
    return v


class DecodeGraph:
    def __init__(self, model, storage, packed: PackedBatch, device) -> None:
        self.size = int(packed.buf.size)
        self.host = torch.empty(self.size, dtype=torch.int32, pin_memory=True)
        self.dev = torch.empty(self.size, dtype=torch.int32, device=device)
        self.batch = batch_from_device(packed, self.dev)
        self._load(packed)
        # run once outside the graph: code objects are loaded and buffers exist
        # before the capture starts (what it writes, the replay writes again)
        model.forward(self.batch, storage)
        torch.cuda.synchronize(device)
        self.batch.memo.clear()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.logits = model.forward(self.batch, storage)
        self.replays = 0

    def _load(self, packed: PackedBatch) -> None:
        if packed.buf.size != self.size:
            raise ValueError("descriptor does not have the shape this graph was captured for")
        self.host.numpy()[:] = packed.buf
        self.dev.copy_(self.host, non_blocking=True)

    def run(self, packed: PackedBatch) -> torch.Tensor:
        """Replay with a new descriptor; the returned logits live in the graph's
        own memory and are overwritten by the next replay."""
        self._load(packed)
        self.graph.replay()
        self.replays += 1
        return self.logits
