"""The model the engine runs: parts put together as a ``ModelPlan`` says."""

from __future__ import annotations

from dataclasses import dataclass

import torch

from tokamak_amd.cache.pages import CacheGroupSpec
from tokamak_amd.config.model_config import ModelPlan, PartSpec
from tokamak_amd.config.registry import get_part
from tokamak_amd.parts.base import Block, CacheRequest
from tokamak_amd.weights.spec import TensorSpec


def _build(family: str, spec: PartSpec, dtype, device):
    return get_part(family, spec.kind)(**spec.as_dict(), dtype=dtype, device=device)


@dataclass
class SlotLayout:
    """Where one cache slot lives: its group, and what its mixer asked for."""

    group: int
    request: CacheRequest


class LayeredModel:
    """Embedding, layers run in the plan's order, final norm, head.

    ``forward`` runs exactly the tokens of the batch against the cache and
    returns float32 logits at ``batch.logit_rows``.
    """

    def __init__(self, plan: ModelPlan, *, dtype: torch.dtype, device: str | torch.device) -> None:
        self.plan = plan
        self.dtype = dtype
        self.device = torch.device(device)
        self.embedding = _build("embedding", plan.embedding, dtype, device)
        self.blocks: list[Block] = []
        for spec in plan.layers:
            block_cls = get_part("block", spec.block.kind)
            self.blocks.append(block_cls(
                _build("mixer", spec.mixer, dtype, device),
                _build("feed_forward", spec.feed_forward, dtype, device),
                _build("norm", spec.mixer_norm, dtype, device),
                _build("norm", spec.feed_forward_norm, dtype, device),
                **spec.block.as_dict(),
            ))
        self.final_norm = _build("norm", plan.final_norm, dtype, device)
        self.head = _build("head", plan.head, dtype, device)

    @property
    def capturable(self) -> bool:
        """Whether a decode step of this model may be recorded into a HIP graph."""
        parts = [self.embedding, self.final_norm, self.head]
        for block in self.blocks:
            parts += [block.mixer, block.feed_forward, block.mixer_norm, block.feed_forward_norm]
            position = getattr(block.mixer, "position", None)
            if position is not None:
                parts.append(position)
        return all(getattr(p, "capturable", False) for p in parts)

    # -- weights -------------------------------------------------------------
    def _named_parts(self):
        p = self.plan
        yield p.embedding_prefix, self.embedding
        for i, (spec, block) in enumerate(zip(p.layers, self.blocks)):
            base = p.layer_prefix.format(i)
            yield base + spec.mixer_norm_prefix, block.mixer_norm
            yield base + spec.mixer_prefix, block.mixer
            yield base + spec.feed_forward_norm_prefix, block.feed_forward_norm
            yield base + spec.feed_forward_prefix, block.feed_forward
        yield p.final_norm_prefix, self.final_norm
        yield p.head_prefix, self.head

    def expected_tensors(self) -> dict[str, TensorSpec]:
        out: dict[str, TensorSpec] = {}
        for prefix, part in self._named_parts():
            for name, spec in part.expected_tensors(prefix).items():
                if name in out:
                    raise ValueError(f"two parts claim tensor {name!r}")
                out[name] = spec
        return out

    def bind(self, fetch) -> None:
        for prefix, part in self._named_parts():
            part.bind(prefix, fetch)
        if self.plan.tie_word_embeddings:
            self.head.tie(self.embedding)

    # -- cache ---------------------------------------------------------------
    def cache_layout(self) -> tuple[list[CacheGroupSpec], dict[int, SlotLayout]]:
        """Cache groups (slots that share a retention rule) and each slot's layout."""
        requests: dict[int, CacheRequest] = {}
        for call in self.plan.order:
            if not call.writes_cache:
                continue
            req = self.blocks[call.layer].mixer.cache_request()
            if req is None:
                continue
            if call.cache in requests and requests[call.cache] != req:
                raise ValueError(f"cache slot {call.cache} is written with two different layouts")
            requests[call.cache] = req
        windows: list[int | None] = []
        for req in requests.values():
            if req.window not in windows:
                windows.append(req.window)
        windows.sort(key=lambda w: (w is not None, w or 0))
        groups = [
            CacheGroupSpec(
                name="full" if w is None else f"window{w}",
                slots=tuple(s for s, r in sorted(requests.items()) if r.window == w),
                window=w,
            )
            for w in windows
        ]
        slots = {s: SlotLayout(windows.index(r.window), r) for s, r in requests.items()}
        return groups, slots

    def state_shapes(self) -> dict[int, tuple[int, ...]]:
        """Cache slot -> shape of the fixed-size per-request state its mixer keeps."""
        out: dict[int, tuple[int, ...]] = {}
        for call in self.plan.order:
            shape = self.blocks[call.layer].mixer.state_shape()
            if shape is not None and call.writes_cache:
                out[call.cache] = tuple(shape)
        return out

    # -- compute -------------------------------------------------------------
    def forward(self, batch, storage) -> torch.Tensor:
        resid = self.embedding.forward(batch.token_ids)
        pending = None
        for call in self.plan.order:
            pending = self.blocks[call.layer].forward(
                resid, pending, batch, storage.slot(call.cache), call.writes_cache)
        if batch.num_logit_rows == 0:
            return torch.empty((0, self.plan.vocab_size), dtype=torch.float32, device=self.device)
        h = self.final_norm.forward(resid, pending, rows=batch.logit_rows, write_resid=False)
        return self.head.forward(h)
