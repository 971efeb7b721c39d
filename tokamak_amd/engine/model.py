"""The model the engine runs: parts put together as a ``ModelPlan`` says."""

from __future__ import annotations

from dataclasses import dataclass

import torch

from tokamak_amd.cache.pages import CacheGroupSpec
from tokamak_amd.config.model_config import ModelPlan, PartSpec
from tokamak_amd.config.registry import get_part
from tokamak_amd.engine import layer_replay
from tokamak_amd.kernels import ops
from tokamak_amd.kernels.linear import Added
from tokamak_amd.parts.base import Block, CacheRequest, Part, StateArray
from tokamak_amd.weights.spec import TensorSpec


@dataclass
class SlotLayout:
    """Where one cache slot lives: its group, and what its mixer asked for."""

    group: int
    request: CacheRequest


class LayeredModel:
    """Embedding, layers run in the plan's order, final norm, head.

    ``forward`` runs exactly the tokens of the batch against the cache and
    returns float32 logits at ``batch.logit_rows``.  Sub-parts marked ``shared``
    with equal family and spec (position encodings) are built once, so what they
    prepare for a step is prepared once.
    """

    def __init__(self, plan: ModelPlan, *, dtype: torch.dtype, device: str | torch.device) -> None:
        self.plan = plan
        self.dtype = dtype
        self.device = torch.device(device)
        self._shared: dict[tuple[str, PartSpec], Part] = {}
        self.embedding = self._build("embedding", plan.embedding)
        self.blocks: list[Block] = []
        for spec in plan.layers:
            parts = {role: self._build(sub.family, sub.spec, shared=sub.shared) for role, sub in spec.parts}
            self.blocks.append(get_part("block", spec.block.kind)(parts, **spec.block.as_dict()))
        self.final_norm = self._build("norm", plan.final_norm)
        self.head = self._build("head", plan.head)
        # Layers of one kind (equal parts, block and arguments; only their tensors differ) launch
        # the same kernels in a step: one is recorded, the others replayed (engine/layer_replay.py).
        self.replay_layers = True
        kinds: dict[tuple, int] = {}
        self._layer_kind = [
            kinds.setdefault((spec.block, tuple((role, sub.family, sub.spec, sub.shared) for role, sub in spec.parts)), i)
            for i, spec in enumerate(plan.layers)
        ]
        self._own_tensors: dict[tuple[int, int], tuple] = {}

    def _build(self, family: str, spec: PartSpec, shared: bool = False) -> Part:
        if shared and (family, spec) in self._shared:
            return self._shared[(family, spec)]
        part = get_part(family, spec.kind)(**spec.as_dict(), dtype=self.dtype, device=self.device)
        if shared:
            self._shared[(family, spec)] = part
        return part

    def _all_parts(self):
        yield self.embedding
        for block in self.blocks:
            yield from block.parts.values()
        yield self.final_norm
        yield self.head

    @property
    def capturable(self) -> bool:
        """Whether a decode step of this model may be recorded into a HIP graph."""
        return all(getattr(p, "capturable", False) for p in self._all_parts())

    # -- weights -------------------------------------------------------------
    def _named_parts(self):
        p = self.plan
        yield p.embedding_prefix, self.embedding
        for i, (spec, block) in enumerate(zip(p.layers, self.blocks)):
            base = p.layer_prefix.format(i)
            for role, sub in spec.parts:
                yield base + sub.prefix, block.parts[role]
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
        self._own_tensors.clear()
        if self.plan.tie_word_embeddings:
            self.head.tie(self.embedding)

    # -- what the parts ask of a step ------------------------------------------
    def step_planners(self) -> list:
        """The parts' planners of work lists, one per name, in the order first met."""
        found: dict[str, object] = {}
        for part in self._all_parts():
            planner = part.step_planner()
            if planner is not None:
                if not planner.name:
                    raise ValueError(f"{type(part).__name__}'s step planner has no name")
                found.setdefault(planner.name, planner)
        return list(found.values())

    def check_page_size(self, page_size: int) -> None:
        for part in self._all_parts():
            part.check_page_size(page_size)

    # -- cache ---------------------------------------------------------------
    def _mixers_of(self, call):
        """(mixer, cache slot) pairs of a layer call."""
        mixers = list(self.blocks[call.layer].mixers.values())
        if mixers and len(call.slots) != len(mixers):
            raise ValueError(f"layer {call.layer} has {len(mixers)} mixer(s) but its call brings "
                             f"{len(call.slots)} cache slot(s)")
        return list(zip(mixers, call.slots))

    def _store_of(self, call, storage):
        """What the block of a call receives as ``store``: its mixer's slot, or with several
        mixers a dict of slots by their roles."""
        block = self.blocks[call.layer]
        if len(block.mixers) <= 1:
            return storage.slot(call.slots[0])
        return {role: storage.slot(slot) for role, slot in zip(block.mixers, call.slots)}

    def cache_layout(self) -> tuple[list[CacheGroupSpec], dict[int, SlotLayout]]:
        """Cache groups (slots that share a retention rule) and each slot's layout."""
        requests: dict[int, CacheRequest] = {}
        for call in self.plan.order:
            if not call.writes_cache:
                continue
            for mixer, slot in self._mixers_of(call):
                req = mixer.cache_request()
                if req is None:
                    continue
                if slot in requests and requests[slot] != req:
                    raise ValueError(f"cache slot {slot} is written with two different layouts")
                requests[slot] = req
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

    def state_requests(self) -> dict[int, dict[str, StateArray]]:
        """Cache slot -> arrays of the fixed-size per-request state its mixer keeps."""
        out: dict[int, dict[str, StateArray]] = {}
        for call in self.plan.order:
            if not call.writes_cache:
                continue
            for mixer, slot in self._mixers_of(call):
                request = mixer.state_request()
                if request:
                    out[slot] = dict(request)
        return out

    # -- compute -------------------------------------------------------------
    def forward(self, batch, storage) -> torch.Tensor:
        resid = self.embedding.forward(batch)
        pending = None
        order = self.plan.order
        replay = self.replay_layers and ops.can_record()
        recordings: dict[tuple, layer_replay.LayerRecording | None] = {}
        for at, call in enumerate(order):
            block = self.blocks[call.layer]
            store = self._store_of(call, storage)
            kwargs = {}
            if block.fuses_residual:
                # the norm that reads the stream after this block: its last product may prepare for it
                kwargs["then"] = self.blocks[order[at + 1].layer].entry_norm if at + 1 < len(order) else self.final_norm
            elif isinstance(pending, Added):
                pending = None      # the sum is in the stream already
            if not (replay and block.replayable):
                pending = block.forward(resid, pending, batch, store, call.writes_cache, **kwargs)
                continue
            then = kwargs.get("then")
            held = self._own_tensors.get((call.layer, call.cache))
            if held is None or held[0] is not storage:      # (another cache storage: its arrays lie elsewhere)
                held = self._own_tensors[(call.layer, call.cache)] = (storage, layer_replay.own_tensors(block, store))
            own = held[1]
            tensors = layer_replay.call_tensors(own, pending, then)
            key = (self._layer_kind[call.layer], call.writes_cache, layer_replay.store_groups(store), type(then),
                   layer_replay.pending_kind(pending))
            if key in recordings:
                recorded = recordings[key]
                if recorded is not None:
                    pending = recorded.launch(tensors, then)
                else:
                    pending = block.forward(resid, pending, batch, store, call.writes_cache, **kwargs)
                continue
            pending, recordings[key] = layer_replay.record(
                lambda: block.forward(resid, pending, batch, store, call.writes_cache, **kwargs), tensors)
        if batch.num_logit_rows == 0:
            return torch.empty((0, self.plan.vocab_size), dtype=torch.float32, device=self.device)
        if isinstance(pending, Added) and not self.final_norm.fuses_residual:
            pending = None
        h = self.final_norm.forward(resid, pending, rows=batch.logit_rows, write_resid=False)
        return self.head.forward(h)
