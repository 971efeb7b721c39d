"""The step function: run a batch of (request, its next tokens) from the cache.

One ``ModelRunner`` owns the model, the cache manager and the cache memory.
``step`` runs only the tokens it is given, as one batch, against what earlier
steps left in the cache, and returns float32 logits at the wanted places.
Generation (``LLM``), the scheduler and trace replay all drive this one
function.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from pathlib import Path

import torch

from tokamak_amd.cache.manager import CacheManager, OutOfSlotsError
from tokamak_amd.cache.pages import OutOfPagesError
from tokamak_amd.config.registry import load_model_description
from tokamak_amd.engine.batch import StepBatch, StepSpan, batch_from_device, pack_batch
from tokamak_amd.engine.decode_graph import DecodeGraph, pow2_at_least
from tokamak_amd.engine.model import LayeredModel
from tokamak_amd.engine.storage import CacheStorage
from tokamak_amd.kernels import ops
from tokamak_amd.weights.loader import load_weights
from tokamak_amd.weights.sources import SafetensorsSource

MAX_GRAPHS = 256   # captured decode shapes kept; the one used longest ago goes first
MAX_GRAPH_BATCH = 64   # larger decode batches use the library product, which is not recorded
GRAPH_MEMORY_BYTES = 8 << 30   # device memory the captured shapes may hold together

DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32,
          torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}


def resolve_dtype(dtype) -> torch.dtype:
    try:
        return DTYPES[dtype]
    except KeyError:
        raise ValueError(f"dtype must be 'bfloat16' or 'float32', got {dtype!r}") from None


@dataclass
class StepEntry:
    """A request's next tokens, and the offsets among them whose logits are wanted.

    ``feed``: the entry brings one token that the host does not know yet: row ``feed`` of
    ``ModelRunner.sampled``, where the sampler of the step before has left it (``tokens``
    holds a placeholder).  With it a decode step is launched while the step before it still
    runs, and the host reads that step's tokens meanwhile."""

    request: object
    tokens: list[int]
    want: list[int] = field(default_factory=list)
    feed: int | None = None


class ModelRunner:
    """Model, cache manager and cache memory of one GPU, and the step function.

    ``kv_pool_tokens``: capacity of the page pool; None sizes it from the memory
    that is free once the weights are loaded: ``memory_fraction`` of it, less
    what the largest steps need for their activations (measured: one step of
    ``max_step_tokens`` tokens and one of ``max_requests`` single tokens run
    against a small throw-away cache) and less ``graph_memory_bytes`` for the
    captured decode shapes, and no more than ``max_requests`` requests of
    ``tokens_per_request`` tokens can use.
    """

    def __init__(self, plan, source, *, dtype="bfloat16", page_size: int = 16,
                 kv_pool_tokens: int | None, max_requests: int = 64,
                 device: str | torch.device = "cuda:0", use_graphs: bool = True,
                 min_pool_tokens: int = 0, tokens_per_request: int | None = None,
                 memory_fraction: float = 0.9, max_step_tokens: int = 2048,
                 graph_memory_bytes: int = GRAPH_MEMORY_BYTES) -> None:
        self.dtype = resolve_dtype(dtype)
        self.device = torch.device(device)
        if self.device.type != "cuda" or not torch.cuda.is_available():
            raise RuntimeError("tokamak_amd runs on a GPU only; no GPU is visible")
        if page_size < 1:
            raise ValueError(f"page_size must be >= 1, got {page_size}")
        self.plan = plan
        self.page_size = page_size
        self.model = LayeredModel(plan, dtype=self.dtype, device=self.device)
        self.model.check_page_size(page_size)      # what the parts' kernels take
        self._planners = self.model.step_planners()
        self.num_tensors = load_weights(self.model, source, dtype=self.dtype, device=self.device)
        groups, layouts = self.model.cache_layout()
        self.num_groups = len(groups)
        self._groups = groups
        self._ctx_len: dict[object, int] = {}
        self._graphs: dict[tuple, DecodeGraph] = {}
        # where a sampler leaves its tokens for entries of the next step that ``feed`` on them
        self.sampled = torch.zeros(max(max_requests, 1), dtype=torch.int32, device=self.device)
        self.graph_memory_bytes = int(graph_memory_bytes)
        self.step_memory_bytes = 0
        self.use_graphs = False
        if kv_pool_tokens is None:
            per_token = sum(lay.request.bytes_per_token(self.dtype) for lay in layouts.values())
            self.step_memory_bytes = self._measure_step_memory(max_step_tokens, max_requests)
            free, _ = torch.cuda.mem_get_info(self.device)
            room = int(free * memory_fraction) - self.step_memory_bytes - self.graph_memory_bytes
            fits = max(0, room) // max(per_token, 1)
            longest = tokens_per_request or plan.max_position_embeddings
            kv_pool_tokens = max(min_pool_tokens, min(max_requests * longest, fits))
        self.kv_pool_tokens = int(kv_pool_tokens)
        self._make_cache(max(1, -(-int(kv_pool_tokens) // page_size)), max_requests)
        self.use_graphs = use_graphs and self.model.capturable

    def _make_cache(self, num_pages: int, max_requests: int) -> None:
        self.manager = CacheManager(self._groups, num_pages, self.page_size, max_requests)
        self.storage = CacheStorage(self.model, [num_pages] * self.num_groups, self.page_size, max_requests,
                                    dtype=self.dtype, device=self.device)

    def _measure_step_memory(self, max_step_tokens: int, max_requests: int) -> int:
        """Peak device memory, beyond weights and cache, of the two largest kinds of
        step: one request bringing ``max_step_tokens`` tokens, and ``max_requests``
        requests bringing one token each.  Run for real against a throw-away cache
        just large enough, so whatever the parts allocate is counted, workspaces of
        library products included."""
        tokens = max(1, min(max_step_tokens, self.plan.max_position_embeddings))
        self._make_cache(-(-tokens // self.page_size) + max_requests, max_requests)
        torch.cuda.synchronize(self.device)
        before = torch.cuda.memory_allocated(self.device)
        torch.cuda.reset_peak_memory_stats(self.device)
        self.step([StepEntry("measure", [0] * tokens, [tokens - 1])])
        self.end("measure")
        self.step([StepEntry(("measure", i), [0], [0]) for i in range(max_requests)])
        self.end_all()
        torch.cuda.synchronize(self.device)
        peak = torch.cuda.max_memory_allocated(self.device) - before
        kept = torch.cuda.memory_allocated(self.device) - before    # workspaces that stay
        del self.manager, self.storage
        torch.cuda.empty_cache()
        return max(0, peak - max(0, kept))

    @classmethod
    def from_folder(cls, folder: str | Path, **kwargs) -> ModelRunner:
        _, _, plan = load_model_description(folder)
        return cls(plan, SafetensorsSource(folder), **kwargs)

    # -- request lifetime ------------------------------------------------------
    def cached_tokens(self, request) -> int:
        return self._ctx_len.get(request, 0)

    def is_live(self, request) -> bool:
        return request in self._ctx_len

    def forget(self, request) -> None:
        """Drop the record of what the cache holds for ``request`` (its pages were
        already given back by whoever preempted it)."""
        self._ctx_len.pop(request, None)

    def end(self, request) -> None:
        """The request is finished: give back what it holds."""
        self._ctx_len.pop(request, None)
        self.manager.free(request)

    def end_all(self) -> None:
        for request in list(self._ctx_len):
            self.end(request)

    # -- the step --------------------------------------------------------------
    def _validate(self, entries: list[StepEntry]) -> None:
        """Refuse a step that cannot run, before anything is reserved for it: the
        cache manager and the live requests are as they were when this raises."""
        vocab, limit = self.plan.vocab_size, self.plan.max_position_embeddings
        seen = set()
        newcomers = 0
        for e in entries:
            if not e.tokens:
                raise ValueError(f"request {e.request!r} brings no tokens to this step")
            if min(e.tokens) < 0 or max(e.tokens) >= vocab:
                raise ValueError(f"request {e.request!r} has a token id outside [0, {vocab})")
            if e.request in seen:
                raise ValueError(f"request {e.request!r} appears twice in one step")
            seen.add(e.request)
            total = self._ctx_len.get(e.request, 0) + len(e.tokens)
            if total > limit:
                raise ValueError(
                    f"request {e.request!r} would reach {total} tokens; the model's limit is {limit}")
            if any(not 0 <= w < len(e.tokens) for w in e.want):
                raise ValueError(f"request {e.request!r} wants logits outside its {len(e.tokens)} tokens")
            if e.feed is not None and (len(e.tokens) != 1 or not 0 <= e.feed < self.sampled.numel()):
                raise ValueError(f"request {e.request!r}: a fed token is one token, from a row of the "
                                 f"{self.sampled.numel()} that the sampler's output holds")
            if e.request not in self._ctx_len and self.manager.slots.slot_of(e.request) is None:
                newcomers += 1
        if newcomers > self.manager.slots.num_free:
            raise OutOfSlotsError(f"{newcomers} new request(s) in this step, but only "
                                  f"{self.manager.slots.num_free} of {self.manager.slots.num_slots} state slots are free")
        # pages: what every group has free, plus what the windows hand back first, against the step's growth
        for gi, group in enumerate(self.manager.groups):
            need = 0
            for e in entries:
                ctx = self._ctx_len.get(e.request, 0)
                need += group.shortfall(e.request, ctx + len(e.tokens))
                if group.spec.window is not None:
                    need -= group.releasable_before(e.request, ctx - group.spec.window + 1)
            if need > group.pool.num_free:
                raise OutOfPagesError(
                    f"this step needs {need} more page(s) of group {group.spec.name!r}, but only "
                    f"{group.pool.num_free} of {group.pool.num_pages} are free")

    def _spans(self, entries: list[StepEntry]) -> list[StepSpan]:
        self._validate(entries)
        # first everything that gives pages back, then everything that takes them: the
        # validation counted the step as a whole
        for e in entries:
            if e.request not in self._ctx_len:
                self.storage.reset_state(self.manager.admit(e.request))
                self._ctx_len[e.request] = 0
            self.manager.release_behind_window(e.request, self._ctx_len[e.request])
        spans = []
        for e in entries:
            ctx = self._ctx_len[e.request]
            self.manager.ensure_capacity(e.request, ctx + len(e.tokens))
            spans.append(StepSpan(
                request=e.request, tokens=list(e.tokens), ctx_len=ctx,
                state_slot=self.manager.slots.slot_of(e.request),
                tables=[self.manager.block_table(e.request, g) for g in range(self.num_groups)],
                want=list(e.want), feed=e.feed))
        return spans

    def _feed(self, batch: StepBatch) -> None:
        """Put the tokens that are still on the GPU into the descriptor's token ids."""
        if batch.num_feed:
            ops.feed_tokens(batch.token_ids, self.sampled, batch.feed_slots, batch.feed_rows, batch.num_feed,
                            self.sampled.numel())

    def prepare(self, entries: list[StepEntry]) -> StepBatch:
        """Reserve what the entries need and build the step's descriptor."""
        packed = pack_batch(self._spans(entries), self.num_groups, self._planners)
        host = torch.from_numpy(packed.buf)
        batch = batch_from_device(packed, host.pin_memory().to(self.device, non_blocking=True))
        self._feed(batch)
        return batch

    def _graph_step(self, entries: list[StepEntry]) -> torch.Tensor:
        """All entries bring one token: replay the captured step of this shape."""
        spans = self._spans(entries)
        wanted = [i for i, s in enumerate(spans) if s.want]
        for s in spans:
            s.want = [0]            # the captured step computes every row's logits
        widths = [pow2_at_least(max(len(s.tables[g]) for s in spans), 16) for g in range(self.num_groups)]
        # the parts' facts of the step (rounded as their planners ask) are part of the shape
        packed = pack_batch(spans, self.num_groups, self._planners, fixed_widths=widths, bucket=True)
        key = (len(spans), tuple(widths), packed.shape_key())
        graph = self._graphs.pop(key, None)
        if graph is None:
            # a new shape: this step runs eagerly, once, and is recorded for the next ones
            graph = DecodeGraph(self.model, self.storage, packed, self.device, self._feed)
            logits, graph.first_logits = graph.first_logits, None
            self._graphs[key] = graph
            self._trim_graphs()
        else:
            self._graphs[key] = graph                # most recently used last
            logits = graph.run(packed, self._feed)
        if len(wanted) == len(spans):
            return logits
        return logits[torch.tensor(wanted, dtype=torch.long, device=self.device)] if wanted else logits[:0]

    def _trim_graphs(self) -> None:
        """Keep the captured shapes within their count and their memory: the shape
        used longest ago goes first, the newest always stays."""
        def total() -> int:
            return sum(g.bytes for g in self._graphs.values())

        while len(self._graphs) > 1 and (len(self._graphs) > MAX_GRAPHS or total() > self.graph_memory_bytes):
            self._graphs.pop(next(iter(self._graphs)))

    @torch.inference_mode()
    def step(self, entries: list[StepEntry]) -> torch.Tensor:
        """Run the entries as one batch; logits float32 [wanted, vocab], in the
        order of the entries and of each entry's ``want``.  The tensor may be
        reused by the next step: read it before stepping again."""
        if not entries:
            return torch.empty((0, self.plan.vocab_size), dtype=torch.float32, device=self.device)
        with torch.cuda.device(self.device):
            if (self.use_graphs and len(entries) <= MAX_GRAPH_BATCH
                    and all(len(e.tokens) == 1 for e in entries)
                    and all(list(e.want) in ([], [0]) for e in entries)):
                logits = self._graph_step(entries)
            else:
                with ops.pinned_stream():
                    logits = self.model.forward(self.prepare(entries), self.storage)
        for e in entries:
            self._ctx_len[e.request] += len(e.tokens)
        return logits
