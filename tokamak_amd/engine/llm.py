"""Offline batch generation: ``LLM(model).generate(prompts, SamplingParams(...))``.

The shape of the interface follows the reference (src/tokamak/engine/llm.py:54-334):
load once, then ``generate`` runs a scheduler-driven step loop and returns one
``RequestOutput`` per prompt in input order.  Not thread-safe.
"""

from __future__ import annotations

import logging
import random
import time
from collections.abc import Sequence as AbcSequence
from dataclasses import dataclass
from pathlib import Path

import torch

from tokamak_amd.config.registry import get_architecture, load_model_description
from tokamak_amd.engine import text
from tokamak_amd.engine.outputs import RequestOutput
from tokamak_amd.engine.runner import ModelRunner, StepEntry, resolve_dtype
from tokamak_amd.kernels import ops
from tokamak_amd.engine.request import Request
from tokamak_amd.engine.scheduler import Scheduler, StepPlan
from tokamak_amd.sampling.params import SamplingParams
from tokamak_amd.sampling.sampler import sample_tokens
from tokamak_amd.weights.random_init import expected_tensors_of
from tokamak_amd.weights.sources import RandomSource, SafetensorsSource

logger = logging.getLogger(__name__)


@dataclass
class _InFlight:
    """A launched step whose sampled tokens the host has not read yet."""

    requests: list[Request]         # in the order of the sampler's rows
    tokens: torch.Tensor            # pinned host copy of those rows ...
    copied: torch.cuda.Event        # ... complete after this


class LLM:
    """Loads a model folder once and serves batch generation requests.

    Args (names and meanings as the reference's where it has them,
    src/tokamak/engine/llm.py:64-104):
        model: folder with ``config.json`` and ``*.safetensors``; or an architecture's
            typed configuration (e.g. ``Qwen3Config``) for seeded random weights
            (``seed``; the same weights ``write_random_model`` would put in a folder, unless
            ``random_weights_on_gpu`` draws them on the GPU, which is what a large shape needs).
        dtype: ``"bfloat16"`` (default) or ``"float32"`` (everything in true 32-bit).
        max_seq_len: cap on one request's context; default the model's maximum.
        block_size: tokens per cache page (a multiple of 8).
        kv_pool_tokens: capacity of the page pool in tokens; must be at least
            ``max_seq_len`` so a request can always finish alone.  Default: room for
            ``max_batch_size`` requests of ``max_seq_len`` tokens, within 90 % of the
            memory that the weights leave free (the reference's default, ``max_seq_len``,
            would serve one long request at a time).
        max_batch_size: most sequences running at once.
        max_num_batched_tokens: token budget of one step (new).
        tune_library_products: time the library's candidate algorithms for each new
            shape of a long portion's matrix products and keep the fastest (new; off by
            default: the library's first choice is taken, so that two runs of the same
            input compute the same bits).
        prefill_chunk: longest prompt portion in one step (new; default the budget).
        steps_ahead: launch every step before the tokens of the step before are read
            (new; default on: the host's work between two steps is hidden behind the GPU's;
            the tokens generated are the same either way).
        device: ``"auto"`` or a cuda device; there is no CPU path.
        kv_backend, scheduling, attention_backend, attention_policy, draft_model: the
            reference's further options; this engine has one choice for each
            (``"paged"``, ``"continuous"``, ``"auto"``, ``"full"``, ``None``) and
            refuses any other with a clear error.
    """

    _ONLY = {"kv_backend": ("paged",), "scheduling": ("continuous",),
             "attention_backend": ("auto", "hip"), "attention_policy": ("full",), "draft_model": (None,)}

    def __init__(self, model: str | Path, *, dtype: str | torch.dtype = "auto",
                 max_seq_len: int | None = None, block_size: int = 16,
                 kv_pool_tokens: int | None = None, max_batch_size: int = 16,
                 max_num_batched_tokens: int = 2048, prefill_chunk: int | None = None,
                 device: str | torch.device = "auto", kv_backend: str = "paged",
                 scheduling: str = "continuous", attention_backend: str = "auto",
                 attention_policy: str = "full", draft_model=None, seed: int = 0,
                 random_weights_on_gpu: bool = False, tune_library_products: bool = False,
                 steps_ahead: bool = True) -> None:
        given = {"kv_backend": kv_backend, "scheduling": scheduling, "attention_backend": attention_backend,
                 "attention_policy": attention_policy, "draft_model": draft_model}
        for name, value in given.items():
            if value not in self._ONLY[name]:
                raise ValueError(f"{name}={value!r} is not supported by this engine; "
                                 f"supported: {', '.join(map(repr, self._ONLY[name]))}")
        if dtype == "auto":
            dtype = "bfloat16"
        if device == "auto":
            device = "cuda:0"
        if torch.device(device).type != "cuda":
            raise ValueError(f"device={device!r}: this engine runs on the GPU only")
        if block_size < 1:
            raise ValueError(f"block_size must be >= 1, got {block_size}")
        if max_batch_size < 1:
            raise ValueError(f"max_batch_size must be >= 1, got {max_batch_size}")
        self.dtype = resolve_dtype(dtype)
        if hasattr(model, "architecture") and not isinstance(model, (str, Path)):
            # a typed configuration: seeded random weights, no folder
            folder = None
            self.architecture = get_architecture(model.architecture)
            self.model_config = model
            plan = self.architecture.plan(model)
            expected = {n: s for n, s in expected_tensors_of(plan).items() if not s.ignored}
            # drawn on the CPU they equal a folder written with the same seed; on the GPU
            # they differ from that but take seconds for tens of billions of parameters
            source = RandomSource(expected, seed, device=device if random_weights_on_gpu else "cpu")
        else:
            folder = Path(model)
            if not folder.is_dir():
                raise FileNotFoundError(f"model folder {folder} does not exist (no download is attempted)")
            self.architecture, self.model_config, plan = load_model_description(folder)
            source = SafetensorsSource(folder)
        model_max = plan.max_position_embeddings
        self.max_seq_len = min(max_seq_len or model_max, model_max)
        if kv_pool_tokens is not None and kv_pool_tokens < self.max_seq_len:
            raise ValueError(
                f"kv_pool_tokens ({kv_pool_tokens}) must be >= max_seq_len ({self.max_seq_len}) "
                f"so any single request can complete alone")
        self.max_batch_size = max_batch_size
        self.max_num_batched_tokens = max(max_num_batched_tokens, max_batch_size)
        self.prefill_chunk = prefill_chunk
        self.eos_token_ids = tuple(plan.eos_token_ids)
        ops.set_library_tuning(tune_library_products)
        # what the reference reports at load (src/tokamak/engine/llm.py:180-189, model/loader.py:95)
        logger.info("Loading %s (%s) on %s as %s (max_seq_len=%d, max_batch_size=%d, block_size=%d)",
                    folder if folder is not None else "seeded random weights", self.architecture.name, device,
                    self.dtype, self.max_seq_len, max_batch_size, block_size)
        started = time.perf_counter()
        self.runner = ModelRunner(plan, source, dtype=self.dtype,
                                  page_size=block_size, kv_pool_tokens=kv_pool_tokens,
                                  max_requests=max_batch_size, device=device,
                                  min_pool_tokens=self.max_seq_len, tokens_per_request=self.max_seq_len,
                                  max_step_tokens=self.max_num_batched_tokens)
        if self.runner.kv_pool_tokens < self.max_seq_len:
            raise RuntimeError(f"the GPU has no room for a cache of max_seq_len ({self.max_seq_len}) tokens")
        logger.info("Loaded %d tensors in %.1f s; cache pool of %d tokens in pages of %d",
                    self.runner.num_tensors, time.perf_counter() - started, self.runner.kv_pool_tokens, block_size)
        self.folder = folder
        self.tokenizer = text.load_tokenizer(folder)
        self.num_steps = 0
        self.num_preemptions = 0
        # the step loop runs one step ahead of the tokens it has read (see generate)
        self.steps_ahead = steps_ahead
        self._host_tokens = [torch.empty(max_batch_size, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        self._copied = [torch.cuda.Event(), torch.cuda.Event()]
        self._turn = 0
        self._progress = None
        self.last_progress = ""   # finished/all requests of the last generate() that showed a bar

    def chat_prompt(self, user_text: str) -> str:
        """``user_text`` as a single user turn, ready to tokenize: by the folder's chat
        template, else the architecture's (engine/text.py)."""
        return text.chat_prompt(self.folder, self.architecture, user_text)

    # ------------------------------------------------------------------
    def generate(self, prompts: str | AbcSequence[str] | None = None,
                 sampling_params: SamplingParams | AbcSequence[SamplingParams] | None = None, *,
                 prompt_token_ids: AbcSequence[AbcSequence[int]] | None = None,
                 use_tqdm: bool = True) -> list[RequestOutput]:
        """One completion per prompt, in input order
        (interface of reference: src/tokamak/engine/llm.py:265-334)."""
        if (prompts is None) == (prompt_token_ids is None):
            raise ValueError("provide exactly one of `prompts` or `prompt_token_ids`")
        texts: list[str | None]
        if prompt_token_ids is not None:
            id_lists = [list(ids) for ids in prompt_token_ids]
            texts = [None] * len(id_lists)
        else:
            if self.tokenizer is None:
                raise ValueError("the model folder has no tokenizer.json: pass prompt_token_ids")
            texts = [prompts] if isinstance(prompts, str) else list(prompts)
            id_lists = [self.tokenizer.encode(t).ids for t in texts]
        if sampling_params is None or isinstance(sampling_params, SamplingParams):
            per_request = [sampling_params or SamplingParams()] * len(id_lists)
        else:
            per_request = list(sampling_params)
            if len(per_request) != len(id_lists):
                raise ValueError(f"Got {len(per_request)} SamplingParams for {len(id_lists)} prompts")

        now = time.perf_counter()
        requests = [self.new_request(rid, ids, params, now)
                    for rid, (ids, params) in enumerate(zip(id_lists, per_request))]
        scheduler = Scheduler(self.runner.manager, self.max_batch_size, self.max_num_batched_tokens,
                              self.prefill_chunk)
        for request in requests:
            scheduler.submit(request)
        # a bar over finished requests, as the reference shows (src/tokamak/engine/llm.py:299)
        self._progress = None
        if use_tqdm:
            try:
                from tqdm.auto import tqdm
                self._progress = tqdm(total=len(requests), desc="Generating")
            except ImportError:
                pass
        try:
            self.run(scheduler)
        finally:
            if self._progress is not None:
                self.last_progress = f"{self._progress.n}/{self._progress.total}"
                self._progress.close()
                self._progress = None
            # also what the scheduler reserved for requests that never reached a step
            self.runner.end_all()
            for request in scheduler.live_requests():
                self.runner.manager.free(request.rid)
        return [self._output(request, text) for request, text in zip(requests, texts)]

    def new_request(self, rid: int, ids: list[int], params: SamplingParams, now: float | None = None) -> Request:
        """A checked request for ``ids``, with its seed and its limit of tokens."""
        seed = params.seed if params.seed is not None else random.getrandbits(62)
        request = Request.from_prompt(rid, ids, params, seed)
        request.arrived_at = time.perf_counter() if now is None else now
        self._check_request(request)
        request.context_limit = self._context_limit(request)
        return request

    def run(self, scheduler: Scheduler) -> None:
        """The step loop: until the scheduler has nothing left, plan a step, launch it, and
        read the tokens of the step before it.

        One step ahead: a step is planned and launched while the one before it runs; the
        tokens that one sampled are read (and stop rules applied) meanwhile.  A decoding
        request's next step takes its token from the sampler's output on the GPU.  With
        ``steps_ahead`` off every step's tokens are read before the next is planned.
        ``generate`` runs this loop, and so does the benchmark's timed decoding."""
        in_flight = None
        while scheduler.busy or in_flight is not None:
            plan = scheduler.plan() if scheduler.busy else None
            launched = self.launch(plan) if plan is not None else None
            if in_flight is not None:
                self.read(in_flight)
            elif plan is None or not plan.spans:
                raise RuntimeError("the scheduler has unfinished requests but plans no step")
            in_flight = launched
            if in_flight is not None and not self.steps_ahead:
                self.read(in_flight)
                in_flight = None

    def launch(self, plan: StepPlan) -> _InFlight | None:
        """Run the plan's step and draw its tokens, all without waiting for the GPU; None
        if the step samples nothing (or the plan is empty)."""
        for victim in plan.evicted:
            self.runner.forget(victim.rid)      # the scheduler has already freed its pages
            self.num_preemptions += 1
        for leaver in plan.released:
            self.runner.forget(leaver.rid)      # ends with the token on its way; nothing is recomputed
        if not plan.spans:
            return None
        entries, sampling = [], []
        for span in plan.spans:
            request = span.request
            held = self.runner.cached_tokens(request.rid)
            if span.start != held or span.start != request.cached:
                raise RuntimeError(f"request {request.rid}: span starts at {span.start}, the cache holds {held}")
            entries.append(StepEntry(request.rid, request.span(span.length), [span.length - 1] if span.samples else [],
                                     span.feed))
            if span.samples:
                sampling.append(request)
        logits = self.runner.step(entries)
        self.num_steps += 1
        for span in plan.spans:
            span.request.advance(span.length)
        if not sampling:
            return None
        drawn = sample_tokens(logits, [r.params for r in sampling], [r.seed for r in sampling],
                              [r.num_drawn for r in sampling], out=self.runner.sampled)
        for row, request in enumerate(sampling):
            request.unknown += 1
            request.feed_row = row
        turn = self._turn
        self._turn = 1 - turn
        host = self._host_tokens[turn][:len(sampling)]
        host.copy_(drawn, non_blocking=True)
        self._copied[turn].record()
        return _InFlight(sampling, host, self._copied[turn])

    def read(self, step: _InFlight) -> None:
        """Wait for a launched step's tokens and give them to their requests."""
        step.copied.synchronize()
        stamp = time.perf_counter()
        for request, token in zip(step.requests, step.tokens.tolist()):
            if request.finished:
                continue    # it ended with an earlier token while this step already ran: one token for nothing
            if request.first_token_at is None:
                request.first_token_at = stamp
            if request.accept(token, eos_token_ids=self.eos_token_ids, context_limit=request.context_limit):
                request.finished_at = stamp
                self.runner.end(request.rid)
                if self._progress is not None:
                    self._progress.update(1)

    # ------------------------------------------------------------------
    def _context_limit(self, request: Request) -> int:
        """Most tokens the request may ever hold: its prompt plus ``max_new_tokens``,
        within ``max_seq_len`` (reference: src/tokamak/engine/llm.py:483-485)."""
        return min(self.max_seq_len, request.prompt_len + request.params.max_new_tokens)

    def _check_request(self, request: Request) -> None:
        """Refuse at submission what could never finish: a prompt that leaves no room
        to generate, ids outside the vocabulary, more pages than the pool has
        (reference: src/tokamak/engine/llm.py:487-499)."""
        if request.prompt_len >= self.max_seq_len:
            raise ValueError(f"prompt {request.rid} has {request.prompt_len} tokens and does not fit "
                             f"max_seq_len={self.max_seq_len}: at least one token must be generated")
        vocab = self.runner.plan.vocab_size
        if min(request.tokens) < 0 or max(request.tokens) >= vocab:
            raise ValueError(f"prompt {request.rid} has a token id outside [0, {vocab})")
        manager = self.runner.manager
        pages = manager.pages_needed(self._context_limit(request))
        smallest = min(manager.num_pages(g) for g in range(len(manager.groups))) if manager.groups else pages
        if pages > smallest:
            raise ValueError(f"prompt {request.rid} may grow to {pages} cache pages, the pool has {smallest}: "
                             f"raise kv_pool_tokens or lower max_new_tokens")

    def _text(self, ids: list[int]) -> str | None:
        return None if self.tokenizer is None else self.tokenizer.decode(ids, skip_special_tokens=True)

    def _output(self, request: Request, prompt_text: str | None) -> RequestOutput:
        if not request.finished:
            raise RuntimeError(f"request {request.rid} left the step loop unfinished")
        since = request.arrived_at

        def elapsed(t):
            return None if t is None or since is None else t - since

        return RequestOutput(
            request_id=request.rid,
            prompt=prompt_text if prompt_text is not None else self._text(request.prompt),
            prompt_token_ids=request.prompt,
            output_text=self._text(request.generated),
            output_token_ids=request.generated,
            finish_reason=request.finish_reason,
            ttft_s=elapsed(request.first_token_at),
            latency_s=elapsed(request.finished_at),
        )
