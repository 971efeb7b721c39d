"""Offline batch generation: ``LLM(model).generate(prompts, SamplingParams(...))``.

The shape of the interface follows the reference (src/tokamak/engine/llm.py:54-334):
load once, then ``generate`` runs a scheduler-driven step loop and returns one
``RequestOutput`` per prompt in input order.  Not thread-safe.
"""

from __future__ import annotations

import random
import time
from collections.abc import Sequence as AbcSequence
from pathlib import Path

import torch

from tokamak_amd.config.registry import get_architecture, load_model_description
from tokamak_amd.engine.outputs import RequestOutput
from tokamak_amd.engine.runner import ModelRunner, StepEntry, resolve_dtype
from tokamak_amd.engine.scheduler import ScheduledStep, Scheduler
from tokamak_amd.engine.sequence import Sequence
from tokamak_amd.sampling.params import SamplingParams
from tokamak_amd.sampling.sampler import sample_tokens
from tokamak_amd.weights.random_init import expected_tensors_of
from tokamak_amd.weights.sources import RandomSource, SafetensorsSource


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
        prefill_chunk: longest prompt portion in one step (new; default the budget).
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
                 random_weights_on_gpu: bool = False) -> None:
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
        self.runner = ModelRunner(plan, source, dtype=self.dtype,
                                  page_size=block_size, kv_pool_tokens=kv_pool_tokens,
                                  max_requests=max_batch_size, device=device,
                                  min_pool_tokens=self.max_seq_len, tokens_per_request=self.max_seq_len)
        if self.runner.kv_pool_tokens < self.max_seq_len:
            raise RuntimeError(f"the GPU has no room for a cache of max_seq_len ({self.max_seq_len}) tokens")
        self.tokenizer = self._load_tokenizer(folder) if folder is not None else None
        self.num_steps = 0
        self.num_preemptions = 0

    @staticmethod
    def _load_tokenizer(folder: Path):
        path = folder / "tokenizer.json"
        if not path.is_file():
            return None
        try:
            from tokenizers import Tokenizer
        except ImportError:
            return None
        return Tokenizer.from_file(str(path))

    # ------------------------------------------------------------------
    def generate(self, prompts: str | AbcSequence[str] | None = None,
                 sampling_params: SamplingParams | AbcSequence[SamplingParams] | None = None, *,
                 prompt_token_ids: AbcSequence[AbcSequence[int]] | None = None,
                 use_tqdm: bool = False) -> list[RequestOutput]:
        """One completion per prompt, in input order
        (reference: src/tokamak/engine/llm.py:265-334)."""
        texts, token_lists = self._resolve_prompts(prompts, prompt_token_ids)
        params_list = self._broadcast_params(sampling_params, len(token_lists))
        arrival = time.perf_counter()
        sequences = []
        for i, (ids, params) in enumerate(zip(token_lists, params_list)):
            seq = Sequence(i, list(ids), params)
            seq.arrival_time = arrival
            seq.seed = params.seed if params.seed is not None else random.getrandbits(62)
            self._validate_fits(seq)
            sequences.append(seq)

        manager = self.runner.manager
        scheduler = Scheduler(manager, self.max_batch_size, self.max_num_batched_tokens, self.prefill_chunk)
        for seq in sequences:
            scheduler.add(seq)
        try:
            while scheduler.has_unfinished():
                step = scheduler.schedule()
                if step is None:
                    raise RuntimeError("scheduler returned no work but is unfinished")
                self._run(step)
        finally:
            self.runner.end_all()
        return [self._to_output(seq, texts[seq.seq_id] if texts else None) for seq in sequences]

    def _run(self, step: ScheduledStep) -> None:
        for victim in step.preempted:
            self.runner.forget(victim.seq_id)  # the scheduler has already freed its pages
            self.num_preemptions += 1
        entries = []
        sampling = []
        for span in step.spans:
            seq = span.seq
            if span.start != self.runner.cached_tokens(seq.seq_id):
                raise RuntimeError(f"sequence {seq.seq_id}: span starts at {span.start}, cache holds "
                                   f"{self.runner.cached_tokens(seq.seq_id)}")
            tokens = seq.tokens_between(span.start, span.start + span.length)
            entries.append(StepEntry(seq.seq_id, tokens, [span.length - 1] if span.samples else []))
            if span.samples:
                sampling.append(seq)
        logits = self.runner.step(entries)
        self.num_steps += 1
        for span in step.spans:
            span.seq.num_cached = span.start + span.length
        if not sampling:
            return
        chosen = sample_tokens(logits, [s.sampling_params for s in sampling],
                               [s.seed for s in sampling], [s.num_output_tokens for s in sampling])
        now = None
        for seq, token in zip(sampling, chosen.tolist()):
            finished = seq.append_checked(token, eos_token_ids=self.eos_token_ids,
                                          max_total_tokens=self._max_total_tokens(seq))
            if seq.first_token_time is None:
                now = now or time.perf_counter()
                seq.first_token_time = now
            if finished:
                seq.finish_time = time.perf_counter()
                self.runner.end(seq.seq_id)

    # ------------------------------------------------------------------
    def _max_total_tokens(self, seq: Sequence) -> int:
        """reference: src/tokamak/engine/llm.py:483-485"""
        return min(self.max_seq_len, seq.num_prompt_tokens + seq.sampling_params.max_new_tokens)

    def _validate_fits(self, seq: Sequence) -> None:
        """reference: src/tokamak/engine/llm.py:487-499"""
        if seq.num_prompt_tokens >= self.max_seq_len:
            raise ValueError(
                f"Prompt of {seq.num_prompt_tokens} tokens does not fit in "
                f"max_seq_len={self.max_seq_len} (room for generation is required)")
        vocab = self.runner.plan.vocab_size
        if min(seq.prompt_token_ids) < 0 or max(seq.prompt_token_ids) >= vocab:
            raise ValueError(f"prompt {seq.seq_id} has a token id outside [0, {vocab})")
        manager = self.runner.manager
        needed = manager.pages_needed(self._max_total_tokens(seq))
        for g in range(len(manager.groups)):
            if needed > manager.num_pages(g):
                raise ValueError(
                    f"Request needs {needed} cache pages but the pool has {manager.num_pages(g)}; "
                    f"raise kv_pool_tokens")

    def _resolve_prompts(self, prompts, prompt_token_ids):
        if (prompts is None) == (prompt_token_ids is None):
            raise ValueError("provide exactly one of `prompts` or `prompt_token_ids`")
        if prompt_token_ids is not None:
            return None, [list(ids) for ids in prompt_token_ids]
        if isinstance(prompts, str):
            prompts = [prompts]
        texts = list(prompts)
        if self.tokenizer is None:
            raise ValueError("the model folder has no tokenizer.json: pass prompt_token_ids")
        return texts, [self.tokenizer.encode(t).ids for t in texts]

    def _decode(self, ids: list[int]) -> str | None:
        if self.tokenizer is None:
            return None
        return self.tokenizer.decode(ids, skip_special_tokens=True)

    def _to_output(self, seq: Sequence, prompt_text: str | None) -> RequestOutput:
        if seq.finish_reason is None:
            raise RuntimeError(f"Sequence {seq.seq_id} completed without a finish reason")
        ttft = latency = None
        if seq.arrival_time is not None:
            if seq.first_token_time is not None:
                ttft = seq.first_token_time - seq.arrival_time
            if seq.finish_time is not None:
                latency = seq.finish_time - seq.arrival_time
        return RequestOutput(
            request_id=seq.seq_id,
            prompt=prompt_text if prompt_text is not None else self._decode(seq.prompt_token_ids),
            prompt_token_ids=seq.prompt_token_ids,
            output_text=self._decode(seq.output_token_ids),
            output_token_ids=seq.output_token_ids,
            finish_reason=seq.finish_reason,
            ttft_s=ttft,
            latency_s=latency,
        )

    @staticmethod
    def _broadcast_params(sampling_params, num_prompts: int) -> list[SamplingParams]:
        """reference: src/tokamak/engine/llm.py:544-556"""
        if sampling_params is None:
            return [SamplingParams()] * num_prompts
        if isinstance(sampling_params, SamplingParams):
            return [sampling_params] * num_prompts
        params_list = list(sampling_params)
        if len(params_list) != num_prompts:
            raise ValueError(f"Got {len(params_list)} SamplingParams for {num_prompts} prompts")
        return params_list
