"""Per-request token state (reference: src/tokamak/engine/sequence.py:32-138)."""

from __future__ import annotations

import enum

from tokamak_amd.sampling.params import SamplingParams


class SequenceStatus(enum.Enum):
    WAITING = enum.auto()
    RUNNING = enum.auto()
    FINISHED = enum.auto()


class FinishReason(enum.Enum):
    STOP = "stop"      # an EOS token was generated
    LENGTH = "length"  # max_new_tokens or the context limit was reached


class Sequence:
    """Tokens, lifecycle and timestamps of one request.

    ``num_cached`` is how many of its tokens the cache holds.  A preempted
    sequence goes back to WAITING with ``num_cached = 0`` and its generated
    tokens intact; resuming recomputes over prompt + generated
    (reference: src/tokamak/engine/sequence.py:35-36,86-89).
    """

    def __init__(self, seq_id: int, prompt_token_ids: list[int], sampling_params: SamplingParams) -> None:
        if not prompt_token_ids:
            raise ValueError("prompt_token_ids must not be empty")
        self.seq_id = seq_id
        self.prompt_token_ids = list(prompt_token_ids)
        self.output_token_ids: list[int] = []
        self.sampling_params = sampling_params
        self.status = SequenceStatus.WAITING
        self.finish_reason: FinishReason | None = None
        self.num_cached = 0
        self.seed: int = 0
        self.arrival_time: float | None = None
        self.first_token_time: float | None = None
        self.finish_time: float | None = None

    @property
    def num_prompt_tokens(self) -> int:
        return len(self.prompt_token_ids)

    @property
    def num_output_tokens(self) -> int:
        return len(self.output_token_ids)

    @property
    def num_tokens(self) -> int:
        return len(self.prompt_token_ids) + len(self.output_token_ids)

    @property
    def num_uncached(self) -> int:
        """Tokens that still have to run before the next one can be sampled."""
        return self.num_tokens - self.num_cached

    @property
    def all_token_ids(self) -> list[int]:
        return self.prompt_token_ids + self.output_token_ids

    def tokens_between(self, start: int, stop: int) -> list[int]:
        p = self.num_prompt_tokens
        if stop <= p:
            return self.prompt_token_ids[start:stop]
        if start >= p:
            return self.output_token_ids[start - p:stop - p]
        return self.prompt_token_ids[start:] + self.output_token_ids[:stop - p]

    @property
    def is_finished(self) -> bool:
        return self.status is SequenceStatus.FINISHED

    def append_output_token(self, token_id: int) -> None:
        if self.is_finished:
            raise RuntimeError(f"Sequence {self.seq_id} is already finished")
        self.output_token_ids.append(token_id)

    def append_checked(self, token_id: int, *, eos_token_ids: tuple[int, ...], max_total_tokens: int) -> bool:
        """Append and apply the stop rules in the reference's order
        (sequence.py:109-127): EOS unless ignore_eos, then max_new_tokens, then
        the context budget.  True when finished."""
        self.append_output_token(token_id)
        params = self.sampling_params
        if not params.ignore_eos and token_id in eos_token_ids:
            self.finish(FinishReason.STOP)
        elif self.num_output_tokens >= params.max_new_tokens or self.num_tokens >= max_total_tokens:
            self.finish(FinishReason.LENGTH)
        return self.is_finished

    def finish(self, reason: FinishReason) -> None:
        self.status = SequenceStatus.FINISHED
        self.finish_reason = reason

    def __repr__(self) -> str:
        return (f"Sequence(id={self.seq_id}, prompt={self.num_prompt_tokens} tok, "
                f"output={self.num_output_tokens} tok, cached={self.num_cached}, status={self.status.name})")
