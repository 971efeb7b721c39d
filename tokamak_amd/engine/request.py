"""One generation request as the scheduler and the step loop see it.

A request is a single growing token list (the prompt, then what was sampled)
and a mark ``cached``: how many of those tokens the cache holds.  Everything the
scheduler decides is a span ``[cached, cached + n)`` of that list; a request is
"decoding" exactly when one token is left to run.  Eviction sets the mark back
to zero and keeps the tokens, so resuming recomputes prompt and generated
tokens alike (the reference's policy, src/tokamak/engine/sequence.py:35-36).

The step loop runs one step ahead of what it has read back: ``unknown`` counts the tokens
that have been sampled for the request but are still on the GPU.  They belong to the
request's length (a span may end with one; the step then takes it from the sampler's
output), and when the request is certain to end with them by its length (``closing``) it is
planned no further.
"""

from __future__ import annotations

import enum
from dataclasses import dataclass, field

from tokamak_amd.sampling.params import SamplingParams


class FinishReason(enum.Enum):
    """Why generation ended; the values are what users see
    (reference: src/tokamak/engine/sequence.py:25-29)."""

    STOP = "stop"
    LENGTH = "length"


@dataclass
class Request:
    rid: int
    prompt_len: int
    tokens: list[int]
    params: SamplingParams
    seed: int = 0
    cached: int = 0
    finish_reason: FinishReason | None = None
    arrived_at: float | None = None
    first_token_at: float | None = None
    finished_at: float | None = None
    evictions: int = field(default=0, repr=False)
    context_limit: int | None = None    # most tokens the request may ever hold (set by the step loop)
    unknown: int = 0                    # tokens sampled for it that the host has not read yet
    feed_row: int = -1                  # row of the sampler's last output that holds its newest token

    @classmethod
    def from_prompt(cls, rid: int, prompt: list[int], params: SamplingParams, seed: int = 0) -> Request:
        if len(prompt) == 0:
            raise ValueError(f"request {rid}: the prompt has no tokens")
        return cls(rid=rid, prompt_len=len(prompt), tokens=[int(t) for t in prompt], params=params, seed=seed)

    # -- what the scheduler asks ---------------------------------------------
    @property
    def finished(self) -> bool:
        return self.finish_reason is not None

    @property
    def length(self) -> int:
        """Tokens of the request, those still on the GPU included."""
        return len(self.tokens) + self.unknown

    @property
    def pending(self) -> int:
        """Tokens that must still run before the next one can be sampled."""
        return self.length - self.cached

    @property
    def closing(self) -> bool:
        """Tokens are on their way with which the request ends by its length, whatever they are."""
        if self.unknown == 0 or self.finished:
            return False
        return (self.num_generated + self.unknown >= self.params.max_new_tokens
                or (self.context_limit is not None and self.length >= self.context_limit))

    @property
    def decoding(self) -> bool:
        return self.cached > 0 and self.pending == 1 and not self.closing

    def span(self, length: int) -> list[int]:
        """The next ``length`` tokens to run (0 in place of one that is still on the GPU)."""
        known = self.tokens[self.cached:self.cached + length]
        return known + [0] * (length - len(known))

    def advance(self, length: int) -> None:
        if length < 0 or self.cached + length > self.length:
            raise ValueError(f"request {self.rid}: cannot advance {length} past {self.length} tokens")
        self.cached += length

    def rewind(self) -> None:
        """The cache no longer holds anything of this request."""
        self.cached = 0
        self.evictions += 1

    # -- what the step loop tells ---------------------------------------------
    @property
    def prompt(self) -> list[int]:
        return self.tokens[:self.prompt_len]

    @property
    def generated(self) -> list[int]:
        return self.tokens[self.prompt_len:]

    @property
    def num_generated(self) -> int:
        return len(self.tokens) - self.prompt_len

    @property
    def num_drawn(self) -> int:
        """Tokens drawn for the request so far, read back or not: the next draw's counter."""
        return self.num_generated + self.unknown

    def accept(self, token: int, *, eos_token_ids: tuple[int, ...], context_limit: int) -> bool:
        """Take a sampled token; True if the request ends with it.  Order of the
        rules as in the reference (src/tokamak/engine/sequence.py:109-127): an EOS
        token (unless ``ignore_eos``) stops, and is kept in the output; otherwise the
        request ends on length when it has ``max_new_tokens`` or fills its context."""
        if self.finished:
            raise RuntimeError(f"request {self.rid} has ended ({self.finish_reason.value}); it takes no more tokens")
        self.tokens.append(int(token))
        self.unknown = max(0, self.unknown - 1)
        if token in eos_token_ids and not self.params.ignore_eos:
            self.finish_reason = FinishReason.STOP
        elif self.num_generated >= self.params.max_new_tokens or len(self.tokens) >= context_limit:
            self.finish_reason = FinishReason.LENGTH
        return self.finished
