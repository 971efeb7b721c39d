"""One generation request as the scheduler and the step loop see it.

A request is a single growing token list (the prompt, then what was sampled)
and a mark ``cached``: how many of those tokens the cache holds.  Everything the
scheduler decides is a span ``[cached, cached + n)`` of that list; a request is
"decoding" exactly when one token is left to run.  Eviction sets the mark back
to zero and keeps the tokens, so resuming recomputes prompt and generated
tokens alike (the reference's policy, src/tokamak/engine/sequence.py:35-36).
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
    def pending(self) -> int:
        """Tokens that must still run before the next one can be sampled."""
        return len(self.tokens) - self.cached

    @property
    def decoding(self) -> bool:
        return self.cached > 0 and self.pending == 1

    def span(self, length: int) -> list[int]:
        """The next ``length`` tokens to run."""
        return self.tokens[self.cached:self.cached + length]

    def advance(self, length: int) -> None:
        if length < 0 or self.cached + length > len(self.tokens):
            raise ValueError(f"request {self.rid}: cannot advance {length} past {len(self.tokens)} tokens")
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

    def accept(self, token: int, *, eos_token_ids: tuple[int, ...], context_limit: int) -> bool:
        """Take a sampled token; True if the request ends with it.  Order of the
        rules as in the reference (src/tokamak/engine/sequence.py:109-127): an EOS
        token (unless ``ignore_eos``) stops, and is kept in the output; otherwise the
        request ends on length when it has ``max_new_tokens`` or fills its context."""
        if self.finished:
            raise RuntimeError(f"request {self.rid} has ended ({self.finish_reason.value}); it takes no more tokens")
        self.tokens.append(int(token))
        if token in eos_token_ids and not self.params.ignore_eos:
            self.finish_reason = FinishReason.STOP
        elif self.num_generated >= self.params.max_new_tokens or len(self.tokens) >= context_limit:
            self.finish_reason = FinishReason.LENGTH
        return self.finished
