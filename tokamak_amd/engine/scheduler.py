"""Iteration-level scheduler: admission, prompt portions under a token budget,
decode, eviction when pages run out.

Policy kept from the reference (src/tokamak/engine/scheduler.py:67-188):
first come first served; nothing overtakes the head of the waiting queue; when
the pool cannot cover a running request's next token the newest arrival is
evicted by recomputation (pages freed, generated tokens kept, back to the
*front* of the waiting queue); a prompt the pool can never hold raises.

Different from the reference, which runs either one whole prompt or one decode
token of every running request: every step takes one token of each decoding
request first, then fills what is left of ``max_num_batched_tokens`` with
portions (at most ``prefill_chunk`` tokens) of requests whose tokens are not yet
all cached, then admits from the waiting queue while slots, budget and pages
allow.  Pages are reserved portion by portion.

The step loop plans a step before it has read the tokens of the step before
(``Request.unknown``): a decoding request's span may be that unread token (``Span.feed``);
a request that is certain to end with it is left alone (and when it is the victim of an
eviction its pages go back and it is not queued again: ``StepPlan.released``); one that was
evicted with it waits at the head of the queue until it is read; and a plan may come back
empty because everything left waits for tokens (``StepPlan.spans == []``).  A request may
end while it waits (it was evicted with its EOS token on its way): a finished request is
never planned, wherever it sits.
"""

from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field

from tokamak_amd.cache.manager import CacheManager
from tokamak_amd.cache.pages import OutOfPagesError
from tokamak_amd.engine.request import Request


@dataclass
class Span:
    """Run ``request.tokens[start : start + length]``; ``samples``: the span ends
    at the request's last token, so a next token is drawn from its last row."""

    request: Request
    start: int
    length: int
    samples: bool
    feed: int | None = None     # its one token is still on the GPU: this row of the sampler's last output


@dataclass
class StepPlan:
    spans: list[Span]
    evicted: list[Request] = field(default_factory=list)     # pages freed, queued again at the front
    released: list[Request] = field(default_factory=list)    # pages freed, ending with the token on its way

    @property
    def num_tokens(self) -> int:
        return sum(s.length for s in self.spans)


class Scheduler:
    def __init__(self, manager: CacheManager, max_batch_size: int, max_num_batched_tokens: int,
                 prefill_chunk: int | None = None) -> None:
        if max_batch_size < 1:
            raise ValueError(f"max_batch_size must be >= 1, got {max_batch_size}")
        if max_num_batched_tokens < max_batch_size:
            raise ValueError(
                f"max_num_batched_tokens ({max_num_batched_tokens}) must be >= max_batch_size "
                f"({max_batch_size}) so every running request can decode in one step")
        if prefill_chunk is not None and prefill_chunk < 1:
            raise ValueError(f"prefill_chunk must be >= 1, got {prefill_chunk}")
        self.manager = manager
        self.max_batch_size = max_batch_size
        self.token_budget = max_num_batched_tokens
        self.chunk = prefill_chunk or max_num_batched_tokens
        self.waiting: deque[Request] = deque()
        self.running: list[Request] = []        # oldest first

    def submit(self, request: Request) -> None:
        self.waiting.append(request)

    @property
    def busy(self) -> bool:
        return any(not r.finished for r in self.waiting) or any(not r.finished for r in self.running)

    def live_requests(self) -> list[Request]:
        """Every request that may hold pages or a slot."""
        return [*self.running, *self.waiting]

    # ------------------------------------------------------------------
    def plan(self) -> StepPlan | None:
        """The next step, or None when nothing is left to do."""
        self.running = [r for r in self.running if not r.finished]
        if any(r.finished for r in self.waiting):
            # evicted with its last token on its way, and ended when that was read: whoever read
            # it has given back what it held
            self.waiting = deque(r for r in self.waiting if not r.finished)
        evicted: list[Request] = []
        released: list[Request] = []
        while True:
            spans = self._fill(evicted, released)
            if spans:
                return StepPlan(spans, evicted, released)
            if any(r.unknown for r in self.running) or (self.waiting and self.waiting[0].unknown):
                return StepPlan([], evicted, released)   # what is left waits for tokens that are still on the GPU
            if self.running:
                # nobody could move: every running request waits for pages
                self._evict_newest(evicted, released)
            elif self.waiting:
                raise OutOfPagesError(
                    f"request {self.waiting[0].rid} needs more pages than the pool can ever provide")
            else:
                return None

    def _fill(self, evicted: list[Request], released: list[Request]) -> list[Span]:
        spans: list[Span] = []
        left = self.token_budget
        # 1. a token for every decoding request, oldest first.  When the pool cannot give
        # one its page the newest running request makes room; walking from the old end and
        # evicting from the new end, a victim never has a span in this step yet.
        at = 0
        while at < len(self.running):
            request = self.running[at]
            if not request.decoding:
                at += 1
            elif self._reserve(request, 1):
                spans.append(Span(request, request.cached, 1, True, request.feed_row if request.unknown else None))
                left -= 1
                at += 1
            else:
                self._evict_newest(evicted, released)    # may be ``request`` itself
        # 2. portions of running requests whose tokens are not all cached yet
        for request in self.running:
            if left <= 0:
                break
            if request.decoding or request.closing:
                continue
            length = self._affordable(request, left)
            if length > 0 and self._reserve(request, length):
                spans.append(Span(request, request.cached, length, length == request.pending))
                left -= length
        # 3. newcomers, in arrival order, never past a head that does not fit
        while self.waiting and left > 0 and len(self.running) < self.max_batch_size:
            head = self.waiting[0]
            if head.unknown:
                break       # evicted with a token still on the GPU: its tokens are complete after the next read
            # the pool must be able to hold all the request has so far (reference:
            # scheduler.py:144-148); only its first portion is reserved
            if not self.manager.can_hold(head.rid, len(head.tokens)):
                break
            if self.manager.slots.num_free == 0 and self.manager.slots.slot_of(head.rid) is None:
                break
            length = self._affordable(head, left)
            if length <= 0:
                break
            self.waiting.popleft()
            self.manager.admit(head.rid)
            self.manager.ensure_capacity(head.rid, length)
            self.running.append(head)
            spans.append(Span(head, 0, length, length == head.pending))
            left -= length
        return spans

    def _reserve(self, request: Request, length: int) -> bool:
        try:
            self.manager.ensure_capacity(request.rid, request.cached + length)
        except OutOfPagesError:
            return False
        return True

    def _affordable(self, request: Request, left: int) -> int:
        """Longest next portion of ``request`` within budget, chunk and free pages."""
        manager = self.manager
        page = manager.page_size
        reserved = len(manager.block_table(request.rid)) * page
        free = min(manager.num_free_pages(g) for g in range(len(manager.groups))) * page
        return max(0, min(request.pending, self.chunk, left, reserved + free - request.cached))

    def _evict_newest(self, evicted: list[Request], released: list[Request]) -> None:
        """Free the newest running request's pages and slot; it keeps its tokens and
        goes to the front of the queue (it is older than anything waiting).  A victim that
        is certain to end with the token on its way will never run again: it only gives
        back what it holds, and whoever reads that token finishes it."""
        victim = self.running.pop()
        self.manager.free(victim.rid)
        if victim.closing:
            released.append(victim)
            return
        victim.rewind()
        self.waiting.appendleft(victim)
        evicted.append(victim)
