"""Iteration-level scheduler: admission, prompt portions under a token budget,
decode, preemption when pages run out.

Policy kept from the reference (src/tokamak/engine/scheduler.py:67-188):
first come first served; no bypass of the head of the waiting queue; when the
pool cannot cover a running sequence's next tokens the newest arrival is
preempted by recomputation (pages freed, generated tokens kept, back to the
*front* of the waiting queue); an impossible prompt raises.

Different from the reference, which runs either one whole prompt or one decode
token of every running sequence: every step takes one token of each decoding
sequence first, then fills what is left of ``max_num_batched_tokens`` with
portions (at most ``prefill_chunk`` tokens) of sequences whose prompt is not
yet cached, then admits from the waiting queue while slots, budget and pages
allow.  Pages are reserved per portion.
"""

from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field

from tokamak_amd.cache.manager import CacheManager
from tokamak_amd.cache.pages import OutOfPagesError
from tokamak_amd.engine.sequence import Sequence, SequenceStatus


@dataclass
class ScheduledSpan:
    """Run ``seq``'s tokens [start, start + length); ``samples`` when the span
    reaches the sequence's last token, so a next token is drawn from it."""

    seq: Sequence
    start: int
    length: int
    samples: bool


@dataclass
class ScheduledStep:
    spans: list[ScheduledSpan]
    preempted: list[Sequence] = field(default_factory=list)

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
                f"({max_batch_size}) so every running sequence can decode in one step")
        if prefill_chunk is not None and prefill_chunk < 1:
            raise ValueError(f"prefill_chunk must be >= 1, got {prefill_chunk}")
        self._manager = manager
        self._max_batch_size = max_batch_size
        self._budget = max_num_batched_tokens
        self._chunk = prefill_chunk or max_num_batched_tokens
        self.waiting: deque[Sequence] = deque()
        self.running: list[Sequence] = []

    def add(self, seq: Sequence) -> None:
        seq.status = SequenceStatus.WAITING
        self.waiting.append(seq)

    def has_unfinished(self) -> bool:
        return bool(self.waiting) or any(not s.is_finished for s in self.running)

    # ------------------------------------------------------------------
    def schedule(self) -> ScheduledStep | None:
        """Plan the next step; None when everything is finished."""
        self.running = [s for s in self.running if not s.is_finished]
        preempted: list[Sequence] = []
        while True:
            spans: list[ScheduledSpan] = []
            budget = self._budget
            budget = self._schedule_decodes(spans, budget, preempted)
            budget = self._schedule_portions(spans, budget)
            self._admit(spans, budget)
            if spans:
                return ScheduledStep(spans, preempted)
            if self.running:
                # every running sequence waits for pages: make room
                victim = self.running[-1]
                self._preempt(victim)
                preempted.append(victim)
                continue
            if self.waiting:
                head = self.waiting[0]
                raise OutOfPagesError(
                    f"sequence {head.seq_id} needs more pages than the pool can ever provide")
            return None

    # ------------------------------------------------------------------
    def _schedule_decodes(self, spans, budget, preempted) -> int:
        for seq in list(self.running):
            if seq not in self.running or seq.num_uncached != 1 or seq.num_cached == 0:
                continue
            while True:
                try:
                    self._manager.ensure_capacity(seq.seq_id, seq.num_tokens)
                    spans.append(ScheduledSpan(seq, seq.num_cached, 1, True))
                    budget -= 1
                    break
                except OutOfPagesError:
                    victim = self.running[-1]  # newest arrival = lowest priority
                    self._preempt(victim)
                    preempted.append(victim)
                    spans[:] = [s for s in spans if s.seq is not victim]
                    if victim is seq:
                        break
        return budget

    def _portion(self, seq: Sequence, budget: int) -> int:
        """Largest portion of ``seq`` that budget, chunk size and free pages allow."""
        want = min(seq.num_uncached, self._chunk, budget)
        if want <= 0:
            return 0
        ps = self._manager.page_size
        have = len(self._manager.block_table(seq.seq_id)) * ps
        room = have + min(self._manager.num_free_pages(g) for g in range(len(self._manager.groups))) * ps
        return max(0, min(want, room - seq.num_cached))

    def _schedule_portions(self, spans, budget) -> int:
        for seq in self.running:
            if budget <= 0:
                break
            if seq.num_uncached <= 1 and seq.num_cached > 0:
                continue  # decoding; handled above
            if any(s.seq is seq for s in spans):
                continue
            length = self._portion(seq, budget)
            if length <= 0:
                continue
            self._manager.ensure_capacity(seq.seq_id, seq.num_cached + length)
            spans.append(ScheduledSpan(seq, seq.num_cached, length,
                                       seq.num_cached + length == seq.num_tokens))
            budget -= length
        return budget

    def _admit(self, spans, budget) -> int:
        while self.waiting and len(self.running) < self._max_batch_size and budget > 0:
            head = self.waiting[0]
            # admit only when the pool could hold everything the sequence has so far
            # (reference: scheduler.py:144-148), but reserve only the first portion
            if not self._manager.can_hold(head.seq_id, head.num_tokens):
                break
            if self._manager.slots.num_free == 0 and self._manager.slots.slot_of(head.seq_id) is None:
                break
            length = self._portion(head, budget)
            if length <= 0:
                break
            self.waiting.popleft()
            self._manager.admit(head.seq_id)
            self._manager.ensure_capacity(head.seq_id, length)
            head.status = SequenceStatus.RUNNING
            head.num_cached = 0
            self.running.append(head)
            spans.append(ScheduledSpan(head, 0, length, length == head.num_tokens))
            budget -= length
        return budget

    def _preempt(self, victim: Sequence) -> None:
        """Evict by recomputation: free pages and slot, requeue at the front."""
        self._manager.free(victim.seq_id)
        self.running.remove(victim)
        victim.status = SequenceStatus.WAITING
        victim.num_cached = 0
        self.waiting.appendleft(victim)
