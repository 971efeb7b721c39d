"""The step descriptor: one flat batch of tokens from several requests.

The reference runs either one whole sequence or B single tokens, in a padded
[batch, seq] layout (src/tokamak/engine/llm.py:347-388).  Here a step is N
tokens from R requests; request r contributes ``q_len[r]`` consecutive tokens
that start at absolute position ``ctx_len[r]`` (what its cache already holds).
A decode token is a span of length one, a prompt portion a longer one; any
mixture is one batch.

The descriptor itself knows nothing of how a part cuts a step into work for its
kernels.  A part that wants lists of its own (tiles of a portion's tokens, chunks
of a scan, rows that run alone) declares a ``StepPlanner``: it is
asked once a step, with the step's span lengths and cached lengths, and what it
returns travels to the device in the same buffer as the descriptor and is found
under the planner's name (``batch.lists["<planner>.<list>"]``,
``batch.facts["<planner>.<fact>"]``).
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Sequence

import numpy as np
import torch


class StepPlanner:
    """How a part's kernels want a step cut into work.

    ``lists(q_lens, ctx_lens)`` is called once a step with, per request of the step, the
    number of tokens it brings and the number its cache already holds.  It returns
    (arrays, facts): ``arrays`` maps a key to a list of integers, which reaches the device
    as int32 in the same copy as the step's descriptor and is found as
    ``batch.lists["<name>.<key>"]``; ``facts`` maps a key to a host integer (a count, a
    longest context) from which the part picks kernels and grids,
    ``batch.facts["<name>.<key>"]``.  The length of every array must follow from ``q_lens``
    and the facts alone.

    ``bucket(facts)`` is applied before a step of single tokens is recorded for replay:
    a recorded step serves every later step with equal facts, so a fact that moves with
    every token (a longest context) is rounded up here to a few values; the kernels must
    be right for any true value up to the rounded one.

    Parts that return planners of the same ``name`` share one (the lists are made once).
    """

    name = ""

    def lists(self, q_lens: list[int], ctx_lens: list[int]) -> tuple[dict[str, list[int]], dict[str, int]]:
        return {}, {}

    def bucket(self, facts: dict[str, int]) -> dict[str, int]:
        return facts


@dataclass
class StepSpan:
    """One request's share of a step."""

    request: object
    tokens: list[int]
    ctx_len: int                 # tokens of this request already in the cache
    state_slot: int
    tables: list[list[int]]      # block table per cache group
    want: list[int] = field(default_factory=list)  # offsets within ``tokens`` whose logits are wanted
    feed: int | None = None      # the span's one token is row ``feed`` of the sampler's last output, still on the GPU


@dataclass
class StepBatch:
    num_tokens: int
    num_requests: int
    num_logit_rows: int
    token_ids: torch.Tensor      # [N] int32
    positions: torch.Tensor      # [N] int32
    req_of_token: torch.Tensor   # [N] int32, row of the request in this batch
    q_start: torch.Tensor        # [R+1] int32, first token of each request
    ctx_len: torch.Tensor        # [R] int32, cached tokens before this step
    state_slots: torch.Tensor    # [R] int32
    logit_rows: torch.Tensor     # [M] int32, token rows whose logits are wanted
    block_tables: list[torch.Tensor]  # per cache group [R, max_pages] int32
    feed_slots: torch.Tensor | None = None      # [N] int32: the first num_feed name token rows whose id ...
    feed_rows: torch.Tensor | None = None       # [N] int32: ... is that row of the sampler's last output
    num_feed: int = 0
    # what the parts' planners asked for: int32 device arrays, and host integers that
    # choose kernels and grids, both under "<planner name>.<key>"
    lists: dict[str, torch.Tensor] = field(default_factory=dict)
    facts: dict[str, int] = field(default_factory=dict)
    # host copies, for choosing kernels and grids
    q_lens: list[int] = field(default_factory=list)
    ctx_lens: list[int] = field(default_factory=list)
    max_q_len: int = 0
    max_seq_len: int = 0
    memo: dict = field(default_factory=dict)  # per-step data shared between layers


NUM_FIXED = 9      # arrays in the packed buffer before the block tables


@dataclass
class PackedBatch:
    """The descriptor packed into one host int32 buffer, plus what is needed to
    cut the device copy of that buffer back into arrays."""

    buf: np.ndarray
    offsets: list[int]
    widths: list[int]
    num_tokens: int
    num_requests: int
    num_logit_rows: int
    q_lens: list[int]
    ctx_lens: list[int]
    list_names: list[str] = field(default_factory=list)   # planners' lists, in buffer order after the tables
    facts: dict[str, int] = field(default_factory=dict)
    num_feed: int = 0
    max_feed_row: int = -1

    def shape_key(self) -> tuple:
        """What two steps must share to use one recorded step: the buffer's cut and the
        planners' facts (kernels and grids are chosen from them)."""
        return (tuple(self.offsets), tuple(sorted(self.facts.items())))


def table_width(longest: int, fixed: int | None = None) -> int:
    if fixed is not None:
        if longest > fixed:
            raise ValueError(f"a block table of {longest} pages does not fit the fixed width {fixed}")
        return fixed
    return max(4, -(-longest // 4) * 4)


def pack_batch(spans: list[StepSpan], num_groups: int, planners: Sequence = (),
               fixed_widths: list[int] | None = None, bucket: bool = False) -> PackedBatch:
    """``planners``: the ``StepPlanner`` objects of the model's parts (one per name).
    ``bucket``: round the planners' facts as they ask for recorded steps, so that steps of
    nearly the same shape share a recording."""
    r = len(spans)
    n = sum(len(s.tokens) for s in spans)
    widths = [table_width(max((len(s.tables[g]) for s in spans), default=0),
                          None if fixed_widths is None else fixed_widths[g])
              for g in range(num_groups)]
    m = sum(len(s.want) for s in spans)
    q_lens = [len(s.tokens) for s in spans]
    ctx_lens = [s.ctx_len for s in spans]
    extra: list[tuple[str, Sequence[int]]] = []
    facts: dict[str, int] = {}
    for planner in planners:
        arrays, found = planner.lists(q_lens, ctx_lens)
        if bucket:
            found = planner.bucket(dict(found))
        for key, values in arrays.items():
            extra.append((f"{planner.name}.{key}", values))
        for key, value in found.items():
            facts[f"{planner.name}.{key}"] = int(value)
    sizes = [n, n, n, r + 1, r, r, m, n, n] + [r * w for w in widths] + [len(values) for _, values in extra]
    offsets = [0]
    for size in sizes:
        offsets.append(offsets[-1] + size)
    buf = np.zeros(offsets[-1], dtype=np.int32)
    tok, pos, req, qs, ctx, slots, rows, fslots, frows = (
        buf[offsets[i]:offsets[i + 1]] for i in range(NUM_FIXED))
    tabs = [buf[offsets[NUM_FIXED + g]:offsets[NUM_FIXED + 1 + g]].reshape(r, widths[g])
            for g in range(num_groups)]
    for i, (_, values) in enumerate(extra):
        at = NUM_FIXED + num_groups + i
        buf[offsets[at]:offsets[at + 1]] = values
    at = 0
    mi = 0
    fed = 0
    for i, s in enumerate(spans):
        q = len(s.tokens)
        if s.feed is not None:
            if q != 1 or s.feed < 0:
                raise ValueError("only a span of one token can take its token from the sampler's output")
            fslots[fed], frows[fed] = at, s.feed
            fed += 1
        tok[at:at + q] = s.tokens
        pos[at:at + q] = np.arange(s.ctx_len, s.ctx_len + q, dtype=np.int32)
        req[at:at + q] = i
        qs[i] = at
        ctx[i] = s.ctx_len
        slots[i] = s.state_slot
        for w in s.want:
            if not 0 <= w < q:
                raise ValueError(f"wanted offset {w} is outside a span of {q} tokens")
            rows[mi] = at + w
            mi += 1
        for g in range(num_groups):
            t = s.tables[g]
            # entries released behind a window are never read; keep them in range
            tabs[g][i, :len(t)] = [p if p >= 0 else 0 for p in t]
        at += q
    qs[r] = at
    return PackedBatch(
        buf=buf, offsets=offsets, widths=widths, num_tokens=n, num_requests=r, num_logit_rows=m,
        q_lens=q_lens, ctx_lens=ctx_lens, list_names=[name for name, _ in extra], facts=facts,
        num_feed=fed, max_feed_row=max((s.feed for s in spans if s.feed is not None), default=-1))


def batch_from_device(packed: PackedBatch, dev: torch.Tensor) -> StepBatch:
    """Cut the device copy ``dev`` of ``packed.buf`` into the descriptor's arrays."""
    o, r, widths = packed.offsets, packed.num_requests, packed.widths
    parts = [dev[o[i]:o[i + 1]] for i in range(len(o) - 1)]
    first_list = NUM_FIXED + len(widths)
    return StepBatch(
        num_tokens=packed.num_tokens, num_requests=r, num_logit_rows=packed.num_logit_rows,
        token_ids=parts[0], positions=parts[1], req_of_token=parts[2], q_start=parts[3],
        ctx_len=parts[4], state_slots=parts[5], logit_rows=parts[6],
        block_tables=[parts[NUM_FIXED + g].view(r, widths[g]) for g in range(len(widths))],
        feed_slots=parts[7], feed_rows=parts[8], num_feed=packed.num_feed,
        lists={name: parts[first_list + i] for i, name in enumerate(packed.list_names)},
        facts=dict(packed.facts),
        q_lens=packed.q_lens, ctx_lens=packed.ctx_lens,
        max_q_len=max(packed.q_lens, default=0),
        max_seq_len=max((c + q for c, q in zip(packed.ctx_lens, packed.q_lens)), default=0),
    )


def build_batch(spans: list[StepSpan], num_groups: int, device, planners: Sequence = ()) -> StepBatch:
    """Pack the descriptor into one host buffer and copy it to the device once."""
    packed = pack_batch(spans, num_groups, planners)
    host = torch.from_numpy(packed.buf)
    if torch.device(device).type == "cuda":
        dev = host.pin_memory().to(device, non_blocking=True)
    else:
        dev = host.to(device)
    return batch_from_device(packed, dev)
