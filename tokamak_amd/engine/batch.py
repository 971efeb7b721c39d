"""The step descriptor: one flat batch of tokens from several requests.

The reference runs either one whole sequence or B single tokens, in a padded
[batch, seq] layout (src/tokamak/engine/llm.py:347-388).  Here a step is N
tokens from R requests; request r contributes ``q_len[r]`` consecutive tokens
that start at absolute position ``ctx_len[r]`` (what its cache already holds).
A decode token is a span of length one, a prompt portion a longer one; any
mixture is one batch.
"""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch


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
    # work lists for the attention kernels: single (decode) tokens, and tiles of up to
    # 16, and of up to 32, consecutive tokens of the longer spans
    decode_tokens: torch.Tensor | None = None   # [num_decode] int32 token rows
    tile_first: torch.Tensor | None = None      # [num_tiles] int32 first token row
    tile_count: torch.Tensor | None = None      # [num_tiles] int32 tokens in the tile
    wide_first: torch.Tensor | None = None      # [num_wide] int32 first token row of a 32-token tile
    wide_count: torch.Tensor | None = None      # [num_wide] int32 tokens in it
    feed_slots: torch.Tensor | None = None      # [N] int32: the first num_feed name token rows whose id ...
    feed_rows: torch.Tensor | None = None       # [N] int32: ... is that row of the sampler's last output
    num_feed: int = 0
    num_decode: int = 0
    num_tiles: int = 0
    num_wide: int = 0
    num_tile_tokens: int = 0                    # tokens of the spans that are cut into tiles
    max_decode_len: int = 0                     # longest context among the decode tokens
    max_tile_len: int = 0                       # longest context (with the portion) among the tiled spans
    min_tile_ctx: int = 0                       # shortest cached context among the tiled spans
    # host copies, for choosing kernels and grids
    q_lens: list[int] = field(default_factory=list)
    ctx_lens: list[int] = field(default_factory=list)
    max_q_len: int = 0
    max_seq_len: int = 0
    memo: dict = field(default_factory=dict)  # per-step data shared between layers


TILE_TOKENS = 16   # tokens per attention tile of a prompt portion
WIDE_TOKENS = 32   # and per tile of the wide attention kernel
NUM_FIXED = 14     # arrays in the packed buffer before the block tables


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
    num_decode: int
    num_tiles: int
    num_wide: int
    q_lens: list[int]
    ctx_lens: list[int]
    max_decode_len: int
    max_tile_len: int = 0
    min_tile_ctx: int = 0
    num_feed: int = 0
    max_feed_row: int = -1


def table_width(longest: int, fixed: int | None = None) -> int:
    if fixed is not None:
        if longest > fixed:
            raise ValueError(f"a block table of {longest} pages does not fit the fixed width {fixed}")
        return fixed
    return max(4, -(-longest // 4) * 4)


def pack_batch(spans: list[StepSpan], num_groups: int, fixed_widths: list[int] | None = None) -> PackedBatch:
    r = len(spans)
    n = sum(len(s.tokens) for s in spans)
    widths = [table_width(max((len(s.tables[g]) for s in spans), default=0),
                          None if fixed_widths is None else fixed_widths[g])
              for g in range(num_groups)]
    m = sum(len(s.want) for s in spans)
    decode_rows, tiles, wide = [], [], []
    at = 0
    for s in spans:
        q = len(s.tokens)
        if q == 1:
            decode_rows.append(at)
        else:
            tiles.extend((at + t, min(TILE_TOKENS, q - t)) for t in range(0, q, TILE_TOKENS))
            wide.extend((at + t, min(WIDE_TOKENS, q - t)) for t in range(0, q, WIDE_TOKENS))
        at += q
    nd, nt, nw = len(decode_rows), len(tiles), len(wide)
    sizes = [n, n, n, r + 1, r, r, m, nd, nt, nt, nw, nw, n, n] + [r * w for w in widths]
    offsets = [0]
    for size in sizes:
        offsets.append(offsets[-1] + size)
    buf = np.zeros(offsets[-1], dtype=np.int32)
    tok, pos, req, qs, ctx, slots, rows, dec, tfirst, tcount, wfirst, wcount, fslots, frows = (
        buf[offsets[i]:offsets[i + 1]] for i in range(NUM_FIXED))
    tabs = [buf[offsets[NUM_FIXED + g]:offsets[NUM_FIXED + 1 + g]].reshape(r, widths[g])
            for g in range(num_groups)]
    dec[:] = decode_rows
    tfirst[:] = [t[0] for t in tiles]
    tcount[:] = [t[1] for t in tiles]
    wfirst[:] = [t[0] for t in wide]
    wcount[:] = [t[1] for t in wide]
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
        num_decode=nd, num_tiles=nt, num_wide=nw, q_lens=[len(s.tokens) for s in spans],
        ctx_lens=[s.ctx_len for s in spans],
        max_decode_len=max((s.ctx_len + 1 for s in spans if len(s.tokens) == 1), default=0),
        max_tile_len=max((s.ctx_len + len(s.tokens) for s in spans if len(s.tokens) > 1), default=0),
        min_tile_ctx=min((s.ctx_len for s in spans if len(s.tokens) > 1), default=0),
        num_feed=fed, max_feed_row=max((s.feed for s in spans if s.feed is not None), default=-1))


def batch_from_device(packed: PackedBatch, dev: torch.Tensor) -> StepBatch:
    """Cut the device copy ``dev`` of ``packed.buf`` into the descriptor's arrays."""
    o, r, widths = packed.offsets, packed.num_requests, packed.widths
    parts = [dev[o[i]:o[i + 1]] for i in range(len(o) - 1)]
    return StepBatch(
        num_tokens=packed.num_tokens, num_requests=r, num_logit_rows=packed.num_logit_rows,
        token_ids=parts[0], positions=parts[1], req_of_token=parts[2], q_start=parts[3],
        ctx_len=parts[4], state_slots=parts[5], logit_rows=parts[6],
        block_tables=[parts[NUM_FIXED + g].view(r, widths[g]) for g in range(len(widths))],
        decode_tokens=parts[7], tile_first=parts[8], tile_count=parts[9],
        wide_first=parts[10], wide_count=parts[11], feed_slots=parts[12], feed_rows=parts[13],
        num_feed=packed.num_feed, num_decode=packed.num_decode, num_tiles=packed.num_tiles, num_wide=packed.num_wide,
        num_tile_tokens=sum(q for q in packed.q_lens if q > 1),
        max_decode_len=packed.max_decode_len, max_tile_len=packed.max_tile_len,
        min_tile_ctx=packed.min_tile_ctx,
        q_lens=packed.q_lens, ctx_lens=packed.ctx_lens,
        max_q_len=max(packed.q_lens, default=0),
        max_seq_len=max((c + q for c, q in zip(packed.ctx_lens, packed.q_lens)), default=0),
    )


def build_batch(spans: list[StepSpan], num_groups: int, device) -> StepBatch:
    """Pack the descriptor into one host buffer and copy it to the device once."""
    packed = pack_batch(spans, num_groups)
    host = torch.from_numpy(packed.buf)
    if torch.device(device).type == "cuda":
        dev = host.pin_memory().to(device, non_blocking=True)
    else:
        dev = host.to(device)
    return batch_from_device(packed, dev)
