"""Dispatch of paged attention to the kernel that fits the shape, and the work lists
those kernels read: how a step's spans are cut into single tokens and tiles."""

from __future__ import annotations

import functools
import math

import torch

from tokamak_amd.kernels import ops
from tokamak_amd.engine.batch import StepPlanner

TILE_TOKENS = 16   # tokens per attention tile of a prompt portion (csrc/attention_generic.hip: kTileTokens)
WIDE_TOKENS = 32   # and per tile of the wide matrix-core kernel

MFMA_HEAD_DIMS = (64, 128)
DECODE_WAVES = 16           # waves of a decode block (csrc/attention_mfma.hip: kDecodeWaves)
TILE_SPLIT_UP_TO_BLOCKS = 640   # a portion with no more blocks of the narrow form than this has its keys split ...
TILE_SPLIT_MIN_KEYS = 512       # ... into pieces no shorter than this (twice this from TILE_SPLIT_FEW_BLOCKS blocks on) ...
TILE_SPLIT_FEW_BLOCKS = 128
TARGET_TILE_BLOCKS = 2048       # ... so that about this many blocks run
GROUP_OVER_SPLIT_FILL = 512     # blocks times shares from which the group form is taken rather than split tiles
DENSE_TILES_FROM = 2048         # every tiled span starts at least this deep: the four-wave kernel
WIDE_FROM_KEYS = 4096           # longest context from which the 32-token tiles of the wide kernel pay (+15-20 %;
                                # for shorter walks the narrow one's smaller tiles balance better)
WIDE_FROM_TOKENS = 20           # ... if a 32-token tile holds at least this many tokens on average
GROUP_FROM_KEYS = 1024          # longest context from which the group form (a block a CU, all heads of a kv head) pays
GROUP_FILL = 128                # ... if its blocks times their shares of the keys are at least this many (half the CUs)


def quarter_octave_at_least(n: int, floor: int) -> int:
    """The smallest of floor, 1.25 floor, 1.5 floor, 1.75 floor, 2 floor, 2.5 floor, ...
    that is >= n: four buckets an octave, so a bucket overshoots by a quarter at most."""
    v = floor
    while 2 * v < n:
        v *= 2
    if n <= v:
        return v
    step = v // 4
    return v + -(-(n - v) // step) * step


class AttentionWork(StepPlanner):
    """The attention kernels' cut of a step: spans of one token run alone (``single``: their
    token rows, the one with the longest context first), longer spans are cut into tiles of up to 16 consecutive tokens
    (``tile_first``, ``tile_count``) and, for the wide kernel, of up to 32 (``wide_first``,
    ``wide_count``).  Facts: how many of each, the tokens in tiled spans, the longest
    context among the single tokens (it fixes how their keys are split), the longest
    among the tiled spans, and the shortest cached length among them."""

    name = "attention"

    def lists(self, q_lens, ctx_lens):
        single, tiles, wide = [], [], []
        at = 0
        for q, ctx in zip(q_lens, ctx_lens):
            if q == 1:
                single.append((-ctx, at))
            else:
                tiles.extend((ctx + t, at + t, min(TILE_TOKENS, q - t)) for t in range(0, q, TILE_TOKENS))
                wide.extend((ctx + t, at + t, min(WIDE_TOKENS, q - t)) for t in range(0, q, WIDE_TOKENS))
            at += q
        # Longest context first: blocks start in the list's order, and a long walk that starts
        # last is what the whole kernel waits for (50 requests of 48 to 1,280 keys, 16 query heads
        # over 8 kv heads: 33 us in the order of the requests, 25 longest first).
        single = [row for _, row in sorted(single)]
        # Tiles by the keys they walk, shortest first: the kernels take the list from its end (as
        # they do for one prompt from position zero, whose later tiles walk further), so that the
        # tiles of several requests' portions start longest first too.
        tiles = [t[1:] for t in sorted(tiles)]
        wide = [t[1:] for t in sorted(wide)]
        arrays = {"single": single, "tile_first": [t[0] for t in tiles], "tile_count": [t[1] for t in tiles],
                  "wide_first": [t[0] for t in wide], "wide_count": [t[1] for t in wide]}
        tiled = [(q, c) for q, c in zip(q_lens, ctx_lens) if q > 1]
        facts = {
            "num_single": len(single), "num_tiles": len(tiles), "num_wide": len(wide),
            "num_tile_tokens": sum(q for q, _ in tiled),
            "max_single_len": max((c + 1 for q, c in zip(q_lens, ctx_lens) if q == 1), default=0),
            "max_tile_len": max((c + q for q, c in tiled), default=0),
            "min_tile_ctx": min((c for _, c in tiled), default=0),
        }
        return arrays, facts

    def bucket(self, facts):
        # the longest context fixes how the decode kernel splits the keys: four buckets an octave
        facts["max_single_len"] = quarter_octave_at_least(facts["max_single_len"], 256)
        return facts


ATTENTION_WORK = AttentionWork()


class _Work:
    """The attention planner's lists and facts of a step, by attribute."""

    def __init__(self, batch) -> None:
        lists, facts = batch.lists, batch.facts
        try:
            self.single = lists["attention.single"]
            self.tile_first, self.tile_count = lists["attention.tile_first"], lists["attention.tile_count"]
            self.wide_first, self.wide_count = lists["attention.wide_first"], lists["attention.wide_count"]
            self.num_single, self.num_tiles = facts["attention.num_single"], facts["attention.num_tiles"]
            self.num_wide, self.num_tile_tokens = facts["attention.num_wide"], facts["attention.num_tile_tokens"]
            self.max_single_len, self.max_tile_len = facts["attention.max_single_len"], facts["attention.max_tile_len"]
            self.min_tile_ctx = facts["attention.min_tile_ctx"]
        except KeyError as missing:
            raise ops.KernelError(f"the step's descriptor lacks {missing}: it was packed without the attention "
                                  f"part's planner (kernels.attention.ATTENTION_WORK)") from None


def work_of(batch) -> _Work:
    work = batch.memo.get("attention.work")
    if work is None:
        work = batch.memo["attention.work"] = _Work(batch)
    return work


def check_page_size(page_size: int) -> None:
    """Pages hold a multiple of 8 tokens: the value layout groups tokens in quads of four,
    the key layout in pieces of 8 numbers, and the generic kernel walks pages 8 keys at a time."""
    if page_size < 8 or page_size % 8:
        raise ValueError(f"page_size must be a multiple of 8 for the attention kernels, got {page_size}")


def mfma_fits(dtype, head_dim, page_size, group, window) -> bool:
    return (dtype == torch.bfloat16 and head_dim in MFMA_HEAD_DIMS and page_size >= 16
            and page_size & (page_size - 1) == 0 and group <= 16 and window is None)


# What the choice of the decode splits is priced with (seconds, bytes a second; fitted to 154
# measured cases of 9 to 64 requests over 300 to 16,384 keys in 1 to 8 splits and checked on
# 1 to 8 requests up to 32,768 keys: the cheapest split by this price is on average 1 % and at
# worst 18 % slower than the best measured one; the rule it replaced, "as few splits as put
# 4,096 waves on the GPU", 5 % and 49 % on such cases).
DECODE_CUS = 256                 # blocks that run at once: a block of sixteen waves has a CU to itself
DECODE_RATE = 5.8e12             # bytes a second of a round of DECODE_CUS blocks
DECODE_BLOCK_RATE = 60e9         # ... and of one block with the GPU to itself
DECODE_START = 3e-6              # a launch
DECODE_ROUND = 3e-6              # a further round of blocks
DECODE_MERGE = (2e-6, 0.1e-6)    # the merge kernel, and each split it reads
DECODE_MOST_SPLITS = 64          # candidates looked at (beside the finest split)


@functools.lru_cache(maxsize=4096)
def decode_split(num_decode: int, num_kv_heads: int, max_len: int, head_dim: int = 128) -> tuple[int, int]:
    """(keys per split, number of splits) for the decode tokens of a step.  A block of
    DECODE_WAVES waves walks one split of one request and kv head, every wave a share of
    it (a split is a whole number of 16 keys for every wave); the splits of a token are
    merged by a second kernel.

    The blocks run in rounds of one a CU, so what a split costs follows from how its blocks
    fill the rounds: full rounds stream at the GPU's rate; the last, partial round at that
    rate or, if its blocks are few, at the rate of a block alone (17 requests of 2,048 keys in
    two splits are 272 blocks, 256 and then 16 that take as long again: 45 us against 34 in
    three splits; 33 requests unsplit are 264 blocks: 71 us against 60 in three splits).  The
    cheapest of the candidates by that price is taken; equal prices go to fewer splits.  The
    kernel cuts every token's own keys evenly in that many splits (csrc/attention_mfma.hip:
    decode_share), so a step's shorter requests, and lengths below the step's rounded longest
    one, still give every block of a token the same share."""
    pairs = max(1, num_decode * num_kv_heads)
    least = 16 * DECODE_WAVES
    most = max(1, -(-max_len // least))
    key_bytes = 4 * head_dim          # a key and a value of one kv head, bfloat16
    best = None
    for want in list(range(1, min(most, DECODE_MOST_SPLITS) + 1)) + [most]:
        split = -(-(-(-max_len // want)) // least) * least
        nsplit = max(1, -(-max_len // split))
        share = max_len / nsplit * key_bytes                       # bytes a block walks, on average
        full, rest = divmod(pairs * nsplit, DECODE_CUS)
        price = full * DECODE_CUS * share / DECODE_RATE
        if rest:
            price += math.hypot(rest * share / DECODE_RATE, share / DECODE_BLOCK_RATE)
        price += DECODE_START + DECODE_ROUND * max(0, full + (rest > 0) - 1)
        if nsplit > 1:
            price += DECODE_MERGE[0] + DECODE_MERGE[1] * nsplit
        if best is None or price < best[0] * (1 - 1e-9):
            best = (price, split, nsplit)
    return best[1], best[2]


def tile_split(num_tiles: int, blocks_per_tile: int, max_len: int) -> tuple[int, int]:
    """(keys per split, number of splits) for the 16-token tiles of prompt portions.
    A block walks its tile's keys 64 at a time, one after the other; a portion of a few
    hundred tokens over a long context (the last piece of a long prompt, a small token
    budget) has few tiles, and a CU holds three such blocks, so up to some hundreds of
    blocks the GPU is mostly idle for a long walk: the keys are cut into pieces that run
    side by side, about TARGET_TILE_BLOCKS blocks in all, and merged afterwards (256 tokens
    of a layer with 64 query heads over 16,384 keys: 447 us unsplit, 228 in eight pieces;
    128 tokens with five heads a kv head over 16,384: 432 -> 220)."""
    blocks = num_tiles * blocks_per_tile
    least = TILE_SPLIT_MIN_KEYS if blocks <= TILE_SPLIT_FEW_BLOCKS else 2 * TILE_SPLIT_MIN_KEYS
    if blocks > TILE_SPLIT_UP_TO_BLOCKS or max_len < 2 * least or num_tiles * 16 > 65535:
        return 1 << 30, 1
    nsplit = min(max_len // least, -(-TARGET_TILE_BLOCKS // blocks))
    if nsplit < 2:
        return 1 << 30, 1
    split = -(-(-(-max_len // nsplit)) // 64) * 64
    return split, -(-max_len // split)


def group_fill(group: int, num_kv_heads: int, num_wide: int) -> int:
    """Blocks of the group form times the shares of the keys a block holds."""
    nblk = -(-group // 8)
    heads = -(-group // nblk)                   # heads a block
    shares = 4 if heads <= 2 else 2 if heads <= 4 else 1
    return num_wide * num_kv_heads * nblk * shares


def group_form_pays(group: int, num_kv_heads: int, num_wide: int, max_len: int) -> bool:
    """Whether the tiles of a step's portions take the group form (csrc/attention_mfma.hip: a block
    holds a CU, the query heads of a kv head times 4, 2 or 1 shares of each stage of keys).  Measured
    against the other forms for 2, 4, 5 and 8 heads a kv head, 64 to 2,048 tokens over 0 to 16,384
    cached ones: it needs enough blocks to fill the GPU (with few tiles the narrow form, whose
    tiles are half as long and whose keys can be split over blocks, is up to 40 % ahead); with an
    odd group it wins from there on (the narrow form computes on one wave of four then); with one
    share a block it needs the longer walks the fewer its blocks; with two heads a kv head it wins
    (by 27-35 %) while its blocks are no more than the CUs, beyond that the wide form does."""
    nblk = -(-group // 8)
    heads = -(-group // nblk)                   # heads a block
    shares = 4 if heads <= 2 else 2 if heads <= 4 else 1
    blocks = num_wide * num_kv_heads * nblk
    if group_fill(group, num_kv_heads, num_wide) < GROUP_FILL:
        return False
    if group <= 2:
        return blocks <= 256 and max_len >= 2 * GROUP_FROM_KEYS
    if group % 2 == 1 or shares >= 2:
        return max_len >= GROUP_FROM_KEYS
    return max_len >= 2 * GROUP_FROM_KEYS * max(1, 256 // blocks)


def fused_decode_fits(dtype, head_dim, page_size, group, window, rotary_dim, batch) -> bool:
    """A step of decode tokens only, at shapes the one-kernel form takes."""
    work = work_of(batch)
    return (work.num_tiles == 0 and work.num_single == batch.num_tokens and work.num_single > 0
            and mfma_fits(dtype, head_dim, page_size, group, window) and group <= ops.FUSED_DECODE_MAX_GROUP
            and rotary_dim in (0, head_dim))


def decode_attention_fused(qkv, q_weight, k_weight, cos, sin, k_cache, v_cache, block_tables, batch, out, *,
                           num_heads, num_kv_heads, head_dim, rotary_dim, page_size, eps, scale, store) -> bool:
    """q/k norm, rotation, cache write and attention of a decode-only step in one kernel
    (plus the merge of the splits, if a token's keys are split)."""
    work = work_of(batch)
    split, nsplit = decode_split(work.num_single, num_kv_heads, work.max_single_len, head_dim)
    if ops._profile is not None:
        keys = sum(c + 1 for c in batch.ctx_lens)
        ops._note(f"decode {work.num_single} tokens, fused", keys * 2 * num_kv_heads * head_dim * 2,
                  keys * 4.0 * num_heads * head_dim)
    return ops.attention_decode_fused(
        qkv, q_weight, k_weight, cos, sin, k_cache, v_cache, block_tables, batch.positions, batch.req_of_token,
        work.single, work.num_single, out, num_heads=num_heads, num_kv_heads=num_kv_heads,
        head_dim=head_dim, rotary_dim=rotary_dim, page_size=page_size, eps=eps, scale=scale, store=store,
        split_keys=split, num_splits=nsplit)


def paged_attention(q, k_cache, v_cache, block_tables, batch, out, *, num_heads, num_kv_heads,
                    head_dim, page_size, scale, window=None) -> None:
    """out[n] = softmax(q[n] . K[0..pos_n] * scale) V, per head, over the pages
    of each token's request.

    bfloat16 with head size 64 or 128: the MFMA kernels, once over the single
    (decode) tokens with their context split, once over the tiles of the prompt
    portions: tiles of 32 tokens in the group form (a block a CU: all query heads
    of a kv head and shares of the keys) when the tiles are mostly full and walk
    a thousand keys or more; tiles of 16 otherwise, their keys split over blocks
    when the tiles are few and the context long.  Everything else, and whatever
    the MFMA library does not instantiate: the generic float32-arithmetic kernel.
    """
    work = work_of(batch)
    profiling = ops._profile is not None
    if profiling:
        # keys each query sees; the cache bytes of a request are read once per kv head
        decode_keys = sum(c + 1 for c, n in zip(batch.ctx_lens, batch.q_lens) if n == 1)
        tile_pairs = sum(n * c + n * (n + 1) // 2 for c, n in zip(batch.ctx_lens, batch.q_lens) if n > 1)
        tile_keys = sum(c + n for c, n in zip(batch.ctx_lens, batch.q_lens) if n > 1)
        kv_token_bytes = 2 * num_kv_heads * head_dim * q.element_size()
        flops_per_pair = 4.0 * num_heads * head_dim
    if mfma_fits(q.dtype, head_dim, page_size, num_heads // num_kv_heads, window):
        if _paged_attention_mfma(q, k_cache, v_cache, block_tables, batch, work, out, num_heads=num_heads,
                                 num_kv_heads=num_kv_heads, head_dim=head_dim, page_size=page_size, scale=scale,
                                 note=(decode_keys, tile_keys, tile_pairs, kv_token_bytes, flops_per_pair) if profiling else None):
            return
    if profiling:
        ops._note(f"{batch.num_tokens} tokens", (decode_keys + tile_keys) * kv_token_bytes,
                  (decode_keys + tile_pairs) * flops_per_pair)
    ops.paged_attention_generic(
        q, k_cache, v_cache, block_tables, batch.positions, batch.req_of_token, out,
        num_heads=num_heads, num_kv_heads=num_kv_heads, head_dim=head_dim, page_size=page_size,
        scale=scale, window=window,
        tiles=(work.tile_first, work.tile_count, work.num_tiles, work.single, work.num_single))


def _paged_attention_mfma(q, k_cache, v_cache, block_tables, batch, work, out, *, num_heads, num_kv_heads,
                          head_dim, page_size, scale, note) -> bool:
    """The matrix-core kernels over the step's single tokens and tiles.  False if the
    library has no instance for the shape: nothing of ``out`` counts then, and the caller
    runs the generic kernel over the whole step."""
    common = dict(num_heads=num_heads, num_kv_heads=num_kv_heads, head_dim=head_dim,
                  page_size=page_size, scale=scale)
    if note is not None:
        decode_keys, tile_keys, tile_pairs, kv_token_bytes, flops_per_pair = note
    if work.num_single:
        split, nsplit = decode_split(work.num_single, num_kv_heads, work.max_single_len, head_dim)
        if note is not None:
            ops._note(f"decode {work.num_single} tokens", decode_keys * kv_token_bytes, decode_keys * flops_per_pair)
        if not ops.attention_mfma("heads", q, k_cache, v_cache, block_tables, batch.positions,
                                  batch.req_of_token, work.single, None, work.num_single, out,
                                  split_keys=split, num_splits=nsplit, **common):
            return False
    if work.num_tiles:
        group = num_heads // num_kv_heads
        per_tile = num_kv_heads * (group // (4 if group % 4 == 0 else 2 if group % 2 == 0 else 1))
        split, nsplit = tile_split(work.num_tiles, per_tile, work.max_tile_len)
        full = work.num_tile_tokens >= WIDE_FROM_TOKENS * work.num_wide
        grouped = full and group_form_pays(group, num_kv_heads, work.num_wide, work.max_tile_len)
        if (nsplit > 1 and grouped and work.num_tiles * per_tile > 2 * TILE_SPLIT_FEW_BLOCKS
                and group_fill(group, num_kv_heads, work.num_wide) >= GROUP_OVER_SPLIT_FILL):
            split, nsplit = 1 << 30, 1      # enough blocks for the group form: ahead of split tiles there
        if nsplit == 1 and grouped:
            # tiles of 32 tokens mostly full: the group form, whose blocks hold a CU each
            if note is not None:
                ops._note(f"portions {work.num_wide} wide tiles", tile_keys * kv_token_bytes, tile_pairs * flops_per_pair)
            return ops.attention_mfma("tokens_group", q, k_cache, v_cache, block_tables, batch.positions,
                                      batch.req_of_token, work.wide_first, work.wide_count, work.num_wide,
                                      out, **common)
        if nsplit == 1 and work.max_tile_len >= WIDE_FROM_KEYS and full:
            # long walks over the keys, tiles of 32 tokens mostly full: the wide kernel
            if note is not None:
                ops._note(f"portions {work.num_wide} wide tiles", tile_keys * kv_token_bytes, tile_pairs * flops_per_pair)
            return ops.attention_mfma("tokens_wide", q, k_cache, v_cache, block_tables, batch.positions,
                                      batch.req_of_token, work.wide_first, work.wide_count, work.num_wide,
                                      out, **common)
        dense = nsplit == 1 and work.min_tile_ctx >= DENSE_TILES_FROM
        if note is not None:
            ops._note(f"portions {work.num_tiles} tiles", tile_keys * kv_token_bytes, tile_pairs * flops_per_pair)
        return ops.attention_mfma("tokens_dense" if dense else "tokens", q, k_cache, v_cache, block_tables, batch.positions,
                                  batch.req_of_token, work.tile_first, work.tile_count, work.num_tiles,
                                  out, split_keys=split, num_splits=nsplit, **common)
    return True
