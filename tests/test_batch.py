"""The step descriptor on the CPU: what is packed, and that the work lists in it are
those the parts' planners asked for, under their names."""

import numpy as np
import pytest
import torch

from tokamak_amd.engine.batch import StepPlanner, StepSpan, batch_from_device, pack_batch
from tokamak_amd.kernels.attention import ATTENTION_WORK, quarter_octave_at_least


def spans_of(*shapes):
    """(tokens, cached) per request."""
    return [StepSpan(request=i, tokens=list(range(10 * i, 10 * i + n)), ctx_len=ctx, state_slot=i + 3,
                     tables=[list(range(4 * i, 4 * i + -(-(ctx + n) // 8)))], want=[n - 1])
            for i, (n, ctx) in enumerate(shapes)]


def unpack(packed):
    return batch_from_device(packed, torch.from_numpy(packed.buf))


def test_the_descriptor_holds_tokens_positions_tables_and_wanted_rows():
    batch = unpack(pack_batch(spans_of((3, 0), (1, 17), (5, 8)), 1))
    assert batch.num_tokens == 9 and batch.num_requests == 3 and batch.num_logit_rows == 3
    assert batch.token_ids.tolist() == [0, 1, 2, 10, 20, 21, 22, 23, 24]
    assert batch.positions.tolist() == [0, 1, 2, 17, 8, 9, 10, 11, 12]
    assert batch.req_of_token.tolist() == [0, 0, 0, 1, 2, 2, 2, 2, 2]
    assert batch.q_start.tolist() == [0, 3, 4, 9] and batch.ctx_len.tolist() == [0, 17, 8]
    assert batch.state_slots.tolist() == [3, 4, 5] and batch.logit_rows.tolist() == [2, 3, 8]
    assert batch.block_tables[0].shape == (3, 4) and batch.block_tables[0][1].tolist() == [4, 5, 6, 0]
    assert batch.q_lens == [3, 1, 5] and batch.max_q_len == 5 and batch.max_seq_len == 18
    assert batch.lists == {} and batch.facts == {}        # no part asked for anything


def test_the_attention_kernels_lists_are_made_by_their_planner():
    packed = pack_batch(spans_of((40, 100), (1, 300), (1, 7), (17, 0)), 1, [ATTENTION_WORK])
    batch = unpack(packed)
    lists = {k: v.tolist() for k, v in batch.lists.items()}
    assert lists["attention.single"] == [40, 41]
    # tiles by the keys they walk, shortest first (the kernels start from the list's end)
    assert lists["attention.tile_first"] == [42, 58, 0, 16, 32] and lists["attention.tile_count"] == [16, 1, 16, 16, 8]
    assert lists["attention.wide_first"] == [42, 0, 32] and lists["attention.wide_count"] == [17, 32, 8]
    assert batch.facts == {"attention.num_single": 2, "attention.num_tiles": 5, "attention.num_wide": 3,
                           "attention.num_tile_tokens": 57, "attention.max_single_len": 301,
                           "attention.max_tile_len": 140, "attention.min_tile_ctx": 0}
    # every token is named exactly once by the singles and the tiles
    rows = lists["attention.single"] + [f + i for f, c in zip(lists["attention.tile_first"], lists["attention.tile_count"])
                                        for i in range(c)]
    assert sorted(rows) == list(range(batch.num_tokens))
    # single tokens are listed longest context first (blocks start in that order), ties in step order
    mixed = unpack(pack_batch(spans_of((1, 7), (1, 300), (2, 5), (1, 300), (1, 41)), 1, [ATTENTION_WORK]))
    assert mixed.lists["attention.single"].tolist() == [1, 4, 5, 0]


def test_a_recorded_step_rounds_the_facts_as_the_planner_asks():
    one = pack_batch(spans_of((1, 299), (1, 12)), 1, [ATTENTION_WORK], fixed_widths=[64], bucket=True)
    two = pack_batch(spans_of((1, 310), (1, 80)), 1, [ATTENTION_WORK], fixed_widths=[64], bucket=True)
    far = pack_batch(spans_of((1, 400), (1, 80)), 1, [ATTENTION_WORK], fixed_widths=[64], bucket=True)
    assert one.facts["attention.max_single_len"] == two.facts["attention.max_single_len"] == 320
    assert one.shape_key() == two.shape_key() != far.shape_key()
    assert one.buf.size == two.buf.size
    assert [quarter_octave_at_least(n, 256) for n in (1, 256, 257, 320, 321, 512, 513, 700)] == [
        256, 256, 320, 320, 384, 512, 640, 768]
    with pytest.raises(ValueError, match="fixed width"):
        pack_batch(spans_of((1, 600)), 1, [ATTENTION_WORK], fixed_widths=[64])


def test_any_part_may_bring_a_planner_of_its_own():
    class Pairs(StepPlanner):
        name = "pairs"

        def lists(self, q_lens, ctx_lens):
            first = [sum(q_lens[:i]) + t for i, q in enumerate(q_lens) for t in range(0, q, 2)]
            return {"first": first}, {"count": len(first), "deepest": max(ctx_lens)}

        def bucket(self, facts):
            facts["deepest"] = -(-facts["deepest"] // 100) * 100
            return facts

    packed = pack_batch(spans_of((5, 0), (2, 41)), 1, [ATTENTION_WORK, Pairs()])
    batch = unpack(packed)
    assert batch.lists["pairs.first"].tolist() == [0, 2, 4, 5]
    assert batch.facts["pairs.count"] == 4 and batch.facts["pairs.deepest"] == 41
    assert batch.lists["attention.tile_first"].tolist() == [0, 5]      # the attention lists are beside them
    assert pack_batch(spans_of((5, 0), (2, 41)), 1, [Pairs()], bucket=True).facts["pairs.deepest"] == 100
    # the lists lie in the one buffer that is copied to the device
    assert packed.buf.dtype == np.int32 and packed.offsets[-1] == packed.buf.size
    assert packed.list_names[-1] == "pairs.first"


def test_a_layer_call_brings_one_cache_slot_for_each_mixer():
    from tokamak_amd.config import LayerCall

    assert LayerCall(0, 3).slots == (3,) and LayerCall(0, (1, 2)).slots == (1, 2)
