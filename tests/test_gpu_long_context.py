"""Attention at the longest contexts the model allows (32,768 and 40,960 keys), compared
with a float64 reference: a decode token (dozens of key splits and the merge over more than
64 of them), a 64-token portion (few tiles, their keys split), a 2,048-token portion (the
wide form at its real threshold).  Pages of 16 scattered over the pool, unused slots NaN.

Random queries and keys would average tens of thousands of values to nearly nothing and
hide a lost split or page, so the queries are scaled until a few keys anywhere in the
context carry each softmax, and chosen queries are pointed at chosen keys: the first key,
keys on both sides of a split's edge, the last key before the portion.  The reference's
longest such test is 4,089 tokens (tests/unit/test_paged_attention_kernel.py:108-124)."""

import pytest
import torch

from kernel_util import make_batch, pack_pages_whole, reference_attention_blocked

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = {torch.float32: dict(rtol=1e-4, atol=2e-5), torch.bfloat16: dict(rtol=2e-2, atol=1e-2)}
HD, PS = 128, 16


def long_case(dtype, nh, nkv, ctx, qlen, seed, targets):
    """One request with ``ctx`` cached tokens and ``qlen`` new ones.  ``targets``: (query
    index, key position) pairs: that query (all heads) points at that key."""
    g = torch.Generator().manual_seed(seed)
    T = ctx + qlen
    pages = -(-T // PS)
    order = torch.randperm(pages + 7, generator=g).tolist()
    table = order[:pages]
    k = torch.randn(T, nkv, HD, generator=g)
    v = torch.randn(T, nkv, HD, generator=g)
    q = torch.randn(qlen, nh, HD, generator=g) * 5.0          # a few keys carry each softmax
    for query, key in targets:
        direction = torch.nn.functional.normalize(torch.randn(HD, generator=g), dim=0)
        k[key] = direction * 14.0
        q[query] = direction * 40.0                          # score 560 * scale = 49: nothing else comes near
    k, v, q = k.to(dtype), v.to(dtype), q.to(dtype)
    k_cache = torch.full((pages + 7, nkv * HD * PS), float("nan"), dtype=dtype)
    v_cache = torch.full((pages + 7, nkv * HD * PS), float("nan"), dtype=dtype)
    pack_pages_whole(k_cache, v_cache, k, v, table, PS)
    # the padding of the last page is NaN again: nothing may read past the request's end
    if T % PS:
        last = k_cache[table[-1]].view(nkv, HD // 8, PS, 8)
        last[:, :, T % PS:, :] = float("nan")
        lastv = v_cache[table[-1]].view(nkv, HD // 16, PS // 4, 16, 4)
        for slot in range(T % PS, PS):
            lastv[:, :, slot // 4, :, slot % 4] = float("nan")
    return q, k, v, k_cache, v_cache, table


def run(dtype, nh, nkv, ctx, qlen, seed, targets, expect_modes=None, monkeypatch=None):
    from tokamak_amd.kernels import attention

    q, k, v, k_cache, v_cache, table = long_case(dtype, nh, nkv, ctx, qlen, seed, targets)
    batch = make_batch([(qlen, ctx, table)])
    launched = []
    if monkeypatch is not None:
        real = attention.ops.attention_mfma
        monkeypatch.setattr(attention.ops, "attention_mfma",
                            lambda mode, *a, **kw: (launched.append((mode, kw.get("num_splits", 1))), real(mode, *a, **kw))[1])
    q_dev = q.reshape(qlen, nh * HD).to(DEV)
    out = torch.full_like(q_dev, float("nan"))
    attention.paged_attention(q_dev, k_cache.to(DEV), v_cache.to(DEV), batch.block_tables[0], batch, out,
                              num_heads=nh, num_kv_heads=nkv, head_dim=HD, page_size=PS, scale=HD ** -0.5)
    got = out.cpu().float().reshape(qlen, nh, HD)
    want = reference_attention_blocked(q.float(), k.float(), v.float(), range(ctx, ctx + qlen), HD ** -0.5).float()
    assert torch.isfinite(got).all(), "a slot past the request's end, or a page it does not own, was read"
    torch.testing.assert_close(got, want, **TOL[dtype])
    for query, key in targets:       # the pointed queries return their key's value
        torch.testing.assert_close(got[query], v[key].float().repeat_interleave(nh // nkv, dim=0),
                                   rtol=0, atol=3e-2 if dtype == torch.bfloat16 else 1e-4)
    return launched


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("keys", [32768, 40960])
@pytest.mark.parametrize("far", [0, 255, 256, 20479, 20480, -2])
def test_a_decode_token_over_the_longest_context(dtype, keys, far, monkeypatch):
    """One token over ``keys`` keys (itself the last), pointed at one far key: the first, the
    last of the first split's first wave share, both sides of a split's edge, the one before
    itself."""
    from tokamak_amd.kernels import attention

    ctx = keys - 1
    key = far if far >= 0 else ctx + far + 1
    chosen = attention.decode_split(1, 2, keys, HD)[1]
    assert 32 <= chosen <= 64            # as priced: two blocks a split, each split a merge read
    for finest in (False, True):
        if finest:                       # and the finest split there is: the merge walks more than 64 splits
            monkeypatch.setattr(attention, "decode_split", lambda *sizes: (256, keys // 256))
        launched = run(dtype, 8, 2, ctx, 1, seed=keys + (far % 997), targets=[(0, key)],
                       monkeypatch=monkeypatch if dtype == torch.bfloat16 else None)
        if dtype == torch.bfloat16:
            assert launched == [("heads", keys // 256 if finest else chosen)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("keys", [32768, 40960])
def test_a_short_portion_over_the_longest_context(dtype, keys, monkeypatch):
    """64 tokens at the end of ``keys``: four tiles, their keys cut into dozens of pieces."""
    from tokamak_amd.kernels.attention import tile_split

    ctx = keys - 64
    targets = [(0, 0), (5, 511), (6, 512), (17, ctx - 1), (40, ctx + 39), (63, ctx // 2 + 3)]
    launched = run(dtype, 8, 2, ctx, 64, seed=keys + 1, targets=targets,
                   monkeypatch=monkeypatch if dtype == torch.bfloat16 else None)
    if dtype == torch.bfloat16:
        split, nsplit = tile_split(4, 2, keys)
        assert nsplit > 16 and launched == [("tokens", nsplit)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("keys", [32768, 40960])
def test_a_long_portion_over_the_longest_context(dtype, keys, monkeypatch):
    """2,048 tokens at the end of ``keys``: with four kv heads the group form (tiles of 32 tokens,
    a block a CU) at its real threshold; with two, too few blocks for it: the 16-token tiles with
    their keys cut into pieces."""
    ctx = keys - 2048
    targets = [(0, 0), (31, 63), (32, 64), (1000, ctx - 1), (1500, ctx + 1499), (2047, ctx // 3), (777, 4095), (778, 4096)]
    launched = run(dtype, 16, 4, ctx, 2048, seed=keys + 2, targets=targets,
                   monkeypatch=monkeypatch if dtype == torch.bfloat16 else None)
    if dtype == torch.bfloat16:
        assert launched == [("tokens_group", 1)]
        launched = run(dtype, 8, 2, ctx, 2048, seed=keys + 6, targets=targets, monkeypatch=monkeypatch)
        assert len(launched) == 1 and launched[0][0] == "tokens" and launched[0][1] > 1


@pytest.mark.parametrize("keys", [32768, 40960])
def test_a_long_portion_of_pairs_of_heads_over_the_longest_context(keys, monkeypatch):
    """The same with two query heads a kv head: the wide form when the tiles are more than the CUs
    (eight kv heads), the group form with four shares of the keys a block when they are not (four)."""
    ctx = keys - 2048
    targets = [(0, 0), (31, 63), (32, 64), (1000, ctx - 1), (1500, ctx + 1499), (2047, ctx // 3)]
    launched = run(torch.bfloat16, 16, 8, ctx, 2048, seed=keys + 4, targets=targets, monkeypatch=monkeypatch)
    assert launched == [("tokens_wide", 1)]
    launched = run(torch.bfloat16, 8, 4, ctx, 2048, seed=keys + 5, targets=targets, monkeypatch=monkeypatch)
    assert launched == [("tokens_group", 1)]


@pytest.mark.parametrize("keys", [32768, 40960])
def test_a_long_portion_of_few_heads_over_the_longest_context(keys, monkeypatch):
    """The same with one kv head: too few blocks to fill the GPU, so the 16-token tiles' keys
    are cut into pieces and merged."""
    ctx = keys - 2048
    targets = [(0, 0), (1000, ctx - 1), (1500, ctx + 1499), (2047, ctx // 3), (777, 4095), (778, 4096)]
    launched = run(torch.bfloat16, 4, 1, ctx, 2048, seed=keys + 3, targets=targets, monkeypatch=monkeypatch)
    assert len(launched) == 1 and launched[0][0] == "tokens" and launched[0][1] > 1


# ---------------------------------------------------------------------------
# the whole model at the longest context: a tiny configuration whose positions go to 40,960
# ---------------------------------------------------------------------------
LONGEST = 40960


@pytest.fixture(scope="module")
def long_model(tmp_path_factory):
    """Two layers, two query heads on one kv head of 128, positions to 40,960.  The q norm's
    weight is raised threefold so that each softmax rests on a handful of keys anywhere in
    the context (scores with a spread of 3: about 40,960 / e^9 = 5 keys carry it) instead of
    averaging all of them to nothing: a lost page, split or portion then moves the logits.
    (A sharper softmax would also magnify the rounding of bfloat16 queries and keys beyond
    the suite's bound.)  The plain logits are computed once, for all positions."""
    import json

    from safetensors.torch import load_file, save_file

    import plain_qwen3 as plain
    from replay_util import random_ids
    from tokamak_amd.models.qwen3 import Qwen3Config
    from tokamak_amd.weights import write_random_model

    cfg = Qwen3Config("Qwen3ForCausalLM", vocab_size=97, hidden_size=64, num_layers=2, num_attention_heads=2,
                      num_kv_heads=1, head_dim=128, intermediate_size=96, rms_norm_eps=1e-6, rope_theta=1000000.0,
                      max_position_embeddings=LONGEST, tie_word_embeddings=False)
    folder = write_random_model(tmp_path_factory.mktemp("long") / "model", cfg, seed=12, matrix_std=0.05, vector_jitter=0.1)
    tensors = load_file(folder / "model.safetensors")
    for layer in range(2):
        name = f"model.layers.{layer}.self_attn.q_norm.weight"
        tensors[name] = (tensors[name].float() * 3.0).to(tensors[name].dtype)
    save_file(tensors, str(folder / "model.safetensors"), metadata={"format": "pt"})
    assert json.loads((folder / "config.json").read_text())["max_position_embeddings"] == LONGEST
    ids = random_ids(cfg.vocab_size, LONGEST, 99)
    pcfg, w = plain.read_folder(folder)
    want = plain.logits(ids, pcfg, w, query_block=1024)
    return folder, ids, want


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_to_the_models_last_position(long_model, dtype):
    """40,960 tokens through the step function: portions of 2,048 (logits wanted here and
    there: at a portion's first and last row, across 4,095/4,096 and 32,767/32,768), then a
    portion of 61 that stops short of the end, then three tokens one by one up to the very last
    position the model allows."""
    from replay_util import TOL
    from tokamak_amd.engine.runner import ModelRunner, StepEntry

    folder, ids, want = long_model
    runner = ModelRunner.from_folder(folder, dtype=dtype, page_size=16, kv_pool_tokens=LONGEST, max_requests=2)
    wanted_at = {0, 2047, 2048, 4095, 4096, 20000, 32767, 32768, LONGEST - 65, LONGEST - 64}
    got = {}
    at = 0
    cuts = [2048] * 19 + [LONGEST - 64 - 19 * 2048, 61, 1, 1, 1]
    assert sum(cuts) == LONGEST
    for n in cuts:
        rows = [p - at for p in range(at, at + n) if p in wanted_at or p >= LONGEST - 64]
        out = runner.step([StepEntry("long", ids[at:at + n], rows)]).cpu()
        for row, logits in zip(rows, out):
            got[at + row] = logits
        at += n
    assert runner.cached_tokens("long") == LONGEST
    with pytest.raises(ValueError, match="limit"):
        runner.step([StepEntry("long", [1], [0])])               # one more than the model allows
    runner.end("long")
    runner.manager.check()
    assert runner.manager.num_free_pages() == runner.manager.num_pages()
    positions = sorted(got)
    assert len(positions) == len(wanted_at) - 1 + 64             # (LONGEST - 64 is in both sets)
    bound = TOL[dtype]
    for p in positions:
        slack = bound["tol_abs"] + bound.get("tol_rel_to_scale", 0.0) * float(want[p].abs().max())
        error = float((got[p] - want[p]).abs().max())
        assert error <= slack, f"position {p}: logits differ by {error:.2e} (allowed {slack:.2e})"
