"""Each kernel alone against a plain float32/float64 reference, at sizes other
than the engine's tiny models, with inputs made so that faults show."""

import math

import pytest
import torch

import plain_qwen3 as plain
from kernel_util import make_batch, pack_pages, reference_attention, unpack_pages

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = {torch.float32: dict(rtol=1e-4, atol=1e-5), torch.bfloat16: dict(rtol=2e-2, atol=1e-2)}


def rand(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


# ---------------------------------------------------------------------------
# attention
# ---------------------------------------------------------------------------
def run_attention(dtype, nh, nkv, hd, ps, requests, *, window=None, poison=True, force_generic=False,
                  seed=0, boost=None, share_heads=None):
    """requests: list of (ctx_len, q_len).  Builds scattered tables, fills pages,
    runs the dispatcher (or the generic kernel) and returns (got, want) lists."""
    from tokamak_amd.kernels import ops
    from tokamak_amd.kernels.attention import paged_attention

    g = torch.Generator().manual_seed(seed)
    total_pages = sum(-(-(c + q) // ps) for c, q in requests) + 5
    order = torch.randperm(total_pages, generator=g).tolist()
    fill = float("nan") if poison else 0.0
    k_cache = torch.full((total_pages, nkv * hd * ps), fill, dtype=dtype)
    v_cache = torch.full((total_pages, nkv * hd * ps), fill, dtype=dtype)
    spans, seqs, qs = [], [], []
    for ctx, qlen in requests:
        T = ctx + qlen
        npages = -(-T // ps)
        table, order = order[:npages], order[npages:]
        k = torch.randn(T, nkv, hd, generator=g).to(dtype)
        v = torch.randn(T, nkv, hd, generator=g).to(dtype)
        q = torch.randn(qlen, nh, hd, generator=g).to(dtype)
        if boost is not None:
            boost(q, k, v, ctx, qlen)
        pack_pages(k_cache, v_cache, k, v, table, ps)
        spans.append((qlen, ctx, table))
        seqs.append((k, v))
        qs.append(q)
    batch = make_batch(spans)
    q_all = torch.cat(qs).reshape(-1, nh * hd).to(DEV)
    out = torch.full_like(q_all, float("nan"))
    scale = hd ** -0.5
    kc, vc = k_cache.to(DEV), v_cache.to(DEV)
    if force_generic:
        ops.paged_attention_generic(q_all, kc, vc, batch.block_tables[0], batch.positions, batch.req_of_token,
                                    out, num_heads=nh, num_kv_heads=nkv, head_dim=hd, page_size=ps,
                                    scale=scale, window=window, share_heads=share_heads)
    else:
        paged_attention(q_all, kc, vc, batch.block_tables[0], batch, out, num_heads=nh, num_kv_heads=nkv,
                        head_dim=hd, page_size=ps, scale=scale, window=window)
    out = out.cpu().float().reshape(-1, nh, hd)
    got, want, at = [], [], 0
    for (ctx, qlen), (k, v), q in zip(requests, seqs, qs):
        got.append(out[at:at + qlen])
        want.append(reference_attention(q.float(), k.float(), v.float(), range(ctx, ctx + qlen), scale, window).float())
        at += qlen
    return got, want


SHAPES = [
    (4, 2, 16, 8), (7, 1, 16, 16), (16, 8, 128, 16), (32, 8, 128, 16), (8, 2, 64, 32), (5, 5, 48, 16),
    (6, 2, 256, 16), (24, 2, 64, 16), (3, 1, 128, 16), (14, 2, 128, 16), (8, 2, 128, 64), (4, 4, 64, 128),
    (2, 1, 128, 24), (16, 1, 128, 16), (20, 2, 128, 32),
]
MIXES = {
    "decode": [(48, 1), (15, 1), (0, 1), (300, 1), (16, 1)],
    "prefill": [(0, 33), (0, 1), (0, 16), (0, 70)],
    "portions": [(17, 2), (30, 19), (64, 32), (5, 40)],
    "mixed": [(100, 1), (0, 50), (31, 1), (47, 18), (16, 1)],
}


@pytest.mark.parametrize("mix", list(MIXES))
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("nh, nkv, hd, ps", SHAPES)
def test_attention_matches_reference(nh, nkv, hd, ps, dtype, mix):
    got, want = run_attention(dtype, nh, nkv, hd, ps, MIXES[mix], seed=hd + nh)
    for g, w in zip(got, want):
        assert torch.isfinite(g).all(), "a page that the request does not own, or a slot past its end, was read"
        torch.testing.assert_close(g, w, **TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_generic_kernel_at_mfma_shapes(dtype):
    got, want = run_attention(dtype, 16, 4, 128, 16, MIXES["mixed"], force_generic=True)
    for g, w in zip(got, want):
        torch.testing.assert_close(g, w, **TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("hd", [64, 128, 80])
def test_long_context_over_shuffled_pages(dtype, hd):
    """4,089 tokens over 256 scattered pages (reference
    tests/unit/test_paged_attention_kernel.py:108-124), decoded and as a portion."""
    got, want = run_attention(dtype, 4, 2, hd, 16, [(4088, 1), (4000, 89)], seed=2)
    for g, w in zip(got, want):
        torch.testing.assert_close(g, w, **TOL[dtype])


@pytest.mark.parametrize("nh, nkv, hd, ps", [(8, 2, 128, 16), (6, 3, 64, 32), (3, 1, 128, 16)])
def test_short_portions_over_long_contexts_split_their_keys(nh, nkv, hd, ps):
    """Few tiles over thousands of keys: the dispatcher cuts the keys of the tiles into
    pieces (checked) that are merged afterwards; portions of other requests in the same
    step are short, start at zero or end inside a piece, and a decode token rides along."""
    from tokamak_amd.kernels.attention import tile_split

    requests = [(5000, 37), (0, 20), (700, 3), (2047, 2), (1300, 1)]
    tiles = sum(-(-q // 16) for _, q in requests if q > 1)
    group = nh // nkv
    per_tile = nkv * (group // (4 if group % 4 == 0 else 2 if group % 2 == 0 else 1))
    split, nsplit = tile_split(tiles, per_tile, 5037)
    assert nsplit > 1 and split % 64 == 0 and (nsplit - 1) * split < 5037 <= nsplit * split
    got, want = run_attention(torch.bfloat16, nh, nkv, hd, ps, requests, seed=11)
    for g, w in zip(got, want):
        assert torch.isfinite(g).all()
        torch.testing.assert_close(g, w, **TOL[torch.bfloat16])


def test_many_tiles_over_long_contexts_use_the_four_wave_kernel(monkeypatch):
    """Two portions that both start beyond 2,048 cached tokens, with too many tiles for their
    keys to be split and (pairs of heads, more blocks than CUs, under 4,096 keys) neither the
    group nor the wide form: the dispatcher takes the kernel variant built for four waves a
    SIMD (checked), with the same results."""
    from tokamak_amd.kernels import attention

    nh, nkv, hd, ps = 16, 8, 128, 16
    requests = [(2100, 700), (2500, 650)]
    tiles = sum(-(-q // 16) for _, q in requests)
    assert attention.tile_split(tiles, nkv, 3150)[1] == 1 and min(c for c, _ in requests) >= attention.DENSE_TILES_FROM
    launched = []
    real = attention.ops.attention_mfma
    monkeypatch.setattr(attention.ops, "attention_mfma", lambda mode, *a, **k: (launched.append(mode), real(mode, *a, **k))[1])
    got, want = run_attention(torch.bfloat16, nh, nkv, hd, ps, requests, seed=13)
    assert launched == ["tokens_dense"]
    for g, w in zip(got, want):
        assert torch.isfinite(g).all()
        torch.testing.assert_close(g, w, **TOL[torch.bfloat16])


@pytest.mark.parametrize("nh, nkv, hd, ps", [(8, 2, 128, 16), (6, 3, 64, 32), (3, 1, 128, 16), (32, 8, 128, 16), (4, 4, 64, 64),
                                             (5, 1, 128, 16), (12, 2, 64, 16), (7, 1, 128, 32), (16, 2, 128, 16), (20, 2, 64, 16),
                                             (6, 1, 128, 16), (9, 1, 64, 16)])
def test_tiles_of_32_tokens_for_long_walks(nh, nkv, hd, ps, monkeypatch):
    """Portions cut into tiles of 32 tokens, the 32x32 matrix-core forms: taken (checked by
    their conditions, here with the thresholds on the context lowered) when tiles are mostly
    full; portions that start at zero, in the middle of a page, end inside a tile, a
    one-token tail tile, and a decode token beside them.  Groups of three query heads and
    more take the group form (a block of all the group's heads, up to eight, and shares of
    the keys that are merged in the block), smaller ones the wide form."""
    from tokamak_amd.kernels import attention

    monkeypatch.setattr(attention, "WIDE_FROM_KEYS", 64)
    monkeypatch.setattr(attention, "group_form_pays", lambda group, *rest: group >= 3)
    requests = [(0, 200), (37, 150), (900, 33), (5, 32), (300, 1), (0, 450)]
    tiles = [q for _, q in requests if q > 1]
    assert sum(tiles) >= attention.WIDE_FROM_TOKENS * sum(-(-q // 32) for q in tiles)
    launched = []
    real = attention.ops.attention_mfma
    monkeypatch.setattr(attention.ops, "attention_mfma", lambda mode, *a, **k: (launched.append(mode), real(mode, *a, **k))[1])
    got, want = run_attention(torch.bfloat16, nh, nkv, hd, ps, requests, seed=21)
    assert launched == ["heads", "tokens_group" if nh // nkv >= 3 else "tokens_wide"]
    for g, w in zip(got, want):
        assert torch.isfinite(g).all(), "a page that the request does not own, or a slot past its end, was read"
        torch.testing.assert_close(g, w, **TOL[torch.bfloat16])


@pytest.mark.parametrize("nh, nkv", [(8, 2), (4, 2), (5, 1)])
def test_tiles_of_32_tokens_find_a_far_key_and_respect_the_causal_edge(nh, nkv, monkeypatch):
    """The group form (and for groups of two the wide form) on inputs made to show faults: one key far back dominates one query's
    softmax (its value must come out), and the key right after a query's position is made
    enormous (reading it would show).  (Three tiles are too few for these forms to be chosen: they are asked for.)"""
    from tokamak_amd.kernels import attention

    hd = 128
    launched = []
    real = attention.ops.attention_mfma
    monkeypatch.setattr(attention, "group_form_pays", lambda group, *rest: group >= 3)
    monkeypatch.setattr(attention, "tile_split", lambda *sizes: (1 << 30, 1))    # (so few tiles would have their keys split)
    monkeypatch.setattr(attention.ops, "attention_mfma", lambda mode, *a, **k: (launched.append(mode), real(mode, *a, **k))[1])
    seen = {}

    def boost(q, k, v, ctx, qlen):
        direction = torch.nn.functional.normalize(torch.randn(hd, generator=torch.Generator().manual_seed(9)), dim=0)
        k[7, :, :] = (direction * 16.0).to(k.dtype)                 # far back, first page
        q[40, :, :] = (direction * 16.0).to(q.dtype)                # query at position ctx + 40
        other = torch.nn.functional.normalize(torch.randn(hd, generator=torch.Generator().manual_seed(10)), dim=0)
        q[10, :, :] = (other * 4.0).to(q.dtype)
        k[ctx + 11, :, :] = (other * 50.0).to(k.dtype)              # the key right after query 10: hidden from it
        v[ctx + 11, :, :] = 1000.0
        seen["far"] = v[7].float().clone()

    got, want = run_attention(torch.bfloat16, nh, nkv, hd, 16, [(4100, 96)], boost=boost, seed=5)
    assert attention.WIDE_FROM_KEYS <= 4196
    assert launched == ["tokens_group" if nh // nkv >= 3 else "tokens_wide"]
    torch.testing.assert_close(got[0], want[0], **TOL[torch.bfloat16])
    expected = seen["far"].repeat_interleave(nh // nkv, dim=0)
    torch.testing.assert_close(got[0][40], expected, rtol=0, atol=2e-2)
    assert got[0][10].abs().max() < 50           # nothing of the hidden key's value of 1000


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("far", [0, 3, 255, 256, 511, 777])
def test_a_far_key_among_hundreds_is_found(dtype, far):
    """One key (position ``far``) and the query are scaled so that its score
    stands out: the output must be that key's value.  Random weights alone would
    spread the softmax so thin that a skipped key could not be seen."""
    hd, nh, nkv = 128, 8, 2
    far_values = []

    def boost(q, k, v, ctx, qlen):
        direction = torch.nn.functional.normalize(torch.randn(hd, generator=torch.Generator().manual_seed(9)), dim=0)
        k[far, :, :] = (direction * 16.0).to(k.dtype)
        q[-1, :, :] = (direction * 16.0).to(q.dtype)
        far_values.append(v[far].float().clone())

    got, want = run_attention(dtype, nh, nkv, hd, 16, [(1023, 1), (1000, 24)], boost=boost, seed=4)
    for g, w, v_far in zip(got, want, far_values):
        torch.testing.assert_close(g, w, **TOL[dtype])
        # the last query's score for the far key is 256 / sqrt(128) = 22.6, a thousand others
        # lie around zero: its softmax weight is one to 1e-6, so the output is that key's value
        # for every head of its group.  Should the boost stop dominating, this fails and says
        # so, instead of leaving a comparison on random data that hides a skipped key.
        expected = v_far.repeat_interleave(nh // nkv, dim=0)
        torch.testing.assert_close(w[-1], expected, rtol=0, atol=1e-4)
        torch.testing.assert_close(g[-1], expected, rtol=0, atol=1e-4 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_window_edge(dtype):
    """Keys just inside and just outside a window of 24; the key right outside is
    made enormous, so reading it would show."""
    window = 24

    def boost(q, k, v, ctx, qlen):
        p = ctx + qlen - 1          # last query's position
        outside = p - window        # first position it must not see
        k[outside] = q[-1, :1].expand_as(k[outside]) * 30
        v[outside] = 1000.0

    for hd, nh, nkv in [(16, 4, 2), (128, 8, 2)]:
        got, want = run_attention(dtype, nh, nkv, hd, 16, [(40, 1), (10, 30), (100, 7)], window=window, boost=boost, seed=5)
        for g, w in zip(got, want):
            torch.testing.assert_close(g, w, **TOL[dtype])
            assert g[-1].abs().max() < 50


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("nh, nkv, hd, ps, window", [(4, 2, 16, 8, None), (5, 5, 48, 16, None), (6, 2, 256, 16, None),
                                                      (8, 2, 128, 16, 37), (3, 1, 80, 32, 70), (2, 1, 512, 8, None)])
def test_generic_attention_gives_equal_bits_for_tokens_alone_and_in_tiles(dtype, nh, nkv, hd, ps, window):
    """The generic kernel takes the tokens of a prompt portion in tiles that share the keys
    and values they load; a token's result is the same bit for bit as when it runs alone
    (rounds of 64 keys go to waves by their place in the context, sums keep their order),
    with a window too, whose first key differs from token to token of a tile."""
    requests = [(0, 70), (130, 21), (64, 1), (5, 16), (300, 1), (63, 2)]
    tiled, want = run_attention(dtype, nh, nkv, hd, ps, requests, window=window, seed=11)
    alone, _ = run_attention(dtype, nh, nkv, hd, ps, requests, window=window, seed=11, force_generic=True)
    for a, b, w in zip(tiled, alone, want):
        torch.testing.assert_close(a, w, **TOL[dtype])
        assert torch.equal(a, b)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("nh, nkv, hd", [(6, 2, 48), (16, 2, 80), (4, 4, 32)])
def test_generic_attention_gives_equal_bits_whether_heads_share_a_block_or_not(dtype, nh, nkv, hd):
    """With many single tokens the query heads of a group share a block and the keys it loads;
    with few every head has a block of its own.  Both give the same bits."""
    requests = [(3 + 37 * i, 1) for i in range(12)] + [(0, 5), (70, 3)]
    many, want = run_attention(dtype, nh, nkv, hd, 16, requests, seed=13, force_generic=True, share_heads=True)
    few, _ = run_attention(dtype, nh, nkv, hd, 16, requests, seed=13, force_generic=True, share_heads=False)
    for a, b, w in zip(many, few, want):
        torch.testing.assert_close(a, w, **TOL[dtype])
        assert torch.equal(a, b)


def test_unsupported_sizes_are_refused_not_wrong():
    from tokamak_amd.kernels import ops

    q = torch.zeros(1, 4 * 12, device=DEV)
    cache = torch.zeros(2, 2 * 12 * 16, device=DEV)
    tables = torch.zeros(1, 4, dtype=torch.int32, device=DEV)
    idx = torch.zeros(1, dtype=torch.int32, device=DEV)
    with pytest.raises(ops.KernelError, match="multiple of 16"):
        ops.paged_attention_generic(q, cache, cache, tables, idx, idx, q.clone(), num_heads=4, num_kv_heads=2,
                                    head_dim=12, page_size=16, scale=1.0)
    with pytest.raises(ops.KernelError, match="GPU"):
        ops.silu_mul(torch.zeros(2, 8), torch.zeros(2, 4))


# ---------------------------------------------------------------------------
# per-head norm + rotation + cache write
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("nh, nkv, hd, ps, rot", [(4, 2, 16, 8, 16), (5, 1, 48, 16, 48), (8, 2, 128, 16, 128), (3, 3, 64, 32, 32)])
def test_qknorm_rope_store(dtype, nh, nkv, hd, ps, rot):
    from tokamak_amd.kernels import ops

    eps, theta = 1e-5, 50000.0
    spans = [(5, 11, [3, 0]), (1, 16, [6, 2]), (20, 0, [5, 1])]      # (tokens, ctx, table)
    if ps == 8:
        spans = [(5, 11, [3, 0]), (1, 16, [6, 2, 7]), (20, 0, [5, 1, 4])]
    batch = make_batch(spans)
    N = batch.num_tokens
    qkv = rand(N, (nh + 2 * nkv) * hd, seed=1).to(dtype)
    qw, kw = 1 + 0.3 * rand(hd, seed=2), 1 + 0.3 * rand(hd, seed=3)
    positions = batch.positions.cpu()
    inv_freq = 1.0 / (theta ** (torch.arange(0, rot, 2, dtype=torch.float32) / rot))
    cos = torch.empty(N, rot // 2, device=DEV)
    sin = torch.empty(N, rot // 2, device=DEV)
    ops.rope_tables(batch.positions, inv_freq.to(DEV), cos, sin)
    want_cos, want_sin = plain.rope_tables(positions, rot, theta)
    torch.testing.assert_close(cos.cpu(), want_cos[:, : rot // 2], rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(sin.cpu(), want_sin[:, : rot // 2], rtol=1e-5, atol=1e-6)

    k_cache = torch.full((8, nkv * hd * ps), 7.0, dtype=dtype, device=DEV)
    v_cache = torch.full((8, nkv * hd * ps), 7.0, dtype=dtype, device=DEV)
    q_out = torch.empty(N, nh * hd, dtype=dtype, device=DEV)
    ops.qknorm_rope_store(qkv.to(DEV), qw.to(DEV), kw.to(DEV), cos, sin, batch.positions, batch.req_of_token,
                          batch.block_tables[0], q_out, k_cache, v_cache, num_heads=nh, num_kv_heads=nkv,
                          head_dim=hd, rotary_dim=rot, page_size=ps, eps=eps)
    x = qkv.float().view(N, nh + 2 * nkv, hd)
    q, k, v = x[:, :nh], x[:, nh:nh + nkv], x[:, nh + nkv:]

    def expect(t, w, rows=slice(None)):
        t = plain.rmsnorm(t, w, eps)
        rotated = plain.apply_rope(t[..., :rot], want_cos[rows], want_sin[rows])
        return torch.cat([rotated, t[..., rot:]], dim=-1)

    tol = TOL[dtype]
    torch.testing.assert_close(q_out.cpu().float().view(N, nh, hd), expect(q, qw), **tol)
    at = 0
    for n, ctx, table in spans:
        kk, vv = unpack_pages(k_cache.cpu(), v_cache.cpu(), table, ctx + n, nkv, hd, ps)
        torch.testing.assert_close(kk[ctx:].float(), expect(k[at:at + n], kw, slice(at, at + n)), **tol)
        torch.testing.assert_close(vv[ctx:].float(), v[at:at + n].to(dtype).float(), rtol=0, atol=0)  # v untouched
        assert (kk[:ctx] == 7.0).all() and (vv[:ctx] == 7.0).all()   # earlier positions are not written
        at += n


@pytest.mark.parametrize("form", ["float32", "bfloat16", "partial sums", "no norm", "queries only"])
@pytest.mark.parametrize("nh, nkv, hd, ps", [(8, 2, 128, 16), (3, 3, 64, 32), (14, 1, 128, 64), (5, 5, 64, 16)])
@pytest.mark.parametrize("lengths", [[(300, 11), (1, 77), (41, 0)], [(300, 12), (1, 77), (3, 5), (41, 8), (2, 30)]],
                         ids=["inside a quad", "quads of four"])
def test_qknorm_rope_store_of_long_portions(form, nh, nkv, hd, ps, lengths):
    """Portions of 300 and 41 tokens that start inside a page, beside a decode token, with a
    number of heads that is no multiple of a wave's share; pages scattered; partial sums as
    input; what is not written stays as it was.  "quads of four": the long portions start where
    both their first token's place in the step and its position are multiples of four, so
    that the values of four tokens are written as one piece of the page (and a portion's
    last, broken quad, a short portion in between and the others token by token)."""
    from tokamak_amd.kernels import ops

    dtype = torch.float32 if form == "float32" else torch.bfloat16
    eps, theta = 1e-5, 50000.0
    g = torch.Generator().manual_seed(nh + hd)
    need = [-(-(n + ctx) // ps) for n, ctx in lengths]
    order = torch.randperm(sum(need) + 3, generator=g).tolist()
    spans, at = [], 0
    for (n, ctx), pages in zip(lengths, need):
        spans.append((n, ctx, order[at:at + pages]))
        at += pages
    batch = make_batch(spans)
    N = batch.num_tokens
    stores = form != "queries only"
    width = (nh + (2 * nkv if stores else 0)) * hd
    qkv = rand(N, width, seed=1)
    qw, kw = 1 + 0.3 * rand(hd, seed=2), 1 + 0.3 * rand(hd, seed=3)
    cos = torch.empty(N, hd // 2, device=DEV)
    sin = torch.empty(N, hd // 2, device=DEV)
    inv_freq = 1.0 / (theta ** (torch.arange(0, hd, 2, dtype=torch.float32) / hd))
    ops.rope_tables(batch.positions, inv_freq.to(DEV), cos, sin)
    want_cos, want_sin = plain.rope_tables(batch.positions.cpu(), hd, theta)
    if form == "partial sums":
        pieces = rand(3, N, width, seed=5)
        pieces[2] = qkv - pieces[0] - pieces[1]
        given, qkv = pieces.to(DEV), pieces.sum(0)
    else:
        qkv = qkv.to(dtype).float()
        given = qkv.to(dtype).to(DEV)
    k_cache = torch.full((len(order), nkv * hd * ps), 7.0, dtype=dtype, device=DEV)
    v_cache = torch.full((len(order), nkv * hd * ps), 7.0, dtype=dtype, device=DEV)
    q_out = torch.empty(N, nh * hd, dtype=dtype, device=DEV)
    normed = form != "no norm"
    ops.qknorm_rope_store(given, qw.to(DEV) if normed else None, kw.to(DEV) if normed else None, cos, sin,
                          batch.positions, batch.req_of_token, batch.block_tables[0], q_out,
                          k_cache if stores else None, v_cache if stores else None, num_heads=nh, num_kv_heads=nkv,
                          head_dim=hd, rotary_dim=hd, page_size=ps, eps=eps, store=stores)
    x = qkv.view(N, -1, hd)

    def expect(t, w, rows=slice(None)):
        if normed:
            t = plain.rmsnorm(t, w, eps)
        return plain.apply_rope(t, want_cos[rows], want_sin[rows])

    tol = TOL[dtype]
    torch.testing.assert_close(q_out.cpu().float().view(N, nh, hd), expect(x[:, :nh], qw), **tol)
    if not stores:
        assert (k_cache == 7.0).all() and (v_cache == 7.0).all()
        return
    k, v = x[:, nh:nh + nkv], x[:, nh + nkv:]
    at = 0
    for n, ctx, table in spans:
        kk, vv = unpack_pages(k_cache.cpu(), v_cache.cpu(), table, len(table) * ps, nkv, hd, ps)
        torch.testing.assert_close(kk[ctx:ctx + n].float(), expect(k[at:at + n], kw, slice(at, at + n)), **tol)
        torch.testing.assert_close(vv[ctx:ctx + n].float(), v[at:at + n].to(dtype).float(), **tol)
        assert (kk[:ctx] == 7.0).all() and (vv[:ctx] == 7.0).all() and (kk[ctx + n:] == 7.0).all() and (vv[ctx + n:] == 7.0).all()
        at += n
    untouched = [p for p in range(len(order)) if all(p not in t for _, _, t in spans)]
    assert (k_cache[untouched] == 7.0).all() and (v_cache[untouched] == 7.0).all()


# ---------------------------------------------------------------------------
# norms, activation, embedding, matrix product
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("H", [64, 200, 4096, 5120 + 24])
def test_add_rmsnorm(dtype, H):
    from tokamak_amd.kernels import ops

    M, eps = 7, 1e-5
    resid, delta, w = rand(M, H, seed=1, scale=3.0), rand(M, H, seed=2).to(dtype), 1 + 0.2 * rand(H, seed=3)
    r = resid.to(DEV)
    out = torch.empty(M, H, dtype=dtype, device=DEV)
    ops.add_rmsnorm(r, delta.to(DEV), w.to(DEV), eps, out)
    x = resid + delta.float()
    torch.testing.assert_close(r.cpu(), x, rtol=0, atol=0)                      # the sum is float32 and stored
    torch.testing.assert_close(out.cpu().float(), plain.rmsnorm(x, w, eps), **TOL[dtype])
    # no delta; and row-indexed without touching the residual
    out2 = torch.empty(M, H, dtype=dtype, device=DEV)
    ops.add_rmsnorm(r, None, w.to(DEV), eps, out2)
    torch.testing.assert_close(out2.cpu().float(), plain.rmsnorm(x, w, eps), **TOL[dtype])
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=DEV)
    out3 = torch.empty(3, H, dtype=dtype, device=DEV)
    before = r.clone()
    ops.add_rmsnorm(r, delta.to(DEV), w.to(DEV), eps, out3, rows=rows, write_resid=False)
    torch.testing.assert_close(out3.cpu().float(), plain.rmsnorm(x[[5, 0, 5]] + delta.float()[[5, 0, 5]], w, eps), **TOL[dtype])
    assert torch.equal(r, before)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_silu_mul_and_embedding(dtype):
    from tokamak_amd.kernels import ops

    N, I = 5, 200
    gu = rand(N, 2 * I, seed=1, scale=4.0).to(dtype)
    out = torch.empty(N, I, dtype=dtype, device=DEV)
    ops.silu_mul(gu.to(DEV), out)
    g, u = gu.float()[:, :I], gu.float()[:, I:]
    torch.testing.assert_close(out.cpu().float(), plain.silu(g) * u, **TOL[dtype])

    table = rand(331, 120, seed=2).to(dtype)
    ids = torch.tensor([0, 330, 17, 17, 5], dtype=torch.int32)
    resid = torch.empty(5, 120, device=DEV)
    ops.embed_gather(table.to(DEV), ids.to(DEV), resid)
    torch.testing.assert_close(resid.cpu(), table.float()[ids.long()], rtol=0, atol=0)
    bad = torch.tensor([331, -1], dtype=torch.int32, device=DEV)
    resid2 = torch.zeros(2, 120, device=DEV)
    ops.embed_gather(table.to(DEV), bad, resid2)
    assert torch.isnan(resid2).all()        # an id outside the table never reads memory


@pytest.mark.parametrize("M, N, K", [(1, 64, 64), (5, 200, 96), (70, 331, 120), (3, 1000, 4096), (129, 65, 17)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_linear(dtype, M, N, K):
    from tokamak_amd.kernels.linear import linear

    x, w = rand(M, K, seed=1).to(dtype), rand(N, K, seed=2, scale=K ** -0.5).to(dtype)
    want = x.double() @ w.double().T
    for out_dtype in (dtype, torch.float32):
        got = linear(x.to(DEV), w.to(DEV), out_dtype=out_dtype).cpu()
        assert got.dtype == out_dtype
        tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else (
            dict(rtol=2e-2, atol=1e-2) if out_dtype == torch.bfloat16 else dict(rtol=1e-3, atol=1e-3))
        torch.testing.assert_close(got.double(), want, **tol)


def test_float32_product_is_true_32_bit_and_row_independent():
    """Values that a reduced-precision matrix mode would round away survive, and
    a row's result does not depend on which rows are beside it."""
    from tokamak_amd.kernels.linear import linear

    K = 512
    x = torch.ones(4, K)
    x[:, 0] = 1.0 + 2.0 ** -20                 # lost in bf16, tf32 and fp16 inputs
    w = torch.zeros(3, K)
    w[:, 0] = 1.0
    w[1, 1] = -1.0 + 2.0 ** -18
    got = linear(x.to(DEV), w.to(DEV)).cpu()
    assert got[0, 0].item() == 1.0 + 2.0 ** -20
    assert got[0, 1].item() == pytest.approx(2.0 ** -20 + 2.0 ** -18, rel=1e-6)
    big = rand(100, 300, seed=5)
    wt = rand(77, 300, seed=6)
    whole = linear(big.to(DEV), wt.to(DEV)).cpu()
    one = linear(big[41:42].to(DEV), wt.to(DEV)).cpu()
    assert torch.equal(whole[41:42], one)


@pytest.mark.parametrize("M, N, K", [(1, 64, 64), (3, 331, 200), (8, 1000, 4096), (16, 77, 1028), (17, 130, 516),
                                     (40, 200, 260), (64, 65, 12), (5, 70000, 264), (50, 16500, 264), (24, 66000, 40)])
def test_float32_product_of_few_rows_equals_the_tiled_one_bit_for_bit(M, N, K):
    """Up to 64 rows the float32 product streams the weights (a lane a weight row, a wave a
    piece of K or all of them); it sums in the tiled kernel's order, so the same rows inside
    a batch of 100 (the tiled kernel) give the same bits, with and without the split."""
    from tokamak_amd.kernels import ops

    x = rand(100, K, seed=1)
    w = rand(N, K, seed=2, scale=K ** -0.5)
    whole = torch.empty(100, N, device=DEV)
    ops.gemm_tiled(x.to(DEV), w.to(DEV), whole)
    torch.testing.assert_close(whole.cpu().double(), x.double() @ w.double().T, rtol=1e-5, atol=1e-5)
    for at in (0, 100 - M):
        for split in (None, False, True):
            out = torch.full((M, N), float("nan"), device=DEV)
            ops.gemm_tiled(x[at:at + M].to(DEV), w.to(DEV), out, fewrows_split=split)
            assert torch.equal(out, whole[at:at + M]), (at, split)
    # many rows of activations over a matrix with a tile for every CU take the tiled kernel itself
    assert ops.fewrows_pays(64, 4096) and ops.fewrows_pays(16, 200000) and ops.fewrows_pays(40, 16000)
    assert not ops.fewrows_pays(48, 16384) and not ops.fewrows_pays(24, 65536)


@pytest.mark.parametrize("M, N, K", [(1, 64, 64), (8, 6144, 4096), (64, 4096, 4096), (33, 331, 200), (17, 4096, 12288), (64, 1000, 264)])
def test_streaming_product_and_its_partial_sums(M, N, K):
    """The LDS-staged weight-streaming kernel, unsplit and split over K: the
    partial sums add up to the product, whoever adds them."""
    from tokamak_amd.kernels import ops
    check_streaming_product(ops, M, N, K, 0)


@pytest.mark.parametrize("M, N, K", [(64, 6144, 4096), (49, 200, 520), (40, 97, 264), (3, 96, 64), (24, 1000, 1024)])
@pytest.mark.parametrize("waves", [4, 6, 8])
def test_streaming_product_with_every_block_size(M, N, K, waves):
    """Blocks of four, six and eight waves (64, 96 and 128 weight rows): with six, a chunk of
    the activations does not divide evenly among the block's threads."""
    from tokamak_amd.kernels import ops
    check_streaming_product(ops, M, N, K, waves)


@pytest.mark.parametrize("M, N, K", [(65, 4096, 4096), (80, 331, 200), (96, 6144, 1024), (113, 1000, 2056), (128, 4096, 12288),
                                     (128, 130, 264), (127, 64, 64)])
def test_streaming_product_of_65_to_128_rows(M, N, K):
    """Five to eight tiles of 16 rows in blocks of eight waves: one copy of the activations'
    chunk in LDS, fragments read step by step."""
    from tokamak_amd.kernels import ops
    check_streaming_product(ops, M, N, K, 8)
    check_streaming_product(ops, M, N, K, 0)        # eight waves are what is chosen for these rows
    x = rand(M, K, seed=1).to(torch.bfloat16).to(DEV)
    w = rand(N, K, seed=2, scale=K ** -0.5).to(torch.bfloat16).to(DEV)
    with pytest.raises(ops.KernelError):            # blocks of four or six waves are not built for them
        ops.gemm_stream(x, w, torch.empty((M, N), device=DEV), waves=4)
    if N % 2 == 0:                                  # the gated product stops at 64 rows
        with pytest.raises(ops.KernelError):
            ops.gemm_stream_swiglu(x, w, torch.empty((M, N // 2), dtype=torch.bfloat16, device=DEV))


def test_products_of_65_to_128_rows_whose_reader_adds_partial_sums_stream_the_weights():
    """q/k/v, o and down of a step of 65 to 128 tokens: split over K by the streaming kernel where
    that was measured to pay (up to 96 rows; to 128 for matrices of 64 MB and more); a caller
    that wants the product itself gets the library's."""
    from tokamak_amd.kernels import gemm_bf16, ops

    x = rand(90, 1024, seed=1).to(torch.bfloat16).to(DEV)
    w = rand(2048, 1024, seed=2, scale=1 / 32).to(torch.bfloat16).to(DEV)
    want = x.cpu().double() @ w.cpu().double().T
    with ops.KernelProfile() as seen:
        parts = gemm_bf16.gemm(x, w, torch.bfloat16, allow_partials=True)
        whole = gemm_bf16.gemm(x, w, torch.bfloat16)
    assert parts.dim() == 3 and parts.shape[0] > 1 and parts.dtype == torch.float32
    torch.testing.assert_close(parts.sum(0).cpu().double(), want, rtol=1e-3, atol=1e-3)
    assert whole.shape == (90, 2048) and whole.dtype == torch.bfloat16
    torch.testing.assert_close(whole.cpu().double(), want, rtol=2e-2, atol=1e-2)
    assert [name.split()[0] for name, *_ in seen.calls] == ["gemm_stream", "lt_gemm"]
    pays = gemm_bf16.stream_pays_beyond_64_rows
    assert pays(65, 4096, 4096) and pays(96, 2048, 2048) and not pays(97, 4096, 4096) and not pays(64, 4096, 4096)
    assert pays(128, 5120, 17408) and pays(112, 4096, 12288) and not pays(129, 5120, 25600) and not pays(80, 48, 4096)
    more = rand(100, 1024, seed=3).to(torch.bfloat16).to(DEV)
    assert gemm_bf16.gemm(more, w, torch.bfloat16, allow_partials=True).dim() == 2      # a small matrix: the library


def check_streaming_product(ops, M, N, K, waves):

    x = rand(M, K, seed=1).to(torch.bfloat16)
    w = rand(N, K, seed=2, scale=K ** -0.5).to(torch.bfloat16)
    want = x.double() @ w.double().T
    for out_dtype, tol in ((torch.float32, dict(rtol=1e-3, atol=1e-3)), (torch.bfloat16, dict(rtol=2e-2, atol=1e-2))):
        out = torch.full((M, N), float("nan"), dtype=out_dtype, device=DEV)
        assert ops.gemm_stream(x.to(DEV), w.to(DEV), out, waves=waves) == 1
        torch.testing.assert_close(out.cpu().double(), want, **tol)
    for splits in (2, 3, 8):
        parts = torch.full((splits, M, N), float("nan"), device=DEV)
        used = ops.gemm_stream(x.to(DEV), w.to(DEV), parts, splits=splits, waves=waves)
        assert 1 <= used <= splits
        torch.testing.assert_close(parts[:used].sum(0).cpu().double(), want, rtol=1e-3, atol=1e-3)
        if used > 1:
            assert parts[0].abs().max() > 0 and not torch.allclose(parts[0].cpu().double(), want, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("M, N, K", [(65, 64, 64), (300, 1000, 512), (2048, 331, 200), (129, 4096, 1024), (130, 4096, 1024)])
def test_library_product_with_kept_plans_and_measured_algorithms(M, N, K):
    """The hipBLASLt path for more than 64 rows: right for sizes that are no power of
    two, on the first call (which measures the candidates) as on later ones (which
    reuse the kept plan), and two shapes of one class (129 and 130 rows) share the
    algorithm that was measured for the first."""
    from tokamak_amd.kernels import ops

    x = rand(M, K, seed=1).to(torch.bfloat16)
    w = rand(N, K, seed=2, scale=K ** -0.5).to(torch.bfloat16)
    want = x.double() @ w.double().T
    outs = []
    for _ in range(3):
        out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
        assert ops.gemm_library(x.to(DEV), w.to(DEV), out)
        outs.append(out.cpu())
        torch.testing.assert_close(outs[-1].double(), want, rtol=2e-2, atol=1e-2)
    # a view with a row stride (the fused qkv output is sliced like this)
    wide = torch.full((M, N + 64), float("nan"), dtype=torch.bfloat16, device=DEV)
    assert ops.gemm_library(x.to(DEV), w.to(DEV), wide[:, :N])
    torch.testing.assert_close(wide[:, :N].cpu().double(), want, rtol=2e-2, atol=1e-2)
    assert torch.isnan(wide[:, N:]).all()


def test_consumers_add_partial_sums():
    """The norm kernel and the q/k norm kernel take a split-K product's partial
    sums and add them in float32."""
    from tokamak_amd.kernels import ops

    M, H, P, eps = 5, 200, 3, 1e-5
    resid, w = rand(M, H, seed=1), 1 + 0.1 * rand(H, seed=2)
    parts = rand(P, M, H, seed=3)
    total = parts.sum(0)
    r = resid.to(DEV)
    out = torch.empty(M, H, dtype=torch.bfloat16, device=DEV)
    ops.add_rmsnorm(r, parts.to(DEV), w.to(DEV), eps, out)
    torch.testing.assert_close(r.cpu(), resid + total, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(out.cpu().float(), plain.rmsnorm(resid + total, w, eps), **TOL[torch.bfloat16])
    rows = torch.tensor([4, 1], dtype=torch.int32, device=DEV)
    out2 = torch.empty(2, H, dtype=torch.bfloat16, device=DEV)
    r2 = resid.to(DEV)
    ops.add_rmsnorm(r2, parts.to(DEV), w.to(DEV), eps, out2, rows=rows, write_resid=False)
    torch.testing.assert_close(out2.cpu().float(), plain.rmsnorm((resid + total)[[4, 1]], w, eps), **TOL[torch.bfloat16])

    nh, nkv, hd, ps = 4, 2, 32, 16
    batch = make_batch([(6, 3, [1, 0])])
    N = 6
    qkv_parts = rand(P, N, (nh + 2 * nkv) * hd, seed=4)
    whole = qkv_parts.sum(0)
    cos = torch.ones(N, hd // 2, device=DEV)
    sin = torch.zeros(N, hd // 2, device=DEV)
    outs = []
    for inp in (qkv_parts, whole):
        k_cache = torch.zeros(2, nkv * hd * ps, dtype=torch.bfloat16, device=DEV)
        v_cache = torch.zeros_like(k_cache)
        q_out = torch.empty(N, nh * hd, dtype=torch.bfloat16, device=DEV)
        ops.qknorm_rope_store(inp.to(DEV), torch.ones(hd, device=DEV), torch.ones(hd, device=DEV), cos, sin,
                              batch.positions, batch.req_of_token, batch.block_tables[0], q_out, k_cache, v_cache,
                              num_heads=nh, num_kv_heads=nkv, head_dim=hd, rotary_dim=hd, page_size=ps, eps=eps)
        outs.append((q_out.cpu(), k_cache.cpu(), v_cache.cpu()))
    for a, b in zip(*outs):
        torch.testing.assert_close(a.float(), b.float(), rtol=1e-2, atol=1e-2)
    assert outs[0][2].abs().max() > 0


@pytest.mark.parametrize("M, I, K", [(1, 64, 64), (8, 12288, 4096), (64, 200, 96), (33, 3072, 1024), (17, 136, 120), (64, 12288, 4096), (50, 1000, 520)])
@pytest.mark.parametrize("waves", [0, 2, 4, 6, 8], ids=["chosen", "two waves", "four", "six", "eight"])
def test_fused_gate_up_silu_product(M, I, K, waves):
    from tokamak_amd.kernels import ops

    x = rand(M, K, seed=1).to(torch.bfloat16)
    w = rand(2 * I, K, seed=2, scale=2 * K ** -0.5).to(torch.bfloat16)
    out = torch.full((M, I), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.gemm_stream_swiglu(x.to(DEV), w.to(DEV), out, waves=waves)
    g = x.double() @ w[:I].double().T
    u = x.double() @ w[I:].double().T
    torch.testing.assert_close(out.cpu().double(), g / (1 + torch.exp(-g)) * u, rtol=2e-2, atol=1e-2)


# ---------------------------------------------------------------------------
# few rows: the product that adds into the residual stream, and the row scale applied late
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("M, N, K", [(1, 4096, 4096), (8, 4096, 12288), (16, 1000, 264), (5, 100, 72), (3, 64, 2048), (7, 20, 8)])
@pytest.mark.parametrize("waves", [4, 8, 16])
def test_whole_k_product_adds_into_the_stream(M, N, K, waves):
    """resid += x W^T in the product's own kernel, with bf16(resid * gamma) and the rows' sums
    of squares per slab of 16 columns beside it; rows and columns past the ends (NaN around
    the operands) are never touched."""
    from tokamak_amd.kernels import ops

    x = rand(M, K, seed=1).to(torch.bfloat16)
    w = rand(N, K, seed=2, scale=K ** -0.5).to(torch.bfloat16)
    stream = rand(M, N, seed=3)
    gamma = 1 + 0.3 * rand(N, seed=4)
    want = stream.double() + x.double() @ w.double().T
    wide = torch.full((M + 2, N + 8), float("nan"), device=DEV)     # the stream as rows of a wider array
    resid = wide[1:M + 1, 4:N + 4]
    resid.copy_(stream)
    sumsq, scaled = ops.gemm_wholek_add(x.to(DEV), w.to(DEV), resid, gamma.to(DEV), waves=waves)
    torch.testing.assert_close(resid.cpu().double(), want, rtol=1e-3, atol=1e-3)
    assert torch.isnan(wide[0]).all() and torch.isnan(wide[M + 1]).all() and torch.isnan(wide[:, :4]).all() and torch.isnan(wide[:, N + 4:]).all()
    torch.testing.assert_close(scaled.cpu().double(), want * gamma.double(), rtol=1e-2, atol=1e-2)
    assert sumsq.shape == (-(-N // 16), M)
    torch.testing.assert_close(sumsq.sum(0).cpu().double(), (want ** 2).sum(1), rtol=1e-4, atol=1e-4)
    slab3 = (want[:, 48:64] ** 2).sum(1) if N >= 64 else None
    if slab3 is not None:
        torch.testing.assert_close(sumsq[3].cpu().double(), slab3, rtol=1e-4, atol=1e-4)
    # without a norm weight: the stream and the sums only
    resid.copy_(stream)
    sumsq2, none = ops.gemm_wholek_add(x.to(DEV), w.to(DEV), resid, None, waves=waves)
    assert none is None and torch.equal(sumsq2, sumsq)
    # the same call twice gives the same bits (the waves' sums are added in a fixed order)
    resid.copy_(stream)
    again, _ = ops.gemm_wholek_add(x.to(DEV), w.to(DEV), resid, gamma.to(DEV), waves=waves)
    assert torch.equal(again, sumsq)


@pytest.mark.parametrize("M, N, K", [(1, 6144, 4096), (8, 4096, 4096), (16, 1000, 264), (5, 100, 72), (3, 2048, 200),
                                     (4, 96, 8136)])
def test_products_apply_a_pending_row_scale(M, N, K):
    """RMSNorm = row scale x column scale; given bf16(x * gamma) and the rows' sums of squares
    in slabs, the streaming products (plain, split over K, gated) and the whole-K product
    give what they give on the finished norm.  x is far from unit scale and eps is large
    enough to matter, so a scale taken without eps, or from K of the wrong matrix, shows."""
    from tokamak_amd.kernels import ops

    eps = 1e-2
    x = rand(M, K, seed=1) * 0.05
    gamma = 1 + 0.3 * rand(K, seed=2)
    w = rand(N, K, seed=3, scale=K ** -0.5).to(torch.bfloat16)
    slabs = -(-K // 16)
    padded = torch.zeros(M, slabs * 16, dtype=torch.float64)
    padded[:, :K] = x.double()
    sumsq = (padded.view(M, slabs, 16) ** 2).sum(2).T.contiguous().float()
    scaled = (x * gamma).to(torch.bfloat16)
    rstd = torch.rsqrt((x.double() ** 2).mean(1) + eps)
    want = (scaled.double() * rstd[:, None]) @ w.double().T
    tol = dict(rtol=2e-3, atol=2e-3 * want.abs().max().item())
    args = (scaled.to(DEV), w.to(DEV))
    out = torch.full((M, N), float("nan"), device=DEV)
    ops.gemm_stream(*args, out, sumsq=sumsq.to(DEV), eps=eps)
    torch.testing.assert_close(out.cpu().double(), want, **tol)
    parts = torch.full((3, M, N), float("nan"), device=DEV)
    used = ops.gemm_stream(*args, parts, splits=3, sumsq=sumsq.to(DEV), eps=eps)
    torch.testing.assert_close(parts[:used].sum(0).cpu().double(), want, **tol)
    out = torch.full((M, N), float("nan"), device=DEV)
    ops.gemm_wholek(*args, out, sumsq=sumsq.to(DEV), eps=eps)
    torch.testing.assert_close(out.cpu().double(), want, **tol)
    if N % 2 == 0:
        half = N // 2
        g, u = want[:, :half], want[:, half:]
        gated = g / (1 + torch.exp(-g)) * u
        gtol = dict(rtol=2e-2, atol=1e-2 * gated.abs().max().item())
        for fn in (ops.gemm_stream_swiglu, lambda a, b, c, **kw: ops.gemm_stream_swiglu(a, b, c, waves=2, **kw),
                   lambda a, b, c, **kw: ops.gemm_stream_swiglu(a, b, c, waves=4, **kw),
                   lambda a, b, c, **kw: ops.gemm_wholek(a, b, c, gated=True, **kw)):
            out = torch.full((M, half), float("nan"), dtype=torch.bfloat16, device=DEV)
            fn(*args, out, sumsq=sumsq.to(DEV), eps=eps)
            torch.testing.assert_close(out.cpu().double(), gated, **gtol)


def test_fused_forms_refuse_what_they_cannot_take():
    from tokamak_amd.kernels import ops

    x = torch.zeros(17, 64, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(64, 64, dtype=torch.bfloat16, device=DEV)
    resid = torch.zeros(17, 64, device=DEV)
    with pytest.raises(ops.KernelError):
        ops.gemm_wholek_add(x, w, resid)                      # more than sixteen rows
    with pytest.raises(ops.KernelError):
        ops.gemm_wholek_add(x[:4], w[:63], resid[:4, :63])    # N not a multiple of 4
    with pytest.raises(ops.KernelError):
        ops.gemm_stream(x, w, torch.zeros(17, 64, device=DEV), sumsq=torch.zeros(4, 17, device=DEV))
    with pytest.raises(ops.KernelError):
        ops.gemm_stream(x[:4], w, torch.zeros(4, 64, device=DEV), sumsq=torch.zeros(4, 5, device=DEV))  # sums of other rows


# ---------------------------------------------------------------------------
# decode tokens in one kernel: q/k norm, rotation, cache write and attention
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("nh, nkv, hd, ps", [(32, 8, 128, 16), (6, 3, 64, 32), (14, 1, 128, 16), (3, 3, 128, 64)])
@pytest.mark.parametrize("form", ["partial sums", "bfloat16", "no norm", "no rotation", "reads only"])
def test_fused_decode_equals_the_two_kernels(nh, nkv, hd, ps, form):
    """The one-kernel form of a decode-only step against the q/k norm kernel followed by
    the attention kernel, on the same inputs: attention output, and every page of the cache
    afterwards (the token's key and value land in their slots, nothing else is touched).
    Contexts end at a tile's first and last key, at a page's edge, at position zero and
    deep enough for several splits; unowned pages are NaN."""
    from tokamak_amd.kernels import ops
    from tokamak_amd.kernels.attention import decode_attention_fused, fused_decode_fits, paged_attention

    g = torch.Generator().manual_seed(nh * 7 + hd)
    ctxs = [0, 15, 16, 31, 255, 256, 700, 2300, 47]
    stores = form != "reads only"
    width = (nh + (2 * nkv if stores else 0)) * hd
    n = len(ctxs)
    total_pages = sum(-(-(c + 1) // ps) for c in ctxs) + 4
    order = torch.randperm(total_pages, generator=g).tolist()
    k_cache = torch.full((total_pages, nkv * hd * ps), float("nan"), dtype=torch.bfloat16)
    v_cache = torch.full((total_pages, nkv * hd * ps), float("nan"), dtype=torch.bfloat16)
    spans = []
    for c in ctxs:
        npages = -(-(c + 1) // ps)
        table, order = order[:npages], order[npages:]
        keys = c + (0 if stores else 1)            # a reading call finds the token's own key in the cache
        if keys:
            pack_pages(k_cache, v_cache, torch.randn(keys, nkv, hd, generator=g), torch.randn(keys, nkv, hd, generator=g), table, ps)
        spans.append((1, c, table))
    batch = make_batch(spans)
    parts = 3 if form == "partial sums" else 1
    if form == "bfloat16":
        qkv = (torch.randn(n, width, generator=g) * 0.7).bfloat16().to(DEV)
    else:
        qkv = (torch.randn(parts, n, width, generator=g) * 0.5).to(DEV)
        qkv = qkv if parts > 1 else qkv[0]
    q_w = k_w = None
    if form != "no norm":
        q_w, k_w = (1 + 0.2 * torch.randn(hd, generator=g)).to(DEV), (1 + 0.2 * torch.randn(hd, generator=g)).to(DEV)
    rot = 0 if form == "no rotation" else hd
    cos = sin = None
    if rot:
        angle = torch.rand(n, hd // 2, generator=g) * 6.28
        cos, sin = angle.cos().to(DEV), angle.sin().to(DEV)
    common = dict(num_heads=nh, num_kv_heads=nkv, head_dim=hd, page_size=ps)
    assert fused_decode_fits(torch.bfloat16, hd, ps, nh // nkv, None, rot, batch)

    kc1, vc1 = k_cache.to(DEV), v_cache.to(DEV)
    q = torch.empty(n, nh * hd, dtype=torch.bfloat16, device=DEV)
    ops.qknorm_rope_store(qkv, q_w, k_w, cos, sin, batch.positions, batch.req_of_token, batch.block_tables[0], q,
                          kc1, vc1, rotary_dim=rot, eps=1e-5, store=stores, **common)
    want = torch.full((n, nh * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    paged_attention(q, kc1, vc1, batch.block_tables[0], batch, want, scale=hd ** -0.5, **common)

    kc2, vc2 = k_cache.to(DEV), v_cache.to(DEV)
    got = torch.full((n, nh * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    assert decode_attention_fused(qkv, q_w, k_w, cos, sin, kc2, vc2, batch.block_tables[0], batch, got,
                                  rotary_dim=rot, eps=1e-5, scale=hd ** -0.5, store=stores, **common)
    assert torch.isfinite(got).all()
    torch.testing.assert_close(got.float().cpu(), want.float().cpu(), rtol=2e-2, atol=1e-2)
    # the caches agree bit for bit where they hold numbers, and NaN stays where it was
    for a, b in ((kc1, kc2), (vc1, vc2)):
        a, b = a.cpu(), b.cpu()
        assert torch.equal(torch.isnan(a), torch.isnan(b))
        assert torch.equal(torch.nan_to_num(a.float()), torch.nan_to_num(b.float()))
