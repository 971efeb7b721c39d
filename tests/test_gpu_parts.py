"""Each part of a layer alone against the plain implementation's function for
it, at sizes of its own; and the sampler against the plain distribution."""

import pytest
import torch

import plain_qwen3 as plain
from kernel_util import make_batch

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = {torch.float32: dict(rtol=2e-4, atol=2e-5), torch.bfloat16: dict(rtol=3e-2, atol=2e-2)}


def rand(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def fetcher(tensors, dtype):
    def fetch(name):
        t = tensors[name]
        return t.to(DEV, torch.float32 if t.dim() == 1 else dtype).contiguous()
    return fetch


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_rmsnorm_part(dtype):
    from tokamak_amd.config import get_part

    norm = get_part("norm", "rmsnorm")(dim=200, eps=3e-6, dtype=dtype, device=DEV)
    assert list(norm.expected_tensors("n.")) == ["n.weight"]
    w = 1 + 0.2 * rand(200, seed=1)
    norm.bind("n.", fetcher({"n.weight": w}, dtype))
    resid, delta = rand(9, 200, seed=2, scale=2.0), rand(9, 200, seed=3).to(dtype)
    r = resid.to(DEV)
    h = norm.forward(r, delta.to(DEV))
    x = resid + delta.float()
    torch.testing.assert_close(h.cpu().float(), plain.rmsnorm(x, w, 3e-6), **TOL[dtype])
    torch.testing.assert_close(r.cpu(), x, rtol=0, atol=0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_swiglu_part(dtype):
    from tokamak_amd.config import get_part

    H, I = 96, 200
    ff = get_part("feed_forward", "swiglu")(hidden_size=H, intermediate_size=I, dtype=dtype, device=DEV)
    w = {"m.gate_proj.weight": rand(I, H, seed=1, scale=H ** -0.5).to(dtype).float(),
         "m.up_proj.weight": rand(I, H, seed=2, scale=H ** -0.5).to(dtype).float(),
         "m.down_proj.weight": rand(H, I, seed=3, scale=I ** -0.5).to(dtype).float()}
    assert set(ff.expected_tensors("m.")) == set(w)
    ff.bind("m.", fetcher(w, dtype))
    for rows in (1, 7, 70):
        x = rand(rows, H, seed=4).to(dtype)
        got = ff.forward(x.to(DEV), None)
        got = (got.sum(0) if got.dim() == 3 else got).cpu().float()
        torch.testing.assert_close(got, plain.swiglu(x.float(), w, "m."), **TOL[dtype])
    # zero gate weights give zero output (reference tests/unit/test_layers.py:71-79)
    w0 = dict(w)
    w0["m.gate_proj.weight"] = torch.zeros(I, H)
    ff.bind("m.", fetcher(w0, dtype))
    assert ff.forward(rand(3, H, seed=5).to(dtype).to(DEV), None).abs().max().item() == 0.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_rotary_part_tables(dtype):
    from tokamak_amd.config import get_part

    rot = get_part("position", "rotary_half")(rotary_dim=48, theta=50000.0, dtype=dtype, device=DEV)
    batch = make_batch([(5, 1000, list(range(70))), (1, 0, [70])])
    data = rot.prepare(batch)
    cos, sin = data.cos, data.sin
    assert data.rotary_dim == 48 and data.score_slopes is None
    assert rot.prepare(batch) is data              # once per step, shared by the layers
    positions = torch.tensor([1000, 1001, 1002, 1003, 1004, 0])
    want_cos, want_sin = plain.rope_tables(positions, 48, 50000.0)
    torch.testing.assert_close(cos.cpu(), want_cos[:, :24], rtol=1e-5, atol=2e-6)
    torch.testing.assert_close(sin.cpu(), want_sin[:, :24], rtol=1e-5, atol=2e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("nh, nkv, hd, H, ps", [(6, 2, 32, 80, 8), (8, 2, 128, 96, 16), (5, 5, 48, 64, 16)])
def test_attention_part_whole_and_in_portions(dtype, nh, nkv, hd, H, ps):
    """The mixer alone: one request whole, then the same tokens in portions and a
    final single token, against the plain attention block."""
    from tokamak_amd.config import get_part
    from tokamak_amd.engine.storage import SlotStore

    rot = get_part("position", "rotary_half")(rotary_dim=hd, theta=10000.0, dtype=dtype, device=DEV)
    mixer = get_part("mixer", "gqa_attention")(
        hidden_size=H, num_heads=nh, num_kv_heads=nkv, head_dim=hd, qk_norm_eps=1e-6,
        softmax_scale=hd ** -0.5, window=None, dtype=dtype, device=DEV)
    w = {"a.q_proj.weight": rand(nh * hd, H, seed=1, scale=H ** -0.5), "a.k_proj.weight": rand(nkv * hd, H, seed=2, scale=H ** -0.5),
         "a.v_proj.weight": rand(nkv * hd, H, seed=3, scale=H ** -0.5), "a.o_proj.weight": rand(H, nh * hd, seed=4, scale=(nh * hd) ** -0.5),
         "a.q_norm.weight": 1 + 0.2 * rand(hd, seed=5), "a.k_norm.weight": 1 + 0.2 * rand(hd, seed=6)}
    w = {k: (v.to(dtype).float() if v.dim() == 2 else v) for k, v in w.items()}
    assert set(mixer.expected_tensors("a.")) == set(w)
    mixer.bind("a.", fetcher(w, dtype))
    req = mixer.cache_request()
    assert [(n, a.elems_per_token, a.dtype) for n, a in req.arrays] == [("k", nkv * hd, None), ("v", nkv * hd, None)]
    assert req.window is None and req.bytes_per_token(dtype) == 2 * nkv * hd * (4 if dtype == torch.float32 else 2)
    T = 45
    x = rand(T, H, seed=7).to(dtype)
    s = dict(nh=nh, nkv=nkv, hd=hd, eps=1e-6, theta=10000.0)
    want = plain.attention_block(x.float(), w, "a.", s, torch.arange(T))
    pages = 8
    table = [5, 2, 7, 0, 3, 6][: -(-T // ps)] if ps == 16 else [5, 2, 7, 0, 3, 6]
    for cuts in ([T], [16, 7, 2, 19, 1]):
        store = SlotStore(group=0, page_size=ps, arrays={
            "k": torch.full((pages, nkv * hd * ps), float("nan"), dtype=dtype, device=DEV),
            "v": torch.full((pages, nkv * hd * ps), float("nan"), dtype=dtype, device=DEV)})
        at, outs = 0, []
        for n in cuts:
            batch = make_batch([(n, at, table)])
            delta = mixer.forward(x[at:at + n].to(DEV), batch, store, True, rot.prepare(batch))
            outs.append(delta.sum(0) if delta.dim() == 3 else delta)   # split-K partial sums
            at += n
        torch.testing.assert_close(torch.cat(outs).cpu().float(), want, **TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_embedding_and_head_parts(dtype):
    from tokamak_amd.config import get_part

    V, H = 331, 120
    emb = get_part("embedding", "token_embedding")(vocab_size=V, dim=H, dtype=dtype, device=DEV)
    table = rand(V, H, seed=1).to(dtype).float()
    emb.bind("e.", fetcher({"e.weight": table}, dtype))
    from tokamak_amd.engine.batch import StepSpan, build_batch

    ids = [3, 330, 0, 3]
    batch = build_batch([StepSpan(request=0, tokens=ids, ctx_len=0, state_slot=0, tables=[[0]])], 1, DEV)
    torch.testing.assert_close(emb.forward(batch).cpu(), table[torch.tensor(ids)], rtol=0, atol=0)
    head = get_part("head", "linear_head")(vocab_size=V, dim=H, tied=True, dtype=dtype, device=DEV)
    assert head.expected_tensors("h.")["h.weight"].ignored
    head.tie(emb)
    h = rand(5, H, seed=2).to(dtype)
    logits = head.forward(h.to(DEV))
    assert logits.dtype == torch.float32
    torch.testing.assert_close(logits.cpu(), h.float() @ table.T, rtol=1e-3, atol=1e-3)


# -- sampler -------------------------------------------------------------------
def test_argmax_first_maximum_wins():
    from tokamak_amd.sampling.sampler import greedy_tokens

    logits = torch.tensor([[0.1, 2.0, -1.0], [3.0, 0.0, 0.5]], device=DEV)   # reference test_sampler.py:12-15
    assert greedy_tokens(logits).tolist() == [1, 0]
    big = torch.randn(5, 151936, generator=torch.Generator().manual_seed(0))
    big[2, 77] = big[2, 150000] = 50.0          # a tie: the lower index wins
    assert greedy_tokens(big.to(DEV)).tolist() == big.argmax(-1).tolist()
    assert greedy_tokens(big.to(DEV))[2].item() == 77


@pytest.mark.parametrize("V", [5, 331, 151936])
def test_sampling_distribution_matches_plain(V):
    from tokamak_amd import SamplingParams
    from tokamak_amd.sampling.sampler import sample_tokens

    logits = torch.randn(6, V, generator=torch.Generator().manual_seed(V)) * 3
    params = [SamplingParams(temperature=0.8), SamplingParams(temperature=1.3, top_k=4),
              SamplingParams(temperature=1.0, top_p=0.7), SamplingParams(temperature=0.5, top_k=50, top_p=0.9),
              SamplingParams(temperature=0.0), SamplingParams(temperature=2.0, top_k=1)]
    tokens, probs = sample_tokens(logits.to(DEV), params, [1, 2, 3, 4, 5, 6], [0] * 6, return_probs=True)
    tokens, probs = tokens.cpu(), probs.cpu()
    for i, p in enumerate(params):
        if p.is_greedy:
            assert tokens[i].item() == logits[i].argmax().item()
            continue
        want = plain.sampling_probs(logits[i], p.temperature, p.top_k, p.top_p).float()
        torch.testing.assert_close(probs[i], want, rtol=2e-3, atol=1e-6)
        assert (probs[i] > 0).sum() == (want > 0).sum()
        assert probs[i][tokens[i]] > 0
    assert tokens[5].item() == logits[5].argmax().item()       # top_k = 1 is greedy at any temperature


@pytest.mark.parametrize("V", [20000, 151936])
def test_sampling_thresholds_when_the_logits_are_nearly_all_alike(V):
    """The threshold searches copy the values that may hold a threshold into LDS when they are
    few.  Here they are not: every logit lies in [1, 1.06), one bin of the first level, so the
    searches walk the row at every level; and a row with a few hundred values far above the
    rest, where the copies are used.  Both against the plain distribution."""
    from tokamak_amd import SamplingParams
    from tokamak_amd.sampling.sampler import sample_tokens

    gen = torch.Generator().manual_seed(V)
    alike = 1.0 + 0.06 * torch.rand(3, V, generator=gen)
    peaked = torch.randn(3, V, generator=gen)
    peaked[:, torch.randperm(V, generator=gen)[:300]] += 12.0
    logits = torch.cat([alike, peaked])
    params = [SamplingParams(temperature=1.0, top_k=50), SamplingParams(temperature=0.9, top_p=0.5),
              SamplingParams(temperature=1.1, top_k=9000, top_p=0.97)] * 2
    tokens, probs = sample_tokens(logits.to(DEV), params, list(range(6)), [0] * 6, return_probs=True)
    tokens, probs = tokens.cpu(), probs.cpu()
    for i, p in enumerate(params):
        want = plain.sampling_probs(logits[i], p.temperature, p.top_k, p.top_p).float()
        torch.testing.assert_close(probs[i], want, rtol=2e-3, atol=1e-9)
        assert (probs[i] > 0).sum() == (want > 0).sum()
        assert probs[i][tokens[i]] > 0


def _uniform(seed: int, draw: int) -> float:
    """The sampler's uniform number of (request seed, draws so far): a splitmix64-style mix, its top 24 bits."""
    mask = (1 << 64) - 1
    z = (seed * 0x9E3779B97F4A7C15 + (draw + 1) * 0xBF58476D1CE4E5B9) & mask
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & mask
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & mask
    z ^= z >> 31
    return (z >> 40) / 16777216.0


@pytest.mark.parametrize("V", [331, 1001, 151936])
def test_the_drawn_token_is_where_the_uniform_number_falls_in_index_order(V):
    """The draw is the inverse of the cumulative distribution over the kept tokens in index
    order: with the request's uniform number u, the first token whose cumulative probability
    exceeds u.  Checked against a float64 walk on the host, to the rounding of the float32 sums;
    many seeds, so that targets fall in every part of the row (the first tokens, the last, the
    edges of the chunks the kernel cuts the row into)."""
    from tokamak_amd import SamplingParams
    from tokamak_amd.sampling.sampler import sample_tokens

    rows = 48
    logits = torch.randn(rows, V, generator=torch.Generator().manual_seed(V + 1)) * 2
    logits[1] = 0.0                                     # a uniform row: the target's place is the token's index
    logits[2, : V // 2] = float("-inf")                 # nothing in the first half
    logits[3, V // 3:] = float("-inf")                  # nothing after the first third
    params = [SamplingParams(temperature=1.0) if i % 3 else SamplingParams(temperature=0.7, top_k=V // 2 + 1, top_p=0.95)
              for i in range(rows)]
    seeds = [1000 + 7 * i for i in range(rows)]
    for draw in (0, 1, 2):
        tokens, probs = sample_tokens(logits.to(DEV), params, seeds, [draw] * rows, return_probs=True)
        tokens, probs = tokens.cpu().tolist(), probs.cpu().double()
        for i in range(rows):
            cum = probs[i].cumsum(0)
            u = _uniform(seeds[i], draw) * cum[-1].item()
            t = tokens[i]
            assert probs[i, t] > 0
            assert cum[t] > u - 2e-5 and cum[t] - probs[i, t] <= u + 2e-5, (i, draw, t, u, cum[t].item())
    # the uniform row: token = floor(u V) to the same rounding
    assert abs(tokens[1] - int(_uniform(seeds[1], 2) * V)) <= max(1, V // 20000)


def test_sampling_vectors_and_seeds():
    """Vectors of reference tests/unit/test_sampler.py:26-56."""
    from tokamak_amd import SamplingParams
    from tokamak_amd.sampling.sampler import sample_tokens

    def draws(logits, params, n=200):
        rows = logits.repeat(n, 1).to(DEV)
        return sample_tokens(rows, [params] * n, list(range(n)), [0] * n).cpu().tolist()

    assert set(draws(torch.tensor([[1.0, 2.0, 3.0, 4.0, 5.0]]), SamplingParams(top_k=2))) == {3, 4}
    assert set(draws(torch.tensor([[0.5, 0.3, 0.2]]).log(), SamplingParams(top_p=0.7))) == {0, 1}
    assert set(draws(torch.tensor([[0.9, 0.06, 0.04]]).log(), SamplingParams(top_p=0.05), 50)) == {0}
    logits = torch.randn(1, 1000, generator=torch.Generator().manual_seed(7))
    p = SamplingParams(temperature=0.8, top_p=0.95)
    a = sample_tokens(logits.repeat(4, 1).to(DEV), [p] * 4, [42, 42, 43, 42], [0, 0, 0, 1]).cpu().tolist()
    assert a[0] == a[1]                     # same seed and draw count: same token
    counts = torch.bincount(torch.tensor(draws(torch.tensor([[0.5, 0.3, 0.2]]).log(), SamplingParams(), 4000)), minlength=3)
    torch.testing.assert_close(counts.float() / 4000, torch.tensor([0.5, 0.3, 0.2]), rtol=0, atol=0.03)


def test_sampling_odd_rows():
    """A NaN or -inf logit is never drawn; a row that holds nothing but those keeps
    token 0 like the argmax; a vocabulary that is no multiple of four."""
    from tokamak_amd import SamplingParams
    from tokamak_amd.sampling.sampler import sample_tokens

    V = 1001
    logits = torch.randn(4, V, generator=torch.Generator().manual_seed(3))
    logits[0, ::2] = float("nan")
    logits[1, 1::2] = float("-inf")
    logits[2, :] = float("-inf")
    logits[3, :] = float("nan")
    logits[3, 777] = -5.0
    for params in (SamplingParams(temperature=1.5), SamplingParams(temperature=0.7, top_k=30, top_p=0.9)):
        for draw in range(20):
            t = sample_tokens(logits.to(DEV), [params] * 4, [11, 12, 13, 14], [draw] * 4).cpu().tolist()
            assert t[0] % 2 == 1 and t[1] % 2 == 0 and t[2] == 0 and t[3] == 777
