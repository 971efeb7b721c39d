"""The framework takes parts it has never seen: a toy mixer with state of its
own, a toy routed feed-forward and a toy position encoding, defined here,
registered, built into a model with a run order that names a layer twice and
lets a layer read another layer's cache, and stepped under every cutting.  None
of them is a model of anyone's; they show the interfaces of the parts."""

import pytest
import torch

from replay_util import random_ids

pytestmark = pytest.mark.gpu
DEV = "cuda"


def register_toys():
    from tokamak_amd.config import register_part
    from tokamak_amd.parts.base import (Block, CacheRequest, FeedForward, Mixer, PagedArray, PositionData,
                                        PositionEncoding, StateArray, StepPlanner)
    from tokamak_amd.weights.spec import TensorSpec

    class RunningMeanMixer(Mixer):
        """out[t] = W (mean of h[0..t]): two state arrays per request, a float32 sum
        vector and an int32 count."""

        def __init__(self, *, hidden_size, dtype, device):
            super().__init__(dtype=dtype, device=device)
            self.h = hidden_size
            self.w = None

        def expected_tensors(self, prefix):
            return {prefix + "mix.weight": TensorSpec((self.h, self.h))}

        def bind(self, prefix, fetch):
            self.w = fetch(prefix + "mix.weight")

        def state_request(self):
            return {"sum": StateArray((self.h,)), "count": StateArray((1,), torch.int32)}

        def forward(self, h, batch, store, writes_cache=True, position=None):
            out = torch.empty_like(h)
            starts = batch.q_start.tolist()
            slots = batch.state_slots.tolist()
            for i, slot in enumerate(slots):
                x = h[starts[i]:starts[i + 1]].float()
                sums = store.state["sum"][slot] + torch.cumsum(x, 0)
                counts = store.state["count"][slot] + torch.arange(1, x.shape[0] + 1, device=h.device, dtype=torch.int32)
                out[starts[i]:starts[i + 1]] = ((sums / counts[:, None].float()) @ self.w.float().T).to(h.dtype)
                store.state["sum"][slot] = sums[-1]
                store.state["count"][slot] = counts[-1]
            return out

    class LastTokenMixer(Mixer):
        """out[t] = W h[t-1] (zero for a request's first token): the state is the
        previous token's row.  Every request brings one token or the host loop below
        handles a portion; in a one-token step nothing touches the host, so the part
        may be recorded into a graph: a step that ran twice would read its own row."""

        capturable = True

        def __init__(self, *, hidden_size, dtype, device):
            super().__init__(dtype=dtype, device=device)
            self.h = hidden_size
            self.w = None

        def expected_tensors(self, prefix):
            return {prefix + "mix.weight": TensorSpec((self.h, self.h))}

        def bind(self, prefix, fetch):
            self.w = fetch(prefix + "mix.weight")

        def state_request(self):
            return {"last": StateArray((self.h,))}

        def forward(self, h, batch, store, writes_cache=True, position=None):
            state = store.state["last"]
            slots = batch.state_slots.long()
            if batch.max_q_len == 1:                     # one token a request: index math only
                previous = state[slots]
                state[slots] = h.float()
            else:
                previous = torch.empty(h.shape, dtype=torch.float32, device=h.device)
                starts = batch.q_start.tolist()
                for i, slot in enumerate(slots.tolist()):
                    a, b = starts[i], starts[i + 1]
                    previous[a] = state[slot]
                    previous[a + 1:b] = h[a:b - 1].float()
                    state[slot] = h[b - 1].float()
            return (previous @ self.w.float().T).to(h.dtype)

    class TwoWidthCacheMixer(Mixer):
        """out[t] = W_a mean(a[0..t]) + W_b mean(b[0..t]) read back from pages, where a
        (8 numbers a token, compute dtype) and b (3 numbers a token, float32) are cached
        in two arrays of unlike width and dtype."""

        def __init__(self, *, hidden_size, dtype, device):
            super().__init__(dtype=dtype, device=device)
            self.h = hidden_size

        def expected_tensors(self, prefix):
            return {prefix + "a.weight": TensorSpec((8, self.h)), prefix + "b.weight": TensorSpec((3, self.h)),
                    prefix + "out_a.weight": TensorSpec((self.h, 8)), prefix + "out_b.weight": TensorSpec((self.h, 3))}

        def bind(self, prefix, fetch):
            self.wa, self.wb = fetch(prefix + "a.weight"), fetch(prefix + "b.weight")
            self.oa, self.ob = fetch(prefix + "out_a.weight"), fetch(prefix + "out_b.weight")

        def cache_request(self):
            return CacheRequest.of(a=8, b=PagedArray(3, torch.float32))

        def forward(self, h, batch, store, writes_cache=True, position=None):
            ps = store.page_size
            a_pages = store.arrays["a"].view(-1, ps, 8)
            b_pages = store.arrays["b"].view(-1, ps, 3)
            assert store.arrays["b"].dtype == torch.float32 and store.arrays["a"].dtype == h.dtype
            tables = batch.block_tables[store.group].tolist()
            starts = batch.q_start.tolist()
            out = torch.empty_like(h)
            for i, ctx in enumerate(batch.ctx_lens):
                x = h[starts[i]:starts[i + 1]].float()
                a_new, b_new = x @ self.wa.float().T, x @ self.wb.float().T
                for t in range(x.shape[0]):
                    pos = ctx + t
                    a_pages[tables[i][pos // ps], pos % ps] = a_new[t].to(a_pages.dtype)
                    b_pages[tables[i][pos // ps], pos % ps] = b_new[t]
                total = ctx + x.shape[0]
                pages = torch.tensor(tables[i][: -(-total // ps)], device=h.device)
                a_all = a_pages[pages].reshape(-1, 8)[:total].float()
                b_all = b_pages[pages].reshape(-1, 3)[:total]
                counts = torch.arange(1, total + 1, device=h.device)[:, None]
                mean_a = (torch.cumsum(a_all, 0) / counts)[ctx:]
                mean_b = (torch.cumsum(b_all, 0) / counts)[ctx:]
                out[starts[i]:starts[i + 1]] = (mean_a @ self.oa.float().T + mean_b @ self.ob.float().T).to(h.dtype)
            return out

    class ScanChunks(StepPlanner):
        """The cut of a step that the decaying-sum mixer below wants: every span in chunks of up
        to 64 consecutive tokens, each with its request's row, in the order they must run."""

        name = "toy_scan"

        def lists(self, q_lens, ctx_lens):
            first, count, request = [], [], []
            at = 0
            for row, q in enumerate(q_lens):
                for t in range(0, q, SCAN_CHUNK):
                    first.append(at + t)
                    count.append(min(SCAN_CHUNK, q - t))
                    request.append(row)
                at += q
            return ({"first": first, "count": count, "request": request},
                    {"num_chunks": len(first), "longest": max(count, default=0)})

        def bucket(self, facts):
            facts["longest"] = 1 if facts["longest"] <= 1 else SCAN_CHUNK
            return facts

    scan_chunks = ScanChunks()

    class DecayingSumMixer(Mixer):
        """out[t] = W s[t], s[t] = decay * s[t-1] + h[t]: state of fixed size, advanced chunk
        by chunk from a work list of the mixer's own (``batch.lists["toy_scan.*"]``), which the
        step's descriptor carries because ``step_planner`` asks for it.  It refuses pages that
        do not divide its chunk, although it has none: the engine only passes the question on."""

        def __init__(self, *, hidden_size, decay, dtype, device):
            super().__init__(dtype=dtype, device=device)
            self.h, self.decay = hidden_size, float(decay)
            self.w = None

        def expected_tensors(self, prefix):
            return {prefix + "mix.weight": TensorSpec((self.h, self.h), held="float32")}    # a matrix kept in 32-bit

        def bind(self, prefix, fetch):
            self.w = fetch(prefix + "mix.weight")

        def state_request(self):
            return {"s": StateArray((self.h,))}

        def step_planner(self):
            return scan_chunks

        def check_page_size(self, page_size):
            if SCAN_CHUNK % page_size:
                raise ValueError(f"the toy scan's chunks of {SCAN_CHUNK} need a page size that divides them, got {page_size}")

        def forward(self, h, batch, store, writes_cache=True, position=None):
            assert self.w.dtype == torch.float32
            n = batch.facts["toy_scan.num_chunks"]
            first = batch.lists["toy_scan.first"].tolist()
            count = batch.lists["toy_scan.count"].tolist()
            request = batch.lists["toy_scan.request"].tolist()
            assert len(first) == n and sum(count) == batch.num_tokens and max(count) <= batch.facts["toy_scan.longest"]
            slots = batch.state_slots.tolist()
            out = torch.empty_like(h)
            state = store.state["s"]
            for a, c, r in zip(first, count, request):
                # a chunk at once: s[t] = decay^(t+1) s_in + sum_{u<=t} decay^(t-u) h[u]
                x = h[a:a + c].float()
                steps = torch.arange(c, device=h.device, dtype=torch.float32)
                powers = self.decay ** (steps[:, None] - steps[None, :]).clamp(min=0) * (steps[:, None] >= steps[None, :])
                s = powers @ x + (self.decay ** (steps + 1))[:, None] * state[slots[r]][None, :]
                out[a:a + c] = (s @ self.w.T).to(h.dtype)
                state[slots[r]] = s[-1]
            return out

    class Top1RoutedFF(FeedForward):
        """Two experts, each one matrix; a router picks one per token."""

        def __init__(self, *, hidden_size, dtype, device):
            super().__init__(dtype=dtype, device=device)
            self.h = hidden_size

        def expected_tensors(self, prefix):
            return {prefix + "router.weight": TensorSpec((2, self.h)),
                    prefix + "experts.0.weight": TensorSpec((self.h, self.h)),
                    prefix + "experts.1.weight": TensorSpec((self.h, self.h))}

        def bind(self, prefix, fetch):
            self.router = fetch(prefix + "router.weight")
            self.experts = [fetch(prefix + f"experts.{i}.weight") for i in range(2)]

        def forward(self, h, batch):
            choice = (h.float() @ self.router.float().T).argmax(-1)     # router logits in 32-bit
            outs = torch.stack([h.float() @ e.float().T for e in self.experts], 1)
            return outs[torch.arange(h.shape[0]), choice].to(h.dtype)

    class NoRotation(PositionEncoding):
        """cos = 1, sin = 0: attention that ignores positions."""

        capturable = True

        def __init__(self, *, rotary_dim, dtype, device):
            super().__init__(dtype=dtype, device=device)
            self.rotary_dim = rotary_dim

        def prepare(self, batch):
            n = batch.num_tokens
            return PositionData(cos=torch.ones(n, self.rotary_dim // 2, device=self.device),
                                sin=torch.zeros(n, self.rotary_dim // 2, device=self.device),
                                rotary_dim=self.rotary_dim)

    class ScoreSlopes(PositionEncoding):
        """A position encoding of another kind: a slope per head on the scores."""

        def __init__(self, *, heads, dtype, device):
            super().__init__(dtype=dtype, device=device)
            self.heads = heads

        def prepare(self, batch):
            return PositionData(score_slopes=torch.ones(self.heads, device=self.device))

    class SandwichBlock(Block):
        """Four norms a layer: each sub-layer's output is normed again before it joins
        the residual stream.  x += post_a(mixer(pre_a(x))); x += post_f(ff(pre_f(x)))."""

        roles = ("pre_mixer_norm", "mixer", "post_mixer_norm", "pre_ff_norm", "feed_forward", "post_ff_norm")
        optional = ("position",)

        def forward(self, resid, pending, batch, store, writes_cache):
            p = self.parts
            position = p["position"].prepare(batch) if "position" in p else None
            h = p["pre_mixer_norm"].forward(resid, pending)
            out = p["mixer"].forward(h, batch, store, writes_cache, position)
            out = out.sum(0) if out.dim() == 3 else out
            zero = torch.zeros_like(resid)
            normed = p["post_mixer_norm"].forward(zero, out, write_resid=False)   # norm of the sub-layer's output alone
            h = p["pre_ff_norm"].forward(resid, normed)
            out = p["feed_forward"].forward(h, batch)
            out = out.sum(0) if out.dim() == 3 else out
            return p["post_ff_norm"].forward(zero, out, write_resid=False)

    class ParallelBlock(Block):
        """One norm feeds the mixer and the feed-forward side by side:
        x += mixer(n(x)) + ff(n(x))."""

        roles = ("norm", "mixer", "feed_forward")
        optional = ("position",)

        def forward(self, resid, pending, batch, store, writes_cache):
            p = self.parts
            position = p["position"].prepare(batch) if "position" in p else None
            h = p["norm"].forward(resid, pending)
            a = p["mixer"].forward(h, batch, store, writes_cache, position)
            f = p["feed_forward"].forward(h, batch)
            a = a.sum(0) if a.dim() == 3 else a
            f = f.sum(0) if f.dim() == 3 else f
            return a.float() + f.float()

    class MixerOnlyBlock(Block):
        """A layer without a feed-forward: x += mixer(norm(x))."""

        roles = ("norm", "mixer")

        def forward(self, resid, pending, batch, store, writes_cache):
            return self.parts["mixer"].forward(self.parts["norm"].forward(resid, pending), batch, store, writes_cache, None)

    class TwoMixerBlock(Block):
        """Two mixers side by side behind one norm, each with a cache slot of its own:
        x += attend(n(x)) + remember(n(x)).  ``store`` is a dict of slot stores by role."""

        roles = ("norm", "attend", "remember")
        optional = ("position",)

        def forward(self, resid, pending, batch, store, writes_cache):
            p = self.parts
            assert set(store) == {"attend", "remember"} and list(self.mixers) == ["attend", "remember"]
            position = p["position"].prepare(batch) if "position" in p else None
            h = p["norm"].forward(resid, pending)
            a = p["attend"].forward(h, batch, store["attend"], writes_cache, position)
            b = p["remember"].forward(h, batch, store["remember"], writes_cache, None)
            a = a.sum(0) if a.dim() == 3 else a
            return a.float() + b.float()

    for family, kind, cls in (("mixer", "toy_running_mean", RunningMeanMixer),
                              ("mixer", "toy_decaying_sum", DecayingSumMixer),
                              ("block", "toy_two_mixers", TwoMixerBlock),
                              ("mixer", "toy_last_token", LastTokenMixer),
                              ("mixer", "toy_two_width", TwoWidthCacheMixer),
                              ("feed_forward", "toy_top1", Top1RoutedFF),
                              ("position", "toy_none", NoRotation),
                              ("position", "toy_slopes", ScoreSlopes),
                              ("block", "toy_sandwich", SandwichBlock),
                              ("block", "toy_parallel", ParallelBlock),
                              ("block", "toy_mixer_only", MixerOnlyBlock)):
        register_part(family, kind, cls, replace=True)


H, V = 64, 100
SCAN_CHUNK = 64


def _specs():
    from tokamak_amd.config import PartSpec, SubPart

    norm = PartSpec.of("rmsnorm", dim=H, eps=1e-5)
    attn = lambda window=None: PartSpec.of("gqa_attention", hidden_size=H, num_heads=4, num_kv_heads=2, head_dim=16,   # noqa: E731
                                           qk_norm_eps=1e-5, softmax_scale=0.25, window=window)
    return dict(
        norm=norm, attn=attn,
        rope=SubPart("position", PartSpec.of("rotary_half", rotary_dim=16, theta=10000.0), shared=True),
        none=SubPart("position", PartSpec.of("toy_none", rotary_dim=16), shared=True),
        swiglu=SubPart("feed_forward", PartSpec.of("swiglu", hidden_size=H, intermediate_size=96), "mlp."),
        n=lambda prefix: SubPart("norm", norm, prefix),
    )


def _plan(layers, order):
    from tokamak_amd.config import ModelPlan, PartSpec

    norm = PartSpec.of("rmsnorm", dim=H, eps=1e-5)
    return ModelPlan(vocab_size=V, hidden_size=H, max_position_embeddings=512, tie_word_embeddings=True,
                     embedding=PartSpec.of("token_embedding", vocab_size=V, dim=H), layers=tuple(layers),
                     order=tuple(order), final_norm=norm,
                     head=PartSpec.of("linear_head", vocab_size=V, dim=H, tied=True),
                     embedding_prefix="tok.", layer_prefix="blocks.{}.", final_norm_prefix="out_norm.",
                     head_prefix="head.")


def toy_plan():
    from tokamak_amd.config import LayerCall, LayerSpec, PartSpec, SubPart

    s = _specs()

    def pre_norm(mixer, ff, position=None):
        roles = dict(mixer_norm=s["n"]("ln1."), mixer=mixer, feed_forward_norm=s["n"]("ln2."), feed_forward=ff)
        if position is not None:
            roles["position"] = position
        return LayerSpec.of(PartSpec.of("pre_norm"), **roles)

    layers = (
        pre_norm(SubPart("mixer", s["attn"](), "attn."), s["swiglu"], s["rope"]),                  # 0: ordinary
        pre_norm(SubPart("mixer", PartSpec.of("toy_running_mean", hidden_size=H), "mean."),        # 1: state + routing,
                 SubPart("feed_forward", PartSpec.of("toy_top1", hidden_size=H), "moe.")),         #    no position part
        pre_norm(SubPart("mixer", s["attn"](window=24), "attn."), s["swiglu"], s["none"]),         # 2: window, no rotation
    )
    order = (LayerCall(0, 0), LayerCall(1, 1), LayerCall(2, 2),
             LayerCall(0, 3),                          # layer 0 again, with a cache slot of its own
             LayerCall(0, 0, writes_cache=False))      # and once more, reading what call 0 stored
    return _plan(layers, order)


def arrangements_plan():
    """Other arrangements of a layer, none of which the framework has: four norms,
    one norm for two branches, a layer of a mixer only, attention with no position
    part at all, a cache of two unlike arrays."""
    from tokamak_amd.config import LayerCall, LayerSpec, PartSpec, SubPart

    s = _specs()
    layers = (
        LayerSpec.of(PartSpec.of("toy_sandwich"), pre_mixer_norm=s["n"]("n1."), mixer=SubPart("mixer", s["attn"](), "attn."),
                     post_mixer_norm=s["n"]("n2."), pre_ff_norm=s["n"]("n3."), feed_forward=s["swiglu"],
                     post_ff_norm=s["n"]("n4."), position=s["rope"]),
        LayerSpec.of(PartSpec.of("toy_parallel"), norm=s["n"]("n."), mixer=SubPart("mixer", s["attn"](), "attn."),
                     feed_forward=s["swiglu"]),                                                # attention without positions
        LayerSpec.of(PartSpec.of("toy_mixer_only"), norm=s["n"]("n."),
                     mixer=SubPart("mixer", PartSpec.of("toy_two_width", hidden_size=H), "mem.")),
    )
    return _plan(layers, (LayerCall(0, 0), LayerCall(1, 1), LayerCall(2, 2)))


def state_plan():
    """Attention, then a mixer with per-request state that may be recorded into a graph."""
    from tokamak_amd.config import LayerCall, LayerSpec, PartSpec, SubPart

    s = _specs()
    layers = (
        LayerSpec.of(PartSpec.of("pre_norm"), mixer_norm=s["n"]("ln1."), mixer=SubPart("mixer", s["attn"](), "attn."),
                     feed_forward_norm=s["n"]("ln2."), feed_forward=s["swiglu"], position=s["none"]),
        LayerSpec.of(PartSpec.of("pre_norm"), mixer_norm=s["n"]("ln1."),
                     mixer=SubPart("mixer", PartSpec.of("toy_last_token", hidden_size=H), "prev."),
                     feed_forward_norm=s["n"]("ln2."), feed_forward=s["swiglu"]),
    )
    return _plan(layers, (LayerCall(0, 0), LayerCall(1, 1)))


def make_runner(dtype, pool_tokens=256, plan=None, **kw):
    from tokamak_amd.engine.model import LayeredModel
    from tokamak_amd.engine.runner import ModelRunner
    from tokamak_amd.weights.sources import RandomSource

    register_toys()
    plan = plan or toy_plan()
    expected = {n: s for n, s in LayeredModel(plan, dtype=torch.float32, device="meta").expected_tensors().items() if not s.ignored}
    source = RandomSource(expected, seed=5, matrix_std=0.15, vector_jitter=0.1)
    return ModelRunner(plan, source, dtype=dtype, page_size=8, kv_pool_tokens=pool_tokens, max_requests=4, **kw)


def cutting_tolerance(dtype, whole, plan, prompts, continuous=True):
    """How far a request's logits may move when its tokens are cut differently.

    float32: 5e-5, the suite's bound (summation order only).

    bfloat16: kernels differ between cuttings (split-K partial sums, other attention
    tiles), so logits move by rounding.  For a model that is a continuous function of its
    weights, how large bfloat16 rounding is for THIS model is measured, not assumed: the
    distance between the bfloat16 and the float32 logits of the same whole prompts; a
    cutting may move a logit by no more than that.  A model with a hard choice inside (the
    toy router's argmax) is not continuous: bfloat16 and float32 pick other experts for a
    few tokens and their logits differ by the logits' own scale, so that distance measures
    nothing.  There the suite's bound for bfloat16 stands (replay_util.TOL: 2e-3 + 2 % of
    the largest logit): bfloat16 keeps 8 bits, 0.4 % a rounding, and a logit here is the
    end of some twenty rounded products and sums through five layer calls; a wrong page, a
    stale state slot or a skipped token moves logits by their own scale, fifty times as far."""
    if dtype == "float32":
        return dict(rtol=0, atol=5e-5)
    scale = max(float(w.abs().max()) for w in whole.values())
    if not continuous:
        print(f"bfloat16 logit scale {scale:.2f}: cutting bound {2e-3 + 2e-2 * scale:.4f}")
        return dict(rtol=0, atol=2e-3 + 2e-2 * scale)
    exact = make_runner("float32", pool_tokens=256, plan=plan)
    rounding = 0.0
    for rid, toks in prompts.items():
        ref = exact.step([StepEntry_(rid, toks, list(range(len(toks))))]).cpu()
        exact.end(rid)
        rounding = max(rounding, float((whole[rid] - ref).abs().max()))
    print(f"bfloat16 against float32, whole prompts: {rounding:.4f} at a logit scale of {scale:.2f}")
    assert 0 < rounding < 0.05 * scale, "bfloat16 is further from float32 than rounding explains"
    return dict(rtol=0, atol=rounding)


def StepEntry_(*args):
    from tokamak_amd.engine.runner import StepEntry

    return StepEntry(*args)


def test_plan_groups_and_state():
    runner = make_runner("float32")
    groups = runner.manager.groups
    assert [(g.spec.name, g.spec.slots, g.spec.window) for g in groups] == [("full", (0, 3), None), ("window24", (2,), 24)]
    state = runner.storage.slot(1).state                       # the toy mixer's per-request state: two arrays
    assert state["sum"].shape == (4, 64) and state["sum"].dtype == torch.float32
    assert state["count"].shape == (4, 1) and state["count"].dtype == torch.int32
    assert runner.storage.slot(1).arrays == {}                 # and no pages
    assert set(runner.model.expected_tensors()) >= {"blocks.1.mean.mix.weight", "blocks.1.moe.router.weight", "tok.weight"}
    # layers 0 and 2 have unlike encodings, hence unlike position parts; layer 1 has none
    assert runner.model.blocks[0].parts["position"] is not runner.model.blocks[2].parts["position"]
    assert "position" not in runner.model.blocks[1].parts


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_model_is_invariant_under_cutting(dtype):
    """Whole, in portions, and mixed with another request whose pages and state
    slot are reused: the logits of a request do not change (beyond rounding)."""
    from tokamak_amd.engine.runner import StepEntry

    runner = make_runner(dtype, pool_tokens=192)
    a, b, c = (random_ids(100, n, 60 + i) for i, n in enumerate([70, 33, 41]))
    whole = {}
    for rid, toks in (("a", a), ("b", b), ("c", c)):
        whole[rid] = runner.step([StepEntry(rid, toks, list(range(len(toks))))]).cpu()
        runner.end(rid)
    tol = cutting_tolerance(dtype, whole, toy_plan(), {"a": a, "b": b, "c": c}, continuous=False)   # it has a router
    # portions down to two tokens, then single tokens
    got, at = [], 0
    for n in (16, 7, 2, 30, 2, 1, 1, 11):
        got.append(runner.step([StepEntry("a", a[at:at + n], list(range(n)))]).cpu())
        at += n
    runner.end("a")
    torch.testing.assert_close(torch.cat(got), whole["a"], **tol)
    # mixed: b and c interleaved, b ends, a starts in b's pages and state slot
    rows = {"a": [], "b": [], "c": []}
    done = {"a": 0, "b": 0, "c": 0}
    toks = {"a": a, "b": b, "c": c}
    plan = [[("b", 20), ("c", 5)], [("b", 1), ("c", 30)], [("b", 12), ("c", 1)], [("c", 1)], [("c", 4), ("a", 40)],
            [("a", 1)], [("a", 29)]]
    for step in plan:
        entries = [StepEntry(r, toks[r][done[r]:done[r] + n], list(range(n))) for r, n in step]
        out = runner.step(entries).cpu()
        at = 0
        for r, n in step:
            rows[r].append(out[at:at + n])
            at += n
            done[r] += n
            if done[r] == len(toks[r]):
                runner.end(r)
    for r in rows:
        torch.testing.assert_close(torch.cat(rows[r]), whole[r], **tol)
    runner.manager.check()
    assert runner.manager.num_free_pages(0) == runner.manager.num_pages(0)


def test_window_group_returns_pages_while_decoding():
    from tokamak_amd.engine.runner import StepEntry

    runner = make_runner("float32", pool_tokens=256)
    toks = random_ids(100, 120, 3)
    runner.step([StepEntry("w", toks[:100], [99])])
    runner.step([StepEntry("w", toks[100:101], [0])])
    full, windowed = runner.manager.groups
    assert full.live_pages("w") == 13                    # 101 tokens of 8
    assert windowed.live_pages("w") <= 5                 # a window of 24 tokens, plus edges
    assert runner.manager.num_free_pages(1) >= 27


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_other_arrangements_of_a_layer(dtype):
    """Blocks the framework does not have (four norms; one norm for two branches; a
    mixer alone), attention with no position part, and a mixer whose cache has two
    arrays of unlike width and dtype: registered here, built from a plan, loaded with
    full-coverage validation, and invariant under cutting and page reuse."""
    from tokamak_amd.engine.runner import StepEntry

    plan = arrangements_plan()
    runner = make_runner(dtype, pool_tokens=128, plan=plan)
    names = set(runner.model.expected_tensors())
    assert {"blocks.0.n1.weight", "blocks.0.n4.weight", "blocks.1.n.weight", "blocks.2.mem.out_b.weight"} <= names
    arrays = runner.storage.slot(2).arrays
    assert arrays["a"].shape[1] == 8 * 8 and arrays["b"].shape[1] == 3 * 8 and arrays["b"].dtype == torch.float32
    prompts = {"a": random_ids(V, 50, 1), "b": random_ids(V, 37, 2)}
    whole = {}
    for rid, toks in prompts.items():
        whole[rid] = runner.step([StepEntry(rid, toks, list(range(len(toks))))]).cpu()
        runner.end(rid)
    tol = cutting_tolerance(dtype, whole, plan, prompts)
    rows = {"a": [], "b": []}
    done = {"a": 0, "b": 0}
    for step in ([("a", 9)], [("a", 2), ("b", 30)], [("a", 1), ("b", 1)], [("a", 38), ("b", 6)]):
        out = runner.step([StepEntry(r, prompts[r][done[r]:done[r] + n], list(range(n))) for r, n in step]).cpu()
        at = 0
        for r, n in step:
            rows[r].append(out[at:at + n])
            at += n
            done[r] += n
    for r in rows:
        torch.testing.assert_close(torch.cat(rows[r]), whole[r], **tol)


def test_attention_refuses_position_data_it_has_no_kernel_for():
    from tokamak_amd.config import LayerCall, LayerSpec, PartSpec, SubPart
    from tokamak_amd.engine.runner import StepEntry
    from tokamak_amd.kernels.ops import KernelError

    register_toys()
    s = _specs()
    layer = LayerSpec.of(PartSpec.of("pre_norm"), mixer_norm=s["n"]("ln1."), mixer=SubPart("mixer", s["attn"](), "attn."),
                         feed_forward_norm=s["n"]("ln2."), feed_forward=s["swiglu"],
                         position=SubPart("position", PartSpec.of("toy_slopes", heads=4), shared=True))
    runner = make_runner("float32", plan=_plan([layer], [LayerCall(0, 0)]))
    with pytest.raises(KernelError, match="bias on the scores"):
        runner.step([StepEntry("x", [1, 2, 3], [2])])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_state_mixer_recorded_into_a_graph_sees_every_token_once(dtype):
    """The step that meets a new decode shape runs eagerly and is recorded without
    running again; a mixer whose state is the previous token's row would otherwise read
    its own row on that step.  Captured and eager runners must agree bit for bit."""
    from tokamak_amd.engine.runner import StepEntry

    graphed = make_runner(dtype, plan=state_plan(), use_graphs=True)
    eager = make_runner(dtype, plan=state_plan(), use_graphs=False)
    assert graphed.use_graphs and not eager.use_graphs
    prompts = {"a": random_ids(V, 11, 5), "b": random_ids(V, 3, 6)}
    last = {}
    for rid, toks in prompts.items():
        x = graphed.step([StepEntry(rid, toks, [len(toks) - 1])])
        y = eager.step([StepEntry(rid, toks, [len(toks) - 1])])
        assert torch.equal(x, y)
        last[rid] = int(x.argmax())
    for i in range(12):
        if i == 6:                           # a request ends: another batch size, a second shape
            graphed.end("b")
            eager.end("b")
            del last["b"]
        entries = [StepEntry(r, [t], [0]) for r, t in last.items()]
        x = graphed.step(entries).clone()
        y = eager.step(entries)
        assert torch.equal(x, y), f"decode step {i} differs"
        for row, r in enumerate(list(last)):
            last[r] = int(x[row].argmax())
    assert len(graphed._graphs) == 2
    assert sum(g.replays for g in graphed._graphs.values()) == 12 - 2     # each shape's first step ran eagerly


def scan_plan():
    """A mixer with a work list of its own, alone in a layer; then a layer with two mixers
    side by side (attention with pages, the scan with state), a cache slot each."""
    from tokamak_amd.config import LayerCall, LayerSpec, PartSpec, SubPart

    s = _specs()
    scan = lambda prefix: SubPart("mixer", PartSpec.of("toy_decaying_sum", hidden_size=H, decay=0.9), prefix)   # noqa: E731
    layers = (
        LayerSpec.of(PartSpec.of("toy_mixer_only"), norm=s["n"]("n."), mixer=scan("scan.")),
        LayerSpec.of(PartSpec.of("toy_two_mixers"), norm=s["n"]("n."), attend=SubPart("mixer", s["attn"](), "attn."),
                     remember=scan("scan."), position=s["rope"]),
    )
    return _plan(layers, (LayerCall(0, 0), LayerCall(1, (1, 2))))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_mixer_brings_its_own_work_lists_and_a_layer_holds_two_mixers(dtype):
    """The decaying-sum mixer consumes chunks of 64 tokens from lists that its own planner
    makes; the step descriptor carries them beside the attention kernels' lists without the
    engine knowing either.  The second layer has two mixers, each with its own cache slot.
    Logits are those of the formula computed here on whole sequences, under every cutting."""
    from tokamak_amd.engine.runner import StepEntry

    plan = scan_plan()
    runner = make_runner(dtype, pool_tokens=512, plan=plan)
    assert [p.name for p in runner.model.step_planners()] == ["toy_scan", "attention"]
    groups, layouts = runner.model.cache_layout()
    assert sorted(layouts) == [1] and [n for n, _ in layouts[1].request.arrays] == ["k", "v"]
    assert sorted(runner.model.state_requests()) == [0, 2]          # the two scans' state, a slot each
    assert runner.storage.slot(0).state["s"].data_ptr() != runner.storage.slot(2).state["s"].data_ptr()
    assert runner.model.blocks[0].mixer is not None and runner.model.blocks[1].mixer is None
    assert list(runner.model.blocks[1].mixers) == ["attend", "remember"]

    prompts = {"a": random_ids(V, 150, 21), "b": random_ids(V, 70, 22)}
    whole = {}
    for rid, toks in prompts.items():
        whole[rid] = runner.step([StepEntry(rid, toks, list(range(len(toks))))]).cpu()
        runner.end(rid)

    if dtype == "float32":
        # the first layer's formula, written out: s[t] = 0.9 s[t-1] + n(x)[t]; x += W s
        model = runner.model
        x = model.embedding.weight.float()[torch.tensor(prompts["a"], device=DEV)]
        gamma = model.blocks[0].parts["norm"].weight.float()
        n = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + 1e-5) * gamma
        s = torch.zeros(H, device=DEV, dtype=torch.float64)
        rows = []
        for t in range(n.shape[0]):
            s = 0.9 * s + n[t].double()
            rows.append(s)
        after_first = x.double() + torch.stack(rows) @ model.blocks[0].mixer.w.double().T
        # ... which is what the second layer's norm reads: compare through a model of the first layer alone
        first_only = make_runner(dtype, pool_tokens=512, plan=_plan(plan.layers[:1], plan.order[:1]))
        got = first_only.step([StepEntry("a", prompts["a"], list(range(150)))])
        gamma_out = first_only.model.final_norm.weight.double()
        y = after_first * torch.rsqrt((after_first * after_first).mean(-1, keepdim=True) + 1e-5) * gamma_out
        want = y @ first_only.model.head.weight.double().T
        torch.testing.assert_close(got.double(), want, rtol=0, atol=2e-4)

    tol = cutting_tolerance(dtype, whole, plan, prompts)
    # cut at and off the chunk's edges, beside the other request, then token by token
    rows = {"a": [], "b": []}
    done = {"a": 0, "b": 0}
    steps = ([("a", 64)], [("a", 2), ("b", 65)], [("a", 70), ("b", 1)], [("a", 1), ("b", 1)], [("a", 13), ("b", 3)])
    for step in steps:
        batch_entries = [StepEntry(r, prompts[r][done[r]:done[r] + n], list(range(n))) for r, n in step]
        out = runner.step(batch_entries).cpu()
        at = 0
        for r, n in step:
            rows[r].append(out[at:at + n])
            at += n
            done[r] += n
    assert done == {"a": 150, "b": 70}
    for r in rows:
        torch.testing.assert_close(torch.cat(rows[r]), whole[r], **tol)
    runner.end_all()
    runner.manager.check()


def test_a_part_may_refuse_a_page_size():
    """The engine asks every part whether it can work with the cache's page size; it has no
    rule of its own."""
    from tokamak_amd.engine.model import LayeredModel
    from tokamak_amd.engine.runner import ModelRunner
    from tokamak_amd.weights.sources import RandomSource

    register_toys()
    plan = scan_plan()
    expected = {n: s for n, s in LayeredModel(plan, dtype=torch.float32, device="meta").expected_tensors().items() if not s.ignored}
    source = RandomSource(expected, seed=5)
    with pytest.raises(ValueError, match="toy scan's chunks"):
        ModelRunner(plan, source, dtype="float32", page_size=24, kv_pool_tokens=96, max_requests=2)
    with pytest.raises(ValueError, match="attention kernels"):
        ModelRunner(plan, source, dtype="float32", page_size=4, kv_pool_tokens=96, max_requests=2)


# ---------------------------------------------------------------------------
# a whole toy architecture: config.json keys of its own -> registry -> folder -> LLM -> command line
# ---------------------------------------------------------------------------
def register_toy_architecture():
    """An architecture defined in this file: its own config.json keys and tensor names, a state
    mixer between two attention layers (one windowed), a routed feed-forward.  Nothing under
    tokamak_amd/ knows it."""
    from dataclasses import dataclass

    from tokamak_amd.config import LayerCall, LayerSpec, ModelPlan, PartSpec, SubPart
    from tokamak_amd.config.registry import Architecture, register_architecture

    register_toys()
    name = "ToyMemoryForCausalLM"

    @dataclass(frozen=True)
    class ToyConfig:
        architecture: str
        vocab: int
        width: int
        heads: int
        kv_heads: int
        head_size: int
        inner: int
        window: int
        eps: float
        longest: int
        eos_token_ids: tuple = ()

    def parse(raw, eos_ids=()):
        if raw.get("toy_memory_layers", 1) != 1:
            raise ValueError("this toy has one memory layer")
        return ToyConfig(name, int(raw["toy_vocab"]), int(raw["toy_width"]), int(raw["toy_heads"]), int(raw["toy_kv_heads"]),
                         int(raw["toy_head_size"]), int(raw["toy_inner"]), int(raw["toy_window"]),
                         float(raw["toy_eps"]), int(raw["toy_longest"]), tuple(eos_ids))

    def to_json(cfg):
        return {"architectures": [name], "toy_vocab": cfg.vocab, "toy_width": cfg.width, "toy_heads": cfg.heads,
                "toy_kv_heads": cfg.kv_heads, "toy_head_size": cfg.head_size, "toy_inner": cfg.inner,
                "toy_window": cfg.window, "toy_eps": cfg.eps, "toy_longest": cfg.longest}

    def plan(cfg):
        norm = PartSpec.of("rmsnorm", dim=cfg.width, eps=cfg.eps)
        n = lambda prefix: SubPart("norm", norm, prefix)   # noqa: E731
        attn = lambda window: SubPart("mixer", PartSpec.of(   # noqa: E731
            "gqa_attention", hidden_size=cfg.width, num_heads=cfg.heads, num_kv_heads=cfg.kv_heads, head_dim=cfg.head_size,
            qk_norm_eps=cfg.eps, softmax_scale=cfg.head_size ** -0.5, window=window), "attend.")
        rope = SubPart("position", PartSpec.of("rotary_half", rotary_dim=cfg.head_size, theta=5000.0), shared=True)
        dense = SubPart("feed_forward", PartSpec.of("swiglu", hidden_size=cfg.width, intermediate_size=cfg.inner), "ff.")
        routed = SubPart("feed_forward", PartSpec.of("toy_top1", hidden_size=cfg.width), "experts.")
        layers = (
            LayerSpec.of(PartSpec.of("pre_norm"), mixer_norm=n("a."), mixer=attn(None), feed_forward_norm=n("b."),
                         feed_forward=dense, position=rope),
            LayerSpec.of(PartSpec.of("pre_norm"), mixer_norm=n("a."),
                         mixer=SubPart("mixer", PartSpec.of("toy_running_mean", hidden_size=cfg.width), "memory."),
                         feed_forward_norm=n("b."), feed_forward=routed),
            LayerSpec.of(PartSpec.of("pre_norm"), mixer_norm=n("a."), mixer=attn(cfg.window), feed_forward_norm=n("b."),
                         feed_forward=dense, position=rope),
        )
        return ModelPlan(vocab_size=cfg.vocab, hidden_size=cfg.width, max_position_embeddings=cfg.longest,
                         tie_word_embeddings=False, embedding=PartSpec.of("token_embedding", vocab_size=cfg.vocab, dim=cfg.width),
                         layers=layers, order=(LayerCall(0, 0), LayerCall(1, 1), LayerCall(2, 2)), final_norm=norm,
                         head=PartSpec.of("linear_head", vocab_size=cfg.vocab, dim=cfg.width, tied=False),
                         embedding_prefix="words.", layer_prefix="stack.{}.", final_norm_prefix="last.", head_prefix="out.",
                         eos_token_ids=cfg.eos_token_ids)

    presets = {"toy-memory": ToyConfig(name, 90, 48, 3, 1, 16, 80, 24, 1e-5, 160)}
    register_architecture(Architecture(name=name, parse=parse, plan=plan, to_json=to_json, presets=presets), replace=True)
    return presets["toy-memory"]


def test_a_toy_architecture_goes_from_config_json_to_generated_tokens(tmp_path, capsys):
    """Registered from here, the toy is found by the name in its folder's config.json, its weights
    are bound by its own tensor names (and a missing one is reported), it generates the same tokens
    with a roomy pool and whole prompts as with a tight pool and prompts in portions, and the command
    line finds its preset."""
    from safetensors import safe_open
    from safetensors.torch import save_file

    from tokamak_amd import LLM, SamplingParams, cli
    from tokamak_amd.config import find_preset
    from tokamak_amd.weights import write_random_model
    from tokamak_amd.weights.loader import WeightError

    cfg = register_toy_architecture()
    assert find_preset("toy-memory")[1] == cfg
    folder = write_random_model(tmp_path / "toy", cfg, seed=4, matrix_std=0.15, vector_jitter=0.1)
    with safe_open(str(folder / "model.safetensors"), framework="pt") as f:
        names = set(f.keys())
        tensors = {k: f.get_tensor(k) for k in names}
    assert {"words.weight", "out.weight", "last.weight", "stack.1.memory.mix.weight", "stack.1.experts.router.weight",
            "stack.2.attend.q_proj.weight"} <= names

    params = SamplingParams(temperature=0.0, max_new_tokens=40, ignore_eos=True)
    prompts = [random_ids(cfg.vocab, n, 70 + i) for i, n in enumerate([40, 9, 75, 3, 28])]
    roomy = LLM(folder, dtype="float32", block_size=8, max_batch_size=8)
    assert roomy.architecture.name == "ToyMemoryForCausalLM" and roomy.max_seq_len == 160
    want = roomy.generate(prompt_token_ids=prompts, sampling_params=params)
    tight = LLM(folder, dtype="float32", block_size=8, kv_pool_tokens=160, max_batch_size=4, max_num_batched_tokens=16,
                prefill_chunk=7)
    got = tight.generate(prompt_token_ids=prompts, sampling_params=params)
    assert [o.output_token_ids for o in got] == [o.output_token_ids for o in want]
    assert tight.num_preemptions > 0
    tight.runner.manager.check()
    half = LLM(folder, dtype="bfloat16", block_size=8, max_batch_size=8).generate(prompt_token_ids=prompts, sampling_params=params)
    assert all(len(o.output_token_ids) == 40 for o in half)
    # every bfloat16 token is the float32 model's best token for the sequence so far, or one whose
    # float32 logit lies within bfloat16 rounding of the best (twice the replay tests' bound)
    from tokamak_amd.engine.runner import StepEntry

    best = 0
    for prompt, out in zip(prompts, half):
        tokens = out.output_token_ids
        rows = roomy.runner.step([StepEntry("check", prompt + tokens[:-1], list(range(len(prompt) - 1, len(prompt) + 39)))])
        roomy.runner.end("check")
        for i, token in enumerate(tokens):
            slack = 2 * (2e-3 + 2e-2 * float(rows[i].abs().max()))
            assert float(rows[i, token]) >= float(rows[i].max()) - slack, f"bfloat16 token {i} of a {len(prompt)}-token prompt"
            best += int(token == int(rows[i].argmax()))
    assert best >= 0.9 * 40 * len(prompts)

    broken = tmp_path / "broken"
    broken.mkdir()
    (broken / "config.json").write_text((folder / "config.json").read_text())
    del tensors["stack.1.memory.mix.weight"]
    save_file(tensors, str(broken / "model.safetensors"))
    with pytest.raises(WeightError, match="stack.1.memory.mix.weight"):
        LLM(broken, dtype="float32", block_size=8)

    assert cli.main(["--random-weights", "toy-memory", "--prompt-ids", "5,6,7", "--max-new-tokens", "4", "--temperature", "0",
                     "--dtype", "float32", "--page-size", "8", "--quiet"]) == 0
    assert "[completion (length)]" in capsys.readouterr().out
