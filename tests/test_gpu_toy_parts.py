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
    from tokamak_amd.parts.base import FeedForward, Mixer, PositionEncoding
    from tokamak_amd.weights.spec import TensorSpec

    class RunningMeanMixer(Mixer):
        """out[t] = W (mean of h[0..t]): state per request = (sum vector, count)."""

        def __init__(self, *, hidden_size, dtype, device):
            super().__init__(dtype=dtype, device=device)
            self.h = hidden_size
            self.w = None

        def expected_tensors(self, prefix):
            return {prefix + "mix.weight": TensorSpec((self.h, self.h))}

        def bind(self, prefix, fetch):
            self.w = fetch(prefix + "mix.weight")

        def state_shape(self):
            return (self.h + 1,)

        def forward(self, h, batch, store, writes_cache=True):
            out = torch.empty_like(h)
            starts = batch.q_start.tolist()
            slots = batch.state_slots.tolist()
            for i, slot in enumerate(slots):
                x = h[starts[i]:starts[i + 1]].float()
                state = store.state[slot]
                sums = state[: self.h] + torch.cumsum(x, 0)
                counts = state[self.h] + torch.arange(1, x.shape[0] + 1, device=h.device)
                out[starts[i]:starts[i + 1]] = ((sums / counts[:, None]) @ self.w.float().T).to(h.dtype)
                state[: self.h] = sums[-1]
                state[self.h] = counts[-1]
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

        def __init__(self, *, rotary_dim, dtype, device):
            super().__init__(dtype=dtype, device=device)
            self.rotary_dim = rotary_dim

        def prepare(self, batch):
            n = batch.num_tokens
            return (torch.ones(n, self.rotary_dim // 2, device=self.device),
                    torch.zeros(n, self.rotary_dim // 2, device=self.device))

    for family, kind, cls in (("mixer", "toy_running_mean", RunningMeanMixer),
                              ("feed_forward", "toy_top1", Top1RoutedFF),
                              ("position", "toy_none", NoRotation)):
        register_part(family, kind, cls, replace=True)


def toy_plan():
    from tokamak_amd.config import LayerCall, LayerSpec, ModelPlan, PartSpec

    H, V = 64, 100
    norm = PartSpec.of("rmsnorm", dim=H, eps=1e-5)
    rope = PartSpec.of("rotary_half", rotary_dim=16, theta=10000.0)
    none = PartSpec.of("toy_none", rotary_dim=16)

    def attn(position, window=None):
        return PartSpec.of("gqa_attention", hidden_size=H, num_heads=4, num_kv_heads=2, head_dim=16,
                           qk_norm_eps=1e-5, softmax_scale=0.25, position=(position.kind, position.params),
                           window=window)

    swiglu = PartSpec.of("swiglu", hidden_size=H, intermediate_size=96)
    layers = (
        LayerSpec(attn(rope), swiglu, norm, norm),                                   # 0: ordinary
        LayerSpec(PartSpec.of("toy_running_mean", hidden_size=H), PartSpec.of("toy_top1", hidden_size=H), norm, norm),  # 1: state + routing
        LayerSpec(attn(none, window=24), swiglu, norm, norm),                        # 2: window, no rotation
    )
    order = (LayerCall(0, 0), LayerCall(1, 1), LayerCall(2, 2),
             LayerCall(0, 3),                          # layer 0 again, with a cache slot of its own
             LayerCall(0, 0, writes_cache=False))      # and once more, reading what call 0 stored
    return ModelPlan(vocab_size=V, hidden_size=H, max_position_embeddings=512, tie_word_embeddings=True,
                     embedding=PartSpec.of("token_embedding", vocab_size=V, dim=H), layers=layers, order=order,
                     final_norm=norm, head=PartSpec.of("linear_head", vocab_size=V, dim=H, tied=True))


def make_runner(dtype, pool_tokens=256, **kw):
    from tokamak_amd.engine.model import LayeredModel
    from tokamak_amd.engine.runner import ModelRunner
    from tokamak_amd.weights.sources import RandomSource

    register_toys()
    plan = toy_plan()
    expected = {n: s for n, s in LayeredModel(plan, dtype=torch.float32, device="meta").expected_tensors().items() if not s.ignored}
    source = RandomSource(expected, seed=5, matrix_std=0.15, vector_jitter=0.1)
    return ModelRunner(plan, source, dtype=dtype, page_size=8, kv_pool_tokens=pool_tokens, max_requests=4, **kw)


def test_plan_groups_and_state():
    runner = make_runner("float32")
    groups = runner.manager.groups
    assert [(g.spec.name, g.spec.slots, g.spec.window) for g in groups] == [("full", (0, 3), None), ("window24", (2,), 24)]
    assert runner.storage.slot(1).state.shape == (4, 65)       # the toy mixer's per-request state
    assert runner.storage.slot(1).arrays == {}                 # and no pages
    assert set(runner.model.expected_tensors()) >= {"model.layers.1.self_attn.mix.weight", "model.layers.1.mlp.router.weight"}


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
    # the suite's criterion (replay_util.TOL): float32 5e-5; bfloat16 2e-3 + 2% of the logits' scale
    scale = max(float(w.abs().max()) for w in whole.values())
    tol = dict(rtol=0, atol=5e-5) if dtype == "float32" else dict(rtol=0, atol=2e-3 + 2e-2 * scale)
    print(f"toy model {dtype}: logit scale {scale:.2f}, tolerance {tol['atol']:.4f}")
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
