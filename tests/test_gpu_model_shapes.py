"""Layers of Qwen3-8B's shape (width 4096, 32 query and 8 kv heads of 128, feed-forward
12288; two layers and a vocabulary of 8192 to keep it small), of Qwen3-32B's (width 5120,
64 query heads in groups of 8, feed-forward 25600; one layer), of Qwen3-0.6B's (width
1024, 16 query heads in groups of 2, tied embeddings) and of Qwen3-14B's (40 query heads in
groups of 5, feed-forward 17408; one layer): float32 and bfloat16 logits
against the plain implementation, whole, in portions and token by token, and mixed
with a second request."""

import dataclasses

import pytest
import torch

import plain_qwen3 as plain
from replay_util import random_ids
from tokamak_amd.models import qwen3

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", params=[("qwen3-8b", 2), ("qwen3-32b", 1), ("qwen3-0.6b", 2), ("qwen3-14b", 1)],
                ids=["8b", "32b", "0.6b", "14b"])
def model(request):
    from tokamak_amd.weights.random_init import expected_tensors_of
    from tokamak_amd.weights.sources import RandomSource

    preset, layers = request.param
    cfg = dataclasses.replace(qwen3.PRESETS[preset], num_layers=layers, vocab_size=8192, max_position_embeddings=4096)
    plan = qwen3.plan(cfg)
    expected = {n: s for n, s in expected_tensors_of(plan).items() if not s.ignored}
    source = RandomSource(expected, seed=3, matrix_std=0.02, vector_jitter=0.1, dtype=torch.bfloat16)
    weights = {name: source.fetch(name) for name in expected}

    class Fixed:
        def names(self):
            return {n: (tuple(t.shape), t.dtype) for n, t in weights.items()}

        def fetch(self, name):
            return weights[name]

    return cfg, plan, Fixed(), {n: t.float() for n, t in weights.items()}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_full_width_layers_match_plain_under_every_cutting(model, dtype):
    from tokamak_amd.engine.runner import ModelRunner, StepEntry

    cfg, plan, source, w = model
    cfg_json = qwen3.to_config_json(cfg)
    a = random_ids(cfg.vocab_size, 150, 1)
    b = random_ids(cfg.vocab_size, 40, 2)
    want_a = plain.logits(a, cfg_json, w)
    want_b = plain.logits(b, cfg_json, w)
    scale = float(want_a.abs().max())
    tol = 5e-5 if dtype == "float32" else 2e-3 + 2e-2 * scale
    runner = ModelRunner(plan, source, dtype=dtype, page_size=16, kv_pool_tokens=512, max_requests=4)

    whole = runner.step([StepEntry("a", a, list(range(len(a))))]).cpu()
    runner.end("a")
    err = (whole - want_a).abs().max().item()
    print(f"{dtype}: logit scale {scale:.3f}; whole {err:.2e}", end="")
    assert err < tol

    # most of it in one step, the last 32 tokens one by one (replayed decode graph in bf16 and fp32)
    rows = [runner.step([StepEntry("a", a[:118], list(range(118)))]).cpu()]
    for t in a[118:]:
        rows.append(runner.step([StepEntry("a", [t], [0])]).cpu().clone())
    runner.end("a")
    err = (torch.cat(rows) - want_a).abs().max().item()
    print(f"; tail one by one {err:.2e}", end="")
    assert err < tol

    # portions of changing size, mixed with the other request
    got_a, got_b, ia, ib = [], [], 0, 0
    for na, nb in [(64, 3), (17, 1), (2, 20), (50, 1), (1, 1), (16, 14)]:
        entries = []
        if na and ia < len(a):
            entries.append(StepEntry("a", a[ia:ia + na], list(range(len(a[ia:ia + na])))))
        if nb and ib < len(b):
            entries.append(StepEntry("b", b[ib:ib + nb], list(range(len(b[ib:ib + nb])))))
        out = runner.step(entries).cpu()
        at = 0
        if na and ia < len(a):
            n = len(a[ia:ia + na]); got_a.append(out[at:at + n]); at += n; ia += n
        if nb and ib < len(b):
            n = len(b[ib:ib + nb]); got_b.append(out[at:at + n]); at += n; ib += n
    assert ia == len(a) and ib == len(b)
    err = max((torch.cat(got_a) - want_a).abs().max().item(), (torch.cat(got_b) - want_b).abs().max().item())
    print(f"; mixed portions {err:.2e}")
    assert err < tol
