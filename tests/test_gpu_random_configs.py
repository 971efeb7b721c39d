"""Configurations drawn at random, every size of its own kind: head sizes in steps of 16
from 16 to 256, any number of heads and groups, widths, feed-forward sizes and vocabularies
that are no multiple of anything, one to three layers, tied or not, pages of 8 to 64 tokens.
Each is written as a model folder and replayed mixed (up to four live requests, portions
beside decoded tokens, a pool with no page to spare) against the plain implementation, in
32-bit and in bfloat16.  A size that a kernel does not take has to be refused by the host
with a KernelError, never computed wrongly; none of these is refused."""

import random

import pytest

import plain_qwen3 as plain
from replay_util import TOL, compare, mixed
from tokamak_amd.models.qwen3 import Qwen3Config

pytestmark = pytest.mark.gpu


def drawn(seed):
    rng = random.Random(10_000 + seed)
    head_dim = rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 144, 160, 192, 256])
    kv_heads = rng.choice([1, 1, 2, 3, 4, 5, 8])
    groups = rng.choice([1, 1, 2, 3, 4, 5, 7, 8])
    hidden = rng.choice([rng.randrange(24, 400), 8 * rng.randrange(4, 64), 64, 128, 256])
    inter = rng.choice([rng.randrange(24, 600), 8 * rng.randrange(4, 90), 256])
    vocab = rng.choice([rng.randrange(40, 1200), 257, 1000, 1024])
    cfg = Qwen3Config("Qwen3ForCausalLM", vocab_size=vocab, hidden_size=hidden, num_layers=rng.randint(1, 3),
                      num_attention_heads=kv_heads * groups, num_kv_heads=kv_heads, head_dim=head_dim,
                      intermediate_size=inter, rms_norm_eps=rng.choice([1e-6, 1e-5, 3e-4]),
                      rope_theta=rng.choice([1e4, 5e4, 1e6]), max_position_embeddings=1024,
                      tie_word_embeddings=rng.random() < 0.5)
    page_size = rng.choice([8, 16, 32, 64])
    lengths = [rng.choice([1, 2, 17, 40, 70, 130, 200]) + rng.randint(0, 15) for _ in range(rng.randint(2, 5))]
    requests = {f"r{i}": [rng.randrange(vocab) for _ in range(n)] for i, n in enumerate(lengths)}
    return cfg, page_size, requests, rng.choice([0, 3, 6, 20])


@pytest.mark.parametrize("first", range(0, 48, 8))
def test_random_configurations_replayed_mixed_match_plain(tmp_path, first):
    from tokamak_amd.engine.runner import ModelRunner, StepEntry
    from tokamak_amd.weights import write_random_model

    for seed in range(first, first + 8):
        cfg, page_size, requests, tail = drawn(seed)
        what = (f"seed {seed}: width {cfg.hidden_size}, heads {cfg.num_attention_heads}/{cfg.num_kv_heads} of "
                f"{cfg.head_dim}, feed-forward {cfg.intermediate_size}, vocabulary {cfg.vocab_size}, "
                f"{cfg.num_layers} layers, pages of {page_size}")
        folder = write_random_model(tmp_path / f"m{seed}", cfg, seed, matrix_std=0.05, vector_jitter=0.1)
        cfg_json, w = plain.read_folder(folder)
        expected = {rid: plain.logits(toks, cfg_json, w).numpy() for rid, toks in requests.items()}
        steps, peak = mixed(requests, seed, max_live=4, tail=tail)
        for dtype in ("float32", "bfloat16"):
            runner = ModelRunner.from_folder(folder, dtype=dtype, page_size=page_size,
                                             kv_pool_tokens=max(peak, 64), max_requests=4)
            got = {}
            for rec in steps:
                out = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in rec["entries"]])
                if out.shape[0]:
                    got[rec["step"]] = out.cpu().numpy().copy()
                for rid in rec["end"]:
                    runner.end(rid)
            runner.manager.check()
            try:
                compare(steps, got, expected, **TOL[dtype])
            except AssertionError as e:
                raise AssertionError(f"{what}, {dtype}: {e}") from None
            del runner


def drawn_wide(seed):
    """Sizes at which the weight-streaming products, their split plans and the matrix-core
    attention kernels run: widths of 256 to 5,600 in steps of 8, feed-forwards up to 26,000,
    batches of 1 to 64 requests."""
    rng = random.Random(77_000 + seed)
    head_dim = rng.choice([64, 128, 128, 96, 256, 80])
    kv_heads = rng.choice([1, 2, 4, 8])
    groups = rng.choice([1, 2, 3, 4, 5, 6, 7, 8])
    hidden = rng.choice([8 * rng.randrange(32, 700), 256 * rng.randrange(2, 22), 128 * rng.randrange(4, 44)])
    inter = rng.choice([8 * rng.randrange(64, 3300), 256 * rng.randrange(4, 100), 128 * rng.randrange(8, 200)])
    vocab = rng.choice([rng.randrange(1000, 20000), 8192, 16 * rng.randrange(100, 1200)])
    cfg = Qwen3Config("Qwen3ForCausalLM", vocab_size=vocab, hidden_size=hidden, num_layers=rng.randint(1, 2),
                      num_attention_heads=kv_heads * groups, num_kv_heads=kv_heads, head_dim=head_dim,
                      intermediate_size=inter, rms_norm_eps=1e-6, rope_theta=1e6, max_position_embeddings=4096,
                      tie_word_embeddings=rng.random() < 0.5)
    batch = rng.choice([1, 2, 3, 5, 8, 9, 16, 17, 24, 32, 33, 40, 48, 49, 64])
    prompts = [[rng.randrange(vocab) for _ in range(rng.randint(3, 40))] for _ in range(batch)]
    fed = [[rng.randrange(vocab) for _ in range(3)] for _ in range(batch)]
    return cfg, prompts, fed, sorted(rng.sample(range(batch), min(batch, 3)))


@pytest.mark.parametrize("seed", [0, 1, 2, 3, 5, 8, 13, 21])
def test_random_wide_configurations_prefilled_together_and_decoded_match_plain(seed):
    """All prompts in one step, then three decode steps of the whole batch; three of the
    requests are compared with the plain implementation at every step."""
    import torch

    from tokamak_amd.engine.runner import ModelRunner, StepEntry
    from tokamak_amd.models import qwen3
    from tokamak_amd.weights.random_init import expected_tensors_of
    from tokamak_amd.weights.sources import RandomSource

    cfg, prompts, fed, checked = drawn_wide(seed)
    what = (f"seed {seed}: width {cfg.hidden_size}, heads {cfg.num_attention_heads}/{cfg.num_kv_heads} of "
            f"{cfg.head_dim}, feed-forward {cfg.intermediate_size}, vocabulary {cfg.vocab_size}, "
            f"{cfg.num_layers} layers, batch {len(prompts)}")
    plan = qwen3.plan(cfg)
    expected = {n: s for n, s in expected_tensors_of(plan).items() if not s.ignored}
    source = RandomSource(expected, seed=seed, matrix_std=0.02, vector_jitter=0.1, dtype=torch.bfloat16)
    weights = {name: source.fetch(name) for name in expected}

    class Fixed:
        def names(self):
            return {n: (tuple(t.shape), t.dtype) for n, t in weights.items()}

        def fetch(self, name):
            return weights[name]

    cfg_json = qwen3.to_config_json(cfg)
    w = {n: t.float() for n, t in weights.items()}
    want = {i: plain.logits(prompts[i] + fed[i], cfg_json, w) for i in checked}
    for dtype in ("float32", "bfloat16"):
        runner = ModelRunner(plan, Fixed(), dtype=dtype, page_size=16, kv_pool_tokens=64 * 80, max_requests=64)
        steps = [[StepEntry(f"r{i}", p, [len(p) - 1]) for i, p in enumerate(prompts)]]
        steps += [[StepEntry(f"r{i}", [f[t]], [0]) for i, f in enumerate(fed)] for t in range(3)]
        for t, entries in enumerate(steps):
            out = runner.step(entries).cpu()
            for i in checked:
                row = want[i][len(prompts[i]) - 1 + t]
                tol = TOL[dtype]["tol_abs"] + TOL[dtype].get("tol_rel_to_scale", 0.0) * float(row.abs().max())
                err = (out[i] - row).abs().max().item()
                assert err < tol, f"{what}, {dtype}, step {t}, request {i}: {err:.3e} > {tol:.3e}"
        for i in range(len(prompts)):
            runner.end(f"r{i}")
        runner.manager.check()
        del runner
