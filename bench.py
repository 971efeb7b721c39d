"""Decode and prefill throughput of a Qwen3-8B-shaped model with random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 4096] [--layers 36]

Prints one JSON line.  A "step" is one decode step of the whole batch through
the engine's own step function and greedy sampler, each request holding
``context`` tokens at the end of the timed steps.  ``value`` is decoded tokens
per second.  ``prefill`` is one 2,048-token prompt in one step; ``roofline``
prices the decode step against HBM: every weight it uses once plus the cache of
the live requests, divided by its time.  Peaks: HBM 8 TB/s, dense bf16 MFMA
2.5 PFLOP/s (MI355X, published).
"""

from __future__ import annotations

import argparse
import dataclasses
import json
import statistics
import sys
import time
from pathlib import Path

sys.path.insert(0, str(Path(__file__).resolve().parent))

HBM_PEAK = 8.0e12
MFMA_PEAK = {"bf16": 2.5e15, "fp16": 2.5e15, "fp8": 5.0e15, "fp32": 157.3e12}
PREFILL_TOKENS = 2048
SHAPE_NAMES = {"qwen3-0.6b": "Qwen3-0.6B", "qwen3-8b": "Qwen3-8B", "qwen3-32b": "Qwen3-32B"}


def make_runner(cfg, dtype, pool_tokens, max_requests, seed=0):
    import torch

    from tokamak_amd.engine.runner import ModelRunner
    from tokamak_amd.config import get_architecture
    from tokamak_amd.weights.random_init import expected_tensors_of
    from tokamak_amd.weights.sources import RandomSource

    plan = get_architecture(cfg.architecture).plan(cfg)
    expected = {n: s for n, s in expected_tensors_of(plan).items() if not s.ignored}
    tdt = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    source = RandomSource(expected, seed, matrix_std=0.02, vector_jitter=0.0, dtype=tdt, device="cuda:0")
    return ModelRunner(plan, source, dtype=dtype, page_size=16, kv_pool_tokens=pool_tokens,
                       max_requests=max_requests)


def weight_bytes(cfg, elem):
    per_layer = ((cfg.num_attention_heads + 2 * cfg.num_kv_heads) * cfg.head_dim * cfg.hidden_size
                 + cfg.hidden_size * cfg.num_attention_heads * cfg.head_dim
                 + 3 * cfg.hidden_size * cfg.intermediate_size)
    return (per_layer * cfg.num_layers + cfg.vocab_size * cfg.hidden_size) * elem


def kv_bytes_per_token(cfg, elem):
    return 2 * cfg.num_layers * cfg.num_kv_heads * cfg.head_dim * elem


def prefill_flops(cfg, t):
    per_layer = ((cfg.num_attention_heads + 2 * cfg.num_kv_heads) * cfg.head_dim * cfg.hidden_size
                 + cfg.hidden_size * cfg.num_attention_heads * cfg.head_dim
                 + 3 * cfg.hidden_size * cfg.intermediate_size)
    linear = 2.0 * t * per_layer * cfg.num_layers
    attention = 4.0 * cfg.num_attention_heads * cfg.head_dim * (t * (t + 1) / 2) * cfg.num_layers
    head = 2.0 * cfg.vocab_size * cfg.hidden_size
    return linear + attention + head


def random_prompt(vocab, n, seed):
    import torch

    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def fill(runner, request, tokens, chunk=2048):
    """Put ``tokens`` into the cache in portions; return the logits row of the last one."""
    from tokamak_amd.engine.runner import StepEntry

    logits = None
    for at in range(0, len(tokens), chunk):
        part = tokens[at:at + chunk]
        last = at + chunk >= len(tokens)
        logits = runner.step([StepEntry(request, part, [len(part) - 1] if last else [])])
    return logits


def time_prefill(runner, cfg, repeats=5):
    import torch

    from tokamak_amd.engine.runner import StepEntry

    times = []
    for i in range(repeats + 2):  # the first two are untimed (kernel choice of the library products, clocks)
        ids = random_prompt(cfg.vocab_size, PREFILL_TOKENS, 1000 + i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        runner.step([StepEntry("prefill", ids, [PREFILL_TOKENS - 1])])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        runner.end("prefill")
    return statistics.median(times[2:])


def time_decode(runner, cfg, batch, context, steps, warmup):
    """``batch`` requests reach ``context`` tokens at the end of the timed steps."""
    import torch

    from tokamak_amd.engine.runner import StepEntry
    from tokamak_amd.sampling.sampler import greedy_tokens

    start = context - steps - warmup
    assert start >= 1
    last = []
    for r in range(batch):
        logits = fill(runner, r, random_prompt(cfg.vocab_size, start, 7 + r))
        last.append(int(greedy_tokens(logits).item()))

    def one_step():
        nonlocal last
        logits = runner.step([StepEntry(r, [last[r]], [0]) for r in range(batch)])
        last = greedy_tokens(logits).tolist()

    for _ in range(warmup):
        one_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        one_step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    mean_ctx = context - (steps + 1) / 2.0
    for r in range(batch):
        runner.end(r)
    return elapsed / steps, mean_ctx


def run_continuous(args) -> int:
    """Optional extra workload: continuous batching through ``LLM.generate`` (scheduler,
    portions of prompts beside decode tokens, captured decode steps).  Prompt and output
    lengths uniform in the given ranges, greedy, seeded."""
    import random

    import torch

    from tokamak_amd import LLM, SamplingParams
    from tokamak_amd.config import find_preset

    p_lo, p_hi = (int(x) for x in args.prompt_tokens.split(","))
    o_lo, o_hi = (int(x) for x in args.output_tokens.split(","))
    max_len = max(4096, p_hi + o_hi)
    cfg = dataclasses.replace(find_preset(args.model)[1], max_position_embeddings=max_len)
    rng = random.Random(0)
    prompts = [[rng.randrange(cfg.vocab_size) for _ in range(rng.randint(p_lo, p_hi))] for _ in range(args.requests)]
    params = [SamplingParams(temperature=0.0, max_new_tokens=rng.randint(o_lo, o_hi), ignore_eos=True)
              for _ in range(args.requests)]
    pool = args.max_batch * (p_hi + o_hi)  # every running request fits at full length
    llm = LLM(cfg, seed=0, random_weights_on_gpu=True, dtype=args.dtype, max_seq_len=max_len,
              kv_pool_tokens=max(pool, max_len), max_batch_size=args.max_batch, max_num_batched_tokens=2048,
              prefill_chunk=2048)
    runs = []
    for _ in range(2):  # the first run also records the decode graphs
        steps0 = llm.num_steps
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        outs = llm.generate(prompt_token_ids=prompts, sampling_params=params)
        torch.cuda.synchronize()
        runs.append((time.perf_counter() - t0, llm.num_steps - steps0))
    elapsed, steps = runs[-1]
    out_tokens = sum(len(o.output_token_ids) for o in outs)
    print(json.dumps({
        "metric": f"output tok/s, continuous batching of {args.requests} requests ({args.model}-shaped, random weights)",
        "value": round(out_tokens / elapsed, 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": 0,
        "ms_per_step": round(elapsed / steps * 1e3, 3), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic (seeded lengths and token ids, random weights)",
        "config": {"model": f"{args.model}-shaped", "requests": args.requests, "max_batch": args.max_batch,
                   "prompt_tokens": sum(map(len, prompts)), "output_tokens": out_tokens,
                   "total_tok_per_s": round((sum(map(len, prompts)) + out_tokens) / elapsed, 1),
                   "first_run_s": round(runs[0][0], 3), "preemptions": llm.num_preemptions,
                   "parallelism": "single GPU"},
    }))
    return 0


def run_phase(args, runner, cfg, full) -> int:
    """One part alone, so that a profile of the run holds that part's kernels only
    (the decode part still has to fill the requests' caches first)."""
    key = "bf16" if args.dtype == "bfloat16" else "fp32"
    if args.phase == "prefill":
        seconds = time_prefill(runner, cfg, repeats=max(args.steps, 1))
        value, steps, what = PREFILL_TOKENS / seconds, max(args.steps, 1), f"prefill tok/s at {PREFILL_TOKENS} tokens"
    else:
        seconds, _ = time_decode(runner, cfg, args.batch, args.context, args.steps, args.warmup)
        value, steps, what = args.batch / seconds, args.steps, f"decode tok/s at batch {args.batch}"
    print(json.dumps({
        "metric": f"{what} ({SHAPE_NAMES[args.shape]}-shaped, random weights)", "value": round(value, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": steps, "warmup": args.warmup, "ms_per_step": round(seconds * 1e3, 3),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": key,
        "data": "synthetic (uniform random token ids, seeded random weights)",
        "config": {"model": f"{args.shape}-shaped", "layers": cfg.num_layers, "layers_of_model": full.num_layers,
                   "global_batch": args.batch, "seq_len": args.context, "phase": args.phase,
                   "parallelism": "single GPU"},
    }))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (named in config)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 points")
    ap.add_argument("--phase", default="all", choices=["all", "prefill", "decode"],
                    help="run only one part (for profiles); the other part's figures are null")
    ap.add_argument("--workload", default="decode", choices=["decode", "continuous"],
                    help="decode: the headline measurement; continuous: LLM.generate over many requests")
    ap.add_argument("--model", default="qwen3-0.6b", help="preset shape of the continuous workload")
    ap.add_argument("--shape", default="qwen3-8b", choices=["qwen3-0.6b", "qwen3-8b", "qwen3-32b"],
                    help="preset whose layer sizes the decode/prefill measurement uses (default: the headline one)")
    ap.add_argument("--requests", type=int, default=256)
    ap.add_argument("--max-batch", type=int, default=64)
    ap.add_argument("--prompt-tokens", default="32,1024", help="continuous workload: MIN,MAX prompt length")
    ap.add_argument("--output-tokens", default="16,256", help="continuous workload: MIN,MAX output length")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this engine")
        return 2
    if args.workload == "continuous":
        return run_continuous(args)

    import torch

    from tokamak_amd.config import find_preset

    full = find_preset(args.shape)[1]
    cfg = dataclasses.replace(full, num_layers=args.layers or full.num_layers)
    elem = 2 if args.dtype == "bfloat16" else 4
    max_batch = 64 if not (args.no_points or args.phase != "all") else args.batch
    pool = max(max_batch, args.batch) * (args.context + 16)
    runner = make_runner(cfg, args.dtype, pool, max(max_batch, args.batch))

    if args.phase != "all":
        return run_phase(args, runner, cfg, full)
    prefill_s = time_prefill(runner, cfg)
    step_s, mean_ctx = time_decode(runner, cfg, args.batch, args.context, args.steps, args.warmup)
    points = {}
    if not args.no_points:
        for b, k in ((1, min(args.steps, 64)), (64, min(args.steps, 32))):
            s, _ = time_decode(runner, cfg, b, args.context, k, min(args.warmup, 4))
            points[f"decode_b{b}"] = round(b / s, 1)

    step_bytes = weight_bytes(cfg, elem) + args.batch * mean_ctx * kv_bytes_per_token(cfg, elem)
    achieved = step_bytes / step_s
    key = "bf16" if args.dtype == "bfloat16" else "fp32"
    result = {
        "metric": f"decode tok/s at batch {args.batch} ({SHAPE_NAMES[args.shape]}-shaped, random weights); prefill tok/s at 2,048 tokens",
        "value": round(args.batch / step_s, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": key,
        "data": "synthetic (uniform random token ids, seeded random weights N(0, 0.02), norm weights 1)",
        "config": {
            "model": f"{args.shape}-shaped", "layers": cfg.num_layers, "layers_of_model": full.num_layers,
            "hidden_size": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_kv_heads,
            "head_dim": cfg.head_dim, "intermediate_size": cfg.intermediate_size,
            "vocab_size": cfg.vocab_size, "global_batch": args.batch, "seq_len": args.context,
            "page_size": 16, "sampling": "greedy", "parallelism": "single GPU",
        },
        "prefill": {
            "value": round(PREFILL_TOKENS / prefill_s, 1), "tokens": PREFILL_TOKENS,
            "ms": round(prefill_s * 1e3, 3),
            "frac": round(prefill_flops(cfg, PREFILL_TOKENS) / prefill_s / MFMA_PEAK[key], 4),
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK, 4)},
        "points": points,
    }
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
