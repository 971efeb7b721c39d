"""Decode and prefill throughput of a Qwen3-8B-shaped model with random weights.

    python bench.py [--gpus 1] [--steps 256] [--warmup 8] [--batch 8] [--prompt 2048]
                    [--context C] [--layers L] [--shape PRESET] [--profile]

Prints one JSON line.  The default workload is the headline one as written: every
request of the batch has a 2,048-token random prompt and generates 256 tokens
greedily; a "step" is one decode step of the whole batch through the engine's own
step function and sampler; all ``--steps`` steps after the prompt are timed, three
times over (fresh requests each time), and the median run is reported.  ``--warmup``
steps of the same workload run untimed before (they also record the decode graph).
``--context C`` instead times the last ``--steps`` steps before each request holds C
tokens (a longer context than the headline's).

``value`` is decoded tokens per second.  ``prefill`` is one 2,048-token prompt in one
step.  ``roofline`` prices the decode step against HBM: every weight it uses once plus
the cache of the live requests at the mean context of the timed steps, divided by its
time.  Fractions are of the published peaks (HBM 8 TB/s, dense bf16 MFMA 2.5 PFLOP/s);
``peaks`` holds what two microbenchmarks of this program reach on this GPU (streaming
reads and copies of 4 GiB; back-to-back MFMA from registers), and ``frac_of_measured``
the same fractions of those.  ``peak_memory_gib`` is the most GPU memory allocated at any
time of the run.  ``--profile`` adds ``kernels``: one decode step and one
prefill step with every kernel call timed by events, summed by kind of call.

Two further workloads go through ``LLM.generate`` (scheduler, prompt portions beside
decode tokens, captured decode steps) and print a line of the same form:
``--workload continuous`` (256 requests of uniform random lengths, Qwen3-0.6B shape) and
``--workload trace`` (the reference's own 32-request throughput trace at 1, 4 and 16
running requests, with its published figure as ``vs_baseline``).  ``--workload attention``
is the reference's microbenchmark of one layer's decode attention at its six shapes, and
``--workload latency`` its single-sequence latency measurement (512 prompt + 128 new tokens).
"""

from __future__ import annotations

import argparse
import ctypes
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
PAGE_SIZE = 16


# ---------------------------------------------------------------------------
# what this GPU reaches
# ---------------------------------------------------------------------------
def measure_peaks() -> dict:
    """Streaming read and copy of 4 GiB (far beyond every cache) and bf16 MFMA from
    registers, each the best of five launches after an untimed one."""
    import torch

    from tokamak_amd.kernels.build import load_library

    lib = load_library("peaks")
    c_void_p, c_size_t, c_int = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int
    lib.tk_peak_read.argtypes = [c_void_p, c_size_t, c_void_p, c_int, c_void_p]
    lib.tk_peak_copy.argtypes = [c_void_p, c_void_p, c_size_t, c_int, c_void_p]
    lib.tk_peak_mfma.argtypes = [c_int, c_int, c_int, c_void_p, ctypes.POINTER(ctypes.c_double), c_void_p]
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    nbytes = 4 << 30
    src = torch.empty(nbytes, dtype=torch.uint8, device="cuda:0").fill_(1)
    dst = torch.empty(nbytes, dtype=torch.uint8, device="cuda:0")
    sink = torch.zeros(65536, dtype=torch.float32, device="cuda:0")

    def best(launch) -> float:
        times = []
        for _ in range(6):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            assert launch() == 0
            e1.record()
            e1.synchronize()
            times.append(e0.elapsed_time(e1) * 1e-3)
        return min(times[1:])

    blocks = 256 * 16
    read_s = best(lambda: lib.tk_peak_read(src.data_ptr(), nbytes, sink.data_ptr(), blocks, stream))
    copy_s = best(lambda: lib.tk_peak_copy(src.data_ptr(), dst.data_ptr(), nbytes, blocks, stream))
    mfma = {}
    for shape, name in ((0, "16x16x32"), (1, "32x32x16")):
        flops = ctypes.c_double(0.0)
        seconds = best(lambda: lib.tk_peak_mfma(shape, 256 * 8, 20000, sink.data_ptr(), ctypes.byref(flops), stream))
        mfma[name] = flops.value / seconds
    del src, dst
    torch.cuda.empty_cache()
    return {"hbm_read_measured": round(nbytes / read_s / 1e9, 1),
            "hbm_copy_measured": round(2 * nbytes / copy_s / 1e9, 1),
            "mfma_bf16_measured": round(max(mfma.values()) / 1e12, 1),
            "mfma_bf16_16x16x32": round(mfma["16x16x32"] / 1e12, 1),
            "hbm_published": HBM_PEAK / 1e9, "mfma_bf16_published": MFMA_PEAK["bf16"] / 1e12,
            "units": "GB/s, TFLOP/s"}


# ---------------------------------------------------------------------------
# the model and what a step has to move and compute, from the plan
# ---------------------------------------------------------------------------
def make_llm(cfg, dtype, pool_tokens, max_requests, max_seq_len, seed=0, tune=True):
    """The engine's entry point over seeded random weights of ``cfg``'s shape, drawn on the GPU."""
    from tokamak_amd import LLM

    return LLM(cfg, seed=seed, random_weights_on_gpu=True, dtype=dtype, block_size=PAGE_SIZE,
               kv_pool_tokens=pool_tokens, max_batch_size=max_requests, max_seq_len=max_seq_len,
               max_num_batched_tokens=PREFILL_TOKENS, tune_library_products=tune)


def make_runner(arch, cfg, dtype, pool_tokens, max_requests, seed=0):
    import torch

    from tokamak_amd.engine.runner import ModelRunner
    from tokamak_amd.weights.random_init import expected_tensors_of
    from tokamak_amd.weights.sources import RandomSource

    plan = arch.plan(cfg)
    expected = {n: s for n, s in expected_tensors_of(plan).items() if not s.ignored}
    tdt = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    source = RandomSource(expected, seed, matrix_std=0.02, vector_jitter=0.0, dtype=tdt, device="cuda:0")
    return ModelRunner(plan, source, dtype=dtype, page_size=PAGE_SIZE, kv_pool_tokens=pool_tokens,
                       max_requests=max_requests)


class StepCost:
    """Bytes and flops of steps of the model a runner holds, from its own tensors and
    cache layout (nothing here names an architecture)."""

    def __init__(self, runner) -> None:
        model, plan = runner.model, runner.plan
        elem = 2 if runner.dtype.itemsize == 2 else 4
        tensors = {n: s for n, s in model.expected_tensors().items() if not s.ignored}
        size = {n: (4 if s.role != "matrix" else elem) for n, s in tensors.items()}
        numel = {n: _prod(s.shape) for n, s in tensors.items()}
        embedding = set(model.embedding.expected_tensors(plan.embedding_prefix))
        head = {n for n in model.head.expected_tensors(plan.head_prefix) if n in tensors}
        self.hidden = plan.hidden_size
        self.elem = elem
        # every tensor a decode step reads whole: all but the embedding table (a row a token),
        # unless the head is tied to it
        self.weight_bytes = sum(numel[n] * size[n] for n in tensors if n not in embedding or plan.tie_word_embeddings)
        self.embedding_row_bytes = plan.hidden_size * elem
        self.matrix_params = sum(numel[n] for n, s in tensors.items()
                                 if s.role == "matrix" and n not in embedding and n not in head)
        self.head_params = plan.vocab_size * plan.hidden_size
        _, layouts = model.cache_layout()
        self.kv_bytes_per_token = sum(lay.request.bytes_per_token(runner.dtype) for lay in layouts.values())
        # attention flops of a layer call: 4 * heads * head_dim per (query, visible key) pair
        self.pair_flops = sum(mixer.pair_flops() for call in plan.order
                              for mixer in model.blocks[call.layer].mixers.values())

    def decode_bytes(self, batch: int, mean_keys: float) -> float:
        return self.weight_bytes + batch * (self.embedding_row_bytes + mean_keys * self.kv_bytes_per_token)

    def prefill_flops(self, tokens: int) -> float:
        return (2.0 * tokens * self.matrix_params + self.pair_flops * tokens * (tokens + 1) / 2
                + 2.0 * self.head_params)


def _prod(shape) -> int:
    out = 1
    for d in shape:
        out *= int(d)
    return out


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


# ---------------------------------------------------------------------------
# timing
# ---------------------------------------------------------------------------
def time_prefill(runner, vocab, repeats=5):
    import torch

    from tokamak_amd.engine.runner import StepEntry

    times = []
    for i in range(repeats + 2):  # the first two are untimed (plans of the library products, clocks)
        ids = random_prompt(vocab, PREFILL_TOKENS, 1000 + i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        runner.step([StepEntry("prefill", ids, [PREFILL_TOKENS - 1])])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        runner.end("prefill")
    return statistics.median(times[2:])


def decode_pass(llm, vocab, batch, prompt_tokens, steps, seed):
    """``batch`` fresh requests with ``prompt_tokens``-token prompts, then ``steps`` greedy
    decode steps of the whole batch; seconds for those steps.

    The timed steps are run by the generation loop itself (``LLM.run``: the scheduler plans
    every step, each is launched before the tokens of the step before it are read and takes
    them from the sampler's output on the GPU, and the host reads every step's tokens one
    step late).  Before that every prompt runs alone, in portions, and its first token is
    read at once, so that all requests enter the timed steps with the same context."""
    import torch

    from tokamak_amd import SamplingParams
    from tokamak_amd.engine.scheduler import Scheduler, Span, StepPlan

    params = SamplingParams(temperature=0.0, max_new_tokens=steps + 1, ignore_eos=True)
    scheduler = Scheduler(llm.runner.manager, batch, max(batch, llm.max_num_batched_tokens))
    requests = []
    for r in range(batch):
        request = llm.new_request(r, random_prompt(vocab, prompt_tokens, seed * 1000 + r), params)
        for at in range(0, prompt_tokens, PREFILL_TOKENS):
            n = min(PREFILL_TOKENS, prompt_tokens - at)
            flight = llm.launch(StepPlan([Span(request, at, n, at + n == prompt_tokens)]))
            if flight is not None:
                llm.read(flight)
        scheduler.running.append(request)
        requests.append(request)
    assert all(r.num_generated == 1 and r.decoding for r in requests)
    before = llm.num_steps
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    llm.run(scheduler)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    assert llm.num_steps - before == steps, f"{llm.num_steps - before} steps ran, {steps} were to be timed"
    assert all(r.finished and r.num_generated == steps + 1 for r in requests)
    llm.runner.end_all()
    return elapsed


def time_decode(llm, vocab, batch, prompt_tokens, steps, warmup, repeats):
    """Median seconds per step over ``repeats`` timed passes, after one untimed pass of
    ``warmup`` steps; and every pass's figure."""
    if warmup > 0:
        decode_pass(llm, vocab, batch, prompt_tokens, warmup, seed=0)
    runs = [decode_pass(llm, vocab, batch, prompt_tokens, steps, seed=1 + i) / steps for i in range(repeats)]
    return statistics.median(runs), runs


def profile_step(runner, entries, blocker):
    """One step, eagerly, every kernel call between two events.  A few long copies are
    queued first so that the step's launches are all in the queue before the first runs:
    what the events bracket is then the kernels, not the host's launch gaps."""
    from tokamak_amd.kernels import ops

    graphs, runner.use_graphs = runner.use_graphs, False
    try:
        blocker()
        with ops.KernelProfile() as prof:
            runner.step(entries)
        return prof.rows()
    finally:
        runner.use_graphs = graphs


def kernel_table(rows, key, top=14):
    out = []
    for row in rows[:top]:
        seconds = row["us"] * 1e-6
        rec = {"name": row["name"], "calls": row["calls"], "us": round(row["us"], 1)}
        if row["bytes"]:
            rec["GBps"] = round(row["bytes"] / seconds / 1e9, 1)
        if row["flops"]:
            rec["TFLOPs"] = round(row["flops"] / seconds / 1e12, 1)
        fracs = [row["bytes"] / seconds / HBM_PEAK, row["flops"] / seconds / MFMA_PEAK[key]]
        rec["frac"] = round(max(fracs), 3)
        rec["bound"] = "hbm" if fracs[0] >= fracs[1] else "mfma"
        out.append(rec)
    rest = rows[top:]
    if rest:
        out.append({"name": f"{len(rest)} other kinds", "calls": sum(r["calls"] for r in rest),
                    "us": round(sum(r["us"] for r in rest), 1)})
    return out


def profile_kernels(runner, vocab, batch, prompt_tokens, key, blocker):
    from tokamak_amd.engine.runner import StepEntry

    for r in range(batch):
        fill(runner, r, random_prompt(vocab, prompt_tokens + 127, 77 + r))
    graphs, runner.use_graphs = runner.use_graphs, False
    runner.step([StepEntry(r, [1 + r], [0]) for r in range(batch)])          # untimed: code objects, allocator
    runner.use_graphs = graphs
    decode = profile_step(runner, [StepEntry(r, [2 + r], [0]) for r in range(batch)], blocker)
    for r in range(batch):
        runner.end(r)
    ids = random_prompt(vocab, PREFILL_TOKENS, 5)
    prefill = profile_step(runner, [StepEntry("prefill", ids, [PREFILL_TOKENS - 1])], blocker)
    runner.end("prefill")
    return {"decode": kernel_table(decode, key), "prefill": kernel_table(prefill, key),
            "decode_sum_us": round(sum(r["us"] for r in decode), 1),
            "prefill_sum_us": round(sum(r["us"] for r in prefill), 1)}


def make_blocker():
    """A callable that queues ~25 ms of copies on the current stream."""
    import torch

    a = torch.empty(1 << 30, dtype=torch.uint8, device="cuda:0")
    b = torch.empty(1 << 30, dtype=torch.uint8, device="cuda:0")

    def blocker():
        for _ in range(40):
            b.copy_(a)

    return blocker


# ---------------------------------------------------------------------------
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
              prefill_chunk=2048, tune_library_products=not args.no_tune)
    runs = []
    for _ in range(2):  # the first run also records the decode graphs
        steps0 = llm.num_steps
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        outs = llm.generate(prompt_token_ids=prompts, sampling_params=params, use_tqdm=False)
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
                   "tuned_products": not args.no_tune, "parallelism": "single GPU"},
    }))
    return 0


# ---------------------------------------------------------------------------
def reference_trace(num_requests: int, max_new_cap: int, seed: int, vocab_size: int):
    """The lengths of the reference's throughput trace (benchmarks/workload.py:23-42): per
    request, drawn in this order from ``random.Random(seed)``: a prompt length, log-normal
    (mu 5.0, sigma 0.7) cut to 16..512; a number of new tokens, floor of an exponential of
    mean 120, plus 8, at most ``max_new_cap``; then the prompt's ids (ids past the first
    special token are folded back, which keeps the stream of draws as published).  With 32
    requests, cap 256 and seed 0 this gives the 4,915 prompt and 2,901 output tokens of
    benchmarks/README.md:87-90."""
    import random

    first_special = 151_643
    rng = random.Random(seed)
    prompts, new_tokens = [], []
    for _ in range(num_requests):
        length = int(min(512.0, max(16.0, rng.lognormvariate(5.0, 0.7))))
        new_tokens.append(min(max_new_cap, 8 + int(rng.expovariate(1.0 / 120.0))))
        prompts.append([rng.randrange(vocab_size) % first_special for _ in range(length)])
    return prompts, new_tokens


def run_trace(args) -> int:
    """The reference's "throughput under concurrency" measurement (benchmarks/benchmark_throughput.py:
    30-68, README.md:87-129): its seeded 32-request trace through ``LLM.generate`` on the
    Qwen3-0.6B shape (random weights here), greedy, EOS ignored, a 16,384-token pool,
    sequences of at most 1,024 tokens, at most 1, 4 and 16 running requests.  Every setting
    runs twice; the second run is reported (the first also records the decode graphs)."""
    import statistics

    import torch

    from tokamak_amd import LLM, SamplingParams
    from tokamak_amd.config import find_preset

    cfg = find_preset(args.model)[1]
    prompts, new_tokens = reference_trace(32, 256, 0, cfg.vocab_size)
    params = [SamplingParams(temperature=0.0, max_new_tokens=n, ignore_eos=True) for n in new_tokens]
    config = {"model": f"{args.model}-shaped", "requests": len(prompts), "prompt_tokens": sum(map(len, prompts)),
              "output_tokens": sum(new_tokens), "kv_pool_tokens": 16384, "max_seq_len": 1024}
    value = steps = elapsed = None
    for batch in (1, 4, 16):
        llm = LLM(cfg, seed=0, random_weights_on_gpu=True, dtype=args.dtype, max_seq_len=1024,
                  kv_pool_tokens=16384, max_batch_size=batch, tune_library_products=not args.no_tune)
        for _ in range(2):
            steps0 = llm.num_steps
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            outs = llm.generate(prompt_token_ids=prompts, sampling_params=params, use_tqdm=False)
            torch.cuda.synchronize()
            elapsed, steps = time.perf_counter() - t0, llm.num_steps - steps0
        assert [len(o.output_token_ids) for o in outs] == new_tokens
        value = sum(new_tokens) / elapsed
        ttft = sorted(o.ttft_s for o in outs)
        config[f"b{batch}_out_tok_per_s"] = round(value, 1)
        config[f"b{batch}_wall_s"] = round(elapsed, 4)
        config[f"b{batch}_ttft_mean_ms"] = round(statistics.mean(ttft) * 1e3, 2)
        config[f"b{batch}_ttft_p95_ms"] = round(ttft[min(int(0.95 * len(ttft)), len(ttft) - 1)] * 1e3, 2)
        del llm
        torch.cuda.empty_cache()
    # the reference's best published figure for its own engine on this trace: continuous b=16 with its
    # Triton kernel under Linux, 236.8 output tok/s on an RTX 3080 Laptop GPU (benchmarks/README.md:196)
    config["baseline"] = "236.8 out tok/s, continuous b=16, RTX 3080 Laptop (reference benchmarks/README.md:196)"
    print(json.dumps({
        "metric": "output tok/s on the reference's 32-request trace, continuous batching, at most 16 running",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": 0,
        "ms_per_step": round(elapsed / steps * 1e3, 3), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": round(value / 236.8, 2), "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic (the reference's seeded trace of lengths and token ids, random weights)", "config": config,
    }))
    return 0


def run_attention(args) -> int:
    """The reference's decode-attention microbenchmark (benchmarks/benchmark_attention.py,
    README.md:41-53): the attention of one layer in one decode step, alone: the new token's key
    and value written to its page, then attention over the request's pages; 16 query heads, 8
    kv heads of 128, pages of 16, bfloat16, every request's pages scattered over the pool
    (request i holds pages i, B + i, 2B + i, ...).  Here that is one kernel (plus the merge of the
    key splits) that also norms and rotates the token's query and key.  ``call_us``: the
    reference's method, one call and a synchronize on the host's clock, median of 50 (mostly the
    launch from Python); ``graph_us``: a call inside a captured graph of 16, as decode steps run."""
    import torch

    from tokamak_amd.engine.batch import StepSpan, build_batch
    from tokamak_amd.kernels import attention as attn

    nh, nkv, hd, ps = 16, 8, 128, 16
    published = {(1, 512): 241, (8, 512): 271, (16, 512): 323, (16, 2048): 806, (32, 512): 440, (32, 2048): 1409}
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    config = {"heads": nh, "kv_heads": nkv, "head_dim": hd, "page_size": ps}
    last = None
    for (batch_size, context), theirs in published.items():
        pages_each = -(-(context + 1) // ps)
        k_cache = torch.randn(pages_each * batch_size, nkv * hd * ps, device=dev, dtype=torch.bfloat16)
        v_cache = torch.randn_like(k_cache)
        spans = [StepSpan(request=i, tokens=[0], ctx_len=context, state_slot=i,
                          tables=[[j * batch_size + i for j in range(pages_each)]]) for i in range(batch_size)]
        batch = build_batch(spans, 1, dev, [attn.ATTENTION_WORK])
        qkv = torch.randn(batch_size, (nh + 2 * nkv) * hd, device=dev, dtype=torch.bfloat16)
        weight = torch.ones(hd, device=dev, dtype=torch.float32)
        angle = torch.rand(batch_size, hd // 2, device=dev, dtype=torch.float32)
        cos, sin = torch.cos(angle), torch.sin(angle)
        out = torch.empty(batch_size, nh * hd, device=dev, dtype=torch.bfloat16)

        def call():
            done = attn.decode_attention_fused(
                qkv, weight, weight, cos, sin, k_cache, v_cache, batch.block_tables[0], batch, out, num_heads=nh,
                num_kv_heads=nkv, head_dim=hd, rotary_dim=hd, page_size=ps, eps=1e-6, scale=hd ** -0.5, store=True)
            assert done

        for _ in range(10):
            call()
        torch.cuda.synchronize()
        times = []
        for _ in range(50):
            t0 = time.perf_counter()
            call()
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
        call_us = statistics.median(times) * 1e6
        stream = torch.cuda.Stream()
        with torch.cuda.stream(stream):
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                for _ in range(16):
                    call()
        graph.replay()
        torch.cuda.synchronize()
        times = []
        for _ in range(20):
            t0 = time.perf_counter()
            graph.replay()
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
        graph_us = statistics.median(times) * 1e6 / 16
        cache_bytes = batch_size * (context + 1) * 2 * nkv * hd * 2
        tag = f"b{batch_size}_c{context}"
        config[f"{tag}_call_us"] = round(call_us, 1)
        config[f"{tag}_graph_us"] = round(graph_us, 2)
        last = (theirs, call_us, graph_us, cache_bytes)
    theirs, call_us, graph_us, cache_bytes = last
    config["baseline"] = "Triton kernel, RTX 3080 Laptop: 241/271/323/806/440/1409 us (reference benchmarks/README.md:48-53)"
    print(json.dumps({
        "metric": "decode attention of one layer and step, batch 32 at context 2,048 (us per call, the reference's method)",
        "value": round(call_us, 1), "unit": "us", "n_gpus": 1, "steps": 50, "warmup": 10,
        "ms_per_step": round(call_us / 1e3, 4), "higher_is_better": False, "scaling": "weak",
        "vs_baseline": round(call_us / theirs, 4), "dtype": "bf16",
        "data": "synthetic (random cache, scattered block tables)",
        "roofline": {"bound": "hbm", "achieved": round(cache_bytes / graph_us / 1e3, 1), "peak": HBM_PEAK / 1e9,
                     "unit": "GB/s", "frac": round(cache_bytes / graph_us * 1e6 / HBM_PEAK, 4)},
        "config": config,
    }))
    return 0


def run_latency(args) -> int:
    """The reference's single-sequence latency measurement (benchmarks/benchmark_latency.py:63-98,
    126-129; README.md:16-24): one random prompt of 512 tokens through the model in one step, its first
    token read on the host (prefill_ms), then 128 greedy tokens one step at a time, every token read on the
    host before the next step starts (decode tok/s, inter-token ms), on the Qwen3-0.6B shape (random weights
    here), pages of 16; one untimed pass, then the median of three.  The published figures are for an RTX
    3080 Laptop GPU: 70.7 ms, 21.0 tok/s and 1.47 GiB with the reference's Triton kernel."""
    import torch

    from tokamak_amd.config import find_preset
    from tokamak_amd.engine.runner import StepEntry
    from tokamak_amd.kernels import ops
    from tokamak_amd.sampling.sampler import greedy_tokens

    prompt_tokens, new_tokens = 512, 128
    arch, cfg = find_preset(args.model)
    ops.set_library_tuning(not args.no_tune)
    runner = make_runner(arch, cfg, args.dtype, prompt_tokens + new_tokens, 1)
    prompt = random_prompt(cfg.vocab_size, prompt_tokens, 0)
    passes = []
    for _ in range(1 + 3):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        token = int(greedy_tokens(runner.step([StepEntry("one", prompt, [prompt_tokens - 1])]))[0])
        t1 = time.perf_counter()
        for _ in range(new_tokens):
            token = int(greedy_tokens(runner.step([StepEntry("one", [token], [0])]))[0])
        t2 = time.perf_counter()
        runner.end("one")
        passes.append((t1 - t0, t2 - t1))
    prefill_s = statistics.median(p for p, _ in passes[1:])
    decode_s = statistics.median(d for _, d in passes[1:])
    value = new_tokens / decode_s
    print(json.dumps({
        "metric": "decode tok/s of one sequence, 512 prompt tokens + 128 greedy tokens, every token read before the next step",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": new_tokens, "warmup": new_tokens,
        "ms_per_step": round(decode_s / new_tokens * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": round(value / 21.0, 2), "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic (seeded random token ids, random weights)",
        "prefill": {"value": round(prompt_tokens / prefill_s, 1), "tokens": prompt_tokens, "ms": round(prefill_s * 1e3, 3)},
        "peak_memory_gib": round(torch.cuda.max_memory_allocated() / 2 ** 30, 2),
        "config": {"model": f"{args.model}-shaped", "prompt_tokens": prompt_tokens, "new_tokens": new_tokens, "page_size": PAGE_SIZE,
                   "baseline": "70.7 ms prefill, 21.0 tok/s, 1.47 GiB: paged cache + Triton kernel, RTX 3080 Laptop "
                               "(reference benchmarks/README.md:24)"},
    }))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256, help="timed decode steps of a pass (the headline workload: 256)")
    ap.add_argument("--warmup", type=int, default=8, help="untimed decode steps before the timed passes")
    ap.add_argument("--repeats", type=int, default=3, help="timed passes; the median is reported")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt", type=int, default=2048, help="prompt tokens of every request")
    ap.add_argument("--context", type=int, default=None,
                    help="instead of --prompt: the timed steps end when each request holds this many tokens")
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (named in config)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 points")
    ap.add_argument("--no-peaks", action="store_true", help="skip the microbenchmarks of this GPU's peaks")
    ap.add_argument("--no-tune", action="store_true",
                    help="take the library's first algorithm for long portions' products instead of timing its candidates")
    ap.add_argument("--profile", action="store_true", help="add per-kernel times of one decode and one prefill step")
    ap.add_argument("--phase", default="all", choices=["all", "prefill", "decode"],
                    help="run only one part (for an external profiler); the other part's figures are null")
    ap.add_argument("--workload", default="decode", choices=["decode", "continuous", "trace", "attention", "latency"],
                    help="decode: the headline measurement; continuous: LLM.generate over many requests; "
                         "trace: the reference's 32-request throughput trace at 1, 4 and 16 running requests; "
                         "attention: the reference's decode-attention microbenchmark; "
                         "latency: its single-sequence latency measurement (512 + 128 tokens)")
    ap.add_argument("--model", default="qwen3-0.6b", help="preset shape of the continuous workload")
    ap.add_argument("--shape", default="qwen3-8b",
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
    if args.workload == "trace":
        return run_trace(args)
    if args.workload == "attention":
        return run_attention(args)
    if args.workload == "latency":
        return run_latency(args)

    from tokamak_amd.config import find_preset
    from tokamak_amd.kernels import ops

    arch, full = find_preset(args.shape)
    cfg = dataclasses.replace(full, num_layers=args.layers or full.num_layers)
    key = "bf16" if args.dtype == "bfloat16" else "fp32"
    prompt_tokens = args.prompt if args.context is None else args.context - args.steps
    if prompt_tokens < 1:
        ap.error("--context must exceed --steps")
    final_context = prompt_tokens + args.steps
    want_points = not args.no_points and args.phase == "all"
    max_batch = max(64 if want_points else 1, args.batch)
    peaks = None if args.no_peaks else measure_peaks()
    deepest = max(final_context, prompt_tokens + 129) if args.profile else final_context   # (the profiled step sits 129 tokens in)
    pool = max_batch * (-(-(deepest + 1) // PAGE_SIZE) * PAGE_SIZE + PAGE_SIZE)
    longest = max(deepest + 1, PREFILL_TOKENS + 1)
    llm = make_llm(cfg, args.dtype, max(pool, PREFILL_TOKENS + PAGE_SIZE, longest), max_batch, longest,
                   tune=not args.no_tune)
    runner = llm.runner
    cost = StepCost(runner)
    vocab = runner.plan.vocab_size

    prefill_s = time_prefill(runner, vocab) if args.phase in ("all", "prefill") else None
    step_s = runs = None
    if args.phase in ("all", "decode"):
        step_s, runs = time_decode(llm, vocab, args.batch, prompt_tokens, args.steps, args.warmup, args.repeats)
    points = {}
    if want_points:
        for b in (1, 64):
            s, _ = time_decode(llm, vocab, b, prompt_tokens, args.steps, min(args.warmup, 4), args.repeats)
            keys = prompt_tokens + (args.steps + 1) / 2.0
            points[f"decode_b{b}"] = round(b / s, 1)
            points[f"decode_b{b}_hbm_frac"] = round(cost.decode_bytes(b, keys) / s / HBM_PEAK, 4)
    kernels = None
    if args.profile:
        kernels = profile_kernels(runner, vocab, args.batch, prompt_tokens, key, make_blocker())

    sizes = arch.to_json(cfg) if arch.to_json else {}
    config = {"model": f"{args.shape}-shaped", "layers": cfg.num_layers, "layers_of_model": full.num_layers}
    for name, short in (("hidden_size", "hidden_size"), ("num_attention_heads", "heads"),
                        ("num_key_value_heads", "kv_heads"), ("head_dim", "head_dim"),
                        ("intermediate_size", "intermediate_size"), ("vocab_size", "vocab_size")):
        if name in sizes:
            config[short] = sizes[name]
    config.update({"global_batch": args.batch, "prompt_tokens": prompt_tokens, "generated_tokens": args.steps,
                   "seq_len": final_context, "page_size": PAGE_SIZE, "repeats": args.repeats,
                   "tuned_products": not args.no_tune, "sampling": "greedy", "parallelism": "single GPU"})
    what = (f"decode tok/s at batch {args.batch} ({args.shape}-shaped, random weights, {prompt_tokens}-token prompts "
            f"+ {args.steps} generated); prefill tok/s at {PREFILL_TOKENS} tokens")
    result = {
        "metric": what, "value": None, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": None, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": key,
        "data": "synthetic (uniform random token ids, seeded random weights N(0, 0.02), norm weights 1)",
        "config": config,
    }
    if step_s is not None:
        mean_keys = prompt_tokens + (args.steps + 1) / 2.0
        achieved = cost.decode_bytes(args.batch, mean_keys) / step_s
        result.update({"value": round(args.batch / step_s, 1), "ms_per_step": round(step_s * 1e3, 3),
                       "runs_ms_per_step": [round(r * 1e3, 3) for r in runs]})
        result["roofline"] = {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9,
                              "unit": "GB/s", "frac": round(achieved / HBM_PEAK, 4)}
        if peaks:
            result["roofline"]["frac_of_measured"] = round(achieved / 1e9 / peaks["hbm_read_measured"], 4)
    if prefill_s is not None:
        flops = cost.prefill_flops(PREFILL_TOKENS)
        result["prefill"] = {"value": round(PREFILL_TOKENS / prefill_s, 1), "tokens": PREFILL_TOKENS,
                             "ms": round(prefill_s * 1e3, 3), "frac": round(flops / prefill_s / MFMA_PEAK[key], 4)}
        if peaks and key == "bf16":
            result["prefill"]["frac_of_measured"] = round(flops / prefill_s / 1e12 / peaks["mfma_bf16_measured"], 4)
        if step_s is None:
            result.update({"value": result["prefill"]["value"], "ms_per_step": result["prefill"]["ms"], "steps": 5})
    result["points"] = points
    # as the reference's latency benchmark reads it (benchmarks/benchmark_latency.py:144-146): weights,
    # the cache pools of every measured batch size (one at a time) and the largest step's activations
    import torch

    result["peak_memory_gib"] = round(torch.cuda.max_memory_allocated() / 2 ** 30, 2)
    if peaks:
        result["peaks"] = peaks
    if kernels:
        result["kernels"] = kernels
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
