"""Choose next tokens from float32 logits on the GPU.

Greedy rows take the first maximum (reference: src/tokamak/sampling/sampler.py:58-59).
Other rows go through temperature -> top-k -> top-p -> softmax -> one draw
(sampler.py:34-39,61).  The draw uses a counter-based generator keyed by the
request's seed and the number of draws it has made, so a request's stream does
not depend on what else is in the batch and survives preemption.  The
reference draws with ``torch.multinomial``; the same distribution is sampled
here, not the same stream.
"""

from __future__ import annotations

import numpy as np
import torch

from tokamak_amd.kernels import ops
from tokamak_amd.sampling.params import SamplingParams


def _output(out: torch.Tensor | None, m: int, device) -> torch.Tensor:
    if out is None:
        return torch.empty((m,), dtype=torch.int32, device=device)
    if out.dtype != torch.int32 or out.dim() != 1 or out.numel() < m or not out.is_contiguous():
        raise ValueError(f"the tokens' place must be a contiguous int32 vector of at least {m}")
    return out[:m]


def greedy_tokens(logits: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """int32 [M]: argmax of every row (written to the head of ``out`` if given)."""
    out = _output(out, logits.shape[0], logits.device)
    ops.argmax(logits, out)
    return out


def sample_tokens(logits: torch.Tensor, params: list[SamplingParams], seeds: list[int],
                  draws: list[int], *, return_probs: bool = False, out: torch.Tensor | None = None):
    """One token per row of ``logits`` [M, V].

    ``seeds[i]`` and ``draws[i]``: row i's request seed and how many tokens it
    has drawn before.  Returns int32 [M] (and the post-filter distributions
    [M, V] when ``return_probs``; greedy rows have none and stay zero).  ``out``: an int32
    vector whose head receives the tokens (the runner's ``sampled``, from which the next
    step may take them on the GPU).
    """
    m = logits.shape[0]
    if not (len(params) == len(seeds) == len(draws) == m):
        raise ValueError("one SamplingParams, seed and draw count per logits row is required")
    if all(p.is_greedy for p in params) and not return_probs:
        return greedy_tokens(logits, out)
    dev = logits.device
    # one host buffer, one copy: [seeds | draws] int64, then [temperature | top_p] float32 and top_k int32
    host = np.empty(7 * m, dtype=np.int32)
    wide = host[:4 * m].view(np.int64)
    wide[:m] = [s & 0x7FFFFFFFFFFFFFFF for s in seeds]
    wide[m:] = draws
    floats = host[4 * m:6 * m].view(np.float32)
    floats[:m] = [p.temperature for p in params]
    floats[m:] = [p.top_p for p in params]
    host[6 * m:] = [p.top_k for p in params]
    # through pinned memory and without waiting: a copy from pageable memory would hold the
    # host until the GPU has run everything queued before it
    packed = torch.from_numpy(host).pin_memory().to(dev, non_blocking=True)
    seed_t, draw_t = packed[:2 * m].view(torch.int64), packed[2 * m:4 * m].view(torch.int64)
    temperature, top_p = packed[4 * m:5 * m].view(torch.float32), packed[5 * m:6 * m].view(torch.float32)
    top_k = packed[6 * m:]
    out = _output(out, m, dev)
    probs = torch.zeros_like(logits) if return_probs else None
    ops.sample(logits, temperature, top_k, top_p, seed_t, draw_t, out, probs)
    return (out, probs) if return_probs else out
