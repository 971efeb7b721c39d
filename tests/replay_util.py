"""Helpers that build traces, drive ``bin/trace_run`` as a user would, and
compare what it wrote with the plain implementation."""

from __future__ import annotations

import json
import random
import subprocess
import sys
from pathlib import Path

import numpy as np
import torch

import plain_qwen3 as plain

ROOT = Path(__file__).resolve().parent.parent
TRACE_RUN = ROOT / "bin" / "trace_run"


def run_trace(folder, dtype, steps, max_tokens, out_dir, page_size=None, timeout=240):
    """Feed ``steps`` one by one (each after the last ``done`` line); return
    {step: float32 array [wanted, vocab]}."""
    cmd = [sys.executable, str(TRACE_RUN), "--model", str(folder), "--dtype", dtype,
           "--out", str(out_dir), "--max-tokens", str(max_tokens)]
    if page_size is not None:
        cmd += ["--page-size", str(page_size)]
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, bufsize=1)
    try:
        for rec in steps:
            proc.stdin.write(json.dumps(rec) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline()
            if line.strip() != f"done {rec['step']}":
                raise AssertionError(f"expected 'done {rec['step']}', got {line!r} (exit {proc.poll()})")
        proc.stdin.close()
        assert proc.wait(timeout=timeout) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    vocab = json.loads((Path(folder) / "config.json").read_text())["vocab_size"]
    out = {}
    for rec in steps:
        wanted = sum(len(e.get("want", [])) for e in rec["entries"])
        path = Path(out_dir) / f"{rec['step']}.f32"
        if wanted:
            out[rec["step"]] = np.fromfile(path, dtype="<f4").reshape(wanted, vocab)
        else:
            assert not path.exists()
    return out


def random_ids(vocab, length, seed):
    return torch.randint(0, vocab, (length,), generator=torch.Generator().manual_seed(seed)).tolist()


# -- trace shapes ---------------------------------------------------------------
def whole(requests):
    """Each request alone and whole, one after the other."""
    return [{"step": i, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}], "end": [rid]}
            for i, (rid, toks) in enumerate(requests.items())]


def tail_one_by_one(rid, toks, tail=32):
    """Most of it in one step, the last ``tail`` tokens one by one."""
    head = max(1, len(toks) - tail)
    steps = [{"step": 0, "entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))}], "end": []}]
    for i in range(head, len(toks)):
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": [toks[i]], "want": [0]}], "end": []})
    steps[-1]["end"] = [rid]
    return steps


def portions(rid, toks, sizes=(16, 7, 2, 5, 3, 2, 11, 2, 64, 1, 9)):
    """Portions of changing size, down to two tokens."""
    steps, at, i = [], 0, 0
    while at < len(toks):
        n = min(sizes[i % len(sizes)], len(toks) - at)
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[at:at + n], "want": list(range(n))}], "end": []})
        at += n
        i += 1
    steps[-1]["end"] = [rid]
    return steps


def mixed(requests, seed, max_live=4, tail=6):
    """Up to ``max_live`` live requests; portions of some beside single decoded
    tokens of others; requests are sometimes left out of a step; finished ones
    end and later ones take their pages.  Returns (steps, max_tokens)."""
    rng = random.Random(seed)
    pending = list(requests.items())
    live: dict[str, int] = {}
    steps = []
    peak = 0
    while pending or live:
        while pending and len(live) < max_live and (not live or rng.random() < 0.6):
            rid, _ = pending.pop(0)
            live[rid] = 0
        entries = []
        for rid in list(live):
            toks = requests[rid]
            done = live[rid]
            if len(live) > 1 and rng.random() < 0.2:
                continue                                   # left out of this step
            left = len(toks) - done
            n = 1 if left <= tail else min(rng.choice([2, 3, 5, 8, 13, 16, 21, 40]), left - tail)
            entries.append({"id": rid, "tokens": toks[done:done + n], "want": list(range(n))})
            live[rid] = done + n
        if not entries:
            continue
        peak = max(peak, sum(-(-n // 64) * 64 for n in live.values()))
        ended = [rid for rid in live if live[rid] == len(requests[rid])]
        for rid in ended:
            del live[rid]
        steps.append({"step": len(steps), "entries": entries, "end": ended})
    return steps, peak


# -- comparison ---------------------------------------------------------------
def expected_logits(folder, requests):
    cfg, w = plain.read_folder(folder)
    return {rid: plain.logits(toks, cfg, w).numpy() for rid, toks in requests.items()}


def compare(steps, got, expected, tol_abs, tol_rel_to_scale=0.0):
    """Every wanted row of every step against the plain logits at that request's
    position.  Returns the worst error; raises naming the first bad place."""
    cursor = {rid: 0 for rid in expected}
    worst = 0.0
    for rec in steps:
        row = 0
        for e in rec["entries"]:
            start = cursor[e["id"]]
            for w in e.get("want", []):
                want = expected[e["id"]][start + w]
                have = got[rec["step"]][row]
                tol = tol_abs + tol_rel_to_scale * float(np.abs(want).max())
                err = float(np.abs(have - want).max())
                if not err <= tol:
                    raise AssertionError(
                        f"step {rec['step']}: request {e['id']!r} position {start + w} "
                        f"(offset {w} of a portion of {len(e['tokens'])} starting at {start}): "
                        f"max abs err {err} > {tol}")
                worst = max(worst, err)
                row += 1
            cursor[e["id"]] = start + len(e["tokens"])
    return worst


TOL = {"float32": dict(tol_abs=5e-5), "bfloat16": dict(tol_abs=2e-3, tol_rel_to_scale=2e-2)}
