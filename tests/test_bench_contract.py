"""The part of the bench.py contract that needs no GPU: more than one GPU is refused
with one line and exit code 2, before anything heavy is imported; and the reference's
throughput trace is the published one."""

import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT))


def test_more_than_one_gpu_is_refused_with_one_line_and_code_2():
    proc = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2", "--steps", "3", "--warmup", "1"],
                          capture_output=True, text=True, timeout=120)
    assert proc.returncode == 2
    lines = [line for line in proc.stdout.splitlines() if line.strip()]
    assert len(lines) == 1 and "one GPU" in lines[0]


def test_the_reference_trace_has_the_published_totals():
    # 32 requests, cap 256, seed 0: 4,915 prompt and 2,901 output tokens
    # (reference: benchmarks/README.md:87-90); every prompt 16..512 tokens, every request
    # within the 1,024 tokens the measurement allows a sequence
    import bench

    prompts, new_tokens = bench.reference_trace(32, 256, 0, 151_936)
    assert len(prompts) == len(new_tokens) == 32
    assert sum(map(len, prompts)) == 4915 and sum(new_tokens) == 2901
    assert all(16 <= len(p) <= 512 for p in prompts) and all(8 <= n <= 256 for n in new_tokens)
    assert all(0 <= t < 151_643 for p in prompts for t in p)
    assert max(len(p) + n for p, n in zip(prompts, new_tokens)) <= 1024
    again, _ = bench.reference_trace(32, 256, 0, 151_936)
    assert again == prompts
