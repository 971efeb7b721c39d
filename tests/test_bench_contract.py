"""The part of the bench.py contract that needs no GPU: more than one GPU is refused
with one line and exit code 2, before anything heavy is imported."""

import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent


def test_more_than_one_gpu_is_refused_with_one_line_and_code_2():
    proc = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2", "--steps", "3", "--warmup", "1"],
                          capture_output=True, text=True, timeout=120)
    assert proc.returncode == 2
    lines = [line for line in proc.stdout.splitlines() if line.strip()]
    assert len(lines) == 1 and "one GPU" in lines[0]
