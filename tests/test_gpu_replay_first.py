"""First end-to-end check on the GPU: whole prompts through the step function
equal the plain implementation, in float32 and in bfloat16."""

import pytest
import torch

import plain_qwen3 as plain
from tiny import TINIES, make_folder

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("which", ["A", "B", "C"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompt_matches_plain(tmp_path, which, dtype):
    from tokamak_amd.engine.runner import ModelRunner, StepEntry

    folder = make_folder(tmp_path, which)
    cfg, w = plain.read_folder(folder)
    gen = torch.Generator().manual_seed(7)
    runner = ModelRunner.from_folder(folder, dtype=dtype, page_size=TINIES[which]["page_size"],
                                     kv_pool_tokens=256)
    for length in (1, 5, 17, 33, 70):
        ids = torch.randint(0, cfg["vocab_size"], (length,), generator=gen).tolist()
        want = plain.logits(ids, cfg, w)
        got = runner.step([StepEntry("r", ids, list(range(length)))]).cpu()
        runner.end("r")
        tol = 2e-4 if dtype == "float32" else 6e-2
        err = (got - want).abs().max().item()
        print(which, dtype, length, "max abs err", err, "logit scale", want.abs().max().item())
        assert err < tol, f"{which} {dtype} len {length}: max abs err {err}"
