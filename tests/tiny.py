"""The tiny test configurations and helpers to make model folders from them."""

from __future__ import annotations

from pathlib import Path

from tokamak_amd.models.qwen3 import Qwen3Config
from tokamak_amd.weights import write_random_model

# Two configurations that differ in every size and option.
TINY_A = dict(
    config=Qwen3Config("Qwen3ForCausalLM", vocab_size=256, hidden_size=64, num_layers=2,
                       num_attention_heads=4, num_kv_heads=2, head_dim=16, intermediate_size=128,
                       rms_norm_eps=1e-6, rope_theta=10000.0, max_position_embeddings=128,
                       tie_word_embeddings=True),
    seed=0, matrix_std=0.02, vector_jitter=0.1, page_size=16)
TINY_B = dict(
    config=Qwen3Config("Qwen3ForCausalLM", vocab_size=384, hidden_size=96, num_layers=3,
                       num_attention_heads=6, num_kv_heads=3, head_dim=32, intermediate_size=200,
                       rms_norm_eps=1e-5, rope_theta=1000000.0, max_position_embeddings=256,
                       tie_word_embeddings=False),
    seed=1, matrix_std=0.03, vector_jitter=0.1, page_size=8)
# A third one with odd sizes: group of 5, head size 48, vocabulary and widths that are no
# power of two, longer context.
TINY_C = dict(
    config=Qwen3Config("Qwen3ForCausalLM", vocab_size=331, hidden_size=120, num_layers=2,
                       num_attention_heads=5, num_kv_heads=1, head_dim=48, intermediate_size=136,
                       rms_norm_eps=3e-6, rope_theta=50000.0, max_position_embeddings=1024,
                       tie_word_embeddings=False),
    seed=2, matrix_std=0.05, vector_jitter=0.2, page_size=16)

TINIES = {"A": TINY_A, "B": TINY_B, "C": TINY_C}


def make_folder(root: Path, which: str, **overrides) -> Path:
    spec = dict(TINIES[which])
    spec.update(overrides)
    folder = Path(root) / f"tiny_{which}"
    return write_random_model(folder, spec["config"], spec["seed"], matrix_std=spec["matrix_std"],
                              vector_jitter=spec["vector_jitter"])
