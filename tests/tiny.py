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

# Three with the head sizes (64, 128) and page sizes (16, 32) that the matrix-core
# attention kernels take: groups of 4, 1 and 6 query heads per kv head.
TINY_D = dict(
    config=Qwen3Config("Qwen3ForCausalLM", vocab_size=300, hidden_size=128, num_layers=2,
                       num_attention_heads=8, num_kv_heads=2, head_dim=64, intermediate_size=192,
                       rms_norm_eps=1e-6, rope_theta=10000.0, max_position_embeddings=1024,
                       tie_word_embeddings=True),
    seed=7, matrix_std=0.05, vector_jitter=0.1, page_size=16)
TINY_E = dict(
    config=Qwen3Config("Qwen3ForCausalLM", vocab_size=263, hidden_size=96, num_layers=2,
                       num_attention_heads=3, num_kv_heads=3, head_dim=128, intermediate_size=160,
                       rms_norm_eps=1e-5, rope_theta=1000000.0, max_position_embeddings=1024,
                       tie_word_embeddings=False),
    seed=8, matrix_std=0.05, vector_jitter=0.1, page_size=32)
TINY_F = dict(
    config=Qwen3Config("Qwen3ForCausalLM", vocab_size=280, hidden_size=64, num_layers=2,
                       num_attention_heads=6, num_kv_heads=1, head_dim=128, intermediate_size=96,
                       rms_norm_eps=1e-6, rope_theta=50000.0, max_position_embeddings=2048,
                       tie_word_embeddings=False),
    seed=9, matrix_std=0.05, vector_jitter=0.1, page_size=16)

TINIES = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D, "E": TINY_E, "F": TINY_F}


def make_folder(root: Path, which: str, **overrides) -> Path:
    spec = dict(TINIES[which])
    spec.update(overrides)
    folder = Path(root) / f"tiny_{which}"
    return write_random_model(folder, spec["config"], spec["seed"], matrix_std=spec["matrix_std"],
                              vector_jitter=spec["vector_jitter"])
