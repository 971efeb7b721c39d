"""Qwen3 dense: typed config from ``config.json`` keys, and its model plan.

Architecture (reference: src/tokamak/model/transformer.py:22-176): token
embedding; per layer RMSNorm -> grouped-query attention with per-head RMSNorm of
queries and keys before a half-split rotary encoding -> residual, RMSNorm ->
SwiGLU feed-forward -> residual; final RMSNorm; linear head, optionally sharing
the embedding matrix.  No biases anywhere.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

from tokamak_amd.config.model_config import (
    LayerSpec,
    ModelPlan,
    PartSpec,
    SubPart,
    default_order,
)
from tokamak_amd.config.registry import Architecture, register_architecture

NAME = "Qwen3ForCausalLM"


@dataclass(frozen=True)
class Qwen3Config:
    """Fields and defaults follow reference: src/tokamak/config.py:98-125."""

    architecture: str
    vocab_size: int
    hidden_size: int
    num_layers: int
    num_attention_heads: int
    num_kv_heads: int
    head_dim: int
    intermediate_size: int
    rms_norm_eps: float
    rope_theta: float
    max_position_embeddings: int
    tie_word_embeddings: bool
    eos_token_ids: tuple[int, ...] = ()

    def __post_init__(self) -> None:
        # reference: src/tokamak/config.py:68-73
        if self.num_attention_heads % self.num_kv_heads != 0:
            raise ValueError(
                f"num_attention_heads ({self.num_attention_heads}) must be divisible "
                f"by num_kv_heads ({self.num_kv_heads})"
            )
        if self.head_dim % 2 != 0:
            raise ValueError(f"head_dim ({self.head_dim}) must be even for rotary encoding")
        for name in ("vocab_size", "hidden_size", "num_layers", "num_attention_heads",
                     "num_kv_heads", "head_dim", "intermediate_size", "max_position_embeddings"):
            if getattr(self, name) < 1:
                raise ValueError(f"{name} must be >= 1, got {getattr(self, name)}")

    @property
    def num_kv_groups(self) -> int:
        return self.num_attention_heads // self.num_kv_heads


def _rope_theta(raw: dict[str, Any]) -> float:
    """reference: src/tokamak/config.py:129-157 (both config layouts; scaling is an error)."""
    rope_parameters = raw.get("rope_parameters")
    if isinstance(rope_parameters, dict):
        rope_type = rope_parameters.get("rope_type", "default")
        if rope_type != "default":
            raise ValueError(f"RoPE scaling type {rope_type!r} is not supported")
        theta = rope_parameters.get("rope_theta")
        if theta is not None:
            return float(theta)
    theta = raw.get("rope_theta")
    if theta is not None:
        if raw.get("rope_scaling") is not None:
            raise ValueError(f"RoPE scaling is not supported (got {raw['rope_scaling']!r})")
        return float(theta)
    raise ValueError("Could not determine rope_theta from the model config")


def _required(raw: dict[str, Any], key: str) -> Any:
    if key not in raw or raw[key] is None:
        raise ValueError(f"config.json lacks required key {key!r}")
    return raw[key]


def parse(raw: dict[str, Any], eos_token_ids: tuple[int, ...] = ()) -> Qwen3Config:
    names = raw.get("architectures") or []
    name = names[0] if names else "<missing>"
    if name != NAME:
        raise ValueError(f"Unsupported architecture {name!r}; supported: {NAME}")
    if raw.get("attention_bias", False):
        raise ValueError("attention_bias=true is not part of Qwen3 dense")
    if raw.get("use_sliding_window", False):
        raise ValueError("use_sliding_window=true is not supported (full causal attention only)")
    if raw.get("hidden_act", "silu") != "silu":
        raise ValueError(f"hidden_act must be 'silu', got {raw['hidden_act']!r}")
    num_heads = int(_required(raw, "num_attention_heads"))
    hidden = int(_required(raw, "hidden_size"))
    head_dim = raw.get("head_dim")
    if head_dim is None:
        head_dim = hidden // num_heads
    num_kv = raw.get("num_key_value_heads")
    return Qwen3Config(
        architecture=name,
        vocab_size=int(_required(raw, "vocab_size")),
        hidden_size=hidden,
        num_layers=int(_required(raw, "num_hidden_layers")),
        num_attention_heads=num_heads,
        num_kv_heads=int(num_heads if num_kv is None else num_kv),
        head_dim=int(head_dim),
        intermediate_size=int(_required(raw, "intermediate_size")),
        rms_norm_eps=float(_required(raw, "rms_norm_eps")),
        rope_theta=_rope_theta(raw),
        max_position_embeddings=int(_required(raw, "max_position_embeddings")),
        tie_word_embeddings=bool(raw.get("tie_word_embeddings", False)),
        eos_token_ids=tuple(int(t) for t in eos_token_ids),
    )


def to_config_json(cfg: Qwen3Config) -> dict[str, Any]:
    """The ``config.json`` dict that parses back to ``cfg``."""
    return {
        "architectures": [cfg.architecture],
        "model_type": "qwen3",
        "vocab_size": cfg.vocab_size,
        "hidden_size": cfg.hidden_size,
        "num_hidden_layers": cfg.num_layers,
        "num_attention_heads": cfg.num_attention_heads,
        "num_key_value_heads": cfg.num_kv_heads,
        "head_dim": cfg.head_dim,
        "intermediate_size": cfg.intermediate_size,
        "rms_norm_eps": cfg.rms_norm_eps,
        "rope_theta": cfg.rope_theta,
        "max_position_embeddings": cfg.max_position_embeddings,
        "tie_word_embeddings": cfg.tie_word_embeddings,
        "attention_bias": False,
        "hidden_act": "silu",
        "use_sliding_window": False,
    }


def plan(cfg: Qwen3Config) -> ModelPlan:
    norm = PartSpec.of("rmsnorm", dim=cfg.hidden_size, eps=cfg.rms_norm_eps)
    position = PartSpec.of("rotary_half", rotary_dim=cfg.head_dim, theta=cfg.rope_theta)
    mixer = PartSpec.of(
        "gqa_attention",
        hidden_size=cfg.hidden_size,
        num_heads=cfg.num_attention_heads,
        num_kv_heads=cfg.num_kv_heads,
        head_dim=cfg.head_dim,
        qk_norm_eps=cfg.rms_norm_eps,
        softmax_scale=float(cfg.head_dim) ** -0.5,
        window=None,
    )
    feed_forward = PartSpec.of(
        "swiglu", hidden_size=cfg.hidden_size, intermediate_size=cfg.intermediate_size
    )
    # checkpoint names as the reference's module tree gives them (transformer.py:1-6)
    layer = LayerSpec.of(
        PartSpec.of("pre_norm"),
        mixer_norm=SubPart("norm", norm, "input_layernorm."),
        mixer=SubPart("mixer", mixer, "self_attn."),
        feed_forward_norm=SubPart("norm", norm, "post_attention_layernorm."),
        feed_forward=SubPart("feed_forward", feed_forward, "mlp."),
        position=SubPart("position", position, shared=True),
    )
    return ModelPlan(
        vocab_size=cfg.vocab_size,
        hidden_size=cfg.hidden_size,
        max_position_embeddings=cfg.max_position_embeddings,
        tie_word_embeddings=cfg.tie_word_embeddings,
        embedding=PartSpec.of("token_embedding", vocab_size=cfg.vocab_size, dim=cfg.hidden_size),
        layers=(layer,) * cfg.num_layers,
        order=default_order(cfg.num_layers),
        final_norm=norm,
        head=PartSpec.of("linear_head", vocab_size=cfg.vocab_size, dim=cfg.hidden_size,
                         tied=cfg.tie_word_embeddings),
        embedding_prefix="model.embed_tokens.",
        layer_prefix="model.layers.{}.",
        final_norm_prefix="model.norm.",
        head_prefix="lm_head.",
        eos_token_ids=cfg.eos_token_ids,
    )


def chat_prompt(user_text: str) -> str:
    """A single user turn in the ChatML form Qwen3 checkpoints are trained on, with
    the empty think block that switches reasoning off (what the reference's example
    asks its tokenizer's template for with enable_thinking=False,
    examples/basic_generation.py:25-30).  Used when the model folder brings no
    template of its own."""
    return f"<|im_start|>user\n{user_text}<|im_end|>\n<|im_start|>assistant\n<think>\n\n</think>\n\n"


def _shape(vocab, hidden, layers, heads, kv, hd, inter, theta, max_pos, tied, eps=1e-6) -> Qwen3Config:
    return Qwen3Config(NAME, vocab, hidden, layers, heads, kv, hd, inter, eps, theta, max_pos, tied)


# Shapes for the random-weights mode (sizes only; no trained weights exist here).
PRESETS = {
    "tiny-a": _shape(256, 64, 2, 4, 2, 16, 128, 10000.0, 128, True),
    "tiny-b": _shape(384, 96, 3, 6, 3, 32, 200, 1000000.0, 256, False, eps=1e-5),
    "qwen3-0.6b": _shape(151936, 1024, 28, 16, 8, 128, 3072, 1000000.0, 40960, True),
    "qwen3-1.7b": _shape(151936, 2048, 28, 16, 8, 128, 6144, 1000000.0, 40960, True),
    "qwen3-4b": _shape(151936, 2560, 36, 32, 8, 128, 9728, 1000000.0, 40960, True),
    "qwen3-8b": _shape(151936, 4096, 36, 32, 8, 128, 12288, 1000000.0, 40960, False),
    "qwen3-14b": _shape(151936, 5120, 40, 40, 8, 128, 17408, 1000000.0, 40960, False),
    "qwen3-32b": _shape(151936, 5120, 64, 64, 8, 128, 25600, 1000000.0, 40960, False),
}


register_architecture(Architecture(name=NAME, parse=parse, plan=plan, to_json=to_config_json,
                                   presets=PRESETS, chat_prompt=chat_prompt))
