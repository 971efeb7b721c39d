"""Configuration and registry (scenarios of reference tests/unit/test_config.py:29-138)."""

import json

import pytest

from tokamak_amd.config import (
    Architecture, LayerCall, ModelPlan, PartSpec, get_architecture, get_part,
    load_model_description, register_architecture, supported_architectures,
)
from tokamak_amd.models import qwen3


def raw(**over):
    d = {
        "architectures": ["Qwen3ForCausalLM"], "vocab_size": 1000, "hidden_size": 64,
        "num_hidden_layers": 2, "num_attention_heads": 4, "num_key_value_heads": 2,
        "head_dim": 32, "intermediate_size": 128, "rms_norm_eps": 1e-6, "rope_theta": 1e6,
        "max_position_embeddings": 512, "tie_word_embeddings": True,
    }
    d.update(over)
    return {k: v for k, v in d.items() if v is not ...}


def test_qwen3_sample_parses():
    cfg = qwen3.parse(raw(), (7,))
    assert cfg.architecture == "Qwen3ForCausalLM"
    assert cfg.head_dim == 32  # decoupled from hidden_size / num_heads
    assert cfg.rope_theta == 1e6
    assert cfg.tie_word_embeddings
    assert cfg.num_kv_groups == 2
    assert cfg.eos_token_ids == (7,)


def test_defaults_when_keys_absent():
    cfg = qwen3.parse(raw(head_dim=..., num_key_value_heads=..., tie_word_embeddings=...))
    assert cfg.head_dim == 16           # hidden_size // num_heads
    assert cfg.num_kv_heads == 4        # = num_attention_heads
    assert cfg.tie_word_embeddings is False


def test_rope_theta_in_rope_parameters_layout():
    cfg = qwen3.parse(raw(rope_theta=..., rope_parameters={"rope_type": "default", "rope_theta": 5e5}))
    assert cfg.rope_theta == 5e5


@pytest.mark.parametrize("over, match", [
    (dict(rope_theta=...), "rope_theta"),
    (dict(rope_scaling={"type": "linear", "factor": 2.0}), "scaling"),
    (dict(rope_theta=..., rope_parameters={"rope_type": "yarn", "rope_theta": 1e6}), "yarn"),
    (dict(num_attention_heads=6, num_key_value_heads=4), "divisible"),
    (dict(architectures=["LlamaForCausalLM"]), "Unsupported architecture"),
    (dict(attention_bias=True), "attention_bias"),
    (dict(use_sliding_window=True), "sliding"),
    (dict(hidden_act="gelu"), "hidden_act"),
    (dict(head_dim=15), "even"),
    (dict(vocab_size=...), "vocab_size"),
])
def test_bad_configs_raise(over, match):
    with pytest.raises(ValueError, match=match):
        qwen3.parse(raw(**over))


def test_registry_rejects_unknown_names_and_lists_supported():
    with pytest.raises(ValueError, match="Unsupported architecture 'NopeForCausalLM'; supported: .*Qwen3ForCausalLM"):
        get_architecture("NopeForCausalLM")
    assert "Qwen3ForCausalLM" in supported_architectures()
    with pytest.raises(ValueError, match="unknown mixer part"):
        get_part("mixer", "does_not_exist")
    with pytest.raises(ValueError, match="already registered"):
        register_architecture(Architecture("Qwen3ForCausalLM", qwen3.parse, qwen3.plan))


def test_config_json_round_trip(tmp_path):
    cfg = qwen3.parse(raw(), ())
    (tmp_path / "config.json").write_text(json.dumps(qwen3.to_config_json(cfg)))
    (tmp_path / "generation_config.json").write_text(json.dumps({"eos_token_id": [3, 9]}))
    arch, parsed, plan = load_model_description(tmp_path)
    assert arch.name == "Qwen3ForCausalLM"
    assert parsed == qwen3.parse(raw(), (3, 9))
    assert plan.eos_token_ids == (3, 9)


def test_eos_as_single_int(tmp_path):
    cfg = qwen3.parse(raw(), ())
    (tmp_path / "config.json").write_text(json.dumps(qwen3.to_config_json(cfg)))
    (tmp_path / "generation_config.json").write_text(json.dumps({"eos_token_id": 5}))
    assert load_model_description(tmp_path)[2].eos_token_ids == (5,)


def test_plan_carries_every_number_as_part_parameters():
    cfg = qwen3.parse(raw(), ())
    plan = qwen3.plan(cfg)
    assert len(plan.layers) == 2 and [c.layer for c in plan.order] == [0, 1]
    layer = plan.layers[0]
    assert [role for role, _ in layer.parts] == ["mixer_norm", "mixer", "feed_forward_norm", "feed_forward", "position"]
    assert layer.block.kind == "pre_norm"
    mixer = layer.role("mixer").spec
    assert mixer.kind == "gqa_attention" and layer.role("mixer").prefix == "self_attn."
    assert mixer["head_dim"] == 32 and mixer["num_kv_heads"] == 2
    assert mixer["softmax_scale"] == 32 ** -0.5   # the configured head_dim, not hidden/heads
    assert mixer["qk_norm_eps"] == 1e-6
    position = layer.role("position")
    assert position.spec.kind == "rotary_half" and position.spec.as_dict() == {"rotary_dim": 32, "theta": 1e6}
    assert position.shared and position.prefix == ""
    assert layer.role("feed_forward").spec["intermediate_size"] == 128
    assert layer.role("mixer_norm").spec["eps"] == 1e-6
    assert plan.head["tied"] is True


def test_run_order_is_validated_data():
    spec = qwen3.plan(qwen3.parse(raw(), ()))
    kw = dict(vocab_size=10, hidden_size=8, max_position_embeddings=16, tie_word_embeddings=False,
              embedding=spec.embedding, layers=spec.layers, final_norm=spec.final_norm, head=spec.head,
              embedding_prefix="e.", layer_prefix="l.{}.", final_norm_prefix="n.", head_prefix="h.")
    ModelPlan(order=(LayerCall(0, 0), LayerCall(1, 1), LayerCall(0, 2), LayerCall(1, 0, writes_cache=False)), **kw)
    with pytest.raises(ValueError, match="names layer 5"):
        ModelPlan(order=(LayerCall(5, 0),), **kw)
    with pytest.raises(ValueError, match="never written"):
        ModelPlan(order=(LayerCall(0, 0), LayerCall(1, 3, writes_cache=False)), **kw)


def test_partspec_is_hashable_and_frozen():
    a = PartSpec.of("x", b=2, a=[1, 2])
    assert a == PartSpec.of("x", a=(1, 2), b=2) and hash(a) == hash(PartSpec.of("x", a=(1, 2), b=2))
    assert a.as_dict() == {"a": (1, 2), "b": 2}


# -- where the EOS ids come from (reference src/tokamak/engine/llm.py:244-263) ---------
def _folder(tmp_path, generation=None, config_eos=..., tokenizer=False):
    from tokamak_amd.config import read_eos_token_ids

    cfg = qwen3.to_config_json(qwen3.parse(raw(), ()))
    if config_eos is not ...:
        cfg["eos_token_id"] = config_eos
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    if generation is not None:
        (tmp_path / "generation_config.json").write_text(json.dumps(generation))
    if tokenizer:
        (tmp_path / "tokenizer_config.json").write_text(json.dumps({"eos_token": "<|end|>"}))
        (tmp_path / "tokenizer.json").write_text(json.dumps(
            {"added_tokens": [{"id": 901, "content": "<|end|>"}], "model": {"vocab": {"a": 0}}}))
    return read_eos_token_ids(tmp_path)


def test_eos_from_generation_config_int_or_list(tmp_path):
    assert _folder(tmp_path, generation={"eos_token_id": 5}, config_eos=9, tokenizer=True) == (5,)
    assert _folder(tmp_path, generation={"eos_token_id": [5, 6]}) == (5, 6)


def test_eos_falls_back_to_config_json_then_to_the_tokenizer(tmp_path):
    assert _folder(tmp_path, generation={"temperature": 0.6}, config_eos=[9, 10], tokenizer=True) == (9, 10)
    (tmp_path / "generation_config.json").unlink()
    assert _folder(tmp_path, config_eos=9, tokenizer=True) == (9,)
    assert _folder(tmp_path, tokenizer=True) == (901,)          # the tokenizer's eos_token, looked up by text
    assert load_model_description(tmp_path)[2].eos_token_ids == (901,)


def test_no_eos_anywhere_means_requests_stop_on_length(tmp_path):
    assert _folder(tmp_path) == ()
    assert _folder(tmp_path, generation={"eos_token_id": True}) == ()     # a bool is no token id


# -- presets and the chat prompt come through the registry -------------------------------
def test_presets_are_found_by_name_through_the_registry():
    from tokamak_amd.config import find_preset, preset_names

    assert {"tiny-a", "tiny-b", "qwen3-0.6b", "qwen3-8b", "qwen3-32b"} <= set(preset_names())
    arch, cfg = find_preset("qwen3-8b")
    assert arch.name == "Qwen3ForCausalLM" and cfg.hidden_size == 4096 and cfg.num_layers == 36
    with pytest.raises(ValueError, match="unknown preset 'nope'.*tiny-a"):
        find_preset("nope")


def test_architecture_brings_its_chat_prompt():
    text = get_architecture("Qwen3ForCausalLM").chat_prompt("hi")
    assert text.startswith("<|im_start|>user\nhi<|im_end|>") and text.endswith("<think>\n\n</think>\n\n")


def test_entry_points_name_no_architecture():
    """The command line and the benchmark reach shapes and models through the registry."""
    from pathlib import Path

    root = Path(__file__).resolve().parent.parent
    for file in (root / "tokamak_amd" / "cli.py", root / "bench.py", root / "bin" / "trace_run",
                 root / "tokamak_amd" / "engine" / "llm.py", root / "tokamak_amd" / "engine" / "runner.py"):
        assert "models.qwen3" not in file.read_text() and "import qwen3" not in file.read_text(), file


def test_a_block_says_which_parts_it_needs():
    import torch

    from tokamak_amd.config import LayerSpec, SubPart
    from tokamak_amd.engine.model import LayeredModel

    plan = qwen3.plan(qwen3.parse(raw(), ()))
    layer = plan.layers[0]
    broken = LayerSpec(tuple((r, p) for r, p in layer.parts if r != "feed_forward_norm")
                       + (("extra", SubPart("norm", layer.role("mixer_norm").spec, "x.")),), layer.block)
    import dataclasses
    with pytest.raises(ValueError, match="missing \\['feed_forward_norm'\\], unknown \\['extra'\\]"):
        LayeredModel(dataclasses.replace(plan, layers=(broken, broken)), dtype=torch.float32, device="meta")
    model = LayeredModel(plan, dtype=torch.float32, device="meta")
    assert model.blocks[0].parts["position"] is model.blocks[1].parts["position"]      # shared: one table a step
    assert model.blocks[0].parts["mixer"] is not model.blocks[1].parts["mixer"]
