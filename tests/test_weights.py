"""Loader errors and the random-weights folder writer."""

import json

import pytest
import torch
from safetensors import safe_open
from safetensors.torch import load_file, save_file

from tiny import TINIES, make_folder
from tokamak_amd.config import load_model_description
from tokamak_amd.engine.model import LayeredModel
from tokamak_amd.weights import SafetensorsSource, WeightError, load_weights, write_random_model


def _model(folder, dtype=torch.float32):
    _, _, plan = load_model_description(folder)
    return LayeredModel(plan, dtype=dtype, device="cpu")


def test_random_folder_has_config_and_bf16_tensors(tmp_path):
    folder = make_folder(tmp_path, "B")
    assert (folder / "config.json").is_file() and (folder / "model.safetensors").is_file()
    tensors = load_file(folder / "model.safetensors")
    assert all(t.dtype == torch.bfloat16 for t in tensors.values())
    cfg = TINIES["B"]["config"]
    assert tensors["model.layers.2.self_attn.q_proj.weight"].shape == (cfg.num_attention_heads * cfg.head_dim, cfg.hidden_size)
    assert tensors["model.layers.0.self_attn.k_norm.weight"].shape == (cfg.head_dim,)
    assert tensors["lm_head.weight"].shape == (cfg.vocab_size, cfg.hidden_size)
    assert "model.rotary_emb.inv_freq" not in tensors
    # statistics of the two kinds of tensors
    w = tensors["model.layers.1.mlp.down_proj.weight"].float()
    assert abs(w.std().item() - 0.03) < 0.003 and abs(w.mean().item()) < 0.003
    n = tensors["model.norm.weight"].float()
    assert abs(n.mean().item() - 1.0) < 0.05 and 0.05 < n.std().item() < 0.15


def test_same_seed_same_bytes_other_seed_differs(tmp_path):
    cfg = TINIES["A"]["config"]
    a = load_file(write_random_model(tmp_path / "a", cfg, 3) / "model.safetensors")
    b = load_file(write_random_model(tmp_path / "b", cfg, 3) / "model.safetensors")
    c = load_file(write_random_model(tmp_path / "c", cfg, 4) / "model.safetensors")
    assert all(torch.equal(a[k], b[k]) for k in a)
    assert not torch.equal(a["model.embed_tokens.weight"], c["model.embed_tokens.weight"])


def test_tied_folder_has_no_lm_head_and_loads(tmp_path):
    folder = make_folder(tmp_path, "A")
    assert "lm_head.weight" not in load_file(folder / "model.safetensors")
    model = _model(folder)
    n = load_weights(model, SafetensorsSource(folder), dtype=torch.float32, device="cpu")
    assert n == len(load_file(folder / "model.safetensors"))
    assert model.head.weight.data_ptr() == model.embedding.weight.data_ptr()  # the embedding itself


def test_tied_folder_with_its_own_lm_head_copy_loads(tmp_path):
    folder = make_folder(tmp_path, "A")
    tensors = load_file(folder / "model.safetensors")
    tensors["lm_head.weight"] = tensors["model.embed_tokens.weight"].clone()
    save_file(tensors, str(folder / "model.safetensors"))
    model = _model(folder)
    load_weights(model, SafetensorsSource(folder), dtype=torch.float32, device="cpu")
    assert model.head.weight.data_ptr() == model.embedding.weight.data_ptr()


def test_dtype_by_role(tmp_path):
    folder = make_folder(tmp_path, "B")
    model = _model(folder, torch.bfloat16)
    load_weights(model, SafetensorsSource(folder), dtype=torch.bfloat16, device="cpu")
    block = model.blocks[0]
    assert block.mixer.qkv.dtype == torch.bfloat16 and model.embedding.weight.dtype == torch.bfloat16
    assert block.mixer_norm.weight.dtype == torch.float32       # vectors are held in 32-bit
    assert block.mixer.q_norm.dtype == torch.float32
    cfg = TINIES["B"]["config"]
    assert block.mixer.qkv.shape == ((cfg.num_attention_heads + 2 * cfg.num_kv_heads) * cfg.head_dim, cfg.hidden_size)
    assert block.feed_forward.gate_up.shape == (2 * cfg.intermediate_size, cfg.hidden_size)


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    folder = make_folder(tmp_path, "B")
    tensors = load_file(folder / "model.safetensors")
    del tensors["model.layers.1.mlp.up_proj.weight"]
    del tensors["lm_head.weight"]                                  # untied: it is required
    tensors["model.layers.0.self_attn.q_proj.bias"] = torch.zeros(4)
    tensors["model.norm.weight"] = torch.ones(7)
    save_file(tensors, str(folder / "model.safetensors"))
    with pytest.raises(WeightError) as err:
        load_weights(_model(folder), SafetensorsSource(folder), dtype=torch.float32, device="cpu")
    e = err.value
    assert e.missing == ["lm_head.weight", "model.layers.1.mlp.up_proj.weight"]
    assert e.unexpected == ["model.layers.0.self_attn.q_proj.bias"]
    assert [m[0] for m in e.mismatched] == ["model.norm.weight"]
    text = str(e)
    for needle in ("missing tensors (2)", "unexpected tensors (1)", "model.norm.weight", "(7,)", "(96,)"):
        assert needle in text


def test_no_safetensors_is_file_not_found(tmp_path):
    folder = make_folder(tmp_path, "A")
    (folder / "model.safetensors").unlink()
    with pytest.raises(FileNotFoundError, match="safetensors"):
        SafetensorsSource(folder)


def test_float32_checkpoint_converts_to_compute_dtype(tmp_path):
    cfg = TINIES["A"]["config"]
    folder = write_random_model(tmp_path / "f32", cfg, 0, dtype=torch.float32)
    with safe_open(folder / "model.safetensors", framework="pt") as f:
        assert f.get_tensor("model.norm.weight").dtype == torch.float32
    model = _model(folder, torch.bfloat16)
    load_weights(model, SafetensorsSource(folder), dtype=torch.bfloat16, device="cpu")
    assert model.embedding.weight.dtype == torch.bfloat16
    assert model.final_norm.weight.dtype == torch.float32  # stored in 32-bit, stays so
    stored = load_file(folder / "model.safetensors")["model.norm.weight"]
    assert torch.equal(model.final_norm.weight, stored)


def test_a_tensor_is_held_as_its_spec_says_whatever_its_role():
    """Matrices in the compute dtype, vectors in float32, tables as int32 by habit; ``held``
    overrides that without changing what kind of numbers the tensor is."""
    from tokamak_amd.weights.loader import target_dtype
    from tokamak_amd.weights.spec import TensorSpec

    bf16, f32 = torch.bfloat16, torch.float32
    assert target_dtype(TensorSpec((4, 4)), bf16, bf16) == bf16
    assert target_dtype(TensorSpec((4, 4)), f32, bf16) == bf16
    assert target_dtype(TensorSpec((4,), role="vector"), bf16, bf16) == f32
    assert target_dtype(TensorSpec((4,), role="table"), torch.int64, bf16) == torch.int32
    router = TensorSpec((2, 4), held="float32")                # a matrix that must not be rounded
    assert router.role == "matrix" and target_dtype(router, f32, bf16) == f32
    assert target_dtype(TensorSpec((4, 4), held="stored"), torch.float16, bf16) == torch.float16
    assert target_dtype(TensorSpec((4,), role="vector", held="compute"), f32, bf16) == bf16
    with pytest.raises(ValueError, match="held"):
        TensorSpec((4,), held="float64")
    with pytest.raises(ValueError, match="role"):
        TensorSpec((4,), role="scalar")
