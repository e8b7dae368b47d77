"""CPU: safetensors loading by name, its one error, random weights, folder writing."""

import json

import pytest
import safetensors.torch
import torch

from conftest import TINY_A, TINY_B
from cie_amd.config import config_from_dict
from cie_amd.parts.model import expected_tensors
from cie_amd.weights import RandomSource, SafetensorsSource, WeightError, write_model_folder, write_tensors


def expected_of(raw):
    return expected_tensors(config_from_dict(raw).model_spec())


def test_expected_names_are_the_checkpoint_names():
    names = expected_of(TINY_B)
    assert names["model.embed_tokens.weight"].shape == (515, 96)
    assert names["lm_head.weight"].shape == (515, 96) and names["model.norm.weight"].shape == (96,)
    assert names["model.layers.2.self_attn.q_proj.weight"].shape == (96, 96)
    assert names["model.layers.2.self_attn.k_proj.weight"].shape == (32, 96)
    assert names["model.layers.0.self_attn.v_proj.bias"].shape == (32,)
    assert names["model.layers.1.mlp.gate_proj.weight"].shape == (328, 96)
    assert names["model.layers.1.mlp.down_proj.weight"].shape == (96, 328)
    assert names["model.layers.1.post_attention_layernorm.weight"].init == "norm"
    assert "lm_head.weight" not in expected_of(TINY_A)  # tied
    assert "model.layers.0.self_attn.q_proj.bias" not in expected_of(dict(TINY_A, attention_bias=False))
    assert len(names) == 3 + 3 * 12


def test_round_trip_keeps_bfloat16_and_values(tmp_path):
    config = config_from_dict(TINY_A)
    write_model_folder(tmp_path, config, seed=3)
    assert json.loads((tmp_path / "config.json").read_text())["hidden_size"] == 64
    expected = expected_of(TINY_A)
    loaded = SafetensorsSource(tmp_path).load(expected, "bfloat16", "cpu")
    drawn = RandomSource(3).load(expected, "bfloat16", "cpu")
    assert list(loaded) == list(expected)
    for name in expected:
        assert loaded[name].dtype == torch.bfloat16 and torch.equal(loaded[name], drawn[name])
    wide = SafetensorsSource(tmp_path).load(expected, "float32", "cpu")
    assert all(t.dtype == torch.float32 for t in wide.values())
    assert torch.equal(wide["model.norm.weight"], loaded["model.norm.weight"].float())


def test_random_weights_follow_seed_and_distribution():
    expected = expected_of(TINY_B)
    a, b, c = (RandomSource(s).load(expected, "float32", "cpu") for s in (1, 1, 2))
    assert all(torch.equal(a[n], b[n]) for n in expected)
    assert not torch.equal(a["lm_head.weight"], c["lm_head.weight"])
    assert abs(a["lm_head.weight"].std().item() - 0.02) < 2e-3 and abs(a["lm_head.weight"].mean().item()) < 2e-3
    assert abs(a["model.norm.weight"].mean().item() - 1.0) < 0.02
    assert not torch.equal(a["model.layers.0.mlp.up_proj.weight"], a["model.layers.0.mlp.gate_proj.weight"])


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    expected = expected_of(TINY_A)
    tensors = RandomSource(0).load(expected, "bfloat16", "cpu")
    del tensors["model.layers.1.mlp.up_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    tensors["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(16, 64, dtype=torch.bfloat16)
    write_tensors(tmp_path, TINY_A, tensors)
    with pytest.raises(WeightError) as caught:
        SafetensorsSource(tmp_path).load(expected, "bfloat16", "cpu")
    error = caught.value
    assert error.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert error.unexpected == ["model.layers.0.self_attn.rotary_emb.inv_freq"]
    assert len(error.wrong_shape) == 1 and "k_proj.weight: expected (32, 64), got (16, 64)" in error.wrong_shape[0]
    text = str(error)
    for piece in ("missing tensors (2)", "unexpected tensors (1)", "wrong shapes (1)", "up_proj", "inv_freq"):
        assert piece in text


def test_no_safetensors_and_duplicates(tmp_path):
    with pytest.raises(FileNotFoundError, match="safetensors"):
        SafetensorsSource(tmp_path)
    expected = expected_of(TINY_A)
    tensors = RandomSource(0).load(expected, "bfloat16", "cpu")
    write_tensors(tmp_path, TINY_A, tensors)
    safetensors.torch.save_file({"model.norm.weight": tensors["model.norm.weight"]}, str(tmp_path / "extra.safetensors"))
    with pytest.raises(ValueError, match="duplicate tensor 'model.norm.weight'"):
        SafetensorsSource(tmp_path).load(expected, "bfloat16", "cpu")


def test_shards_are_read_together(tmp_path):
    expected = expected_of(TINY_A)
    tensors = RandomSource(0).load(expected, "bfloat16", "cpu")
    names = list(tensors)
    (tmp_path / "config.json").write_text(json.dumps(TINY_A))
    safetensors.torch.save_file({n: tensors[n] for n in names[:7]}, str(tmp_path / "model-00001-of-00002.safetensors"))
    safetensors.torch.save_file({n: tensors[n] for n in names[7:]}, str(tmp_path / "model-00002-of-00002.safetensors"))
    loaded = SafetensorsSource(tmp_path).load(expected, "bfloat16", "cpu")
    assert all(torch.equal(loaded[n], tensors[n]) for n in names)


def test_tied_head_in_file_must_equal_embedding(tmp_path):
    expected = expected_of(TINY_A)
    tensors = RandomSource(0).load(expected, "bfloat16", "cpu")
    tied = {"lm_head.weight": "model.embed_tokens.weight"}
    same = dict(tensors, **{"lm_head.weight": tensors["model.embed_tokens.weight"].clone()})
    write_tensors(tmp_path / "same", TINY_A, same)
    loaded = SafetensorsSource(tmp_path / "same").load(expected, "bfloat16", "cpu", tied_optional=tied)
    assert "lm_head.weight" not in loaded
    other = dict(tensors, **{"lm_head.weight": tensors["model.embed_tokens.weight"] * 2})
    write_tensors(tmp_path / "other", TINY_A, other)
    with pytest.raises(WeightError, match="differs from model.embed_tokens.weight"):
        SafetensorsSource(tmp_path / "other").load(expected, "bfloat16", "cpu", tied_optional=tied)
    with pytest.raises(WeightError, match="unexpected"):  # without the tied allowance it is simply unexpected
        SafetensorsSource(tmp_path / "same").load(expected, "bfloat16", "cpu")


def test_tensor_stored_in_32_bit_stays_so(tmp_path):
    expected = expected_of(TINY_A)
    tensors = RandomSource(0).load(expected, "bfloat16", "cpu")
    tensors["model.norm.weight"] = tensors["model.norm.weight"].float() + 1e-4  # not representable in bf16
    write_tensors(tmp_path, TINY_A, tensors)
    loaded = SafetensorsSource(tmp_path).load(expected, "bfloat16", "cpu")
    assert loaded["model.norm.weight"].dtype == torch.float32
    assert torch.equal(loaded["model.norm.weight"], tensors["model.norm.weight"])
    assert loaded["model.layers.0.input_layernorm.weight"].dtype == torch.bfloat16
    assert loaded["model.embed_tokens.weight"].dtype == torch.bfloat16


def test_open_hands_out_tensors_one_by_one_and_checks_the_folder_first(tmp_path):
    config = config_from_dict(TINY_B)
    write_model_folder(tmp_path, config, seed=5)
    expected = expected_of(TINY_B)
    for source in (SafetensorsSource(tmp_path), RandomSource(5)):
        whole = source.load(expected, "bfloat16", "cpu")
        lazy = source.open(expected, "bfloat16", "cpu")
        assert list(lazy) == list(expected) and len(lazy) == len(expected)
        name = "model.layers.1.mlp.down_proj.weight"
        first, second = lazy[name], lazy[name]
        assert torch.equal(first, whole[name]) and first is not second  # made anew each time, not kept
        assert all(torch.equal(lazy[n], whole[n]) for n in reversed(list(expected)))  # in any order
        with pytest.raises(KeyError):
            lazy["model.layers.0.self_attn.rotary_emb.inv_freq"]
    # the folder's faults are reported when it is opened, before a tensor is asked for
    tensors = RandomSource(5).load(expected, "bfloat16", "cpu")
    del tensors["model.norm.weight"]
    write_tensors(tmp_path / "short", TINY_B, tensors)
    with pytest.raises(WeightError, match="missing tensors"):
        SafetensorsSource(tmp_path / "short").open(expected, "bfloat16", "cpu")
