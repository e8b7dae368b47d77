"""Shared fixtures: two tiny Qwen2.5 configurations that differ in every size and
option, model folders with random weights made in a temporary folder, and the
``gpu`` marker."""

from __future__ import annotations

import json
import os
import sys
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))

# Tiny-A: 2 layers, hidden 64, 4 query / 2 KV heads, head 16, tied head.
TINY_A = {
    "architectures": ["Qwen2ForCausalLM"],
    "model_type": "qwen2",
    "hidden_size": 64,
    "num_hidden_layers": 2,
    "num_attention_heads": 4,
    "num_key_value_heads": 2,
    "intermediate_size": 128,
    "vocab_size": 256,
    "rope_theta": 10000.0,
    "rms_norm_eps": 1e-6,
    "attention_bias": True,
    "tie_word_embeddings": True,
    "use_sliding_window": False,
    "max_position_embeddings": 128,
    "eos_token_id": 255,
    "hidden_act": "silu",
}

# Tiny-B: every size and option differs; sizes that are no power of two
# (hidden 96 = 3 heads of 32, intermediate 328, vocabulary 515), one KV head, untied head.
TINY_B = {
    "architectures": ["Qwen2ForCausalLM"],
    "model_type": "qwen2",
    "hidden_size": 96,
    "num_hidden_layers": 3,
    "num_attention_heads": 3,
    "num_key_value_heads": 1,
    "intermediate_size": 328,
    "vocab_size": 515,
    "rope_theta": 1000000.0,
    "rms_norm_eps": 1e-5,
    "attention_bias": True,
    "tie_word_embeddings": False,
    "use_sliding_window": False,
    "max_position_embeddings": 320,
    "eos_token_id": 7,
    "hidden_act": "silu",
}

# Sizes the fast paths refuse: a width and an intermediate size that are no multiples of 8 (no 16-byte rows),
# a head size given in the configuration that is not hidden / heads, five heads on one key head, no biases.
TINY_C = {
    "architectures": ["Qwen2ForCausalLM"],
    "model_type": "qwen2",
    "hidden_size": 100,
    "num_hidden_layers": 2,
    "num_attention_heads": 5,
    "num_key_value_heads": 1,
    "head_dim": 16,
    "intermediate_size": 108,
    "vocab_size": 211,
    "rope_theta": 500000.0,
    "rms_norm_eps": 1e-4,
    "attention_bias": False,
    "tie_word_embeddings": False,
    "use_sliding_window": False,
    "max_position_embeddings": 200,
    "eos_token_id": 2,
}

TINY = {"A": TINY_A, "B": TINY_B, "C": TINY_C}


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real GPU (MI355X); skipped from the CPU run with -m 'not gpu'")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def sharpen(tensors: dict, factor: float = 8.0) -> dict:
    """Scale the query and key projections so that attention is peaked: with
    plain N(0, 0.02) weights every softmax is almost uniform and a wrong key, a
    wrong position or a stale cache page would barely move the logits."""
    out = {}
    for name, tensor in tensors.items():
        if name.endswith(("q_proj.weight", "k_proj.weight", "q_proj.bias", "k_proj.bias")):
            tensor = (tensor.float() * factor).to(tensor.dtype)
        out[name] = tensor
    return out


def make_folder(tmp: Path, raw: dict, seed: int, store_dtype: str = "bfloat16", factor: float = 8.0) -> tuple[Path, dict]:
    """Write config.json + model.safetensors; returns the folder and the stored tensors."""
    from cie_amd.config import config_from_dict
    from cie_amd.parts.model import expected_tensors
    from cie_amd.weights import RandomSource, write_tensors

    config = config_from_dict(raw)
    expected = expected_tensors(config.model_spec())
    tensors = sharpen(RandomSource(seed).load(expected, store_dtype, "cpu"), factor)
    write_tensors(tmp, raw, tensors)
    return tmp, tensors


@pytest.fixture(scope="session")
def tiny_folders(tmp_path_factory):
    """{'A': (folder, raw config, tensors), 'B': ...}; weights stored in bfloat16."""
    out = {}
    for index, (name, raw) in enumerate(TINY.items()):
        folder = tmp_path_factory.mktemp(f"tiny_{name}")
        folder, tensors = make_folder(folder, raw, seed=11 + index)
        out[name] = (folder, raw, tensors)
    return out


def random_tokens(count: int, vocab: int, seed: int) -> list[int]:
    generator = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (count,), generator=generator).tolist()
