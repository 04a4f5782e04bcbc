"""Shared fixtures: two tiny Qwen3 configurations that differ in every size and option (plus a
windowed variant), model folders made from them in a temporary place, and the plain
implementation's logits for fixed token sequences."""
from __future__ import annotations

import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for path in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if path not in sys.path:
        sys.path.insert(0, path)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


TINY_A = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=256, hidden_size=64, intermediate_size=128,
    num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=16, max_position_embeddings=128,
    rms_norm_eps=1e-6, rope_theta=1e4, tie_word_embeddings=True, torch_dtype="bfloat16", attention_bias=False,
    use_sliding_window=False, hidden_act="silu")
TINY_B = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=509, hidden_size=96, intermediate_size=224,
    num_hidden_layers=3, num_attention_heads=6, num_key_value_heads=1, head_dim=32, max_position_embeddings=256,
    rms_norm_eps=1e-5, rope_theta=1e6, tie_word_embeddings=False, torch_dtype="bfloat16", attention_bias=False,
    use_sliding_window=False, hidden_act="silu")
# a third one with yet other sizes (head_dim 48 is no power of two), run with attention windows on some layers: an
# option of the engine (the reference has no windows, so config.json cannot ask for them), given as overrides
TINY_W = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=331, hidden_size=80, intermediate_size=176,
    num_hidden_layers=4, num_attention_heads=6, num_key_value_heads=3, head_dim=48, max_position_embeddings=512,
    rms_norm_eps=3e-6, rope_theta=5e4, tie_word_embeddings=False, torch_dtype="bfloat16", attention_bias=False,
    use_sliding_window=False, hidden_act="silu")
WINDOW_W = 24
TINY = {"A": (TINY_A, 4), "B": (TINY_B, 16), "W": (TINY_W, 8)}  # config, cache page size used with it
OVERRIDES = {"A": None, "B": None, "W": {"layer_windows": [None, None, WINDOW_W, WINDOW_W]}}   # options of the engine


@pytest.fixture(scope="session")
def model_folders(tmp_path_factory):
    """name -> folder with config.json and model.safetensors (random weights, seeded)."""
    from pulse_infer_amd.config import Qwen3Config
    from pulse_infer_amd.weights import write_model_folder

    out = {}
    for seed, (name, (cfg, _)) in enumerate(TINY.items()):
        folder = tmp_path_factory.mktemp(f"tiny{name}")
        write_model_folder(Qwen3Config.from_dict(cfg), str(folder), seed=11 + seed)
        out[name] = str(folder)
    return out


def token_ids(vocab: int, count: int, seed: int):
    return torch.randint(0, vocab, (count,), generator=torch.Generator().manual_seed(seed)).tolist()


@pytest.fixture(scope="session")
def plain_models(model_folders):
    from plain.qwen3_plain import PlainQwen3

    return {name: PlainQwen3.from_folder(folder, windows=(OVERRIDES[name] or {}).get("layer_windows"))
            for name, folder in model_folders.items()}


class _PlainLogits:
    def __init__(self, models):
        self.models = models
        self.memo = {}

    def __call__(self, name, ids):
        key = (name, tuple(ids))
        if key not in self.memo:
            self.memo[key] = self.models[name].logits(list(ids))
        return self.memo[key]


@pytest.fixture(scope="session")
def plain_logits(plain_models):
    return _PlainLogits(plain_models)


def require_gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
