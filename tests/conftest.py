"""Shared fixtures: the tiny configurations and model folders of random weights.

Tests build their models in temporary folders; nothing is read from or written
to the repository.  GPU tests carry the ``gpu`` marker and are skipped by
``-m "not gpu"``.
"""
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP GPU (MI355X)")


def pytest_terminal_summary(terminalreporter):
    """What the bfloat16 comparisons measured, beside their bounds."""
    import helpers
    for kind, (worst, rms) in sorted(helpers.BF16_SEEN.items()):
        terminalreporter.write_line(
            f"[bfloat16 against the plain implementation, {kind}] largest difference {worst:.4f} of the logits' spread "
            f"(bound {helpers.BF16_MAX[kind]}), root mean square {rms:.4f} (bound {helpers.BF16_RMS[kind]})")


# Tiny A and B differ in every size and option: layers, width, heads and groups
# (GQA 2:1 / MQA 3:1), head size, inner width, vocabulary (no powers of two in
# B), rope base, eps, maximum positions, tied or separate head.  C adds what
# neither has: plain multi-head attention, a head size of 48, YaRN scaling with
# its score multiplier, several eos ids.
TINY_A = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2,
    "intermediate_size": 128, "vocab_size": 256, "rope_theta": 10000.0, "rms_norm_eps": 1e-6,
    "max_position_embeddings": 128, "tie_word_embeddings": True, "use_sliding_window": False,
    "hidden_act": "silu", "sliding_window": 131072, "max_window_layers": 2,
}
TINY_B = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 3, "hidden_size": 96, "num_attention_heads": 3, "num_key_value_heads": 1,
    "intermediate_size": 224, "vocab_size": 384, "rope_theta": 1000000.0, "rms_norm_eps": 1e-5,
    "max_position_embeddings": 256, "tie_word_embeddings": False, "use_sliding_window": False,
    "hidden_act": "silu", "eos_token_id": 7,
}
TINY_C = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 2, "hidden_size": 144, "num_attention_heads": 3, "num_key_value_heads": 3,
    "intermediate_size": 200, "vocab_size": 300, "rope_theta": 50000.0, "rms_norm_eps": 3e-5,
    "max_position_embeddings": 512, "tie_word_embeddings": False, "use_sliding_window": False,
    "hidden_act": "silu", "eos_token_id": [5, 9],
    "rope_scaling": {"type": "yarn", "factor": 4.0, "original_max_position_embeddings": 64,
                     "beta_fast": 32.0, "beta_slow": 1.0},
}
TINY = {"A": TINY_A, "B": TINY_B, "C": TINY_C}


@pytest.fixture(scope="session")
def tiny_configs():
    return {k: dict(v) for k, v in TINY.items()}


@pytest.fixture(scope="session")
def model_folders(tmp_path_factory):
    """name -> folder with config.json and bf16 model.safetensors of seeded random weights."""
    from sonicboom_amd.weights import write_random_model
    out = {}
    for i, (name, cfg) in enumerate(TINY.items()):
        folder = str(tmp_path_factory.mktemp(f"tiny_{name}"))
        write_random_model(folder, dict(cfg), seed=1234 + i, dtype="bfloat16")
        out[name] = folder
    return out


# Random N(0, 0.02) weights give attention scores near 0.03: the softmax is almost uniform and a
# wrong scale, rope base, bias or position moves the logits by less than bfloat16's rounding.
# The "sharp" folders hold the same models with the query and key projections times SHARP_QK and
# their biases times SHARP_QK_BIAS (a bias of N(0, 0.02) is an eighth of what the projection of a
# normed row gives; the larger factor makes it a third), which spreads the scores over several
# units so that such mistakes show (tests/test_plain.py::test_sharp_models_show_attention_mistakes
# measures by how much).
SHARP_QK = 10.0
SHARP_QK_BIAS = 30.0


def sharpen_model(src: str, dst: str, factor: float = SHARP_QK, bias_factor: float = SHARP_QK_BIAS) -> None:
    """Copy the model folder ``src`` to ``dst`` with q_proj and k_proj (weights and biases) scaled."""
    import shutil

    import torch
    from safetensors import safe_open
    from safetensors.torch import save_file
    os.makedirs(dst, exist_ok=True)
    shutil.copy(os.path.join(src, "config.json"), os.path.join(dst, "config.json"))
    tensors = {}
    with safe_open(os.path.join(src, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            t = f.get_tensor(name)
            if ".q_proj." in name or ".k_proj." in name:
                t = (t.float() * (bias_factor if name.endswith(".bias") else factor)).to(t.dtype)
            tensors[name] = t.contiguous()
    save_file(tensors, os.path.join(dst, "model.safetensors"), metadata={"format": "pt"})


@pytest.fixture(scope="session")
def sharp_folders(model_folders, tmp_path_factory):
    """name -> folder of the same tiny model with attention scores of several units."""
    out = {}
    for name in ("A", "B", "C"):
        out[name] = str(tmp_path_factory.mktemp(f"sharp_{name}"))
        sharpen_model(model_folders[name], out[name])
    return out


def random_prompt(rng: np.random.Generator, vocab: int, n: int):
    return [int(t) for t in rng.integers(0, vocab, size=n)]
