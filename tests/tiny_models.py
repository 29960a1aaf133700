"""Tiny random-weight model folders for the tests.

Five configurations of the one architecture that differ in every size and option:
A and B are the two tiny workloads the benchmark contract names; C adds what they leave
out (no QKV bias, one KV head per query head, a window on the later layers); D has heads of
64 (the size from which the 128-row prompt attention kernel is built), groups of three, a
window wider than a step of keys and pages of 8; E has a width, a feed-forward width and a
vocabulary that are no multiples of 8 (the matrix-core kernels refuse them: the bfloat16 engine
runs its general kernels), seven heads of 16 and pages of 4; F is the tiny configuration of the
reference's own loader test (/root/reference/tests/test_weight_loading.py:75-84: hidden 16, four heads
of 4 in two groups, eight positions, tied) with pages of 4; G has heads of 24, a size that is no
multiple of 16 (the attention library of 32 serves it), in groups of five, and pages of 16.
"""
import json
from pathlib import Path

import torch

CONFIGS = {
    "A": dict(
        architectures=["Qwen2ForCausalLM"], vocab_size=256, hidden_size=64, num_hidden_layers=2,
        num_attention_heads=4, num_key_value_heads=2, intermediate_size=128, max_position_embeddings=128,
        rope_theta=10000.0, rms_norm_eps=1e-6, tie_word_embeddings=True, use_sliding_window=False,
    ),
    "B": dict(
        architectures=["Qwen2ForCausalLM"], vocab_size=300, hidden_size=96, num_hidden_layers=3,
        num_attention_heads=3, num_key_value_heads=1, head_dim=32, intermediate_size=200,
        max_position_embeddings=256, rope_theta=1000000.0, rms_norm_eps=1e-5, tie_word_embeddings=False,
    ),
    "C": dict(
        architectures=["Qwen2ForCausalLM"], vocab_size=211, hidden_size=80, num_hidden_layers=4,
        num_attention_heads=5, num_key_value_heads=5, head_dim=48, intermediate_size=112,
        max_position_embeddings=512, rope_parameters={"rope_theta": 500000.0}, rms_norm_eps=3e-6,
        attention_bias=False, tie_word_embeddings=False,
        use_sliding_window=True, sliding_window=20, max_window_layers=1,
    ),
    "D": dict(
        architectures=["Qwen2ForCausalLM"], vocab_size=190, hidden_size=72, num_hidden_layers=2,
        num_attention_heads=6, num_key_value_heads=2, head_dim=64, intermediate_size=104,
        max_position_embeddings=400, rope_theta=30000.0, rms_norm_eps=2e-6, tie_word_embeddings=True,
        use_sliding_window=True, sliding_window=70, max_window_layers=1,
    ),
    "E": dict(
        architectures=["Qwen2ForCausalLM"], vocab_size=131, hidden_size=100, num_hidden_layers=2,
        num_attention_heads=7, num_key_value_heads=7, head_dim=16, intermediate_size=75,
        max_position_embeddings=300, rope_theta=20000.0, rms_norm_eps=5e-6, tie_word_embeddings=False,
    ),
    "F": dict(
        architectures=["Qwen2ForCausalLM"], vocab_size=16, hidden_size=16, num_hidden_layers=1,
        num_attention_heads=4, num_key_value_heads=2, intermediate_size=32, max_position_embeddings=8,
        tie_word_embeddings=True,
    ),
    "G": dict(
        architectures=["Qwen2ForCausalLM"], vocab_size=150, hidden_size=88, num_hidden_layers=2,
        num_attention_heads=10, num_key_value_heads=2, head_dim=24, intermediate_size=120,
        max_position_embeddings=320, rope_theta=100000.0, rms_norm_eps=1e-5, tie_word_embeddings=False,
    ),
}
SEEDS = {"A": 0, "B": 1, "C": 5, "D": 8, "E": 9, "F": 12, "G": 13}
PAGE_SIZES = {"A": 16, "B": 8, "C": 16, "D": 8, "E": 4, "F": 4, "G": 16}


def write(name: str, root: Path, dtype=torch.bfloat16) -> Path:
    """Write configuration ``name`` with its seed under ``root`` through the framework's
    random-weights mode, then put the raw dictionary back as config.json so that the
    folder holds exactly the keys listed above (defaults stay implicit)."""
    from torchlet_amd.registry import config_class
    from torchlet_amd.weights.random_init import write_model_folder

    d = CONFIGS[name]
    cfg = config_class(d["architectures"][0]).from_dict(d)
    folder = write_model_folder(cfg, SEEDS[name], root / f"tiny_{name}", dtype)
    (folder / "config.json").write_text(json.dumps(d, indent=2))
    return folder
