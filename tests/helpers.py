"""Tiny configurations, model folders and tolerances shared by the tests.

The tiny configurations differ in every size and option: head counts and
groups, sizes that are no power of two, number of layers, vocabulary, eps,
rope base, tying of the head, norm weights and, in the third, windows.
"""

from __future__ import annotations

import json
import math
import os

import torch

TINY_A = dict(architectures=["Qwen2ForCausalLM"], num_hidden_layers=2, hidden_size=64,
              num_attention_heads=4, num_key_value_heads=2, head_dim=16, intermediate_size=176,
              vocab_size=512, rope_theta=10000.0, rms_norm_eps=1e-6, tie_word_embeddings=True,
              use_sliding_window=False, max_position_embeddings=256, hidden_act="silu")
TINY_B = dict(architectures=["Qwen2ForCausalLM"], num_hidden_layers=3, hidden_size=128,
              num_attention_heads=4, num_key_value_heads=1, head_dim=32, intermediate_size=352,
              vocab_size=1000, rope_theta=1000000.0, rms_norm_eps=1e-5, tie_word_embeddings=False,
              use_sliding_window=False, max_position_embeddings=512, hidden_act="silu")
# windows on the last two of four layers, head_dim 48 (a multiple of 16 that is no power of two),
# three query heads per key/value head, odd hidden width and vocabulary
TINY_C = dict(architectures=["Qwen2ForCausalLM"], num_hidden_layers=4, hidden_size=72,
              num_attention_heads=6, num_key_value_heads=2, head_dim=48, intermediate_size=200,
              vocab_size=777, rope_theta=50000.0, rms_norm_eps=3e-6, tie_word_embeddings=False,
              use_sliding_window=True, sliding_window=24, max_window_layers=2,
              max_position_embeddings=512, hidden_act="silu")

# a shape the matrix-core attention kernels take (head_dim 32, pages of 16), five query heads on
# one key/value head, a window on the second of two layers
TINY_D = dict(architectures=["Qwen2ForCausalLM"], num_hidden_layers=2, hidden_size=160,
              num_attention_heads=5, num_key_value_heads=1, head_dim=32, intermediate_size=400,
              vocab_size=1111, rope_theta=200000.0, rms_norm_eps=2e-6, tie_word_embeddings=False,
              use_sliding_window=True, sliding_window=40, max_window_layers=1,
              max_position_embeddings=1024, hidden_act="silu")

TINY = {"A": (TINY_A, dict(seed=0, norm_std=0.0, block_size=16)),
        "B": (TINY_B, dict(seed=1, norm_std=0.1, block_size=8)),
        "C": (TINY_C, dict(seed=2, norm_std=0.1, block_size=16)),
        "D": (TINY_D, dict(seed=3, norm_std=0.05, block_size=16))}


def make_model_folder(tmp_path, name: str) -> str:
    """Write tiny model `name` with the product's random-weights mode."""
    import paged_attention_engine_amd as pae

    cfg, opts = TINY[name]
    out = os.path.join(str(tmp_path), f"tiny_{name}")
    pae.write_model_folder(pae.read_config_dict(cfg), opts["seed"], out, norm_std=opts["norm_std"])
    return out


def read_folder_plain(folder: str):
    """(config dict, float32 tensors by name) read without the product's loader."""
    from safetensors import safe_open

    with open(os.path.join(folder, "config.json")) as handle:
        cfg = json.load(handle)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), "pt") as handle:
        for key in handle.keys():
            tensors[key] = handle.get_tensor(key).to(torch.float32)
    return cfg, tensors


# float32 engine against the float64 plain implementation: a hundred float32
# roundings relative to the largest logit
FP32_REL = 1e-5


def fp32_atol(reference_logits: torch.Tensor) -> float:
    return FP32_REL * max(float(reference_logits.abs().max()), 1e-3)


def bf16_atol(reference_logits: torch.Tensor) -> float:
    """Four bfloat16 units in the last place at the largest logit: the error model the
    reference states for its reduced-precision parity (tests/test_parity_fp16.py:161-163:
    4 ulp of the logits' binade; bf16 has 8 significant bits, ulp = 2**-7 * 2**exponent)."""
    top = max(float(reference_logits.abs().max()), 1e-6)
    return 4.0 * 2.0 ** -7 * 2.0 ** math.floor(math.log2(top))
