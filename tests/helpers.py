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

# what the serving kernels of the large shapes take, in small: heads of 64 on pages of 16, six query
# heads per key/value head, a window on the second layer.  Query and key projections are drawn
# six times wider than the rest, so that scores spread over several units and attention is peaked:
# a missing rotation or a flat softmax then moves the logits far beyond the bfloat16 tolerance
# (`test_the_peaked_model_shows_mistakes...` in tests/test_plain.py shows by how much).
TINY_E = dict(architectures=["Qwen2ForCausalLM"], num_hidden_layers=2, hidden_size=192,
              num_attention_heads=12, num_key_value_heads=2, head_dim=64, intermediate_size=328,
              vocab_size=1500, rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False,
              use_sliding_window=True, sliding_window=48, max_window_layers=1,
              max_position_embeddings=2048, hidden_act="silu")
PEAKED = {"": 0.02, "q_proj.weight": 0.12, "k_proj.weight": 0.12, "q_proj.bias": 0.3, "k_proj.bias": 0.3,
          "v_proj.weight": 0.06, "o_proj.weight": 0.04}

TINY = {"A": (TINY_A, dict(seed=0, norm_std=0.0, block_size=16)),
        "B": (TINY_B, dict(seed=1, norm_std=0.1, block_size=8)),
        "C": (TINY_C, dict(seed=2, norm_std=0.1, block_size=16)),
        "D": (TINY_D, dict(seed=3, norm_std=0.05, block_size=16)),
        "E": (TINY_E, dict(seed=4, norm_std=0.05, block_size=16, std=PEAKED))}


def make_model_folder(tmp_path, name: str) -> str:
    """Write tiny model `name` with the product's random-weights mode."""
    import paged_attention_engine_amd as pae

    cfg, opts = TINY[name]
    out = os.path.join(str(tmp_path), f"tiny_{name}")
    pae.write_model_folder(pae.read_config_dict(cfg), opts["seed"], out, std=opts.get("std", 0.02),
                           norm_std=opts["norm_std"])
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


def bf16_ulp(reference_logits: torch.Tensor) -> float:
    """One bfloat16 unit in the last place at the largest logit (8 significant bits:
    ulp = 2**-7 * 2**exponent)."""
    top = max(float(torch.as_tensor(reference_logits).abs().max()), 1e-6)
    return 2.0 ** -7 * 2.0 ** math.floor(math.log2(top))


# The reference states its reduced-precision parity as 4 ulp of the logits' binade
# (tests/test_parity_fp16.py:161-163).  With flat attention (weights N(0, 0.02): scores a few
# hundredths wide) this engine stays within 1 ulp, so those models are held to 2 ulp at the worst
# logit.  Model E's scores are some ten units wide:
# rounding q and k to bfloat16 alone moves a score by several hundredths and a softmax weight by
# several per cent, whatever the kernel, so E keeps the reference's 4 ulp; its job is the other direction: a wrong kernel moves its logits by 45 times that.
# The same holds at the real layer sizes ("wide"): with hidden widths of 1,536 to 8,192 the scores of
# N(0, 0.02) weights are one to three units wide by themselves.
BF16_MAX_ULPS = {"E": 4.0, "wide": 4.0}
# The root mean square over all logits is held to a share of the largest logit instead of its
# binade (a bound that halves when the largest logit drops from 1.01 to 0.99 says little about an
# average): 2**-9 of it, half a unit in the last place of a bfloat16 number of that size, for the
# flat models (observed: at most 0.55 of that), and 2.5 times as much where attention is peaked.
BF16_RMS_SHARE = {"E": 2.5, "wide": 2.5}


def bf16_atol(reference_logits: torch.Tensor, name: str = "") -> float:
    return BF16_MAX_ULPS.get(name, 2.0) * bf16_ulp(reference_logits)


def bf16_rms_bound(reference_logits: torch.Tensor, name: str = "") -> float:
    top = max(float(torch.as_tensor(reference_logits).abs().max()), 1e-6)
    return BF16_RMS_SHARE.get(name, 1.0) * 2.0 ** -9 * top


def bounds(dtype: str, reference_logits: torch.Tensor, name: str = ""):
    """(largest error allowed at any logit, largest root-mean-square error over all logits)."""
    if dtype == "float32":
        atol = fp32_atol(reference_logits)
        return atol, atol / 4
    return bf16_atol(reference_logits, name), bf16_rms_bound(reference_logits, name)


def check_logits(got: torch.Tensor, want: torch.Tensor, dtype: str, name: str = "", what: str = "") -> float:
    """Assert both bounds; returns the worst error."""
    got, want = torch.as_tensor(got).double(), torch.as_tensor(want).double()
    atol, rms_bound = bounds(dtype, want, name)
    diff = got - want
    worst, rms = float(diff.abs().max()), float(diff.pow(2).mean().sqrt())
    assert worst <= atol, f"{what}: worst logit error {worst:.3e} > {atol:.3e}"
    assert rms <= rms_bound, f"{what}: root-mean-square logit error {rms:.3e} > {rms_bound:.3e}"
    return worst
