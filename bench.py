"""Decode and prefill throughput of the engine on one MI355X, random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Default run: the layer sizes of the Qwen2.5-1.5B shape (28 layers, hidden 1536,
12 query / 2 key-value heads of 128, intermediate 8960, vocabulary 151936, tied
head), bfloat16, a batch of 8 sequences at a context of 4,096 tokens.  A "step"
is one decode step of the whole batch through the scheduler: planning, the
model's pass, sampling and the copy of the tokens to the host.  One JSON line is
printed: `value` is decoded tokens per second; `prefill` is one 2,048-token
prompt in one step; `roofline` prices the decode step against HBM (every weight
read once plus the cache of the live sequences); `points` holds decoding at
batch 1 and 64.  Token ids are synthetic (seeded, uniform over the vocabulary),
as the reference's own streams are (bench/workload.py:241-254,294-298).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

QWEN25_1P5B = dict(architectures=["Qwen2ForCausalLM"], num_hidden_layers=28, hidden_size=1536,
                   num_attention_heads=12, num_key_value_heads=2, head_dim=128, intermediate_size=8960,
                   vocab_size=151936, rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=True,
                   use_sliding_window=False, max_position_embeddings=32768, hidden_act="silu")
FULL_LAYERS = 28
HBM_PEAK_GBS = 8000.0
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}


def build_model(cfg: dict, dtype: str, seed: int = 0):
    import torch
    import paged_attention_engine_amd as pae
    from paged_attention_engine_amd.engine.model import TORCH_DTYPE
    from paged_attention_engine_amd.weights.random_init import random_tensor

    config = pae.read_config_dict(cfg)
    model = pae.Model(config.plan(), TORCH_DTYPE[dtype], "cuda:0")

    class Lazy(dict):  # tensors are drawn on the device one at a time as parts ask for them
        def __init__(self, shapes):
            super().__init__()
            self.shapes = shapes

        def __missing__(self, name):
            return random_tensor(name, tuple(self.shapes[name]), seed, device="cuda:0")

        def get(self, name, default=None):
            return self[name] if name in self.shapes else default

    model.bind(Lazy(model.expected_tensors()))
    torch.cuda.synchronize()
    return model


def weight_bytes(cfg: dict, elem: int) -> int:
    H, I, V, L = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"], cfg["num_hidden_layers"]
    nh, nkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    qkv = (nh + 2 * nkv) * hd
    per_layer = qkv * H + qkv + nh * hd * H + 3 * H * I + 2 * H
    head = V * H  # read once per step; the tied embedding gather adds only a few rows
    return (L * per_layer + head + H) * elem


def kv_bytes(cfg: dict, tokens: int, elem: int) -> int:
    return tokens * 2 * cfg["num_key_value_heads"] * cfg["head_dim"] * cfg["num_hidden_layers"] * elem


def prefill_flops(cfg: dict, T: int) -> float:
    H, I, V, L = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"], cfg["num_hidden_layers"]
    nh, nkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    linear = 2.0 * T * L * ((nh + 2 * nkv) * hd * H + nh * hd * H + 3 * H * I) + 2.0 * H * V
    attention = 4.0 * hd * nh * (T * (T + 1) / 2) * L
    return linear + attention


def decode_run(model, cfg, batch: int, ctx: int, steps: int, warmup: int, block_size: int = 16):
    """Time `steps` decode steps of `batch` sequences whose context reaches `ctx`."""
    import torch
    import paged_attention_engine_amd as pae

    # Prompts run in portions of at most 2,048 tokens a step, so the first
    # sequences decode while the last still prefill; every sequence holds at
    # least `ctx` tokens when the clock starts.  The context passes `ctx` in the
    # middle of the warm-up: a decode step is recorded anew when its block tables
    # grow past a multiple of 64 pages (once per 1,024 tokens), and at a context
    # of a power of two that recording would otherwise be the first timed step.
    prompt_len = ctx - warmup // 2 - 1
    slack = batch * prompt_len // 2048 + 4
    max_new = warmup + steps + slack + 2
    blocks = batch * (-(-(prompt_len + max_new) // block_size) + 1) + 2
    dtype = "bfloat16" if model.dtype == torch.bfloat16 else "float32"
    engine = pae.Engine(model, dtype=dtype, block_size=block_size, num_blocks=blocks, max_num_seqs=batch,
                        max_num_batched_tokens=2048)
    gen = torch.Generator().manual_seed(1234)
    for b in range(batch):
        prompt = torch.randint(0, cfg["vocab_size"], (prompt_len,), generator=gen).tolist()
        assert engine.add_request(pae.Request(f"b{b}", tuple(prompt), max_new))
    sched = engine.scheduler
    while sched.waiting or any(s.prefilling for s in sched.running):
        engine.step()
    for _ in range(warmup):
        result = engine.step()
        assert len(result.decoded) == batch, result
    held_before = sum(engine.cache.num_tokens(s.seq_id) for s in sched.running)
    generated_before = sum(len(s.generated) for s in sched.running)
    torch.cuda.synchronize()
    start = time.perf_counter()
    # the engine's own loop: the next step is decided and launched while the current one runs,
    # and the clock stops when the last step's tokens are on the host
    ran = engine.run_steps(steps)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - start
    assert ran == steps and len(sched.running) == batch and not any(s.prefilling for s in sched.running)
    assert sum(len(s.generated) for s in sched.running) - generated_before == batch * steps
    assert all(t >= 0 for s in sched.running for t in s.generated)
    held_after = sum(engine.cache.num_tokens(s.seq_id) for s in sched.running)
    del engine, sched
    torch.cuda.empty_cache()
    return elapsed / steps, (held_before + held_after) / 2


def prefill_run(model, cfg, T: int, repeats: int = 3, block_size: int = 16):
    import torch
    import paged_attention_engine_amd as pae

    dtype = "bfloat16" if model.dtype == torch.bfloat16 else "float32"
    gen = torch.Generator().manual_seed(99)
    times = []
    for r in range(repeats + 1):
        engine = pae.Engine(model, dtype=dtype, block_size=block_size, num_blocks=-(-T // block_size) + 4,
                            max_num_seqs=1, max_num_batched_tokens=T)
        prompt = torch.randint(0, cfg["vocab_size"], (T,), generator=gen).tolist()
        engine.add_request(pae.Request("p", tuple(prompt), 1))
        torch.cuda.synchronize()
        start = time.perf_counter()
        result = engine.step()
        torch.cuda.synchronize()
        times.append(time.perf_counter() - start)
        assert result.finished == ("p",), result
        del engine
    return sorted(times[1:])[len(times[1:]) // 2]


def main() -> int:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=64)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--ctx", type=int, default=4096)
    parser.add_argument("--layers", type=int, default=FULL_LAYERS)
    parser.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    parser.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 and prefill runs")
    parser.add_argument("--prefill-only", action="store_true", help="time the 2,048-token prefill alone (for profiles)")
    args = parser.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU only: this engine has no multi-GPU path (run with --gpus 1)")
        return 2

    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 1
    cfg = dict(QWEN25_1P5B, num_hidden_layers=args.layers)
    elem = 2 if args.dtype == "bfloat16" else 4
    model = build_model(cfg, args.dtype)

    if args.prefill_only:
        pre_s = prefill_run(model, cfg, 2048, repeats=max(3, args.steps))
        print(json.dumps({"metric": "prefill tok/s at 2,048 tokens (Qwen2.5-1.5B shape)", "value": round(2048 / pre_s, 1),
                          "unit": "tokens/s", "ms": round(pre_s * 1e3, 3), "dtype": args.dtype,
                          "frac": round(prefill_flops(cfg, 2048) / pre_s / PEAK_FLOPS[args.dtype], 4)}))
        return 0
    step_s, tokens_held = decode_run(model, cfg, args.batch, args.ctx, args.steps, args.warmup)
    value = args.batch / step_s
    step_bytes = weight_bytes(cfg, elem) + kv_bytes(cfg, tokens_held, elem)
    achieved = step_bytes / step_s / 1e9
    record = {
        "metric": f"decode tok/s at batch {args.batch}, context {args.ctx} (Qwen2.5-1.5B shape)",
        "value": round(value, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: seeded uniform token ids, random weights N(0, 0.02)",
        "config": {"model": "Qwen2.5-1.5B shape", "global_batch": args.batch, "seq_len": args.ctx,
                   "parallelism": "single GPU", "layers": args.layers, "layers_of_model": FULL_LAYERS,
                   "hidden": cfg["hidden_size"], "q_heads": cfg["num_attention_heads"],
                   "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"],
                   "intermediate": cfg["intermediate_size"], "vocab": cfg["vocab_size"],
                   "tied_head": True, "block_size": 16, "prefill_tokens": 2048},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }
    if not args.no_points:
        T = 2048
        pre_s = prefill_run(model, cfg, T)
        record["prefill"] = {"value": round(T / pre_s, 1), "tokens": T, "ms": round(pre_s * 1e3, 3),
                             "frac": round(prefill_flops(cfg, T) / pre_s / PEAK_FLOPS[args.dtype], 4)}
        points = {}
        for b in (1, 64):
            s, _ = decode_run(model, cfg, b, args.ctx, max(8, args.steps // 2), 4)
            points[f"decode_b{b}"] = round(b / s, 2)
        record["points"] = points
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    sys.exit(main())
