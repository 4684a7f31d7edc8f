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

Method, after the reference's (bench/run.py:628-702): after the warm-up, three
passes of K steps each are timed (the device is synchronised before the clock
starts and after it stops); the figure is the median pass, with the range beside
it; if the range exceeds 20 % of the median seven passes are timed instead, and
if it still does no figure is given (`value` null, exit code 3).  Every pass must
decode the same number of tokens.  `provenance` says what ran where
(bench/run.py:232-317).
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
# Other shapes of the same architecture (--model): the layer sizes of the other Qwen2.5 models, for decode
# steps and prefills at sizes where a kernel runs longer than a launch costs (7B, 72B) and at the widths in
# between.
OTHER_SHAPES = {
    "0.5b": dict(QWEN25_1P5B, num_hidden_layers=24, hidden_size=896, num_attention_heads=14, num_key_value_heads=2,
                 head_dim=64, intermediate_size=4864),
    "3b": dict(QWEN25_1P5B, num_hidden_layers=36, hidden_size=2048, num_attention_heads=16, num_key_value_heads=2,
               intermediate_size=11008),
    "7b": dict(QWEN25_1P5B, hidden_size=3584, num_attention_heads=28, num_key_value_heads=4,
               intermediate_size=18944, vocab_size=152064, tie_word_embeddings=False),
    "14b": dict(QWEN25_1P5B, num_hidden_layers=48, hidden_size=5120, num_attention_heads=40, num_key_value_heads=8,
                intermediate_size=13824, vocab_size=152064, rms_norm_eps=1e-5, tie_word_embeddings=False),
    "32b": dict(QWEN25_1P5B, num_hidden_layers=64, hidden_size=5120, num_attention_heads=40, num_key_value_heads=8,
                intermediate_size=27648, vocab_size=152064, rms_norm_eps=1e-5, tie_word_embeddings=False),
    "72b": dict(QWEN25_1P5B, num_hidden_layers=80, hidden_size=8192, num_attention_heads=64,
                num_key_value_heads=8, intermediate_size=29568, vocab_size=152064, rms_norm_eps=1e-5,
                tie_word_embeddings=False),
}
HBM_PEAK_GBS = 8000.0
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}


WEIGHT_SEED, DECODE_TOKEN_SEED, PREFILL_TOKEN_SEED = 0, 1234, 99
MEASURED_PASSES, ESCALATED_PASSES, SPREAD_LIMIT = 3, 7, 0.20


def build_model(cfg: dict, dtype: str, seed: int = WEIGHT_SEED):
    """Random weights of the shape `cfg`, drawn on the device tensor by tensor."""
    import torch
    import paged_attention_engine_amd as pae

    model = pae.random_model(cfg, seed, dtype, "cuda:0")
    torch.cuda.synchronize()
    return model


class Unresolved(RuntimeError):
    """The passes of a measurement disagree by more than the limit: no figure is given."""


class Refused(RuntimeError):
    """The run that was asked for cannot be made at this shape; the message says why."""


def settle(passes):
    """(median, range) of the passes' times."""
    ordered = sorted(passes)
    return ordered[len(ordered) // 2], ordered[-1] - ordered[0]


def measured(run_pass, what: str):
    """Three passes; seven if their range exceeds 20 % of the median; Unresolved if it still does.
    Returns (median seconds, range seconds, the passes)."""
    passes = [run_pass() for _ in range(MEASURED_PASSES)]
    median, spread = settle(passes)
    if spread > SPREAD_LIMIT * median:
        passes += [run_pass() for _ in range(ESCALATED_PASSES - MEASURED_PASSES)]
        median, spread = settle(passes)
        if spread > SPREAD_LIMIT * median:
            raise Unresolved(f"{what}: {len(passes)} passes range over {spread / median:.0%} of their median "
                             f"({', '.join(f'{p * 1e3:.3f}' for p in passes)} ms)")
    return median, spread, passes


def provenance(model, extra: dict) -> dict:
    import torch
    import paged_attention_engine_amd as pae
    from paged_attention_engine_amd.kernels import build as kernel_build, lib

    props = torch.cuda.get_device_properties(0)
    out = {"device": props.name, "arch": lib.device_arch(), "compute_units": props.multi_processor_count,
           "hbm_gib": round(props.total_memory / 2**30, 1), "hip": torch.version.hip, "torch": torch.__version__,
           "kernel_sources": kernel_build.source_hash(), "kernel_library": os.path.basename(lib.loaded_library_path() or ""),
           "weight_seed": WEIGHT_SEED, "decode_token_seed": DECODE_TOKEN_SEED, "prefill_token_seed": PREFILL_TOKEN_SEED,
           "weights": "N(0, 0.02), drawn on the device", "passes": MEASURED_PASSES, "spread_limit": SPREAD_LIMIT}
    out.update(extra)
    return out


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
    """Passes of `steps` decode steps of `batch` sequences whose context has reached `ctx`.
    Returns (median seconds a step, range of the passes' seconds a step, mean tokens held, pages)."""
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
    max_new = warmup + ESCALATED_PASSES * steps + slack + 2
    limit = cfg.get("max_position_embeddings")
    if prompt_len < 1 or (limit and prompt_len + max_new > limit):
        raise Refused(f"a context of {ctx} tokens with {max_new} new tokens to decode on top (warm-up, up to "
                      f"{ESCALATED_PASSES} passes of {steps} steps and slack) runs past the shape's "
                      f"max_position_embeddings of {limit}: the scheduler would reject the requests; ask for a "
                      f"context of at most {limit - max_new + warmup // 2 + 1}")
    blocks = batch * (-(-(prompt_len + max_new) // block_size) + 1) + 2
    dtype = "bfloat16" if model.dtype == torch.bfloat16 else "float32"
    engine = pae.Engine(model, dtype=dtype, block_size=block_size, num_blocks=blocks, max_num_seqs=batch,
                        max_num_batched_tokens=2048)
    gen = torch.Generator().manual_seed(DECODE_TOKEN_SEED)
    for b in range(batch):
        prompt = torch.randint(0, cfg["vocab_size"], (prompt_len,), generator=gen).tolist()
        assert engine.add_request(pae.Request(f"b{b}", tuple(prompt), max_new))
    sched = engine.scheduler
    while len(sched.waiting) or any(s.prefilling for s in sched.running):
        engine.step()
    for _ in range(warmup):
        result = engine.step()
        assert len(result.decoded) == batch, result
    held = []

    def one_pass():
        generated_before = sum(len(s.generated) for s in sched.running)
        held.append(sum(engine.cache.num_tokens(s.seq_id) for s in sched.running))
        torch.cuda.synchronize()
        start = time.perf_counter()
        # the engine's own loop: the next step is decided and launched while the current one runs,
        # and the clock stops when the last step's tokens are on the host
        ran = engine.run_steps(steps)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - start
        assert ran == steps and len(sched.running) == batch and not any(s.prefilling for s in sched.running)
        # every pass does the same work: batch * steps tokens, all of them arrived
        assert sum(len(s.generated) for s in sched.running) - generated_before == batch * steps
        assert all(t >= 0 for s in sched.running for t in s.generated)
        held.append(sum(engine.cache.num_tokens(s.seq_id) for s in sched.running))
        return elapsed / steps

    median, spread, _ = measured(one_pass, f"decode at batch {batch}")
    recordings = engine.executor.runner.graph_recordings
    del engine, sched
    torch.cuda.empty_cache()
    return median, spread, sum(held) / len(held), blocks, recordings


def baseline_decode_run(model, cfg, batch: int, prompt_len: int = 512, new_tokens: int = 256, block_size: int = 16):
    """The reference's own decode workload: `batch` requests of `prompt_len`-token prompts, `new_tokens`
    greedy tokens each.  The prompts run first, untimed (each yields its request's first token); the clock
    runs over the decode steps that give the other new_tokens - 1 tokens of every request, to the last
    token's arrival on the host.  One engine serves all passes (its recorded steps are made in the first
    pass, which is discarded).  Returns (median seconds, range, decoded tokens a pass, mean tokens held)."""
    import torch
    import paged_attention_engine_amd as pae

    dtype = "bfloat16" if model.dtype == torch.bfloat16 else "float32"
    blocks = batch * (-(-(prompt_len + new_tokens) // block_size) + 1) + 2
    engine = pae.Engine(model, dtype=dtype, block_size=block_size, num_blocks=blocks, max_num_seqs=batch,
                        max_num_batched_tokens=2048)
    sched = engine.scheduler
    gen = torch.Generator().manual_seed(DECODE_TOKEN_SEED)
    counted, number = [], [0]

    def one_pass():
        number[0] += 1
        names = [f"p{number[0]}b{b}" for b in range(batch)]
        for name in names:
            prompt = torch.randint(0, cfg["vocab_size"], (prompt_len,), generator=gen).tolist()
            assert engine.add_request(pae.Request(name, tuple(prompt), new_tokens))
        while len(sched.waiting) or any(s.prefilling for s in sched.running):
            engine.step()
        before = sum(len(s.generated) for s in sched.running)
        torch.cuda.synchronize()
        start = time.perf_counter()
        engine.run_to_completion()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - start
        done = sum(len(engine.finished[name].generated) for name in names)
        assert done == batch * new_tokens and not sched.running
        counted.append(done - before)
        return elapsed

    one_pass()  # warm-up, discarded
    median, spread, _ = measured(one_pass, f"{prompt_len}+{new_tokens} decode at batch {batch}")
    assert len(set(counted)) == 1, counted  # every pass decodes the same number of tokens
    del engine, sched
    torch.cuda.empty_cache()
    return median, spread, counted[0], batch * (prompt_len + new_tokens / 2)


def prefill_run(model, cfg, T: int, block_size: int = 16):
    """One prompt of T tokens in one step, a fresh engine each pass (first pass discarded).
    Returns (median seconds, range seconds)."""
    import torch
    import paged_attention_engine_amd as pae

    dtype = "bfloat16" if model.dtype == torch.bfloat16 else "float32"
    gen = torch.Generator().manual_seed(PREFILL_TOKEN_SEED)

    def one_pass():
        engine = pae.Engine(model, dtype=dtype, block_size=block_size, num_blocks=-(-T // block_size) + 4,
                            max_num_seqs=1, max_num_batched_tokens=T)
        prompt = torch.randint(0, cfg["vocab_size"], (T,), generator=gen).tolist()
        engine.add_request(pae.Request("p", tuple(prompt), 1))
        torch.cuda.synchronize()
        start = time.perf_counter()
        result = engine.step()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - start
        assert result.finished == ("p",), result
        del engine
        return elapsed

    one_pass()  # warm-up, discarded
    median, spread, _ = measured(one_pass, f"prefill of {T} tokens")
    return median, spread


def main() -> int:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=64)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--ctx", type=int, default=4096)
    parser.add_argument("--model", choices=("0.5b", "1.5b", "3b", "7b", "14b", "32b", "72b"), default="1.5b",
                        help="layer sizes (default: the Qwen2.5-1.5B shape of the headline figure)")
    parser.add_argument("--layers", type=int, default=None, help="fewer layers than the shape has")
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
    shape = QWEN25_1P5B if args.model == "1.5b" else OTHER_SHAPES[args.model]
    args.full_layers = shape["num_hidden_layers"]
    args.layers = args.layers or args.full_layers
    args.shape_name = f"Qwen2.5-{args.model.upper()} shape"
    cfg = dict(shape, num_hidden_layers=args.layers)
    elem = 2 if args.dtype == "bfloat16" else 4
    model = build_model(cfg, args.dtype)

    try:
        return report(args, cfg, elem, model)
    except Refused as err:
        print(f"bench.py: {err}")
        return 2
    except Unresolved as err:
        print(json.dumps({"metric": f"decode tok/s at batch {args.batch}, context {args.ctx} ({args.shape_name})",
                          "value": None, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
                          "invalid": str(err)}))
        return 3


def report(args, cfg, elem, model) -> int:
    if args.prefill_only:
        pre_s, pre_range = prefill_run(model, cfg, 2048)
        print(json.dumps({"metric": f"prefill tok/s at 2,048 tokens ({args.shape_name})", "value": round(2048 / pre_s, 1),
                          "unit": "tokens/s", "ms": round(pre_s * 1e3, 3), "range_ms": round(pre_range * 1e3, 3),
                          "dtype": args.dtype,
                          "frac": round(prefill_flops(cfg, 2048) / pre_s / PEAK_FLOPS[args.dtype], 4)}))
        return 0
    step_s, step_range, tokens_held, pages, recordings = decode_run(model, cfg, args.batch, args.ctx, args.steps,
                                                                     args.warmup)
    value = args.batch / step_s
    step_bytes = weight_bytes(cfg, elem) + kv_bytes(cfg, tokens_held, elem)
    achieved = step_bytes / step_s / 1e9
    record = {
        "metric": f"decode tok/s at batch {args.batch}, context {args.ctx} ({args.shape_name})",
        "value": round(value, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: seeded uniform token ids, random weights N(0, 0.02)",
        "config": {"model": args.shape_name, "global_batch": args.batch, "seq_len": args.ctx,
                   "parallelism": "single GPU", "layers": args.layers, "layers_of_model": args.full_layers,
                   "hidden": cfg["hidden_size"], "q_heads": cfg["num_attention_heads"],
                   "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"],
                   "intermediate": cfg["intermediate_size"], "vocab": cfg["vocab_size"],
                   "tied_head": bool(cfg["tie_word_embeddings"]), "block_size": 16, "prefill_tokens": 2048},
        "passes": MEASURED_PASSES, "range_ms_per_step": round(step_range * 1e3, 4),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }
    if not args.no_points:
        T = 2048
        pre_s, pre_range = prefill_run(model, cfg, T)
        record["prefill"] = {"value": round(T / pre_s, 1), "tokens": T, "ms": round(pre_s * 1e3, 3),
                             "frac": round(prefill_flops(cfg, T) / pre_s / PEAK_FLOPS[args.dtype], 4),
                             "range_ms": round(pre_range * 1e3, 3)}
        # tokens a second, and beside each the share of the HBM peak that its bytes a step come to
        points, fracs = {}, {}
        short = max(8, args.steps // 2)

        def point(name, cfg_, batch, step_seconds, tokens_held):
            points[name] = round(batch / step_seconds, 2)
            moved = weight_bytes(cfg_, elem) + kv_bytes(cfg_, tokens_held, elem)
            fracs[name] = round(moved / step_seconds / 1e9 / HBM_PEAK_GBS, 4)

        for b in (1, 64):
            s, _, held, _, _ = decode_run(model, cfg, b, args.ctx, short, 4)
            point(f"decode_b{b}", cfg, b, s, held)
        if args.model == "1.5b" and args.layers == args.full_layers and args.ctx == 4096:
            # the reference's own decode workload: 512-token prompts, 256 greedy tokens each
            for b in (1, 8, 64):
                s, _, decoded, held = baseline_decode_run(model, cfg, b)
                point(f"decode_512p256_b{b}", cfg, b, s / (decoded / b), held)
            # a longer context at the headline batch
            s, _, held, _, _ = decode_run(model, cfg, 8, 16384, short, 4)
            point("decode_b8_ctx16384", cfg, 8, s, held)
            # the 7B layer sizes at the headline batch and context
            import torch
            del model
            torch.cuda.empty_cache()
            cfg7 = dict(OTHER_SHAPES["7b"])
            model = build_model(cfg7, args.dtype)
            s, _, held, _, _ = decode_run(model, cfg7, 8, 4096, short, 4)
            point("decode_7b_b8", cfg7, 8, s, held)
        record["points"] = points
        record["points_hbm_frac"] = fracs
    record["provenance"] = provenance(model, {"pool_pages": pages, "graph_recordings_in_run": recordings})
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    sys.exit(main())
