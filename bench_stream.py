"""Stream throughput of the engine: many requests through the scheduler, random weights.

    python bench_stream.py --model 7b            # ragged stream of the Qwen2.5-7B shape
    python bench_stream.py --model 72b           # 64 requests of 1,024 + 256 at the 72B shape
    python bench_stream.py --model 72b --num-blocks 4096   # the same in an undersized pool

The reference's published numbers are of this kind (generated tokens / wall time of
`run_to_completion`, prefill and scheduling included, bench/run.py:463-528), on synthetic
streams of uniform random token ids (bench/workload.py:241-254).  Workloads:

  1.5b / 7b   256 requests, prompt lengths uniform in [16, 3072], decode lengths uniform in
              [8, 1024], max_num_seqs 64, max_num_batched_tokens 8192
  72b         64 requests of 1,024-token prompts with 256 greedy new tokens; the pool takes what
              is left of HBM, or --num-blocks pages to force preemption with recompute

One JSON line is printed.  With --check-against N the run is repeated in a pool of N pages and
the two runs' tokens are compared request by request.  With --passes N (after one discarded
pass) the figure is the median pass and its range is given; a range beyond 20 % of the median
gives no figure (bench/run.py:628-702 of the reference).  A run in a pool that even the
smallest `max_num_seqs` requests overflow must record preemptions, or it is invalid and no
figure is given either (bench/run.py:581-622).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

SHAPES = {
    "1.5b": dict(num_hidden_layers=28, hidden_size=1536, num_attention_heads=12, num_key_value_heads=2,
                 head_dim=128, intermediate_size=8960, vocab_size=151936, rms_norm_eps=1e-6,
                 tie_word_embeddings=True),
    "7b": dict(num_hidden_layers=28, hidden_size=3584, num_attention_heads=28, num_key_value_heads=4,
               head_dim=128, intermediate_size=18944, vocab_size=152064, rms_norm_eps=1e-6,
               tie_word_embeddings=False),
    "72b": dict(num_hidden_layers=80, hidden_size=8192, num_attention_heads=64, num_key_value_heads=8,
                head_dim=128, intermediate_size=29568, vocab_size=152064, rms_norm_eps=1e-5,
                tie_word_embeddings=False),
}
COMMON = dict(architectures=["Qwen2ForCausalLM"], rope_theta=1000000.0, use_sliding_window=False,
              max_position_embeddings=32768, hidden_act="silu")


def make_requests(model: str, count: int, seed: int, vocab: int):
    import torch
    import paged_attention_engine_amd as pae

    gen = torch.Generator().manual_seed(seed)
    out = []
    for i in range(count):
        if model == "72b":
            prompt_len, new = 1024, 256
        else:
            prompt_len = int(torch.randint(16, 3073, (1,), generator=gen))
            new = int(torch.randint(8, 1025, (1,), generator=gen))
        prompt = torch.randint(0, vocab, (prompt_len,), generator=gen).tolist()
        out.append(pae.Request(f"s{i}", tuple(prompt), new))
    return out


class InvalidRun(RuntimeError):
    pass


def forced_demand(requests, block_size: int, max_num_seqs: int) -> int:
    """Pages that the `max_num_seqs` smallest requests need at their full lengths: a lower bound on
    any resident set once the queue is longer than that, so a smaller pool must evict."""
    per_request = sorted(-(-r.max_total_len // block_size) for r in requests)
    return sum(per_request[:min(max_num_seqs, len(per_request))])


def run_stream(model, requests, block_size, pool, max_num_seqs, budget):
    """`pool`: keyword arguments of the engine that size its cache (num_blocks / kv_bytes / fill_hbm)."""
    import torch
    import paged_attention_engine_amd as pae

    engine = pae.Engine(model, dtype="bfloat16", block_size=block_size, max_num_seqs=max_num_seqs,
                        max_num_batched_tokens=budget, **pool)
    num_blocks = engine.num_blocks
    for r in requests:
        if not engine.add_request(r):
            raise SystemExit(f"request {r.request_id} rejected: {engine.events_of(pae.EventKind.REJECT)[-1].detail}")
    tokens_to_run = sum(r.max_total_len - 1 for r in requests)  # without replays
    torch.cuda.synchronize()
    start = time.perf_counter()
    steps = 0
    last = start
    sched = engine.scheduler
    while not sched.idle:
        # the engine's own loop (the next step is launched while the current one runs), in
        # stretches so that a long run reports where it is
        steps += engine.run_steps(64)
        if time.perf_counter() - last > 30:
            last = time.perf_counter()
            print(f"[stream] step {steps}: {len(engine.finished)} finished, {len(sched.running)} running, "
                  f"{len(sched.waiting)} waiting, {engine.cache.min_free_blocks()} free pages",
                  file=sys.stderr, flush=True)
    torch.cuda.synchronize()
    wall = time.perf_counter() - start
    tokens_run = tokens_to_run + sum(int(e.detail.split()[1]) for e in engine.events_of(pae.EventKind.RECOMPUTE))
    outputs = {rid: tuple(seq.generated) for rid, seq in engine.finished.items()}
    stats = dict(wall_s=wall, steps=steps, mean_batch_tokens=tokens_run / max(steps, 1),
                 preemptions=len(engine.events_of(pae.EventKind.PREEMPT)),
                 recomputes=len(engine.events_of(pae.EventKind.RECOMPUTE)), num_blocks=num_blocks,
                 graph_recordings=engine.executor.runner.graph_recordings,
                 graph_replays=engine.executor.runner.graph_replays)
    demand = forced_demand(requests, block_size, max_num_seqs)
    if demand > num_blocks and stats["preemptions"] == 0:
        raise InvalidRun(f"no preemption was recorded although the {max_num_seqs} smallest requests alone need "
                         f"{demand} pages and the pool has {num_blocks}: the run did not measure what it claims")
    del engine
    torch.cuda.empty_cache()
    return outputs, stats


def main() -> int:
    p = argparse.ArgumentParser()
    p.add_argument("--model", choices=sorted(SHAPES), default="7b")
    p.add_argument("--requests", type=int, default=None)
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--layers", type=int, default=None, help="fewer layers than the shape has (named in the output)")
    p.add_argument("--block-size", type=int, default=16)
    p.add_argument("--num-blocks", type=int, default=None, help="pages in the pool (default: what the workload needs, "
                   "or for 72b what is left of HBM)")
    p.add_argument("--max-num-seqs", type=int, default=64)
    p.add_argument("--max-num-batched-tokens", type=int, default=8192)
    p.add_argument("--check-against", type=int, default=None, metavar="PAGES",
                   help="repeat in a pool of this many pages and compare the tokens")
    p.add_argument("--passes", type=int, default=1, help="timed passes after one discarded pass (median and range)")
    p.add_argument("--fill-hbm", type=float, default=0.93, help="72b without --num-blocks: share of the free memory "
                   "the cache takes (the rest is for the activations of 8,192-token steps)")
    args = p.parse_args()

    import torch
    from bench import SPREAD_LIMIT, build_model, provenance, settle

    cfg = dict(COMMON, **SHAPES[args.model])
    full_layers = cfg["num_hidden_layers"]
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    print(f"[stream] drawing random weights of the {args.model} shape on the device", file=sys.stderr, flush=True)
    model = build_model(cfg, "bfloat16")
    count = args.requests or (64 if args.model == "72b" else 256)
    requests = make_requests(args.model, count, args.seed, cfg["vocab_size"])
    generated = sum(r.max_new_tokens for r in requests)

    if args.num_blocks is not None:
        pool = dict(num_blocks=args.num_blocks)
    elif args.model == "72b":
        pool = dict(fill_hbm=args.fill_hbm)
    else:
        longest = sorted((r.max_total_len for r in requests), reverse=True)[:args.max_num_seqs]
        pool = dict(num_blocks=sum(-(-n // args.block_size) + 1 for n in longest) + 8)
    print(f"[stream] {count} requests, {generated} tokens to generate, pool {pool}", file=sys.stderr, flush=True)

    def one_pass():
        outputs, stats = run_stream(model, requests, args.block_size, pool, args.max_num_seqs,
                                    args.max_num_batched_tokens)
        assert sum(len(v) for v in outputs.values()) == generated  # every pass does the same work
        return outputs, stats

    try:
        if args.passes > 1:
            one_pass()  # discarded
        runs = [one_pass() for _ in range(max(1, args.passes))]
    except InvalidRun as err:
        print(json.dumps({"metric": f"stream tok/s, {args.model} shape", "value": None, "invalid": str(err)}))
        return 3
    outputs, stats = runs[0]
    assert all(run[0] == outputs for run in runs), "passes of one greedy stream gave different tokens"
    wall, wall_range = settle([run[1]["wall_s"] for run in runs])
    if wall_range > SPREAD_LIMIT * wall:
        print(json.dumps({"metric": f"stream tok/s, {args.model} shape", "value": None,
                          "invalid": f"{len(runs)} passes range over {wall_range / wall:.0%} of their median"}))
        return 3
    num_blocks = stats["num_blocks"]
    record = {
        "metric": f"stream tok/s, {args.model} shape, {count} requests, max_num_seqs {args.max_num_seqs}",
        "value": round(generated / wall, 2), "unit": "tokens/s", "generated_tokens": generated,
        "wall_s": round(wall, 3), "passes": len(runs), "range_s": round(wall_range, 3), "steps": stats["steps"],
        "mean_batch_tokens": round(stats["mean_batch_tokens"], 1), "preemptions": stats["preemptions"],
        "recomputes": stats["recomputes"], "num_blocks": num_blocks, "block_size": args.block_size,
        "pool_gib": round(num_blocks * model.page_bytes(args.block_size) / 2**30, 2),
        "forced_demand_pages": forced_demand(requests, args.block_size, args.max_num_seqs),
        "graph_recordings": stats["graph_recordings"], "graph_replays": stats["graph_replays"],
        "max_num_batched_tokens": args.max_num_batched_tokens, "layers": cfg["num_hidden_layers"],
        "layers_of_model": full_layers, "dtype": "bf16",
        "data": "synthetic: seeded uniform token ids and lengths, random weights N(0, 0.02)",
        "provenance": provenance(model, {"stream_seed": args.seed, "pool_pages": num_blocks}),
    }
    if args.check_against is not None:
        try:
            other, other_stats = run_stream(model, requests, args.block_size, dict(num_blocks=args.check_against),
                                            args.max_num_seqs, args.max_num_batched_tokens)
        except InvalidRun as err:
            print(json.dumps({"metric": f"stream tok/s, {args.model} shape", "value": None, "invalid": str(err)}))
            return 3
        same = sum(outputs[r] == other[r] for r in outputs)
        agree = sum(a == b for r in outputs for a, b in zip(outputs[r], other[r]))
        record["check"] = {"num_blocks": args.check_against, "value": round(generated / other_stats["wall_s"], 2),
                           "preemptions": other_stats["preemptions"], "recomputes": other_stats["recomputes"],
                           "requests_with_identical_tokens": same, "tokens_identical": agree, "tokens": generated}
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    sys.exit(main())
