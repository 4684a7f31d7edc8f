"""Command line: token ids in, generated token ids out.

The reference has no generation command, only benchmark ones
(`python -m bench.run --stream ... --seed S -C N`, bench/run.py:846-885); the
options here carry the names of its scheduler's and cache's settings
(engine/scheduler.py:317-349, engine/cache.py:29-35).  Token ids go in and come
out: the reference's engine never touches a tokenizer either.
"""

from __future__ import annotations

import argparse
import json
import sys
from typing import List, Optional


def _parse_ids(text: str) -> List[int]:
    return [int(t) for t in text.replace(",", " ").split()]


def main(argv: Optional[List[str]] = None) -> int:
    p = argparse.ArgumentParser(prog="paged_attention_engine_amd", description=__doc__,
                                formatter_class=argparse.RawDescriptionHelpFormatter)
    src = p.add_mutually_exclusive_group(required=True)
    src.add_argument("--model", help="folder with config.json and safetensors weights")
    src.add_argument("--random-config", help="a config.json; random weights are drawn from --seed on the GPU "
                     "(nothing is written unless --save-model is given)")
    p.add_argument("--seed", type=int, default=0, help="seed of the random weights")
    p.add_argument("--save-model", help="with --random-config: draw the weights on the CPU, write the model folder "
                   "here and load it")
    p.add_argument("--dtype", choices=("bfloat16", "float32"), default=None,
                   help="default: the torch_dtype of the model's config.json (bfloat16 if it is neither of the two)")
    p.add_argument("--prompt-ids", action="append", default=[], help='one prompt as "1,2,3" (repeatable)')
    p.add_argument("--prompts-file", help="one prompt of token ids per line")
    p.add_argument("--max-new-tokens", type=int, default=16)
    p.add_argument("--temperature", type=float, default=0.0)
    p.add_argument("--sample-seed", type=int, default=0)
    p.add_argument("--block-size", type=int, default=16)
    pool = p.add_mutually_exclusive_group()
    pool.add_argument("--num-blocks", type=int, default=None, help="pages in the cache pool (default 3584)")
    pool.add_argument("--kv-bytes", type=int, default=None, help="or: bytes the cache may take")
    pool.add_argument("--fill-hbm", type=float, default=None,
                      help="or: share of the GPU memory free after loading that the cache takes, in (0, 1]")
    p.add_argument("--stop-token-ids", default="", help='token ids that end a request, as "1,2"')
    p.add_argument("--max-num-seqs", type=int, default=None)
    p.add_argument("--max-num-batched-tokens", type=int, default=None)
    p.add_argument("--admission-margin-blocks", type=int, default=1)
    p.add_argument("--dump-logits", help="write every request's per-token logits to this .pt file")
    args = p.parse_args(argv)

    prompts = [_parse_ids(t) for t in args.prompt_ids]
    if args.prompts_file:
        with open(args.prompts_file) as handle:
            prompts += [_parse_ids(line) for line in handle if line.strip()]
    if not prompts:
        p.error("no prompts: give --prompt-ids or --prompts-file")

    from .. import read_config_dict, write_model_folder
    from .llm import Engine
    from .scheduler import EventKind, Request

    options = dict(dtype=args.dtype, block_size=args.block_size, num_blocks=args.num_blocks, kv_bytes=args.kv_bytes,
                   fill_hbm=args.fill_hbm, max_num_seqs=args.max_num_seqs,
                   max_num_batched_tokens=args.max_num_batched_tokens,
                   admission_margin_blocks=args.admission_margin_blocks, record_logits=bool(args.dump_logits))
    if args.random_config:
        with open(args.random_config) as handle:
            config = read_config_dict(json.load(handle))
        if args.save_model:
            write_model_folder(config, args.seed, args.save_model)
            engine = Engine(args.save_model, **options)
        else:
            engine = Engine.from_random(config, args.seed, **options)
    else:
        engine = Engine(args.model, **options)
    stops = tuple(_parse_ids(args.stop_token_ids))
    for i, prompt in enumerate(prompts):
        ok = engine.add_request(Request(f"r{i}", tuple(prompt), args.max_new_tokens, args.temperature,
                                        args.sample_seed, stops))
        if not ok:
            print(json.dumps({"request_id": f"r{i}", "rejected": engine.events_of(EventKind.REJECT)[-1].detail}))
    outputs = engine.run_to_completion()
    for rid in sorted(outputs, key=lambda r: int(r[1:])):
        print(json.dumps({"request_id": rid, "token_ids": list(outputs[rid])}))
    if args.dump_logits:
        import torch
        torch.save({rid: torch.stack(seq.step_logits) for rid, seq in engine.finished.items()}, args.dump_logits)
    return 0


if __name__ == "__main__":
    sys.exit(main())
