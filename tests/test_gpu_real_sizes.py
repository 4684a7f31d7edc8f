"""Whole-model logits at the layer sizes the engine is measured at, against the plain implementation.

Two-layer models with the real hidden width, head counts, head size, feed-forward width and
vocabulary of the Qwen2.5 1.5B, 7B and 72B shapes (and of the 0.5B and 3B shapes, for the replay schedules),
random weights drawn on the GPU (the product's
`random_model`; the plain implementation gets the same tensors from the same generator and runs in
float64 on the GPU as well).  These are the widths at which the serving kernels differ from what
the tiny models exercise: heads of 128 with 6, 7 and 8 query heads per key/value head in the
matrix-core attention, k ranges added up inside the products, the products for 17 to 64 rows, the
152k-row head, recorded decode steps.  With N(0, 0.02) weights at these widths the scores are one
to three units wide, so attention is peaked by itself.

Every shape is replayed in the four schedules of `tests/test_gpu_replay.py` (whole; the last 32
tokens one by one; portions down to two tokens; four live requests mixed in a pool so small that
pages are used again) through the same `TraceReplayer` that `bin/trace_run` drives; the 1.5B shape
also goes through the program itself, from a folder.  float32 must agree with the plain logits to
1e-5 of the largest logit and bit for bit between schedules; bfloat16 within the bounds of
`tests/helpers.py`.  Then requests are pushed through the scheduler in a pool too small for them,
so that some are preempted and replayed, and every recorded logit row is compared with the plain
logits of the same history.  (The reference's counterparts: tests/test_parity.py:226-330 on a real
checkpoint, tests/test_sched.py:776-825 for preemption.)
"""

import gc
import os

import numpy as np
import pytest
import torch

import paged_attention_engine_amd as pae
from paged_attention_engine_amd.engine.model import random_model
from paged_attention_engine_amd.engine.trace import TraceReplayer
from paged_attention_engine_amd.weights import RandomWeights
from tests import helpers
from tests.plain import qwen2_plain as plain
from tests.test_gpu_replay import build_trace, peak_live_tokens, run_trace

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

COMMON = dict(architectures=["Qwen2ForCausalLM"], num_hidden_layers=2, rope_theta=1000000.0,
              use_sliding_window=False, max_position_embeddings=32768, hidden_act="silu")
SHAPES = {
    "0.5b": dict(hidden_size=896, num_attention_heads=14, num_key_value_heads=2, head_dim=64,
                 intermediate_size=4864, vocab_size=151936, rms_norm_eps=1e-6, tie_word_embeddings=True),
    "3b": dict(hidden_size=2048, num_attention_heads=16, num_key_value_heads=2, head_dim=128,
               intermediate_size=11008, vocab_size=151936, rms_norm_eps=1e-6, tie_word_embeddings=True),
    "1.5b": dict(hidden_size=1536, num_attention_heads=12, num_key_value_heads=2, head_dim=128,
                 intermediate_size=8960, vocab_size=151936, rms_norm_eps=1e-6, tie_word_embeddings=True),
    "7b": dict(hidden_size=3584, num_attention_heads=28, num_key_value_heads=4, head_dim=128,
               intermediate_size=18944, vocab_size=152064, rms_norm_eps=1e-6, tie_word_embeddings=False),
    "72b": dict(hidden_size=8192, num_attention_heads=64, num_key_value_heads=8, head_dim=128,
                intermediate_size=29568, vocab_size=152064, rms_norm_eps=1e-5, tie_word_embeddings=False),
}
SEED = 21
LENGTHS = (70, 100, 45, 130)


def config_of(shape):
    return dict(COMMON, **SHAPES[shape])


def plain_weights(cfg):
    """The tensors `random_model(cfg, SEED)` is built from, as float64 on the GPU."""
    expected = pae.expected_tensors(pae.read_config_dict(cfg).plan())
    drawn = RandomWeights(expected, SEED, device=DEV)
    return {name: drawn[name].double() for name in expected}


def free_gpu():
    gc.collect()
    torch.cuda.empty_cache()


def request_tokens(cfg, lengths, seed):
    gen = torch.Generator().manual_seed(seed)
    return {f"q{i}": torch.randint(0, cfg["vocab_size"], (n,), generator=gen).tolist() for i, n in enumerate(lengths)}


def compare_trace(trace, step_logits, want, dtype, vocab):
    """Every wanted row against the plain logits; float32 rows of one (request, position) must be
    the same bits in every schedule.  Returns (worst, rms, rows)."""
    top = max(float(w.abs().max()) for w in want.values())
    atol, rms_bound = helpers.bounds(dtype, torch.tensor(top), "wide")
    seen, worst, squares, checked = {}, 0.0, 0.0, 0
    for rec in trace.records:
        rows = trace.wanted.get(rec["step"])
        got = step_logits.get(rec["step"])
        assert (got is not None) == bool(rows)
        if not rows:
            continue
        assert got.shape == (len(rows), vocab)
        for row, (req, pos) in zip(got, rows):
            diff = row.double() - want[req][pos].double()
            err = float(diff.abs().max())
            assert err <= atol, f"step {rec['step']} ({req}, position {pos}): error {err:.3e} > {atol:.3e}"
            worst, squares, checked = max(worst, err), squares + float(diff.pow(2).mean()), checked + 1
            if dtype == "float32":
                first = seen.setdefault((req, pos), row)
                assert torch.equal(first, row), f"step {rec['step']} ({req}, {pos}) differs between schedules"
    rms = (squares / checked) ** 0.5
    assert rms <= rms_bound, f"root-mean-square error {rms:.3e} > {rms_bound:.3e}"
    return worst, rms, checked, atol


@pytest.mark.parametrize("shape,dtype", [(shape, dtype) for shape in ("1.5b", "7b", "72b") for dtype in ("float32", "bfloat16")]
                         # the widths in between (other branches of the kernels' rules; heads of 64 at the 0.5B sizes)
                         + [("0.5b", "float32"), ("0.5b", "bfloat16"), ("3b", "bfloat16")])
def test_replay_schedules_at_real_layer_sizes(shape, dtype):
    cfg = config_of(shape)
    tokens = request_tokens(cfg, LENGTHS, 11)
    weights = plain_weights(cfg)
    want = {n: plain.logits(weights, cfg, ids, torch.float64).float().cpu() for n, ids in tokens.items()}
    del weights
    free_gpu()

    model = random_model(cfg, SEED, dtype, DEV)
    trace = build_trace(tokens)
    replayer = TraceReplayer(model, dtype, peak_live_tokens(trace), block_size=16)
    step_logits = {}
    for rec in trace.records:
        out = replayer.step(rec)
        if out is not None:
            step_logits[rec["step"]] = torch.from_numpy(out)
    worst, rms, checked, atol = compare_trace(trace, step_logits, want, dtype, cfg["vocab_size"])
    runner = replayer.runner
    print(f"{shape} {dtype}: {len(trace.records)} steps, {checked} rows, worst error {worst:.3e} (bound {atol:.3e}), "
          f"rms {rms:.3e}, {runner.graph_recordings} recorded steps replayed {runner.graph_replays} times")
    assert runner.graph_replays > 100  # the one-token steps ran as recorded graphs
    assert replayer.cache.free_blocks() == tuple(g.allocator.num_blocks for g in replayer.cache.groups)
    del replayer, model, runner
    free_gpu()


def test_the_replay_program_at_the_1p5b_layer_sizes(tmp_path):
    """`bin/trace_run` itself on a folder of the 1.5B widths, in the precision that serves."""
    cfg = config_of("1.5b")
    folder = pae.write_model_folder(pae.read_config_dict(cfg), SEED, str(tmp_path / "wide"))
    cfg_read, weights = helpers.read_folder_plain(folder)
    weights = {k: v.to(DEV).double() for k, v in weights.items()}
    tokens = request_tokens(cfg, (70, 45), 12)
    want = {n: plain.logits(weights, cfg_read, ids, torch.float64).float().cpu() for n, ids in tokens.items()}
    del weights
    free_gpu()
    trace = build_trace(tokens)
    out_dir = str(tmp_path / "out")
    run_trace(folder, "bfloat16", out_dir, peak_live_tokens(trace), 16, trace.records)
    step_logits = {}
    for rec in trace.records:
        path = os.path.join(out_dir, f"{rec['step']}.f32")
        if os.path.exists(path):
            step_logits[rec["step"]] = torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(-1, cfg["vocab_size"]))
    worst, rms, checked, atol = compare_trace(trace, step_logits, want, "bfloat16", cfg["vocab_size"])
    print(f"bin/trace_run at the 1.5B widths: {checked} rows, worst error {worst:.3e} (bound {atol:.3e}), rms {rms:.3e}")


@pytest.mark.parametrize("shape,dtype", [("1.5b", "float32"), ("1.5b", "bfloat16"), ("7b", "bfloat16"), ("72b", "bfloat16")])
def test_preemption_and_replay_at_real_layer_sizes(shape, dtype):
    """Six requests that grow to 150 tokens each in a pool of 40 pages (they want 60): the newest are
    preempted and replay prompt and generated tokens in portions beside the others' decoding.
    Every logit row the scheduler recorded, replayed or not, is the plain implementation's for the
    same history; in float32 the tokens are those of each request run alone."""
    cfg = config_of(shape)
    model = random_model(cfg, SEED, dtype, DEV)
    gen = torch.Generator().manual_seed(31)
    requests = [pae.Request(f"g{i}", tuple(torch.randint(0, cfg["vocab_size"], (30 + 5 * i,), generator=gen).tolist()),
                            110 - 5 * i) for i in range(6)]
    engine = pae.Engine(model, dtype=dtype, block_size=16, num_blocks=40, max_num_batched_tokens=48,
                        record_logits=True)
    for r in requests:
        assert engine.add_request(r)
    out = engine.run_to_completion()
    preempted = engine.events_of(pae.EventKind.PREEMPT)
    assert preempted and engine.events_of(pae.EventKind.RECOMPUTE)
    assert engine.cache.free_blocks() == (40,)
    recorded = {r.request_id: torch.stack(engine.finished[r.request_id].step_logits) for r in requests}
    alone = {}
    if dtype == "float32":
        for r in requests:
            single = pae.Engine(model, dtype=dtype, block_size=16, num_blocks=16)
            single.add_request(r)
            alone.update(single.run_to_completion())
            del single
        assert out == alone
    del engine, model
    free_gpu()

    weights = plain_weights(cfg)
    worst = 0.0
    for r in requests:
        history = list(r.prompt_token_ids) + list(out[r.request_id])
        want = plain.logits(weights, cfg, history[:-1], torch.float64)[len(r.prompt_token_ids) - 1:].float().cpu()
        assert recorded[r.request_id].shape == want.shape
        worst = max(worst, helpers.check_logits(recorded[r.request_id], want, dtype, "wide", f"{shape} {r.request_id}"))
        atol = helpers.bounds(dtype, want, "wide")[0]
        top2 = want.topk(2, dim=-1).values
        for k, token in enumerate(out[r.request_id]):  # greedy tokens wherever the plain margin allows
            if float(top2[k, 0] - top2[k, 1]) > 2 * atol:
                assert token == int(want[k].argmax()), f"{r.request_id}: token {k}"
    print(f"{shape} {dtype}: {len(preempted)} preemptions, worst logit error {worst:.3e}")
    del weights
    free_gpu()
