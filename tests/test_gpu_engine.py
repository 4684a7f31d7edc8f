"""The engine end to end on the GPU: generation through the entry points, the
scheduler on a real model (mixed batches, portions, preemption with recompute,
temperature sampling), long decoding, the first tokens of a sequence, replayed
HIP graphs against eager steps, and one pass of the model per step."""

import json
import os
import subprocess
import sys

import pytest
import torch

import paged_attention_engine_amd as pae
from tests import helpers
from tests.plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def tokens_of(cfg, n, seed):
    return torch.randint(0, cfg["vocab_size"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def atol_for(dtype, want, name=""):
    return helpers.bounds(dtype, want, name)[0]


def check_teacher_forced(cfg, weights, prompt, generated, step_logits, dtype, exact_tokens, greedy=True, name=""):
    """`step_logits[k]` produced `generated[k]`: compare every row with the plain logits of
    the same history, and the tokens with the plain argmax where the margin allows."""
    history = list(prompt) + list(generated)
    want = plain.logits({k: v.double() for k, v in weights.items()}, cfg, history[:-1], torch.float64).float()
    want = want[len(prompt) - 1:]
    atol = atol_for(dtype, want, name)
    err = helpers.check_logits(step_logits, want, dtype, name, "teacher-forced rows")
    top2 = want.topk(2, dim=-1).values
    for k, token in enumerate(generated if greedy else ()):
        if exact_tokens or float(top2[k, 0] - top2[k, 1]) > 2 * atol:
            assert token == int(want[k].argmax()), f"token {k} differs"
    return err


@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(tmp_path, name, dtype):
    folder = helpers.make_model_folder(tmp_path, name)
    cfg, weights = helpers.read_folder_plain(folder)
    prompt = tokens_of(cfg, 13, 3)
    engine = pae.Engine(folder, dtype=dtype, block_size=helpers.TINY[name][1]["block_size"], num_blocks=16)
    result = engine.generate(prompt, 32)
    assert len(result.token_ids) == 32 and result.step_logits.shape == (32, cfg["vocab_size"])
    err = check_teacher_forced(cfg, weights, prompt, result.token_ids, result.step_logits, dtype, dtype == "float32",
                               name=name)
    print(f"{name} {dtype}: 32 greedy tokens, worst logit error {err:.3e}")
    assert engine.cache.free_blocks() == tuple(g.allocator.num_blocks for g in engine.cache.groups)
    with pytest.raises(ValueError):
        engine.generate([], 4)
    with pytest.raises(ValueError):
        engine.generate(prompt, 0)


def test_command_line_generates_the_same_tokens(tmp_path):
    folder = helpers.make_model_folder(tmp_path, "A")
    cfg, weights = helpers.read_folder_plain(folder)
    want, _ = plain.greedy_generate(weights, cfg, [5, 17, 3, 99], 6)
    out = subprocess.run([sys.executable, "-m", "paged_attention_engine_amd", "--model", folder, "--dtype", "float32",
                          "--prompt-ids", "5,17,3,99", "--prompt-ids", "7 8", "--max-new-tokens", "6",
                          "--num-blocks", "8", "--max-num-batched-tokens", "3"],
                         cwd=ROOT, capture_output=True, text=True, check=True)
    lines = [json.loads(line) for line in out.stdout.splitlines() if line.startswith("{")]
    assert lines[0] == {"request_id": "r0", "token_ids": want}
    assert lines[1]["request_id"] == "r1" and len(lines[1]["token_ids"]) == 6
    # random-weights mode writes the folder itself
    cfg_path = tmp_path / "cfg.json"
    cfg_path.write_text(json.dumps(helpers.TINY_A))
    out = subprocess.run([sys.executable, "-m", "paged_attention_engine_amd", "--random-config", str(cfg_path),
                          "--seed", "0", "--dtype", "float32", "--prompt-ids", "5,17,3,99", "--max-new-tokens", "6",
                          "--num-blocks", "8", "--save-model", str(tmp_path / "saved")],
                         cwd=ROOT, capture_output=True, text=True, check=True)
    assert json.loads(out.stdout.splitlines()[-1])["token_ids"] == want  # same seed as make_model_folder("A")
    assert sorted(os.listdir(tmp_path / "saved")) == ["config.json", "model.safetensors"]


def test_command_line_draws_random_weights_on_the_device_and_sizes_the_pool_by_bytes(tmp_path):
    """`--random-config` without `--save-model` draws the weights on the GPU and writes nothing; the
    pool is sized as a share of the free memory or by a byte budget, which changes no token; without
    `--dtype` the precision is the config's `torch_dtype`."""
    cfg_path = tmp_path / "cfg.json"
    cfg_path.write_text(json.dumps(dict(helpers.TINY_A, torch_dtype="float32")))

    def run(*extra):
        out = subprocess.run([sys.executable, "-m", "paged_attention_engine_amd", "--random-config", str(cfg_path),
                              "--seed", "3", "--prompt-ids", "5,17,3,99", "--prompt-ids", "8 9 10",
                              "--max-new-tokens", "7", "--dump-logits", str(tmp_path / "logits.pt"), *extra],
                             cwd=ROOT, capture_output=True, text=True)
        assert out.returncode == 0, out.stderr[-2000:]
        lines = [json.loads(line) for line in out.stdout.splitlines() if line.startswith("{")]
        return [line["token_ids"] for line in lines], torch.load(tmp_path / "logits.pt", weights_only=True)

    by_share, logits = run("--fill-hbm", "0.05")
    assert [len(t) for t in by_share] == [7, 7]
    assert logits["r0"].dtype == torch.float32 and logits["r0"].shape == (7, helpers.TINY_A["vocab_size"])
    by_bytes, logits_again = run("--kv-bytes", str(1 << 22))
    assert by_bytes == by_share and torch.equal(logits_again["r0"], logits["r0"])  # float32: bit for bit
    in_bf16, _ = run("--kv-bytes", str(1 << 22), "--dtype", "bfloat16")
    assert [len(t) for t in in_bf16] == [7, 7]
    assert sorted(os.listdir(tmp_path)) == ["cfg.json", "logits.pt"]  # no model folder was written


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(tmp_path, dtype):
    """400 decoded tokens: pages fill one after the other and the windowed group of model D gives
    pages back on the way.  (The tables stay below 64 pages here; recorded steps whose tables grow
    past that are covered in tests/test_gpu_long_context.py.)"""
    for name in ("B", "D"):
        folder = helpers.make_model_folder(tmp_path, name)
        cfg, weights = helpers.read_folder_plain(folder)
        prompt = tokens_of(cfg, 9, 8)
        engine = pae.Engine(folder, dtype=dtype, block_size=helpers.TINY[name][1]["block_size"], num_blocks=64)
        result = engine.generate(prompt, 400)
        err = check_teacher_forced(cfg, weights, prompt, result.token_ids, result.step_logits, dtype, False)
        print(f"{name} {dtype}: 400 tokens, worst logit error {err:.3e}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_of_a_sequence(tmp_path, dtype):
    folder = helpers.make_model_folder(tmp_path, "A")
    cfg, weights = helpers.read_folder_plain(folder)
    ids = tokens_of(cfg, 4, 1)
    want = plain.logits({k: v.double() for k, v in weights.items()}, cfg, ids, torch.float64).float()
    model = pae.load_model(folder, dtype)
    cache = model.new_cache(16, 4, 2)
    runner = pae.StepRunner(model, cache)
    cache.create_sequence(0)
    rows = []
    for t in ids:  # one token at a time from the very first
        cache.reserve(0, 1)
        rows.append(runner.run([pae.StepEntry(0, (t,), (0,))]).cpu().clone())
    assert float((torch.cat(rows) - want).abs().max()) <= atol_for(dtype, want)
    # the first token's logits do not depend on anything but the token
    cache.create_sequence(1)
    cache.reserve(1, 1)
    again = runner.run([pae.StepEntry(1, (ids[0],), (0,))]).cpu()
    assert torch.equal(again, rows[0])


def baseline_requests(name):
    """The workloads of the two tiny baseline configurations."""
    cfg = helpers.TINY[name][0]
    if name == "A":
        lens, new, kw = (5, 17, 33, 1), 8, {}
    else:
        lens, new, kw = (3, 9, 40, 64, 2, 27), 12, dict(temperature=0.8, seed=7)
    return [pae.Request(f"r{i}", tuple(tokens_of(cfg, n, 100 + i)), new, **kw) for i, n in enumerate(lens)]


@pytest.mark.parametrize("name,budget", [("A", None), ("B", 32)])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_scheduler_runs_the_baseline_workloads(tmp_path, name, budget, dtype):
    from paged_attention_engine_amd.sampling import uniform_for

    folder = helpers.make_model_folder(tmp_path, name)
    cfg, weights = helpers.read_folder_plain(folder)
    requests = baseline_requests(name)
    block = helpers.TINY[name][1]["block_size"]
    engine = pae.Engine(folder, dtype=dtype, block_size=block, num_blocks=64, max_num_batched_tokens=budget,
                        record_logits=True)
    passes = engine.model.forward_pass_count
    for r in requests:
        assert engine.add_request(r)
    steps = 0
    while engine.scheduler.waiting or engine.scheduler.running:
        result = engine.step()
        steps += 1
        if budget:
            assert result.batched_token_cost <= budget
    assert engine.model.forward_pass_count - passes == steps  # one pass of the model per step
    if budget:  # prompts were cut into portions and ran beside decoded tokens
        assert steps > 12
    for r in requests:
        seq = engine.finished[r.request_id]
        logits = torch.stack(seq.step_logits)
        check_teacher_forced(cfg, weights, r.prompt_token_ids, seq.generated, logits, dtype, False,
                             greedy=r.temperature == 0)
        if r.temperature > 0 and dtype == "float32":
            for k, token in enumerate(seq.generated):  # the draw depends on (seed, request, index) alone
                u = uniform_for(r.seed, r.request_id, k)
                assert token == plain.sample_from_logits(logits[k], r.temperature, u)
    # each request alone gives the same tokens (float32: schedules agree exactly)
    if dtype == "float32":
        for r in requests:
            alone = pae.Engine(engine.model, dtype=dtype, block_size=block, num_blocks=64)
            alone.add_request(r)
            assert alone.run_to_completion()[r.request_id] == tuple(engine.finished[r.request_id].generated)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "D", "E"])
def test_preemption_with_recompute_is_transparent(tmp_path, name, dtype):
    """Four requests that grow far beyond what admission charged them, in a pool that cannot
    hold them all: some are evicted and replayed, and every token equals the run alone.  Models D
    and E take the serving kernels (matrix-core attention over pages that were given back and
    taken again, windows with holes, the few-row products); E's attention is peaked.  In
    bfloat16, where a replay sums in another order than the first run, a request's tokens may part
    from the run alone only at a token where the plain logits nearly tie."""
    folder = helpers.make_model_folder(tmp_path, name)
    cfg, weights = helpers.read_folder_plain(folder)
    weights64 = {k: v.double() for k, v in weights.items()}
    model = pae.load_model(folder, dtype)
    requests = [pae.Request(f"g{i}", tuple(tokens_of(cfg, 4, 50 + i)), 60) for i in range(4)]
    alone = {}
    for r in requests:
        engine = pae.Engine(model, dtype=dtype, block_size=16, num_blocks=16)
        engine.add_request(r)
        alone.update(engine.run_to_completion())
    small = pae.Engine(model, dtype=dtype, block_size=16, num_blocks=6, max_num_batched_tokens=24, record_logits=True)
    for r in requests:
        assert small.add_request(r)
    out = small.run_to_completion()
    assert small.events_of(pae.EventKind.PREEMPT) and small.events_of(pae.EventKind.RECOMPUTE)
    if dtype == "float32":
        assert out == alone
    for r in requests:  # replayed or not, every logit row is that of the plain implementation
        seq = small.finished[r.request_id]
        assert len(seq.step_logits) == 60
        check_teacher_forced(cfg, weights, r.prompt_token_ids, seq.generated, torch.stack(seq.step_logits), dtype,
                             False, name=name)
        got, ref = out[r.request_id], alone[r.request_id]
        if got != ref:
            k = next(i for i in range(60) if got[i] != ref[i])
            history = list(r.prompt_token_ids) + list(got[:k])
            row = plain.logits(weights64, cfg, history, torch.float64)[-1]
            top2 = row.topk(2).values
            bound = atol_for(dtype, row, name)
            assert float(top2[0] - top2[1]) <= 2 * bound, f"{r.request_id}: token {k} differs at a clear margin"
            assert {got[k], ref[k]} <= set(row.topk(4).indices.tolist())
    assert all(n == 6 for n in small.cache.free_blocks())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,num_blocks", [("B", 60), ("B", 14), ("C", 40), ("D", 7), ("E", 7)])
def test_overlapped_steps_give_the_tokens_of_single_steps(tmp_path, name, num_blocks, dtype):
    """`run_to_completion` launches the next step before it has seen the current one's tokens
    (the sampled ids go from step to step on the device).  Greedy and temperature requests,
    prompts cut into portions, a pool so small that requests are evicted and replayed: tokens
    and events are those of `step()` in a loop, bit for bit, because the same kernels run on
    the same inputs."""
    folder = helpers.make_model_folder(tmp_path, name)
    cfg = helpers.TINY[name][0]
    model = pae.load_model(folder, dtype)
    shapes = [(3, 12, 0.0), (9, 30, 0.8), (40, 20, 0.0), (64, 17, 0.7), (2, 40, 0.0), (27, 25, 1.1), (50, 33, 0.0)]
    requests = [pae.Request(f"r{i}", tuple(tokens_of(cfg, n, 70 + i)), new, temp, seed=i)
                for i, (n, new, temp) in enumerate(shapes)]

    def run(overlap):
        engine = pae.Engine(model, dtype=dtype, block_size=helpers.TINY[name][1]["block_size"] if name in "DE" else 8,
                            num_blocks=num_blocks, max_num_seqs=4, max_num_batched_tokens=32)
        for r in requests:
            assert engine.add_request(r)
        assert engine.scheduler.can_overlap()
        out = engine.run_to_completion(overlap=overlap)
        events = [(e.step, e.kind, e.request_id, e.detail) for e in engine.scheduler.events]
        assert all(n == num_blocks for n in engine.cache.free_blocks())  # every group's pool is whole again
        return out, events, engine.executor.runner.graph_replays

    single, overlapped = run(False), run(True)
    assert single[0] == overlapped[0] and single[1] == overlapped[1]
    assert all(len(single[0][r.request_id]) == r.max_new_tokens for r in requests)
    assert all(0 <= t < cfg["vocab_size"] for tokens in overlapped[0].values() for t in tokens)
    if num_blocks in (14, 7):
        assert any(kind is pae.EventKind.PREEMPT for _, kind, _, _ in single[1])
    assert overlapped[2] > 0  # decode steps were replayed graphs fed from the device


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "D"])
def test_replayed_graphs_equal_eager_steps(tmp_path, name, dtype):
    """Decode steps replayed as HIP graphs, with eager work and synchronisation between the
    replays, give bit for bit what the same steps give when every kernel is launched eagerly."""
    folder = helpers.make_model_folder(tmp_path, name)
    cfg = helpers.TINY[name][0]
    model = pae.load_model(folder, dtype)
    assert model.graph_safe
    seqs = [tokens_of(cfg, n, 20 + i) for i, n in enumerate((70, 33, 26))]
    outs = []
    for use_graphs in (True, False):
        cache = model.new_cache(16, 32, 4)
        runner = pae.StepRunner(model, cache, use_graphs=use_graphs)
        rows = []
        for s, ids in enumerate(seqs):
            cache.create_sequence(s)
            cache.reserve(s, len(ids) - 24)
        runner.run([pae.StepEntry(s, tuple(ids[:-24]), ()) for s, ids in enumerate(seqs)])
        for k in range(24):
            for s in range(3):
                cache.reserve(s, 1)
            step = runner.run([pae.StepEntry(s, (ids[len(ids) - 24 + k],), (0,)) for s, ids in enumerate(seqs)])
            rows.append(step.cpu().clone())
            torch.cuda.synchronize()
            if k % 5 == 0:  # eager work between replays: another sequence prefilled and dropped
                cache.create_sequence(99)
                cache.reserve(99, 7)
                runner.run([pae.StepEntry(99, tuple(seqs[0][:7]), (6,))])
                cache.free_sequence(99)
        outs.append(torch.stack(rows))
        if use_graphs:
            assert runner.graph_replays == 24
        else:
            assert runner.graph_replays == 0
    assert torch.equal(outs[0], outs[1])


def test_engine_refuses_what_it_cannot_run(tmp_path):
    folder = helpers.make_model_folder(tmp_path, "A")
    model = pae.load_model(folder, "float32")
    cache = model.new_cache(16, 4, 2)
    runner = pae.StepRunner(model, cache)
    cache.create_sequence(0)
    cache.reserve(0, 2)
    with pytest.raises(ValueError):
        runner.run([pae.StepEntry(0, (5, 99999), ())])  # outside the vocabulary
    with pytest.raises(ValueError):
        runner.run([pae.StepEntry(0, (5, 6, 7), ())])   # more tokens than reserved
    with pytest.raises(ValueError):
        runner.run([pae.StepEntry(0, (5, 6), (2,))])    # a wanted place outside the tokens
    with pytest.raises(ValueError):
        pae.load_model(folder, "float16")
    from paged_attention_engine_amd.kernels import lib
    with pytest.raises(lib.KernelError):
        lib.gemm_plain(torch.empty(2, 2), torch.empty(2, 2), torch.empty(2, 2))  # operands on the CPU
    assert lib.device_arch().startswith("gfx950")
    assert lib.loaded_library_path().endswith(".so")
