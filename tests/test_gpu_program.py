"""A decode step's layers as one resident kernel (a decode program) against the same step launched
kernel by kernel: the same logits and the same cache contents bit for bit, with any number of
resident workgroups (few of them make every phase take several rounds), with recorded steps, at
the tiny peaked model's sizes and at the real layer widths; models whose parts cannot be fused run
as before."""

import pytest
import torch

import paged_attention_engine_amd as pae
from paged_attention_engine_amd.kernels import lib as K
from tests import helpers
from tests.plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu

WIDE = dict(architectures=["Qwen2ForCausalLM"], num_hidden_layers=2, hidden_size=1536, num_attention_heads=12,
            num_key_value_heads=2, head_dim=128, intermediate_size=8960, vocab_size=3000, rope_theta=1000000.0,
            rms_norm_eps=1e-6, tie_word_embeddings=True, use_sliding_window=False, max_position_embeddings=4096,
            hidden_act="silu")


def tokens(vocab, n, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def run_schedule(model, prompts, decode_steps, use_programs, groups=None, use_graphs=False, block_size=16):
    """Prompts in one step each, then `decode_steps` steps of one token a sequence (every sequence's
    logits wanted).  Returns (logits of every decode step, the cache, the runner)."""
    vocab = model.plan.vocab_size
    pages = sum(-(-(len(p) + decode_steps) // block_size) + 1 for p in prompts) + 2
    cache = model.new_cache(block_size, pages, len(prompts))
    runner = pae.StepRunner(model, cache, use_graphs=use_graphs, use_programs=use_programs)
    runner.program_groups = groups
    for s, prompt in enumerate(prompts):
        assert cache.create_sequence(s)
        cache.reserve(s, len(prompt))
        runner.run([pae.StepEntry(s, tuple(prompt), ())])
    out = []
    for step in range(decode_steps):
        entries = []
        for s in range(len(prompts)):
            cache.reserve(s, 1)
            entries.append(pae.StepEntry(s, (tokens(vocab, 1, 1000 * step + s)[0],), (0,)))
        out.append(runner.run(entries).clone())
    torch.cuda.synchronize()
    runner.check_programs()
    K.check_tickets_zero(model.device)
    return torch.stack(out), cache, runner


def same_cache(a, b):
    for group_a, group_b in zip(a.groups, b.groups):
        for name in group_a.pools:
            if not torch.equal(group_a.pools[name], group_b.pools[name]):
                return False
    return True


@pytest.mark.parametrize("groups", [None, 3, 64])
@pytest.mark.parametrize("lengths", [(37,), (5, 130, 64), (300, 1, 17, 129, 255, 256, 33, 2)])
def test_a_decode_program_gives_the_bits_of_the_separate_kernels(tmp_path, groups, lengths):
    folder = helpers.make_model_folder(tmp_path, "E")
    model = pae.load_model(folder, "bfloat16")
    prompts = [tokens(model.plan.vocab_size, n, 7 + n) for n in lengths]
    alone, cache_alone, runner_alone = run_schedule(model, prompts, 20, use_programs=False)
    fused, cache_fused, runner = run_schedule(model, prompts, 20, use_programs=True, groups=groups)
    assert runner_alone._eager_program is None
    program = runner._eager_program
    assert program is not None and program.count == 6 * len(model.plan.schedule)  # six phases a layer
    assert program.groups == (groups or program.groups)
    assert torch.equal(fused, alone)
    assert same_cache(cache_fused, cache_alone)


def test_a_decode_program_at_the_real_layer_widths_and_sixteen_rows(tmp_path):
    model = pae.random_model(WIDE, seed=3, dtype="bfloat16")
    for lengths in ((700,), (9, 100, 250, 31, 64, 65, 1, 2, 3, 4, 127, 128, 129, 300, 16, 17)):
        prompts = [tokens(WIDE["vocab_size"], n, 11 + n) for n in lengths]
        alone, cache_alone, _ = run_schedule(model, prompts, 6, use_programs=False)
        fused, cache_fused, runner = run_schedule(model, prompts, 6, use_programs=True)
        assert runner._eager_program.count == 12
        assert torch.equal(fused, alone)
        assert same_cache(cache_fused, cache_alone)
    # seventeen sequences are more rows than a program takes: the kernels are launched one by one
    prompts = [tokens(WIDE["vocab_size"], 5 + n, n) for n in range(17)]
    _, _, runner = run_schedule(model, prompts, 2, use_programs=True)
    assert runner._eager_program is not None and runner._eager_program.count == 0


def test_a_decode_program_whose_wavefronts_take_a_tile_in_several_chunks():
    """With a width of 2,560 and 6,912 between, a k range is longer than the 14 k steps a wavefront asks
    for at once (20 for QKV and gate/up, 18 for down's three ranges): a tile's weights then come in two
    chunks, the next always on the way.  (Wider still, and a range's activations no longer fit LDS beside
    the attention's: the 7B widths are refused, and run kernel by kernel.)"""
    wider = dict(WIDE, num_hidden_layers=1, hidden_size=2560, num_attention_heads=20, num_key_value_heads=4,
                 intermediate_size=6912, vocab_size=1000)
    model = pae.random_model(wider, seed=4, dtype="bfloat16")
    for lengths in ((130,), (40, 7, 300, 64, 65, 129, 1, 18, 250)):
        prompts = [tokens(wider["vocab_size"], n, 31 + n) for n in lengths]
        alone, cache_alone, _ = run_schedule(model, prompts, 4, use_programs=False)
        fused, cache_fused, runner = run_schedule(model, prompts, 4, use_programs=True)
        assert runner._eager_program.count == 6
        assert torch.equal(fused, alone)
        assert same_cache(cache_fused, cache_alone)
    seven_b = dict(wider, hidden_size=3584, num_attention_heads=28, intermediate_size=18944)
    model = pae.random_model(seven_b, seed=4, dtype="bfloat16")
    _, _, runner = run_schedule(model, [tokens(1000, 20, 1)], 2, use_programs=True)
    assert runner._eager_program.count == 0


def test_recorded_steps_replay_their_programs(tmp_path):
    """Recorded decode steps hold their program's launch; replays with new tokens, positions and tables
    give what eager steps without programs give, and the oracle's logits within the bound."""
    folder = helpers.make_model_folder(tmp_path, "E")
    cfg, weights = helpers.read_folder_plain(folder)
    model = pae.load_model(folder, "bfloat16")
    prompts = [tokens(cfg["vocab_size"], n, 3 + n) for n in (45, 7, 100)]
    alone, _, _ = run_schedule(model, prompts, 40, use_programs=False)
    replayed, _, runner = run_schedule(model, prompts, 40, use_programs=True, use_graphs=True)
    assert runner.graph_recordings == 1 and runner.graph_replays == 40
    assert torch.equal(replayed, alone)
    # the first sequence's rows against the plain implementation
    history = prompts[0] + [tokens(cfg["vocab_size"], 1, 1000 * step)[0] for step in range(40)]
    want = plain.logits({k: v.double() for k, v in weights.items()}, cfg, history, torch.float64).float()[len(prompts[0]):]
    helpers.check_logits(replayed[:, 0].cpu(), want, "bfloat16", "E", "replayed program rows")


@pytest.mark.parametrize("name", ["A", "C"])
def test_models_whose_parts_cannot_be_fused_run_kernel_by_kernel(tmp_path, name):
    folder = helpers.make_model_folder(tmp_path, name)
    model = pae.load_model(folder, "bfloat16")
    prompts = [tokens(model.plan.vocab_size, n, n) for n in (20, 3)]
    bs = helpers.TINY[name][1]["block_size"]
    alone, _, _ = run_schedule(model, prompts, 5, use_programs=False, block_size=bs)
    offered, _, runner = run_schedule(model, prompts, 5, use_programs=True, block_size=bs)
    assert runner._eager_program.count == 0  # head sizes of 16 and 48: the attention part said no
    assert torch.equal(offered, alone)


def test_a_part_that_is_not_recordable_is_refused_while_recording():
    program = K.DecodeProgram("cuda:0", 4)
    x = torch.zeros(4, 64, dtype=torch.bfloat16, device="cuda:0")
    with pytest.raises(K.KernelError, match="cannot be a phase"):
        with K.recording(program):
            K.swiglu(torch.empty(4, 32, dtype=torch.bfloat16, device="cuda:0"), x)
    assert program.count == 0
    K.swiglu(torch.empty(4, 32, dtype=torch.bfloat16, device="cuda:0"), x)  # and works again afterwards


@pytest.mark.parametrize("programs", [False, True])
def test_a_sequences_decoded_logits_do_not_depend_on_the_batch_up_to_16_rows(tmp_path, programs):
    """Decode steps of up to 16 sequences add every product's k in one order and split the attention
    at fixed places: a sequence decoded alone, beside 7 others and beside 15 others gives the same
    logits bit for bit (prompts run alone in all three, so the caches start equal), at the real layer
    widths, with the kernels launched one by one or as a program."""
    model = pae.random_model(WIDE, seed=5, dtype="bfloat16")
    lengths = (200, 9, 100, 250, 31, 64, 65, 1, 300, 4, 127, 128, 129, 77, 16, 17)
    prompts = [tokens(WIDE["vocab_size"], n, 21 + n) for n in lengths]
    steps = 5
    feed = [[tokens(WIDE["vocab_size"], 1, 1000 * step + s)[0] for s in range(16)] for step in range(steps)]

    def decode(which):
        pages = sum(-(-(len(prompts[s]) + steps) // 16) + 1 for s in which) + 2
        cache = model.new_cache(16, pages, len(which))
        runner = pae.StepRunner(model, cache, use_graphs=False, use_programs=programs)
        for s in which:
            assert cache.create_sequence(s)
            cache.reserve(s, len(prompts[s]))
            runner.run([pae.StepEntry(s, tuple(prompts[s]), ())])
        out = []
        for step in range(steps):
            entries = []
            for s in which:
                cache.reserve(s, 1)
                entries.append(pae.StepEntry(s, (feed[step][s],), (0,)))
            out.append(runner.run(entries).clone())
        torch.cuda.synchronize()
        runner.check_programs()
        return torch.stack(out)  # [step, sequence, vocab]

    alone = decode([0])
    eight = decode(list(range(8)))
    sixteen = decode(list(range(16)))
    assert torch.equal(alone[:, 0], eight[:, 0]) and torch.equal(alone[:, 0], sixteen[:, 0])
    assert torch.equal(eight, sixteen[:, :8])
