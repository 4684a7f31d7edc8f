"""Schedules and paths beside the four of the replay test, and negative controls.

* a decode step of more than 64 sequences (in bfloat16 it leaves the recorded-step path and the
  few-row products) against the same sequences in groups of at most 64;
* more shapes of decode steps than recordings are kept, so that recordings are dropped and made
  again, against eager steps;
* recorded steps padded with rows that live in the padding page;
* containment: a step changes the cache pools in the slots of its new tokens and nowhere else
  (the reference's tests/test_fused.py:704-767);
* a negative control: steps that read through identity block tables instead of the real ones
  diverge on a fragmented pool (tests/test_parity.py:333-380), so agreement elsewhere is not an
  accident of sequential allocation.
"""

from array import array

import pytest
import torch

import paged_attention_engine_amd as pae
from paged_attention_engine_amd.engine.step import padded_rows
from tests import helpers
from tests.plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu


def tokens_of(cfg, n, seed):
    return torch.randint(0, cfg["vocab_size"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def prefill_all(runner, cache, seqs, per_step=16):
    """Prompts into the cache, `per_step` sequences a step; all but the last token of each."""
    for first in range(0, len(seqs), per_step):
        entries = []
        for s in range(first, min(first + per_step, len(seqs))):
            assert cache.create_sequence(s)
            assert cache.reserve(s, len(seqs[s]) - 1).ok
            entries.append(pae.StepEntry(s, tuple(seqs[s][:-1]), ()))
        runner.run(entries)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["D", "E"])
def test_a_decode_step_of_more_than_64_sequences(tmp_path, name, dtype):
    folder = helpers.make_model_folder(tmp_path, name)
    cfg, weights = helpers.read_folder_plain(folder)
    weights = {k: v.double() for k, v in weights.items()}
    model = pae.load_model(folder, dtype)
    count = 70
    seqs = [tokens_of(cfg, 3 + (7 * i) % 40, 300 + i) for i in range(count)]
    want = torch.stack([plain.logits(weights, cfg, ids, torch.float64)[-1] for ids in seqs]).float()
    results = []
    for groups in ((70,), (40, 30), (1, 64, 5)):
        cache = model.new_cache(16, 4 * count, count)
        runner = pae.StepRunner(model, cache)
        prefill_all(runner, cache, seqs)
        rows, first = [], 0
        for size in groups:
            entries = []
            for s in range(first, first + size):
                assert cache.reserve(s, 1).ok
                entries.append(pae.StepEntry(s, (seqs[s][-1],), (0,)))
            rows.append(runner.run(entries).cpu().clone())
            first += size
        results.append(torch.cat(rows))
        if dtype == "bfloat16":  # 70 rows at once run eagerly, the groups as recorded steps
            assert runner.graph_replays == (0 if groups == (70,) else len(groups))
    for got in results:
        helpers.check_logits(got, want, dtype, name, f"{name} {dtype}")
    if dtype == "float32":  # every row from that row's data alone, in a fixed order
        assert torch.equal(results[0], results[1]) and torch.equal(results[0], results[2])
    else:
        bound = helpers.bounds(dtype, want, name)[0]
        assert float((results[0] - results[1]).abs().max()) <= bound


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_more_step_shapes_than_recordings_are_kept(tmp_path, dtype):
    """With room for three recordings, decode steps of 1 to 14 sequences, growing and shrinking
    twice, drop and remake recordings all the time (and most are padded): every step's logits are
    those of the same steps launched eagerly, bit for bit."""
    folder = helpers.make_model_folder(tmp_path, "D")
    cfg = helpers.TINY_D
    model = pae.load_model(folder, dtype)
    seqs = [tokens_of(cfg, 5 + 3 * i, 40 + i) + tokens_of(cfg, 12, 90 + i) for i in range(14)]
    sizes = [1, 2, 5, 9, 10, 13, 14, 12, 9, 3, 14, 7]
    outs = []
    for use_graphs in (True, False):
        cache = model.new_cache(16, 64, 16)
        runner = pae.StepRunner(model, cache, use_graphs=use_graphs)
        runner.MAX_GRAPHS = 3
        for s, ids in enumerate(seqs):
            cache.create_sequence(s)
            cache.reserve(s, len(ids) - 12)
        runner.run([pae.StepEntry(s, tuple(ids[:-12]), ()) for s, ids in enumerate(seqs)])
        rows = []
        done = [len(ids) - 12 for ids in seqs]
        for k, size in enumerate(sizes):
            entries = []
            for s in range(size):
                cache.reserve(s, 1)
                entries.append(pae.StepEntry(s, (seqs[s][done[s]],), (0,) if (s + k) % 4 else ()))
                done[s] += 1
            rows.append(runner.run(entries).cpu().clone())
            torch.cuda.synchronize()
        outs.append(rows)
        if use_graphs:
            assert runner.graph_replays == len(sizes) and len(runner._graphs) <= 3
            assert runner.graph_recordings > len(set(padded_rows(n) for n in sizes))  # some were made again
    for a, b in zip(*outs):
        assert a.shape == b.shape and torch.equal(a, b)


def snapshot(cache):
    return {(g.index, name): pool.clone() for g in cache.groups for name, pool in g.pools.items()}


def declared_slots(cache, group, entries):
    """(page, offset) of every token the step brings, in this group."""
    out = set()
    for e in entries:
        held = cache.num_tokens(e.seq_id)
        table = cache.block_table(group.index, e.seq_id)
        for pos in range(held - len(e.token_ids), held):
            out.add((table[pos // cache.block_size], pos % cache.block_size))
    return out


def changed_slots(before, after, tensor_name):
    """(page, offset) pairs at which a pool [stop][block][*page shape] differs, over all stops."""
    diff = before != after
    page_axis = 3 if tensor_name == "k" else 4  # keys [stop][block][kv][PAGE][hd], values [stop][block][kv][hd][PAGE]
    keep = diff.movedim((1, page_axis), (0, 1)).flatten(2).any(dim=2)  # every axis but (block, PAGE) folded
    return {(int(b), int(o)) for b, o in keep.nonzero().tolist()}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["C", "E"])
def test_a_step_changes_only_the_slots_of_its_new_tokens(tmp_path, name, dtype):
    """Mixed steps (portions, decoded tokens, padded recorded steps, a request ending and its pages
    going to the next) on models with a full and a windowed cache group: after every step each
    pool differs from its snapshot exactly in the slots of the step's tokens, in every layer, and
    the padding page aside nothing else has moved."""
    folder = helpers.make_model_folder(tmp_path, name)
    cfg = helpers.TINY[name][0]
    model = pae.load_model(folder, dtype)
    cache = model.new_cache(16, 12, 12)
    assert len(cache.groups) == 2
    runner = pae.StepRunner(model, cache)
    ids = {s: tokens_of(cfg, 90, 500 + s) for s in range(13)}
    done = {s: 0 for s in ids}
    plans = [[(0, 20), (1, 3)], [(0, 1), (1, 30), (2, 2)], [(0, 1), (1, 1), (2, 1)], [(0, 17), (2, 40)],
             [(0, 1), (1, 1), (2, 1)], "end 1", [(3, 33), (0, 1)], [(0, 1), (2, 1), (3, 1)]]
    # nine sequences decoding at once: a recorded step padded to twelve rows
    nine = range(4, 13)
    plans += ["end 0", "end 2", "end 3", [(s, 2) for s in nine], [(s, 1) for s in nine], [(s, 1) for s in nine]]
    live = set()
    for plan in plans:
        if isinstance(plan, str):
            s = int(plan.split()[1])
            cache.free_sequence(s)
            live.discard(s)
            continue
        entries = []
        for s, n in plan:
            if s not in live:
                assert cache.create_sequence(s)
                live.add(s)
            assert cache.reserve(s, n).ok, (s, n, cache.free_blocks())
            entries.append(pae.StepEntry(s, tuple(ids[s][done[s]:done[s] + n]), (n - 1,)))
            done[s] += n
        before = snapshot(cache)
        runner.run(entries)
        torch.cuda.synchronize()
        for group in cache.groups:
            want = declared_slots(cache, group, entries)
            padding = cache.padding_page(group.index)
            for tensor_name, pool in group.pools.items():
                changed = changed_slots(before[(group.index, tensor_name)], pool, tensor_name)
                changed = {(b, o) for b, o in changed if b != padding}
                assert changed <= want, f"{plan}: group {group.index} {tensor_name} changed {sorted(changed - want)} undeclared"
                assert changed == want, f"{plan}: group {group.index} {tensor_name} left {sorted(want - changed)} unwritten"
                # every stop of the group wrote its own copy of each slot
                for b, o in want:
                    page = pool[:, b]
                    cell = page[:, :, o, :] if tensor_name == "k" else page[:, :, :, o]
                    assert bool((cell.float().abs().amax(dim=(1, 2)) > 0).all())
        for s, _ in plan:
            cache.release_passed(s)
    assert runner.graph_recordings >= 2  # decode steps were recorded, one of them padded


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_ignoring_the_block_tables_diverges_on_a_fragmented_pool(tmp_path, dtype):
    """Negative control.  The pool is fragmented first (one-token decoys in every page, freed from
    both ends inward, as in the reference's tests/test_parity.py:196-223), so a sequence's pages
    are neither adjacent nor ascending.  Read through the real tables, the decoded tokens' logits
    are the plain implementation's.  Read through tables that say 0, 1, 2, ... (what a kernel that
    ignored the table, or a host that uploaded a stale one, would amount to), the same steps are
    far off: the agreement is the tables' doing."""
    folder = helpers.make_model_folder(tmp_path, "E")
    cfg, weights = helpers.read_folder_plain(folder)
    weights = {k: v.double() for k, v in weights.items()}
    model = pae.load_model(folder, dtype)
    seq = tokens_of(cfg, 75, 7)
    want = plain.logits(weights, cfg, seq, torch.float64)[-8:].float()

    def run(identity_tables):
        cache = model.new_cache(16, 12, 16)
        for d in range(12):  # a decoy in every page ...
            cache.create_sequence(100 + d)
            cache.reserve(100 + d, 1)
        order = []
        lo, hi = 0, 11
        while lo <= hi:      # ... freed from both ends inward: the free list reads 11, 0, 10, 1, ...
            order += [hi, lo] if lo != hi else [hi]
            lo, hi = lo + 1, hi - 1
        for d in order:
            cache.free_sequence(100 + d)
        runner = pae.StepRunner(model, cache, use_graphs=False)
        cache.create_sequence(0)
        cache.reserve(0, len(seq) - 8)
        runner.run([pae.StepEntry(0, tuple(seq[:-8]), ())])
        table = cache.block_table(0, 0)
        assert list(table) != sorted(table) and table[0] != 0  # really fragmented
        rows = []
        real = cache.table_array
        for t in seq[-8:]:
            cache.reserve(0, 1)
            if identity_tables:
                cache.table_array = lambda group, seq_id: array("i", range(len(real(group, seq_id))))
            rows.append(runner.run([pae.StepEntry(0, (t,), (0,))]).cpu().clone())
            cache.table_array = real
        return torch.cat(rows)

    bound = helpers.bounds(dtype, want, "E")[0]
    helpers.check_logits(run(False), want, dtype, "E", "through the real tables")
    off = float((run(True) - want).abs().max())
    assert off > 10 * bound, f"identity tables moved the logits by {off:.3e} only (bound {bound:.3e})"


def test_ticket_counters_are_zero_between_steps_and_belong_to_one_stream(tmp_path):
    """Products whose k ranges are added up inside the kernel share counters that every launch
    leaves at zero.  With the runner's check switched on, every step of a run at widths that use k
    ranges (prefill portions of 17 to 64 rows, decode steps, a padded recorded step) is followed by
    a look at the counters; and a launch from a second stream is refused instead of racing."""
    from paged_attention_engine_amd.kernels import lib as K

    cfg = dict(helpers.TINY_E, hidden_size=2048, intermediate_size=4096, num_attention_heads=16,
               num_key_value_heads=2, head_dim=128, use_sliding_window=False)
    model = pae.random_model(cfg, 3, "bfloat16")
    cache = model.new_cache(16, 64, 12)
    runner = pae.StepRunner(model, cache)
    runner.check_tickets = True
    ids = {s: tokens_of(cfg, 80, 900 + s) for s in range(9)}
    done = {s: 0 for s in ids}
    for plan in ([(0, 40), (1, 20)], [(0, 1), (1, 1), (2, 64)], [(s, 3) for s in range(3, 9)],
                 [(s, 1) for s in range(9)], [(s, 1) for s in range(9)]):
        entries = []
        for s, n in plan:
            if not cache.has_sequence(s):
                assert cache.create_sequence(s)
            assert cache.reserve(s, n).ok
            entries.append(pae.StepEntry(s, tuple(ids[s][done[s]:done[s] + n]), (n - 1,)))
            done[s] += n
        runner.run(entries)  # raises if a counter is left standing
    assert runner.graph_replays >= 2
    K.check_tickets_zero("cuda:0")
    a = torch.randn(40, 2048, device="cuda:0").to(torch.bfloat16)
    w = torch.randn(4096, 2048, device="cuda:0").to(torch.bfloat16)
    out = torch.empty(40, 4096, device="cuda:0", dtype=torch.bfloat16)
    K.gemm_skinny(out, a, w, None, K.EPI_BF16, 2)  # on the counters' own stream: fine
    with torch.cuda.stream(torch.cuda.Stream()):
        with pytest.raises(K.KernelError, match="another stream"):
            K.gemm_skinny(out, a, w, None, K.EPI_BF16, 2)
    torch.cuda.synchronize()
    K.check_tickets_zero("cuda:0")
