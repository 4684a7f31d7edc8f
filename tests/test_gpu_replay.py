"""Trace replay through bin/trace_run against the plain implementation.

For each tiny model and precision one trace replays the same requests whole, with
the last 32 tokens decoded one by one, in portions of changing size (down to two
tokens), and mixed: up to four live requests, portions of some beside decoded
tokens of others, in a pool so small that pages are given back and used again.
Every logit asked for is compared with the plain implementation (float64 on the
same weights); in float32 the schedules must also agree with each other exactly,
since every kernel of that path computes a row from that row's data alone in a
fixed order.
"""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from tests import helpers
from tests.plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LENGTHS = (70, 100, 45, 130)
PORTIONS = (7, 2, 5, 3, 2, 11, 4, 2, 9)


class Trace:
    """Builds the step records and remembers which (request, position) every wanted row is."""

    def __init__(self):
        self.records = []
        self.wanted = {}  # step -> [(name, position)]

    def step(self, entries, end=()):
        number = len(self.records)
        rec = {"step": number, "entries": [], "end": list(end)}
        rows = []
        for rid, name, start, tokens, want in entries:
            rec["entries"].append({"id": rid, "tokens": list(tokens), "want": list(want)})
            rows += [(name, start + w) for w in want]
        self.records.append(rec)
        if rows:
            self.wanted[number] = rows
        return number


def build_trace(tokens):
    """tokens: name -> list of ids.  Returns the trace and the peak of live tokens (rounded to 64)."""
    t = Trace()
    names = list(tokens)
    # 1. each request alone and whole
    for name in names:
        ids = tokens[name]
        t.step([(f"whole-{name}", name, 0, ids, range(len(ids)))], end=[f"whole-{name}"])
    # 2. most of it in one step, the last 32 tokens one by one
    for name in names:
        ids = tokens[name]
        cut = len(ids) - 32
        rid = f"dec-{name}"
        t.step([(rid, name, 0, ids[:cut], [cut - 1])])
        for p in range(cut, len(ids)):
            t.step([(rid, name, p, ids[p:p + 1], [0])], end=[rid] if p == len(ids) - 1 else [])
    # 3. portions of changing size, down to two tokens
    for k, name in enumerate(names):
        ids = tokens[name]
        rid, p, i = f"por-{name}", 0, k
        while p < len(ids):
            n = min(PORTIONS[i % len(PORTIONS)], len(ids) - p)
            i += 1
            t.step([(rid, name, p, ids[p:p + n], range(n))], end=[rid] if p + n == len(ids) else [])
            p += n
    # 4. mixed: requests arrive staggered; each prefills in portions and then decodes its last 20
    #    tokens one by one beside the portions of later arrivals; a finished request's pages are
    #    taken by the next arrival.  Every request runs twice under different ids.
    queue = [(f"mix{r}-{name}", name) for r in range(2) for name in names]
    live = {}  # rid -> [name, position]
    tick = 0
    while queue or live:
        while queue and len(live) < 4 and (tick % 3 == 0 or not live):
            rid, name = queue.pop(0)
            live[rid] = [name, 0]
            break
        entries, ended = [], []
        for j, (rid, (name, p)) in enumerate(list(live.items())):
            ids = tokens[name]
            if (tick + j) % 5 == 4 and len(live) > 1:
                continue  # a request may be left out of a step and go on later
            decode_from = len(ids) - 20
            n = 1 if p >= decode_from else min(PORTIONS[(tick + j) % len(PORTIONS)], decode_from - p)
            entries.append((rid, name, p, ids[p:p + n], [n - 1] if p + n >= decode_from else ([0] if n > 2 else [])))
            live[rid][1] = p + n
            if p + n == len(ids):
                ended.append(rid)
        t.step(entries, end=ended)
        for rid in ended:
            del live[rid]
        tick += 1
    return t


def peak_live_tokens(trace):
    held, peak = {}, 0
    for rec in trace.records:
        for e in rec["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum(-(-n // 64) * 64 for n in held.values()))
        for rid in rec["end"]:
            del held[rid]
    return peak


def run_trace(folder, dtype, out_dir, max_tokens, block_size, records):
    proc = subprocess.Popen(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
         "--out", out_dir, "--max-tokens", str(max_tokens), "--block-size", str(block_size)],
        stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    for rec in records:
        proc.stdin.write(json.dumps(rec) + "\n")
        proc.stdin.flush()
        line = proc.stdout.readline().strip()
        assert line == f"done {rec['step']}", f"step {rec['step']}: got {line!r}"
    proc.stdin.close()
    assert proc.wait(timeout=60) == 0


@pytest.mark.parametrize("name", ["D", "E"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_with_pages_of_32_tokens(tmp_path, name, dtype):
    """The same trace with twice as many tokens to a page as the models' own tests use: the
    matrix-core attention kernels walk pages of 32, windows pass them half as often."""
    replay_and_compare(tmp_path, name, dtype, 32)


@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_schedules_agree_with_the_plain_implementation(tmp_path, name, dtype):
    replay_and_compare(tmp_path, name, dtype, helpers.TINY[name][1]["block_size"])


def replay_and_compare(tmp_path, name, dtype, block_size):
    folder = helpers.make_model_folder(tmp_path, name)
    cfg, weights = helpers.read_folder_plain(folder)
    weights64 = {k: v.double() for k, v in weights.items()}
    gen = torch.Generator().manual_seed(11)
    tokens = {f"q{i}": torch.randint(0, cfg["vocab_size"], (n,), generator=gen).tolist()
              for i, n in enumerate(LENGTHS)}
    want = {n: plain.logits(weights64, cfg, ids, torch.float64).float().numpy() for n, ids in tokens.items()}
    top = max(float(np.abs(w).max()) for w in want.values())
    atol, rms_bound = helpers.bounds(dtype, torch.tensor(top), name)

    trace = build_trace(tokens)
    max_tokens = peak_live_tokens(trace)
    assert max_tokens <= 4 * 192  # four live requests at most
    out_dir = str(tmp_path / "out")
    run_trace(folder, dtype, out_dir, max_tokens, block_size, trace.records)

    seen = {}  # (name, position) -> first logits seen, to compare schedules with each other
    worst, checked, squares = 0.0, 0, 0.0
    for rec in trace.records:
        path = os.path.join(out_dir, f"{rec['step']}.f32")
        rows = trace.wanted.get(rec["step"])
        assert os.path.exists(path) == bool(rows)
        if not rows:
            continue
        got = np.fromfile(path, dtype="<f4").reshape(len(rows), cfg["vocab_size"])
        for row, (req, pos) in zip(got, rows):
            err = float(np.abs(row - want[req][pos]).max())
            worst = max(worst, err)
            squares += float(np.square(row - want[req][pos]).mean())
            assert err <= atol, f"step {rec['step']} ({req}, position {pos}): error {err:.3e} > {atol:.3e}"
            if dtype == "float32":
                first = seen.setdefault((req, pos), row)
                assert np.array_equal(first, row), f"step {rec['step']} ({req}, {pos}) differs between schedules"
            checked += 1
    print(f"{name} {dtype}: {len(trace.records)} steps, {checked} rows, pool for {max_tokens} tokens, "
          f"worst error {worst:.3e} (bound {atol:.3e}), rms error {(squares / checked) ** 0.5:.3e}")
    assert (squares / checked) ** 0.5 <= rms_bound
    assert checked > 4 * sum(LENGTHS) // 2
