"""Logits and attention outputs at the context lengths that the benchmarks measure.

Kernel level: the matrix-core decode attention over 4,096 / 16,384 / 32,000 keys (32 to 250
splits of 128 keys, the merge over more than 32 splits, block tables of 256 to 2,000 pages) with one
key made to stand out in the first, a middle and the last split, and with a window of 4,096 keys; the
prefill attention for a portion of 2,048 tokens from an empty cache and into a warm cache of 6,000
tokens.  Model level: the peaked tiny model decoding step by step, with recorded steps, over the
points at which its block tables pass 64 and 128 pages (where a recorded step is recorded anew),
teacher-forced against the plain implementation; in float32 the step after a crossing is bit for bit
the row of a whole-sequence step.  The reference checks the same at its own scale
(tests/test_parity.py:226-330).
"""

import math

import pytest
import torch

import paged_attention_engine_amd as pae
from paged_attention_engine_amd.engine.trace import TraceReplayer
from paged_attention_engine_amd.kernels import lib as K
from tests import helpers
from tests.plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
SPLIT = 128  # keys per split of the decode kernel; asserted below against the library's own


def attention_in_float64(q, keys, values, positions, scale, window):
    """q [T, nh, hd] for the tokens at `positions` of one sequence with keys/values [n, nkv, hd]:
    softmax(q k^T * scale) v over keys start..position, in float64 by library calls on the device."""
    T, nh, hd = q.shape
    n, nkv, _ = keys.shape
    g = nh // nkv
    qd, kd, vd = q.double().to(DEV), keys.double().to(DEV), values.double().to(DEV)
    pos = torch.tensor(positions, device=DEV)
    at = torch.arange(n, device=DEV)
    seen = at[None, :] <= pos[:, None]
    if window:
        seen &= at[None, :] > pos[:, None] - window
    out = torch.empty(T, nh, hd, dtype=torch.float64, device=DEV)
    for h in range(nh):
        scores = (qd[:, h] @ kd[:, h // g].T) * scale
        scores.masked_fill_(~seen, float("-inf"))
        out[:, h] = torch.softmax(scores, dim=-1) @ vd[:, h // g]
    return out.view(T, nh * hd).cpu()


def paged(keys, values, bs, seed):
    """Pools with the sequence's pages scattered over them in shuffled order, and its block table."""
    n, nkv, hd = keys.shape
    pages = -(-n // bs)
    num_blocks = pages + 7
    order = torch.randperm(num_blocks, generator=torch.Generator().manual_seed(seed))[:pages]
    pad = pages * bs - n
    kpad = torch.cat([keys, torch.zeros(pad, nkv, hd, dtype=keys.dtype)]).view(pages, bs, nkv, hd)
    vpad = torch.cat([values, torch.zeros(pad, nkv, hd, dtype=values.dtype)]).view(pages, bs, nkv, hd)
    kp = torch.zeros(num_blocks, nkv, bs, hd, dtype=keys.dtype)
    vp = torch.zeros(num_blocks, nkv, hd, bs, dtype=keys.dtype)
    kp[order] = kpad.permute(0, 2, 1, 3)
    vp[order] = vpad.permute(0, 2, 3, 1)
    return kp.to(DEV), vp.to(DEV), order.to(torch.int32)[None, :].contiguous().to(DEV)


def stand_out(q_row, keys, key_pos, hd, gen):
    """One key takes almost all the weight of one query (every head of it)."""
    direction = torch.randn(hd, generator=gen)
    direction /= direction.norm()
    keys[key_pos] = 6.0 * direction * math.sqrt(hd) ** 0.5
    q_row[:] = 6.0 * direction * math.sqrt(hd) ** 0.5


@pytest.mark.parametrize("nh,nkv", [(12, 2), (7, 1), (8, 1)])
@pytest.mark.parametrize("n,window", [(4096, 0), (16384, 0), (32000, 0), (16384, 4096)])
@pytest.mark.parametrize("where", ["first split", "middle split", "last split", "nowhere"])
def test_decode_attention_over_long_contexts(nh, nkv, n, window, where):
    assert K.library().pae_attn_decode_split() == SPLIT
    hd, bs = 128, 16
    gen = torch.Generator().manual_seed(n + nh)
    keys, values = torch.randn(n, nkv, hd, generator=gen), torch.randn(n, nkv, hd, generator=gen)
    q = torch.randn(1, nh, hd, generator=gen)
    first_seen = max(0, n - window) if window else 0
    splits = (n - 1) // SPLIT - first_seen // SPLIT + 1
    assert splits > 30
    if where != "nowhere":
        key_pos = {"first split": first_seen + 5, "middle split": first_seen + (n - first_seen) // 2 // SPLIT * SPLIT + 127,
                   "last split": n - 2}[where]
        stand_out(q[0], keys, key_pos, hd, gen)
    q, keys, values = q.bfloat16(), keys.bfloat16(), values.bfloat16()
    want = attention_in_float64(q, keys, values, [n - 1], hd ** -0.5, window)
    if where != "nowhere":  # the construction works: the output is nearly that key's value
        assert float((want.view(nh, hd)[0] - values[key_pos, 0].double()).abs().max()) < 0.1
    kp, vp, table = paged(keys, values, bs, seed=n)
    assert table.shape[1] >= 256
    out = torch.zeros(1, nh * hd, dtype=torch.bfloat16, device=DEV)
    work = torch.tensor([[0, n - 1, 0, 0]], dtype=torch.int32, device=DEV)
    K.attn_decode(out, q.view(1, nh * hd).to(DEV), kp, vp, work, table, nh, nkv, hd, hd ** -0.5, window)
    err = float((out.double().cpu() - want).abs().max())
    assert err <= 3e-2, err


@pytest.mark.parametrize("nh,nkv", [(12, 2), (7, 1), (8, 1)])
@pytest.mark.parametrize("past", [0, 6000])
def test_prefill_attention_of_a_2048_token_portion(nh, nkv, past):
    hd, bs, run = 128, 16, 2048
    n = past + run
    gen = torch.Generator().manual_seed(past + nh)
    keys, values = torch.randn(n, nkv, hd, generator=gen), torch.randn(n, nkv, hd, generator=gen)
    q = torch.randn(run, nh, hd, generator=gen)
    # three queries each with a key of their own far back, at a page's edge and right before them
    for row, key_pos in ((run - 1, 3), (run // 2, past + run // 2 - 1), (17, max(0, past - 1))):
        stand_out(q[row], keys, key_pos, hd, gen)
    q, keys, values = q.bfloat16(), keys.bfloat16(), values.bfloat16()
    positions = list(range(past, n))
    want = attention_in_float64(q, keys, values, positions, hd ** -0.5, 0)
    kp, vp, table = paged(keys, values, bs, seed=n)
    out = torch.zeros(run, nh * hd, dtype=torch.bfloat16, device=DEV)
    tiles = torch.tensor([[0, first, min(K.PREFILL_TILE, run - first)] for first in range(0, run, K.PREFILL_TILE)],
                         dtype=torch.int32, device=DEV)
    K.attn_prefill(out, q.view(run, nh * hd).to(DEV), kp, vp, tiles,
                   torch.tensor(positions, dtype=torch.int32, device=DEV), table, nh, nkv, hd, hd ** -0.5, 0)
    err = (out.double().cpu() - want).abs().max(dim=1).values
    assert float(err.max()) <= 3e-2, f"worst rows: {torch.topk(err, 5)}"


# the peaked tiny model with room for more positions than its 2,048, so that its tables pass 128 pages of 16
LONG_E = dict(helpers.TINY_E, max_position_embeddings=4096)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_recorded_decode_steps_while_the_block_tables_pass_64_and_128_pages(tmp_path, dtype):
    opts = helpers.TINY["E"][1]
    folder = str(tmp_path / "long_e")
    pae.write_model_folder(pae.read_config_dict(LONG_E), opts["seed"], folder, std=opts["std"], norm_std=opts["norm_std"])
    cfg, weights = helpers.read_folder_plain(folder)
    total = 2100
    ids = torch.randint(0, cfg["vocab_size"], (total,), generator=torch.Generator().manual_seed(21)).tolist()
    # angles as the reference and the engine form them, in float32 (see plain.ANGLE_DTYPE): at these
    # positions a float64 angle alone would put the float32 engine several bounds away
    with plain.angles_in(torch.float32):
        want = plain.logits({k: v.double() for k, v in weights.items()}, cfg, ids, torch.float64).float()
    replayer = TraceReplayer(folder, dtype, max_tokens=2 * 2112, block_size=16)
    runner = replayer.runner
    assert runner.use_graphs
    pages_of = lambda tokens: -(-tokens // 16)
    got = {}

    def portion(first, last):  # tokens [first, last) in one step, the last one's logits wanted
        out = replayer.step({"step": 0, "entries": [{"id": "a", "tokens": ids[first:last], "want": [last - first - 1]}]})
        got[last - 1] = torch.from_numpy(out[0]).clone()

    def one_by_one(first, last):
        for t in range(first, last):
            before, held = runner.graph_recordings, t + 1
            out = replayer.step({"step": 0, "entries": [{"id": "a", "tokens": [ids[t]], "want": [0]}]})
            got[t] = torch.from_numpy(out[0]).clone()
            # a step is recorded anew exactly when the tables' rounded width changes
            crossed = pages_of(held) in (65, 129) and pages_of(held - 1) in (64, 128)
            assert runner.graph_recordings - before == (1 if crossed or t == first and first == 1000 else 0), (t, held)

    portion(0, 1000)
    one_by_one(1000, 1100)   # 63 pages -> 69 pages: past 64 at 1,025 tokens
    assert runner.graph_recordings == 2
    portion(1100, 2020)
    one_by_one(2020, total)  # 127 pages -> 132 pages: past 128 at 2,049 tokens
    assert runner.graph_recordings == 3 and runner.graph_replays == 100 + (total - 2020)
    rows = sorted(got)
    mine = torch.stack([got[t] for t in rows])
    if dtype == "float32":
        helpers.check_logits(mine, want[rows], dtype, "E", "decoded rows around the crossings")
    else:
        # The 4 ulp that the reference states for bfloat16 belong to its sequences of a few hundred tokens;
        # at 2,000 keys this peaked model's logits move further under any bfloat16 arithmetic.  The measure
        # here is the reference's own arithmetic: the plain implementation run in bfloat16 (every product,
        # norm and softmax rounded as engine/model.py rounds them) against the same float64 logits.  The
        # engine must be no further off than that, at the worst logit and in the root mean square.
        in_bf16 = plain.logits({k: v.bfloat16() for k, v in weights.items()}, cfg, ids, torch.bfloat16).float()[rows]
        plain_err, engine_err = (in_bf16 - want[rows]).abs(), (mine - want[rows]).abs()
        print(f"worst: engine {float(engine_err.max()):.3e}, plain bfloat16 {float(plain_err.max()):.3e}; "
              f"rms: engine {float(engine_err.pow(2).mean().sqrt()):.3e}, plain {float(plain_err.pow(2).mean().sqrt()):.3e}")
        assert float(engine_err.max()) <= float(plain_err.max())
        assert float(engine_err.pow(2).mean().sqrt()) <= float(plain_err.pow(2).mean().sqrt())
    if dtype == "float32":
        # the same rows from one step over the whole sequence, bit for bit: the steps right after a
        # crossing (1,024 and 2,048 tokens held before them) among them
        replayer.step({"step": 1, "entries": [], "end": ["a"]})
        whole = replayer.step({"step": 2, "entries": [{"id": "b", "tokens": ids, "want": rows}]})
        assert 1024 in rows and 2048 in rows
        assert torch.equal(torch.from_numpy(whole), torch.stack([got[t] for t in rows]))
