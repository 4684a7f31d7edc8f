"""First end-to-end check on the GPU: whole prompts and decoding through the
trace replayer against the plain implementation."""

import pytest
import torch

from tests import helpers
from tests.plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompt_and_decode(tmp_path, name, dtype):
    from paged_attention_engine_amd.engine.trace import TraceReplayer

    folder = helpers.make_model_folder(tmp_path, name)
    cfg, weights = helpers.read_folder_plain(folder)
    block = helpers.TINY[name][1]["block_size"]
    gen = torch.Generator().manual_seed(5)
    tokens = torch.randint(0, cfg["vocab_size"], (70,), generator=gen).tolist()
    want = plain.logits({k: v.double() for k, v in weights.items()}, cfg, tokens, torch.float64).float()
    atol = helpers.bounds(dtype, want)[0]

    rep = TraceReplayer(folder, dtype, max_tokens=128, block_size=block)
    got = rep.step({"step": 0, "entries": [{"id": "a", "tokens": tokens, "want": list(range(70))}], "end": ["a"]})
    err = float((torch.from_numpy(got) - want).abs().max())
    print(f"{name} {dtype} whole: max err {err:.3e} (atol {atol:.3e}, max logit {float(want.abs().max()):.3f})")
    assert err <= atol

    # most in one step, the last 32 one by one
    rows = [rep.step({"step": 1, "entries": [{"id": "b", "tokens": tokens[:38], "want": [37]}]})]
    for i in range(38, 70):
        rows.append(rep.step({"step": i, "entries": [{"id": "b", "tokens": [tokens[i]], "want": [0]}]}))
    got2 = torch.from_numpy(__import__("numpy").concatenate(rows))
    err2 = float((got2 - want[37:]).abs().max())
    print(f"{name} {dtype} decode: max err {err2:.3e}")
    assert err2 <= atol
