"""The plain implementation pinned by what fixes it beside the reference's text:
closed forms, special cases that reduce to a library routine, invariants, and
the vectors the reference's own tests hold.  Each check is chosen so that a
plausible mistake (a wrong sign or pairing, a norm in the wrong place, a mask
off by one) fails it."""

import math

import pytest
import torch
import torch.nn.functional as F

from tests import helpers
from tests.plain import qwen2_plain as plain


# ------------------------------------------------------------------ RMSNorm
def test_rms_norm_closed_forms():
    c, H, eps = 3.0, 64, 1e-6
    x = torch.full((2, H), c, dtype=torch.float64)
    out = plain.rms_norm(x, torch.ones(H, dtype=torch.float64), eps)
    assert torch.allclose(out, torch.full_like(out, c / math.sqrt(c * c + eps)), atol=1e-12)
    # zero vector gives exactly zero, not NaN (the reference relies on it for pads, engine/model.py:435-436)
    assert torch.equal(plain.rms_norm(torch.zeros(1, H), torch.ones(H), eps), torch.zeros(1, H))
    # equals x / ||x|| * sqrt(H) when eps vanishes; the weight multiplies after normalising
    x = torch.randn(5, H, dtype=torch.float64)
    w = torch.randn(H, dtype=torch.float64)
    want = w * x / x.norm(dim=-1, keepdim=True) * math.sqrt(H)
    assert torch.allclose(plain.rms_norm(x, w, 1e-30), want, atol=1e-10)
    # scale invariance: norm(a x) = norm(x) for a > 0
    assert torch.allclose(plain.rms_norm(7.5 * x, w, 1e-30), plain.rms_norm(x, w, 1e-30), atol=1e-10)
    # mean of squares, not variance about the mean: a constant offset changes the result
    assert not torch.allclose(plain.rms_norm(x + 5, w, 1e-6), plain.rms_norm(x, w, 1e-6))


def test_rms_norm_accumulates_in_float32_for_half_inputs():
    """The reference's vector (tests/test_parity_fp16.py:285-329): fp16 input of
    shape (1, 8, 896), eps 1e-6; the error against float64 must not exceed that of
    a version that squares and averages in fp16."""
    torch.manual_seed(0)
    x = torch.randn(1, 8, 896).to(torch.float16)
    w = torch.ones(896, dtype=torch.float16)
    ours = plain.rms_norm(x, w, 1e-6).float()
    exact = x.double()
    exact = (exact * torch.rsqrt(exact.pow(2).mean(-1, keepdim=True) + 1e-6)).float()
    naive = (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6)).float()
    assert ours.dtype == torch.float32 and plain.rms_norm(x, w, 1e-6).dtype == torch.float16
    assert (ours - exact).abs().max() <= (naive - exact).abs().max()


# ------------------------------------------------------------------ rotary encoding
def _rope(x, positions, theta, dtype=torch.float64):
    hd = x.shape[-1]
    cos, sin = plain.rope_cos_sin(plain.rope_inv_freq(hd, theta, dtype), torch.as_tensor(positions), dtype)
    return plain.apply_rope(x, cos, sin)


def test_rope_tables_shape_and_values():
    inv = plain.rope_inv_freq(16, 10000.0)
    assert inv.shape == (8,) and inv[0] == 1.0  # engine/model.py:148-151: length hd/2
    assert torch.allclose(inv, torch.tensor([10000.0 ** (-2 * i / 16) for i in range(8)]), rtol=1e-6)
    cos, sin = plain.rope_cos_sin(inv, torch.arange(5), torch.float32)
    assert cos.shape == (5, 16) and torch.equal(cos[:, :8], cos[:, 8:])  # emb = cat(freqs, freqs)


def test_rope_position_zero_is_identity_and_two_dims_is_a_plane_rotation():
    x = torch.randn(3, 1, 8, dtype=torch.float64)
    assert torch.allclose(_rope(x, [0], 1e4), x)
    # head_dim 2: one pair, inv_freq[0] = 1 whatever theta: rotation by p radians, counter-clockwise
    v = torch.tensor([[[2.0, 0.5]]], dtype=torch.float64)
    p = 3
    got = _rope(v, [p], 123.0)[0, 0]
    z = complex(2.0, 0.5) * complex(math.cos(p), math.sin(p))
    assert torch.allclose(got, torch.tensor([z.real, z.imag], dtype=torch.float64), atol=1e-12)


def test_rope_pairs_are_i_and_i_plus_half():
    hd = 8
    x = torch.zeros(1, 1, hd, dtype=torch.float64)
    x[0, 0, 1] = 1.0
    out = _rope(x, [5], 1e4)[0, 0]
    nonzero = set(torch.nonzero(out.abs() > 1e-12).flatten().tolist())
    assert nonzero == {1, 1 + hd // 2}  # not {0, 1} as an interleaved pairing would give
    # each pair keeps its length
    y = torch.randn(2, 4, hd, dtype=torch.float64)
    r = _rope(y, [3, 9, 27, 81], 1e4)
    assert torch.allclose(y[..., :4] ** 2 + y[..., 4:] ** 2, r[..., :4] ** 2 + r[..., 4:] ** 2, atol=1e-12)


def test_rope_scores_depend_on_distance_only():
    q = torch.randn(1, 1, 16, dtype=torch.float64)
    k = torch.randn(1, 1, 16, dtype=torch.float64)
    def score(m, n):
        return float((_rope(q, [m], 1e4) * _rope(k, [n], 1e4)).sum())
    assert abs(score(7, 3) - score(107, 103)) < 1e-9
    assert abs(score(7, 3) - score(3, 7)) > 1e-6  # and on its sign


# ------------------------------------------------------------------ attention
def test_attention_special_cases():
    hd = 8
    q = torch.randn(4, 1, hd, dtype=torch.float64)
    k = torch.randn(2, 1, hd, dtype=torch.float64)
    v = torch.randn(2, 1, hd, dtype=torch.float64)
    out = plain.attention(q, k, v, hd ** -0.5)
    # one token: softmax over one score is 1, so every head returns its KV head's value;
    # KV head j serves query heads 2j and 2j+1 (engine/attention.py:72-74)
    for h in range(4):
        assert torch.allclose(out[h, 0], v[h // 2, 0])
    # all value rows equal: that row, whatever the scores
    n = 6
    q = torch.randn(2, n, hd, dtype=torch.float64)
    k = torch.randn(2, n, hd, dtype=torch.float64)
    row = torch.randn(hd, dtype=torch.float64)
    out = plain.attention(q, k, row.expand(2, n, hd), 0.3)
    assert torch.allclose(out, row.expand(2, n, hd))
    # zero queries: uniform weights over the allowed keys, so position p averages values 0..p
    v = torch.randn(2, n, hd, dtype=torch.float64)
    out = plain.attention(torch.zeros(2, n, hd, dtype=torch.float64), k, v, 1.0)
    for p in range(n):
        assert torch.allclose(out[:, p], v[:, : p + 1].mean(dim=1))


@pytest.mark.parametrize("nh,nkv,hd", [(12, 2, 128), (14, 2, 64), (4, 4, 32)])  # tests/test_attention_gqa.py:55-59
def test_attention_reduces_to_library_causal_attention(nh, nkv, hd):
    torch.manual_seed(0)
    n = 9
    q = torch.randn(nh, n, hd, dtype=torch.float64)
    k = torch.randn(nkv, n, hd, dtype=torch.float64)
    v = torch.randn(nkv, n, hd, dtype=torch.float64)
    g = nh // nkv
    want = F.scaled_dot_product_attention(q[None], k.repeat_interleave(g, 0)[None], v.repeat_interleave(g, 0)[None],
                                          is_causal=True, scale=0.125)[0]
    assert torch.allclose(plain.attention(q, k, v, 0.125), want, atol=1e-10)


def test_mask_matches_the_reference_rule_by_double_loop():
    # engine/attention.py:474-487 and tests/test_fused.py:405-456: for a sequence with `past`
    # cached tokens and `new` query tokens, query r may see key j iff j <= past + r.
    for past, new in ((0, 9), (14, 1), (0, 3), (7, 1), (0, 40), (33, 1), (5, 1)):
        total = past + new
        ok = plain.allowed_keys(total, None)
        for r in range(new):
            for j in range(total):
                assert bool(ok[past + r, j]) == (j <= past + r)
        assert ok.any(dim=-1).all()  # no row without a key (tests/test_fused.py:459-477)


def test_window_limits_how_far_back_a_query_sees():
    n, hd = 12, 4
    q = torch.randn(1, n, hd, dtype=torch.float64)
    k = torch.randn(1, n, hd, dtype=torch.float64)
    v = torch.randn(1, n, hd, dtype=torch.float64)
    assert torch.allclose(plain.attention(q, k, v, 0.5, window=n), plain.attention(q, k, v, 0.5))
    assert torch.allclose(plain.attention(q, k, v, 0.5, window=1), v)  # only itself
    ok = plain.allowed_keys(n, 3)
    assert ok.sum(-1).tolist() == [1, 2] + [3] * (n - 2)
    # with zero queries the output is the mean of the last three values
    out = plain.attention(torch.zeros_like(q), k, v, 1.0, window=3)
    assert torch.allclose(out[0, 7], v[0, 5:8].mean(0))


# ------------------------------------------------------------------ projections, feed-forward, head
def test_zero_projection_weights_leave_the_bias_in_head_order():
    cfg = dict(helpers.TINY_A)
    w = plain.random_weights(cfg, 0)
    p = "model.layers.0.self_attn."
    x = torch.randn(3, cfg["hidden_size"])
    y = plain.linear(x, torch.zeros_like(w[p + "q_proj.weight"]), w[p + "q_proj.bias"])
    heads = plain.split_heads(y, 4, 16)
    for j in range(4):  # head j = features [j*hd, (j+1)*hd)
        assert torch.equal(heads[j, 0], w[p + "q_proj.bias"][j * 16:(j + 1) * 16])
    assert torch.equal(plain.merge_heads(heads), y)


def test_swiglu_closed_forms():
    x = torch.randn(7, dtype=torch.float64)
    assert torch.allclose(plain.silu(x), F.silu(x))
    H, I = 6, 10
    w = {"mlp.gate_proj.weight": torch.zeros(I, H), "mlp.up_proj.weight": torch.randn(I, H),
         "mlp.down_proj.weight": torch.randn(H, I)}
    assert torch.equal(plain.swiglu_mlp(w, "", torch.randn(2, H)), torch.zeros(2, H))  # silu(0) = 0
    # a large positive gate passes `up` through: silu(g) * u ~ g * u
    g = torch.full((4,), 30.0, dtype=torch.float64)
    assert torch.allclose(plain.silu(g), g, rtol=1e-9)


def test_head_tying():
    cfg = dict(helpers.TINY_A)
    w = plain.random_weights(cfg, 0)
    assert "lm_head.weight" not in w and plain.lm_head_weight(w, cfg) is w["model.embed_tokens.weight"]
    cfg_b = dict(helpers.TINY_B)
    wb = plain.random_weights(cfg_b, 1)
    base = plain.logits(wb, cfg_b, [1, 2, 3])
    wb["lm_head.weight"] = wb["lm_head.weight"] * 2
    assert torch.allclose(plain.logits(wb, cfg_b, [1, 2, 3]), base * 2, atol=1e-6)  # untied: only the head moved


# ------------------------------------------------------------------ whole model
@pytest.mark.parametrize("name", ["A", "B"])
def test_zero_output_projections_reduce_the_model_to_norm_and_head(name):
    cfg = dict(helpers.TINY[name][0])
    w = plain.random_weights(cfg, 3, norm_std=0.1)
    for i in range(cfg["num_hidden_layers"]):
        w[f"model.layers.{i}.self_attn.o_proj.weight"].zero_()
        w[f"model.layers.{i}.mlp.down_proj.weight"].zero_()
    ids = [4, 9, 2]
    emb = w["model.embed_tokens.weight"][ids]
    want = plain.linear(plain.rms_norm(emb, w["model.norm.weight"], cfg["rms_norm_eps"]), plain.lm_head_weight(w, cfg))
    assert torch.allclose(plain.logits(w, cfg, ids), want, atol=1e-7)


def test_logits_are_invariant_under_a_shift_of_all_positions():
    """Only distances between positions count (rotation of q and k by absolute position)."""
    cfg = dict(helpers.TINY_B)
    w = {k: v.double() for k, v in plain.random_weights(cfg, 1, norm_std=0.1).items()}
    ids = [5, 900, 33, 7, 512, 64, 1]
    base = plain.logits(w, cfg, ids, torch.float64)
    shifted = plain.logits(w, cfg, ids, torch.float64, positions=[p + 37 for p in range(len(ids))])
    assert torch.allclose(base, shifted, atol=1e-9)
    # a change of distances does change them
    stretched = plain.logits(w, cfg, ids, torch.float64, positions=[2 * p for p in range(len(ids))])
    assert not torch.allclose(base, stretched, atol=1e-6)


def test_causality_and_prefix_stability():
    cfg = dict(helpers.TINY_A)
    w = plain.random_weights(cfg, 0)
    ids = [3, 1, 4, 1, 5, 9, 2, 6]
    full = plain.logits(w, cfg, ids)
    assert torch.allclose(plain.logits(w, cfg, ids[:5]), full[:5], atol=1e-6)


def test_greedy_generation_feeds_tokens_back():
    cfg = dict(helpers.TINY_A)
    w = plain.random_weights(cfg, 0)
    tokens, rows = plain.greedy_generate(w, cfg, [7, 8, 9], 4)
    assert len(tokens) == 4 and rows.shape == (4, cfg["vocab_size"])
    assert tokens[0] == int(plain.logits(w, cfg, [7, 8, 9])[-1].argmax())
    assert tokens[1] == int(plain.logits(w, cfg, [7, 8, 9, tokens[0]])[-1].argmax())


# ------------------------------------------------------------------ sampling
def test_sampling_rules():
    row = torch.tensor([0.1, 2.0, 2.0, -1.0])
    assert plain.sample_from_logits(row, 0.0, 0.9) == 1  # first maximum wins
    onehot = torch.full((50,), -1e9)
    onehot[17] = 0.0
    for t in (0.3, 1.0, 4.0):
        for u in (0.0, 0.5, 0.999):
            assert plain.sample_from_logits(onehot, t, u) == 17
    # two equally likely tokens split the unit interval in the middle
    pair = torch.tensor([1.0, 1.0])
    assert plain.sample_from_logits(pair, 1.0, 0.49) == 0 and plain.sample_from_logits(pair, 1.0, 0.51) == 1
    # a low temperature concentrates on the maximum
    assert plain.sample_from_logits(torch.tensor([0.0, 1.0, 0.5]), 1e-3, 0.7) == 1


# ------------------------------------------------------------------ pins that a plausible mistake fails
def _mutated(attribute, replacement):
    """Context manager: the plain module with one of its functions swapped for a mistaken one."""
    import contextlib

    @contextlib.contextmanager
    def swap():
        keep = getattr(plain, attribute)
        setattr(plain, attribute, replacement)
        try:
            yield
        finally:
            setattr(plain, attribute, keep)
    return swap()


def _bias_after_rotation(w, prefix, cfg, x, positions, window):
    """self_attention with the mistake of adding q/k bias after the rotation."""
    nh, nkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], plain.head_dim_of(cfg)
    p = prefix + "self_attn."
    q = plain.split_heads(plain.linear(x, w[p + "q_proj.weight"]), nh, hd)
    k = plain.split_heads(plain.linear(x, w[p + "k_proj.weight"]), nkv, hd)
    v = plain.split_heads(plain.linear(x, w[p + "v_proj.weight"], w[p + "v_proj.bias"]), nkv, hd)
    cos, sin = plain.rope_cos_sin(plain.rope_inv_freq(hd, plain.rope_theta_of(cfg), torch.float64), positions, x.dtype)
    q = plain.apply_rope(q, cos, sin) + plain.split_heads(w[p + "q_proj.bias"][None].to(x.dtype), nh, hd)
    k = plain.apply_rope(k, cos, sin) + plain.split_heads(w[p + "k_proj.bias"][None].to(x.dtype), nkv, hd)
    return plain.linear(plain.merge_heads(plain.attention(q, k, v, hd ** -0.5, window)), w[p + "o_proj.weight"])


def test_the_bias_is_added_before_the_rotation():
    """engine/model.py:303-311: q and k get their bias, then the rotation.  Then scores depend on
    distances only and a shift of all positions changes nothing; with the bias added after the
    rotation the terms <R_m q, b_k> depend on the absolute position m, and the shift shows."""
    cfg = dict(helpers.TINY_B)
    w = {k: v.double() for k, v in plain.random_weights(cfg, 1, std=0.3, norm_std=0.1).items()}
    ids = [5, 900, 33, 7, 512, 64, 1, 77, 3]
    shifted = [p + 211 for p in range(len(ids))]
    assert torch.allclose(plain.logits(w, cfg, ids, torch.float64),
                          plain.logits(w, cfg, ids, torch.float64, positions=shifted), atol=1e-9)
    with _mutated("self_attention", _bias_after_rotation):
        wrong = plain.logits(w, cfg, ids, torch.float64)
        wrong_shifted = plain.logits(w, cfg, ids, torch.float64, positions=shifted)
    assert float((wrong - wrong_shifted).abs().max()) > 1e-3  # the mistake breaks the invariance


def test_the_gate_goes_through_silu_and_up_does_not():
    """engine/model.py:317-320: down(silu(gate) * up).  A strongly negative gate closes the unit
    whatever `up` holds; had SiLU been put on `up`, the same numbers would give about -57."""
    w = {"mlp.gate_proj.weight": torch.tensor([[-20.0]], dtype=torch.float64),
         "mlp.up_proj.weight": torch.tensor([[3.0]], dtype=torch.float64),
         "mlp.down_proj.weight": torch.tensor([[1.0]], dtype=torch.float64)}
    y = plain.swiglu_mlp(w, "", torch.ones(1, 1, dtype=torch.float64))
    assert abs(float(y)) < 1e-6
    assert abs(float(plain.silu(torch.tensor(3.0, dtype=torch.float64)) * -20.0)) > 50  # what the swap would give
    # and an open gate of 1.0 scales `up` by silu(1) = 1 / (1 + e^-1)
    w["mlp.gate_proj.weight"] = torch.tensor([[1.0]], dtype=torch.float64)
    assert abs(float(plain.swiglu_mlp(w, "", torch.ones(1, 1, dtype=torch.float64))) - 3.0 / (1 + math.exp(-1))) < 1e-12


def test_one_layer_one_token_is_a_closed_chain():
    """engine/model.py:340-351 for one token (whose attention is its own value vector, softmax of
    one score being 1): h1 = e + Wo (Wv n1(e) + bv); h2 = h1 + MLP(n2(h1)); logits = head nf(h2).
    Pins the arrangement: each norm feeds its branch only, the residual carries the un-normed sum,
    the final norm comes before the head.  A post-norm block, a norm on the residual, or a
    missing final norm all give other numbers."""
    cfg = dict(helpers.TINY_B, num_hidden_layers=1)
    w = {k: v.double() for k, v in plain.random_weights(cfg, 5, std=0.2, norm_std=0.2).items()}
    p, eps, tok = "model.layers.0.", cfg["rms_norm_eps"], 321
    e = w["model.embed_tokens.weight"][tok][None]
    n1 = plain.rms_norm(e, w[p + "input_layernorm.weight"], eps)
    value = n1 @ w[p + "self_attn.v_proj.weight"].t() + w[p + "self_attn.v_proj.bias"]  # [1, nkv * hd]
    nh, nkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    per_head = value.view(nkv, hd).repeat_interleave(nh // nkv, dim=0).reshape(1, nh * hd)  # kv head j serves heads j*g..
    h1 = e + per_head @ w[p + "self_attn.o_proj.weight"].t()
    n2 = plain.rms_norm(h1, w[p + "post_attention_layernorm.weight"], eps)
    gate, up = n2 @ w[p + "mlp.gate_proj.weight"].t(), n2 @ w[p + "mlp.up_proj.weight"].t()
    h2 = h1 + (gate * torch.sigmoid(gate) * up) @ w[p + "mlp.down_proj.weight"].t()
    want = plain.rms_norm(h2, w["model.norm.weight"], eps) @ w["lm_head.weight"].t()
    got = plain.logits(w, cfg, [tok], torch.float64)
    assert torch.allclose(got, want, atol=1e-10)
    # the branches matter in this check: without them the logits are far away
    bare = plain.rms_norm(e, w["model.norm.weight"], eps) @ w["lm_head.weight"].t()
    assert float((bare - want).abs().max()) > 0.1


def test_the_window_rule():
    """Not in the reference (every layer there sees every earlier key): layers from
    `max_window_layers` on look back `sliding_window` keys.  Parity unpinned; what is pinned is
    that the rule does what it says: a window as long as the sequence changes nothing, the
    layers below `max_window_layers` are not windowed, a window of one sees only the token itself."""
    cfg = dict(helpers.TINY_C)
    assert [plain.layer_window(cfg, i) for i in range(4)] == [None, None, 24, 24]
    assert plain.layer_window(dict(cfg, use_sliding_window=False), 3) is None
    w = {k: v.double() for k, v in plain.random_weights(cfg, 2, std=0.2).items()}
    ids = list(range(3, 33))
    full = plain.logits(w, dict(cfg, use_sliding_window=False), ids, torch.float64)
    assert torch.allclose(plain.logits(w, dict(cfg, sliding_window=len(ids)), ids, torch.float64), full, atol=1e-12)
    assert not torch.allclose(plain.logits(w, cfg, ids, torch.float64), full, atol=1e-6)
    assert torch.allclose(plain.logits(w, cfg, ids, torch.float64)[:24], full[:24], atol=1e-12)  # the first 24 see all
    q = torch.randn(2, 5, 8, dtype=torch.float64)
    v = torch.randn(1, 5, 8, dtype=torch.float64)
    out = plain.attention(q, torch.randn(1, 5, 8, dtype=torch.float64), v, 0.3, window=1)
    assert torch.allclose(out[0], v[0]) and torch.allclose(out[1], v[0])


def test_the_peaked_model_shows_mistakes_far_beyond_the_bfloat16_bound(tmp_path):
    """The bfloat16 tests can fail: on model E (tests/helpers.py) the logits move by more than ten
    times the bound they are held to when the rotation is dropped, when attention is flattened,
    when the window is off by one, when the bias comes after the rotation, and when query heads
    are paired with the wrong key/value head.  (With weights N(0, 0.02) everywhere, as in models
    A to D, the same mistakes move the logits by less than the bound.)"""
    folder = helpers.make_model_folder(tmp_path, "E")
    cfg, w = helpers.read_folder_plain(folder)
    w = {k: v.double() for k, v in w.items()}
    ids = torch.randint(0, cfg["vocab_size"], (130,), generator=torch.Generator().manual_seed(11)).tolist()
    base = plain.logits(w, cfg, ids, torch.float64)
    bound = helpers.bf16_atol(base, "E")

    def moved(logits):
        return float((logits - base).abs().max()) / bound

    with _mutated("apply_rope", lambda x, cos, sin: x):
        assert moved(plain.logits(w, cfg, ids, torch.float64)) > 10
    real_attention = plain.attention
    with _mutated("attention", lambda q, k, v, scale, window=None: real_attention(torch.zeros_like(q), k, v, scale, window)):
        assert moved(plain.logits(w, cfg, ids, torch.float64)) > 10
    for off in (-1, 1):
        assert moved(plain.logits(w, dict(cfg, sliding_window=cfg["sliding_window"] + off), ids, torch.float64)) > 10
    with _mutated("self_attention", _bias_after_rotation):
        assert moved(plain.logits(w, cfg, ids, torch.float64)) > 10
    # heads paired the other way round: query head h reads key/value head h % nkv instead of h // g
    def interleaved(q, k, v, scale, window=None):
        nh, nkv = q.shape[0], k.shape[0]
        order = [(h % nkv) * (nh // nkv) + h // nkv for h in range(nh)]
        return real_attention(q[order], k, v, scale, window)[[order.index(h) for h in range(nh)]]
    with _mutated("attention", interleaved):
        assert moved(plain.logits(w, cfg, ids, torch.float64)) > 10
