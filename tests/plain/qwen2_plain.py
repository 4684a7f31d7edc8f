"""A plain, slow Qwen2 decoder: whole sequences, no cache, one function per part.

This module is the oracle the engine is compared with. It is written from the
formulas of the reference engine (each function cites the file and lines it was
read from, paths relative to the reference's root) and shares no code with the
product package: it does not import it, uses no paging, no batching and no
kernels, and recomputes the whole sequence for every query.

Everything takes a dict of tensors keyed by checkpoint name and a plain dict of
the config.json keys, so the same functions serve any size; index tensors are made
on the device the weights live on, so the same functions run on the CPU or, for the
large shapes, on a GPU in float64.

`dtype` is the storage dtype of activations (float64, float32 or bfloat16).
With bfloat16 the cast points follow the reference's text: the norm's variance
in float32 and its output cast back before the weight multiply, rotary tables
built in float32 then cast, residual adds in the storage dtype.  Attention
scores, softmax and the weighted sum are always taken in at least float32.
"""

from __future__ import annotations

import math

import torch


# --------------------------------------------------------------------------- config


def head_dim_of(cfg: dict) -> int:
    """engine/model.py:66-70 -- `head_dim`, else hidden_size // num_attention_heads."""
    hd = cfg.get("head_dim")
    return int(hd) if hd else cfg["hidden_size"] // cfg["num_attention_heads"]


def rope_theta_of(cfg: dict) -> float:
    """engine/model.py:79 reads rope_parameters["rope_theta"]; plain files keep it top-level."""
    if "rope_theta" in cfg:
        return float(cfg["rope_theta"])
    return float(cfg["rope_parameters"]["rope_theta"])


def layer_window(cfg: dict, layer_idx: int) -> int | None:
    """Window of a layer, or None for full attention.

    The reference has no window at all (every layer is full causal attention,
    engine/attention.py:474-487).  The rule used here for a config that switches
    windows on -- layers with index >= max_window_layers use `sliding_window` --
    is this repository's own reading of the config keys: parity unpinned.
    """
    if not cfg.get("use_sliding_window", False):
        return None
    if layer_idx < int(cfg.get("max_window_layers", cfg["num_hidden_layers"])):
        return None
    return int(cfg["sliding_window"])


# --------------------------------------------------------------------------- parts


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """engine/model.py:117-123 -- variance and scaling in float32 (float64 stays
    float64), cast back to the input dtype, then multiply by the weight."""
    in_dtype = x.dtype
    work = torch.float64 if in_dtype == torch.float64 else torch.float32
    xw = x.to(work)
    variance = xw.pow(2).mean(-1, keepdim=True)
    xw = xw * torch.rsqrt(variance + eps)
    return weight.to(in_dtype) * xw.to(in_dtype)


# The precision in which rotation angles are formed in `self_attention`: None = the working precision
# of the call.  The reference forms them in float32 whatever the activations' type (engine/model.py:
# 132-152: inv_freq and positions * inv_freq "built in float32 then cast"); at position 2,000 a float32
# angle is 1e-4 radians away from the float64 one, which the scores of a peaked model turn into logit
# differences several times the float32 comparison bound, so comparisons of a float32 engine at long
# positions set this to torch.float32 (`angles_in`): everything else stays in the working precision.
ANGLE_DTYPE = None


class angles_in:
    def __init__(self, dtype):
        self.dtype = dtype

    def __enter__(self):
        global ANGLE_DTYPE
        self.saved, ANGLE_DTYPE = ANGLE_DTYPE, self.dtype

    def __exit__(self, *exc):
        global ANGLE_DTYPE
        ANGLE_DTYPE = self.saved


def rope_inv_freq(head_dim: int, theta: float, work: torch.dtype = torch.float32, device=None) -> torch.Tensor:
    """engine/model.py:132-135 -- 1 / theta ** (arange(0, hd, 2) / hd)."""
    exponent = torch.arange(0, head_dim, 2, dtype=torch.int64, device=device).to(work)
    return 1.0 / (theta ** (exponent / head_dim))


def rope_cos_sin(inv_freq: torch.Tensor, positions: torch.Tensor, dtype: torch.dtype):
    """engine/model.py:138-152 -- freqs[p, i] = p * inv_freq[i]; emb = cat(freqs, freqs);
    cos and sin taken in the working precision, then cast to `dtype`."""
    freqs = positions.to(inv_freq.dtype)[:, None] * inv_freq[None, :]
    emb = torch.cat((freqs, freqs), dim=-1)
    if dtype == torch.float64:  # cosine and sine of the angle as formed, not rounded to its precision
        emb = emb.double()
    return emb.cos().to(dtype), emb.sin().to(dtype)


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    """engine/model.py:126-129 -- cat(-x[hd/2:], x[:hd/2])."""
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """engine/model.py:155-161 -- x * cos + rotate_half(x) * sin, x is (heads, n, hd),
    cos/sin are (n, hd) and broadcast over heads."""
    return (x * cos[None]) + (rotate_half(x) * sin[None])


def linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """F.linear as the reference uses it (engine/model.py:303-305,315,318-320):
    x @ W.T + b with W stored (out_features, in_features)."""
    y = x @ weight.to(x.dtype).t()
    if bias is not None:
        y = y + bias.to(x.dtype)
    return y


def split_heads(x: torch.Tensor, num_heads: int, head_dim: int) -> torch.Tensor:
    """engine/model.py:307-309 -- (n, heads*hd) -> (heads, n, hd); head j is the
    features [j*hd, (j+1)*hd)."""
    n = x.shape[0]
    return x.view(n, num_heads, head_dim).transpose(0, 1)


def allowed_keys(num_tokens: int, window: int | None, device=None) -> torch.Tensor:
    """Boolean (n, n): may query i see key j.

    engine/attention.py:474-487: key j is visible to the query at position p iff
    j <= p (and j < kv_len, which holds for a whole sequence).  With a window w
    (not in the reference) additionally p - j < w."""
    i = torch.arange(num_tokens, device=device)[:, None]
    j = torch.arange(num_tokens, device=device)[None, :]
    ok = j <= i
    if window is not None:
        ok = ok & ((i - j) < window)
    return ok


def attention(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, window: int | None = None
) -> torch.Tensor:
    """softmax(q k^T * scale + mask) v with grouped KV heads.

    q is (nh, n, hd); k, v are (nkv, n, hd).  KV head j serves query heads
    j*g .. (j+1)*g-1 (engine/attention.py:72-74, consecutive expansion); scale is
    passed explicitly as hd**-0.5 by the caller (engine/model.py:60-62,
    engine/attention.py:227-235); no dropout."""
    nh, n, hd = q.shape
    nkv = k.shape[0]
    g = nh // nkv
    work = torch.float64 if q.dtype == torch.float64 else torch.float32
    ok = allowed_keys(n, window, q.device)
    out = torch.empty(nh, n, v.shape[-1], dtype=work, device=q.device)
    for h in range(nh):
        kh = k[h // g].to(work)
        vh = v[h // g].to(work)
        scores = (q[h].to(work) @ kh.t()) * scale
        scores = scores.masked_fill(~ok, float("-inf"))
        probs = torch.softmax(scores, dim=-1)
        out[h] = probs @ vh
    return out.to(q.dtype)


def merge_heads(x: torch.Tensor) -> torch.Tensor:
    """engine/model.py:314 -- (nh, n, hd) -> (n, nh*hd)."""
    nh, n, hd = x.shape
    return x.transpose(0, 1).reshape(n, nh * hd)


def self_attention(w: dict, prefix: str, cfg: dict, x: torch.Tensor, positions: torch.Tensor,
                   window: int | None) -> torch.Tensor:
    """engine/model.py:281-315 -- q/k/v projections with bias, heads, rope on q and k
    (after the bias, before attending), attention, merge, o projection without bias."""
    nh, nkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], head_dim_of(cfg)
    p = prefix + "self_attn."
    q = split_heads(linear(x, w[p + "q_proj.weight"], w[p + "q_proj.bias"]), nh, hd)
    k = split_heads(linear(x, w[p + "k_proj.weight"], w[p + "k_proj.bias"]), nkv, hd)
    v = split_heads(linear(x, w[p + "v_proj.weight"], w[p + "v_proj.bias"]), nkv, hd)
    work = torch.float64 if x.dtype == torch.float64 else torch.float32
    angle = ANGLE_DTYPE or work
    cos, sin = rope_cos_sin(rope_inv_freq(hd, rope_theta_of(cfg), angle, x.device), positions, x.dtype)
    q, k = apply_rope(q, cos, sin), apply_rope(k, cos, sin)
    out = attention(q, k, v, hd ** -0.5, window)
    return linear(merge_heads(out), w[p + "o_proj.weight"])


def silu(x: torch.Tensor) -> torch.Tensor:
    """F.silu (engine/model.py:320): x * sigmoid(x)."""
    return x * torch.sigmoid(x)


def swiglu_mlp(w: dict, prefix: str, x: torch.Tensor) -> torch.Tensor:
    """engine/model.py:317-320 -- down(silu(gate(x)) * up(x)), no biases."""
    p = prefix + "mlp."
    gate = linear(x, w[p + "gate_proj.weight"])
    up = linear(x, w[p + "up_proj.weight"])
    return linear(silu(gate) * up, w[p + "down_proj.weight"])


def decoder_layer(w: dict, cfg: dict, layer_idx: int, x: torch.Tensor,
                  positions: torch.Tensor) -> torch.Tensor:
    """engine/model.py:340-349 -- h += Attn(Norm1(h)); h += MLP(Norm2(h))."""
    prefix = f"model.layers.{layer_idx}."
    eps = cfg["rms_norm_eps"]
    h = rms_norm(x, w[prefix + "input_layernorm.weight"], eps)
    x = x + self_attention(w, prefix, cfg, h, positions, layer_window(cfg, layer_idx))
    h = rms_norm(x, w[prefix + "post_attention_layernorm.weight"], eps)
    return x + swiglu_mlp(w, prefix, h)


def lm_head_weight(w: dict, cfg: dict) -> torch.Tensor:
    """engine/model.py:220-222 -- lm_head.weight, else the embedding matrix (tied)."""
    if cfg.get("tie_word_embeddings", False) or "lm_head.weight" not in w:
        return w["model.embed_tokens.weight"]
    return w["lm_head.weight"]


def hidden_states(w: dict, cfg: dict, token_ids, dtype: torch.dtype = torch.float32,
                  positions=None) -> torch.Tensor:
    """Embedding gather (engine/model.py:401), every layer, final norm (:351)."""
    device = w["model.embed_tokens.weight"].device
    ids = torch.as_tensor(token_ids, dtype=torch.long, device=device)
    pos = torch.arange(len(ids), device=device) if positions is None else torch.as_tensor(positions, device=device)
    x = w["model.embed_tokens.weight"][ids].to(dtype)
    for i in range(cfg["num_hidden_layers"]):
        x = decoder_layer(w, cfg, i, x, pos)
    return rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"])


def logits(w: dict, cfg: dict, token_ids, dtype: torch.dtype = torch.float32,
           positions=None) -> torch.Tensor:
    """Logits at every position, (n, vocab): final-norm rows times the head
    matrix, no bias (engine/model.py:406,453-455)."""
    h = hidden_states(w, cfg, token_ids, dtype, positions)
    return linear(h, lm_head_weight(w, cfg))


def greedy_generate(w: dict, cfg: dict, prompt, max_new_tokens: int,
                    dtype: torch.dtype = torch.float32):
    """engine/model.py:459-503 -- argmax of the last position's logits, fed back;
    exactly max_new_tokens tokens, EOS ignored.  Recomputes the whole sequence
    each time (no cache).  Returns (tokens, logits that produced each token)."""
    seq = list(prompt)
    out, rows = [], []
    for _ in range(max_new_tokens):
        row = logits(w, cfg, seq, dtype)[-1].to(torch.float32)
        tok = int(torch.argmax(row))
        out.append(tok)
        rows.append(row)
        seq.append(tok)
    return out, torch.stack(rows)


# --------------------------------------------------------------------------- sampling


def sample_from_logits(row: torch.Tensor, temperature: float, u: float) -> int:
    """Greedy for temperature 0 (engine/scheduler.py:610: argmax, first maximum
    wins); otherwise inverse-CDF sampling from softmax(row / T): the first index
    whose cumulative probability exceeds u * total (not in the reference, which
    samples greedily only)."""
    row = row.to(torch.float64)
    if temperature == 0.0:
        return int(torch.argmax(row))
    z = row / temperature
    p = torch.exp(z - z.max())
    c = torch.cumsum(p, 0)
    idx = int(torch.searchsorted(c, torch.tensor(u, dtype=torch.float64) * c[-1], right=True))
    return min(idx, row.numel() - 1)


# --------------------------------------------------------------------------- weights


def tensor_shapes(cfg: dict) -> dict[str, tuple[int, ...]]:
    """Checkpoint names and shapes as the reference reads them (engine/model.py:198-227)."""
    H, I, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    nh, nkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], head_dim_of(cfg)
    shapes: dict[str, tuple[int, ...]] = {"model.embed_tokens.weight": (V, H)}
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        shapes[p + "self_attn.q_proj.weight"] = (nh * hd, H)
        shapes[p + "self_attn.q_proj.bias"] = (nh * hd,)
        shapes[p + "self_attn.k_proj.weight"] = (nkv * hd, H)
        shapes[p + "self_attn.k_proj.bias"] = (nkv * hd,)
        shapes[p + "self_attn.v_proj.weight"] = (nkv * hd, H)
        shapes[p + "self_attn.v_proj.bias"] = (nkv * hd,)
        shapes[p + "self_attn.o_proj.weight"] = (H, nh * hd)
        shapes[p + "mlp.gate_proj.weight"] = (I, H)
        shapes[p + "mlp.up_proj.weight"] = (I, H)
        shapes[p + "mlp.down_proj.weight"] = (H, I)
        shapes[p + "input_layernorm.weight"] = (H,)
        shapes[p + "post_attention_layernorm.weight"] = (H,)
    shapes["model.norm.weight"] = (H,)
    if not cfg.get("tie_word_embeddings", False):
        shapes["lm_head.weight"] = (V, H)
    return shapes


def random_weights(cfg: dict, seed: int, std: float = 0.02, norm_std: float = 0.0) -> dict:
    """Random tensors of the right names and shapes, values rounded to bfloat16
    (kept as float32 tensors) so that every precision starts from the same numbers.
    The test oracle's own generator: matrices and biases ~N(0, std), norm weights
    1 + N(0, norm_std) (the reference's tests/tiny_model.py:21-50 uses zero biases
    and unit norms; non-zero biases are used here so the bias path is exercised)."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        if name.endswith("norm.weight") or "layernorm" in name:
            t = 1.0 + norm_std * torch.randn(shape, generator=g)
        else:
            t = std * torch.randn(shape, generator=g)
        out[name] = t.to(torch.bfloat16).to(torch.float32)
    return out
