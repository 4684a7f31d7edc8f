"""Each part alone against the plain functions, and the framework's generality: a toy
mixer with state of its own, a toy mixer that caches one tensor of its own shape per token, a toy
position encoding (which only encodes: it never sees a cache) and a toy architecture whose
schedule names a layer twice, lets a stop read another stop's cache and scales its embedding and
its logits, and a toy norm and a toy arrangement of a layer's parts beside the built-in ones are
registered here, built and stepped (in portions, several sequences at once) without touching the
framework's files."""

import math

import pytest
import torch

import paged_attention_engine_amd as pae
from paged_attention_engine_amd import parts as P
from paged_attention_engine_amd.cache import PAGE, CacheManager, PagedSpec, PagedTensor, StateSpec
from paged_attention_engine_amd.parts.attention import WORK_LISTS, attention_work_lists
from paged_attention_engine_amd.config import (FeedForwardSpec, LayerSpec, MixerSpec, ModelPlan, NormSpec, PartSpec,
                                               PositionSpec, ScheduleEntry)
from tests.plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": 2e-5, "bfloat16": 4e-2}


def make_ctx(cache, dtype, seq_ids, q_lens):
    """A step context for sequences that have already reserved `q_lens` new tokens."""
    positions, tok_seq, q_starts, past = [], [], [], []
    for row, (s, n) in enumerate(zip(seq_ids, q_lens)):
        held = cache.num_tokens(s)
        q_starts.append(len(positions))
        past.append(held - n)
        positions += list(range(held - n, held))
        tok_seq += [row] * n
    tables = {}
    for group in cache.groups:
        rows = [cache.block_table(group.index, s) for s in seq_ids]
        width = max(len(r) for r in rows)
        tables[group.index] = torch.tensor([list(r) + [-1] * (width - len(r)) for r in rows], dtype=torch.int32, device=DEV)
    slots = [cache.slot_of(s) for s in seq_ids]
    # the attention kernels' work lists, as the step function would leave them for the mixer
    shape = P.StepShape(tuple(seq_ids), tuple(q_starts), tuple(q_lens), tuple(past), cache.block_size)
    lists = {name: torch.tensor(flat, dtype=torch.int32, device=DEV).view(*((-1, width) if width else (-1,)))
             for name, (flat, width) in attention_work_lists(shape).items()}
    return P.StepContext(
        dtype=dtype, device=torch.device(DEV), num_tokens=len(positions), num_seqs=len(seq_ids),
        positions=torch.tensor(positions, dtype=torch.int32, device=DEV),
        tok_seq=torch.tensor(tok_seq, dtype=torch.int32, device=DEV), block_tables=tables,
        slots=torch.tensor(slots, dtype=torch.int32, device=DEV), cache=cache, seq_ids=list(seq_ids),
        q_starts=q_starts, q_lens=list(q_lens), past_lens=past, host_slots=slots, memo={WORK_LISTS: lists})


# ------------------------------------------------------------------ built-in parts, one at a time
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_norm_part(dtype):
    spec = NormSpec(size=200, eps=3e-6)
    part = P.build_part(P.NORMS, "norm", spec, DT[dtype], DEV)
    assert part.tensors("x.") == {"x.weight": (200,)}
    w = 1 + 0.1 * torch.randn(200)
    part.bind("x.", {"x.weight": w.to(DT[dtype])})
    res = torch.randn(6, 200)
    branch = torch.randn(6, 200).to(DT[dtype])
    stream = P.ResidualStream(res.to(DEV))
    stream.pending = branch.to(DEV)
    out = part.forward(stream)
    want = plain.rms_norm((res + branch.float()).double(), w.to(DT[dtype]).double(), 3e-6)
    assert stream.pending is None and torch.allclose(stream.residual.cpu(), res + branch.float(), atol=1e-6)
    assert (out.double().cpu() - want).abs().max() <= TOL[dtype] * 4
    stream.pending = branch.to(DEV)
    rows = part.forward(stream, torch.tensor([5, 2], dtype=torch.int32, device=DEV))
    want2 = plain.rms_norm((res + 2 * branch.float()).double(), w.to(DT[dtype]).double(), 3e-6)[[5, 2]]
    assert stream.pending is not None and (rows.double().cpu() - want2).abs().max() <= TOL[dtype] * 4


def test_norm_part_and_rows_that_a_product_prepared():
    """A branch's last product may have added itself into the residual and prepared rows for a norm.
    The norm they were prepared for hands them on as they are (no kernel); another norm, or the same
    norm asked for some rows only, normalises the (complete) residual itself."""
    torch.manual_seed(4)
    width, eps = 200, 3e-6
    spec = NormSpec(size=width, eps=eps)
    mine, other = (P.build_part(P.NORMS, "norm", spec, torch.bfloat16, DEV) for _ in range(2))
    w_mine, w_other = (1 + 0.1 * torch.randn(width)).bfloat16(), (1 + 0.3 * torch.randn(width)).bfloat16()
    mine.bind("a.", {"a.weight": w_mine})
    other.bind("b.", {"b.weight": w_other})
    from paged_attention_engine_amd.kernels import lib
    assert mine.folded_for(3) is not None and mine.folded_for(lib.FOLD_MAX_ROWS) is not None
    assert mine.folded_for(lib.FOLD_MAX_ROWS + 1) is None and mine.folded_for(0) is None
    assert P.build_part(P.NORMS, "norm", spec, torch.float32, DEV).folded_for(3) is None  # float32 runs its kernel
    # a wide norm is folded at every row count up to 16, above that only while rows x width stays small
    wide = P.build_part(P.NORMS, "norm", NormSpec(size=lib.FOLD_MAX_ELEMENTS // 32, eps=eps), torch.bfloat16, DEV)
    wide.bind("c.", {"c.weight": torch.ones(lib.FOLD_MAX_ELEMENTS // 32).bfloat16()})
    assert wide.folded_for(16) is not None and wide.folded_for(32) is not None and wide.folded_for(33) is None
    res = torch.randn(3, width)
    rows = (res * w_mine.float()).bfloat16()
    stats = torch.zeros(3, K_stat_tiles(width))
    padded = torch.zeros(3, K_stat_tiles(width) * 16)
    padded[:, :width] = res.pow(2)
    stats = padded.view(3, -1, 16).sum(-1)

    def stream_with_owed(to):
        stream = P.ResidualStream(res.to(DEV))
        stream.owed, stream.owed_to = P.OwedRows(rows.to(DEV), stats.to(DEV), eps), to
        return stream

    stream = stream_with_owed(mine)
    handed = stream.owed
    got = mine.forward(stream)
    assert got is handed and stream.owed is None  # handed on as they are: no kernel ran
    settled = P.plain_rows(got)
    want = plain.rms_norm(res.double(), w_mine.double(), eps)
    assert (settled.double().cpu() - want).abs().max() <= TOL["bfloat16"] * 4
    # prepared for another norm: this one normalises the residual with its own weight
    stream = stream_with_owed(other)
    got = mine.forward(stream)
    assert torch.is_tensor(got) and stream.owed is None
    assert (got.double().cpu() - want).abs().max() <= TOL["bfloat16"] * 4
    # some rows only: the stream keeps what it owes, the rows come from the residual
    stream = stream_with_owed(mine)
    got = mine.forward(stream, torch.tensor([2, 0], dtype=torch.int32, device=DEV))
    assert torch.is_tensor(got) and stream.owed is not None and stream.owed_to is mine
    assert (got.double().cpu() - want[[2, 0]]).abs().max() <= TOL["bfloat16"] * 4


def K_stat_tiles(width):
    from paged_attention_engine_amd.kernels import lib
    return lib.stat_tiles(width)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("hidden,inter", [(96, 208), (72, 200)])  # the second is not a multiple of 16
def test_feed_forward_part(dtype, hidden, inter):
    torch.manual_seed(0)
    spec = FeedForwardSpec(hidden_size=hidden, intermediate_size=inter)
    part = P.build_part(P.FEED_FORWARDS, "feed-forward", spec, DT[dtype], DEV)
    names = part.tensors("m.mlp.")
    assert names == {"m.mlp.gate_proj.weight": (inter, hidden), "m.mlp.up_proj.weight": (inter, hidden),
                     "m.mlp.down_proj.weight": (hidden, inter)}
    w = {n: (torch.randn(shape) * 0.2).to(DT[dtype]) for n, shape in names.items()}
    part.bind("m.mlp.", w)
    for rows in (5, 70):  # the skinny products and the library's
        x = torch.randn(rows, hidden).to(DT[dtype])
        got = part.forward(None, x.to(DEV))
        got = got.sum(0) if got.dim() == 3 else got  # float32 partial sums are added by the next norm
        want = plain.swiglu_mlp({k: v.double() for k, v in w.items()}, "m.", x.double())
        assert (got.double().cpu() - want).abs().max() <= TOL[dtype] * max(1.0, float(want.abs().max()))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nh,nkv,hd,window,bs", [(4, 2, 16, None, 8), (6, 2, 32, 20, 16), (5, 1, 64, None, 16)])
def test_attention_part_in_portions(dtype, nh, nkv, hd, window, bs):
    """The mixer alone, two sequences at once, the first in portions of 9, 1 and 30 tokens."""
    torch.manual_seed(1)
    hidden = 80
    spec = MixerSpec(hidden_size=hidden, num_heads=nh, num_kv_heads=nkv, head_dim=hd, scale=hd ** -0.5,
                     qkv_bias=True, window=window, position=PositionSpec(rotary_dim=hd, theta=12345.0))
    part = P.build_part(P.MIXERS, "mixer", spec, DT[dtype], DEV)
    names = part.tensors("a.self_attn.")
    w = {n: (torch.randn(shape) * 0.15).to(DT[dtype]) for n, shape in names.items()}
    part.bind("a.self_attn.", w)
    cache = CacheManager([part.paged_spec()], [None], bs, 24, 4, DT[dtype], DEV)
    cfg = dict(num_attention_heads=nh, num_key_value_heads=nkv, head_dim=hd, rope_theta=12345.0)
    xs = {0: torch.randn(40, hidden).to(DT[dtype]), 1: torch.randn(17, hidden).to(DT[dtype])}
    want = {s: plain.self_attention({k: v.double() for k, v in w.items()}, "a.", cfg, x.double(),
                                    torch.arange(x.shape[0]), window) for s, x in xs.items()}
    for s in xs:
        cache.create_sequence(s)
    done = {0: 0, 1: 0}
    for step in ([(0, 9), (1, 17)], [(0, 1)], [(0, 30)]):
        for s, n in step:
            cache.reserve(s, n)
        ctx = make_ctx(cache, DT[dtype], [s for s, _ in step], [n for _, n in step])
        x = torch.cat([xs[s][done[s]:done[s] + n] for s, n in step]).to(DEV)
        got = part.forward(ctx, x)
        got = got.sum(0) if got.dim() == 3 else got
        ref = torch.cat([want[s][done[s]:done[s] + n] for s, n in step])
        assert (got.double().cpu() - ref).abs().max() <= TOL[dtype] * max(1.0, float(ref.abs().max()))
        for s, n in step:
            done[s] += n
            cache.release_passed(s)


# ------------------------------------------------------------------ toy parts registered by this test
@P.register_mixer("toy_decay")
class DecayMixer(P.Part):
    """y_t = s_t, s_t = decay * s_{t-1} + W x_t: a mixer that keeps a vector per request
    instead of keys and values.  Written with library calls and host loops (a test part)."""

    def state_spec(self):
        return StateSpec((self.spec.hidden_size,), torch.float32)

    def tensors(self, prefix):
        return {prefix + "in.weight": (self.spec.hidden_size, self.spec.hidden_size)}

    def bind(self, prefix, weights):
        self.w = weights[prefix + "in.weight"].to(device=self.device, dtype=torch.float32)

    def forward(self, ctx, x):
        state = ctx.cache.state_of(ctx.cache_entry)
        u = x.float() @ self.w.t()
        out = torch.empty_like(u)
        for start, n, slot in zip(ctx.q_starts, ctx.q_lens, ctx.host_slots):
            s = state[slot]
            for t in range(start, start + n):
                s = self.spec.decay * s + u[t]
                out[t] = s
            state[slot] = s
        return out.to(x.dtype)


@P.register_position_encoding("toy_shift")
class ShiftEncoding(P.Part):
    """Adds position / 100 to the first feature of every head it is given (a toy).  It encodes in
    place and knows of no cache: the mixer stores keys and values."""

    def encode(self, ctx, x, num_heads, head_dim):
        heads = x[:, :num_heads * head_dim].view(x.shape[0], num_heads, head_dim)
        heads[:, :, 0] += (ctx.positions.float() / 100.0).to(x.dtype)[:, None]


from dataclasses import dataclass


@dataclass(frozen=True)
class RoutedSpec(PartSpec):
    hidden_size: int = 0
    intermediate_size: int = 0
    num_experts: int = 2
    kind: str = "toy_routed"


@P.register_feed_forward("toy_routed")
class RoutedFeedForward(P.Part):
    """y = down_e(relu(up_e(x))) with e = argmax(router x), router logits in float32: a feed-forward
    that sends every token to one of several experts.  The products are the framework's own
    `Linear` (its kernels); the routing is a few library calls (a test part)."""

    def tensors(self, prefix):
        s = self.spec
        out = {prefix + "router.weight": (s.num_experts, s.hidden_size)}
        for e in range(s.num_experts):
            out[prefix + f"experts.{e}.up.weight"] = (s.intermediate_size, s.hidden_size)
            out[prefix + f"experts.{e}.down.weight"] = (s.hidden_size, s.intermediate_size)
        return out

    def bind(self, prefix, weights):
        from paged_attention_engine_amd.parts.linear import Linear
        self.router = weights[prefix + "router.weight"].to(device=self.device, dtype=torch.float32)
        self.up = [Linear(self.matrix(weights[prefix + f"experts.{e}.up.weight"])) for e in range(self.spec.num_experts)]
        self.down = [Linear(self.matrix(weights[prefix + f"experts.{e}.down.weight"])) for e in range(self.spec.num_experts)]

    def forward(self, ctx, x):
        choice = (x.float() @ self.router.t()).argmax(-1)  # a function of the token alone
        out = torch.zeros_like(x)
        for e in range(self.spec.num_experts):
            rows = (choice == e).nonzero().flatten()
            if rows.numel():
                out[rows] = self.down[e](torch.relu(self.up[e](x[rows].contiguous())))
        return out


@dataclass(frozen=True)
class DecaySpec(PartSpec):
    hidden_size: int = 0
    decay: float = 0.5
    kind: str = "toy_decay"


class ToyConfig:
    """config.json of a made-up architecture: attention, a decay mixer, attention again through
    the first stop's weights, and a stop that reads the first stop's cache."""

    def __init__(self, cfg):
        self.cfg = dict(cfg)

    def to_json_dict(self):
        return dict(self.cfg)

    def plan(self):
        c = self.cfg
        H, hd = c["hidden_size"], c["head_dim"]
        # names of this architecture's own: norms are `ln1.scale` / `ln2.scale` / `final_ln.scale`, the
        # attention's projections `wq` .. `wo` (the built-in parts take their names from the specs)
        norm = NormSpec(size=H, eps=c["eps"], weight_name="scale")
        attn = MixerSpec(hidden_size=H, num_heads=c["heads"], num_kv_heads=c["kv_heads"], head_dim=hd,
                         scale=hd ** -0.5, qkv_bias=False, position=PositionSpec(kind="toy_shift"),
                         q_name="wq", k_name="wk", v_name="wv", o_name="wo")
        ffn = FeedForwardSpec(hidden_size=H, intermediate_size=c["inter"])
        names = dict(mixer_norm_prefix="ln1.", feed_forward_norm_prefix="ln2.")
        layers = (LayerSpec("layers.0.", attn, ffn, norm, norm, **names),
                  LayerSpec("layers.1.", DecaySpec(hidden_size=H, decay=c["decay"]), ffn, norm, norm, **names))
        schedule = (ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0), ScheduleEntry(0, cache_from=0), ScheduleEntry(1))
        return ModelPlan("ToyForCausalLM", H, c["vocab"], layers, schedule, norm, "embed.weight", "head.weight", "final_ln.",
                         embedding_scale=c["embedding_scale"], logit_scale=c["logit_scale"], logit_softcap=c["logit_softcap"])


pae.register_architecture("ToyForCausalLM", ToyConfig)
TOY = dict(architectures=["ToyForCausalLM"], hidden_size=48, head_dim=16, heads=3, kv_heads=1, inter=64, vocab=97,
           eps=1e-5, decay=0.6, embedding_scale=3.0, logit_scale=0.25, logit_softcap=2.0)


def toy_plain_logits(w, c, ids):
    """The toy architecture written out plainly (float64, whole sequence, no cache)."""
    x = c["embedding_scale"] * w["embed.weight"][ids].double()
    n = len(ids)
    pos = torch.arange(n, dtype=torch.float64)
    kv_of_stop0 = None

    def attention(prefix, h, borrowed=None):
        nh, nkv, hd = c["heads"], c["kv_heads"], c["head_dim"]
        q = plain.split_heads(plain.linear(h, w[prefix + "wq.weight"].double()), nh, hd).clone()
        q[:, :, 0] += pos / 100.0
        if borrowed is None:
            k = plain.split_heads(plain.linear(h, w[prefix + "wk.weight"].double()), nkv, hd).clone()
            v = plain.split_heads(plain.linear(h, w[prefix + "wv.weight"].double()), nkv, hd)
            k[:, :, 0] += pos / 100.0
        else:
            k, v = borrowed
        out = plain.attention(q, k, v, hd ** -0.5)
        return plain.linear(plain.merge_heads(out), w[prefix + "wo.weight"].double()), (k, v)

    def decay(prefix, h):
        u = h @ w[prefix + "in.weight"].double().t()
        s, rows = torch.zeros(u.shape[1], dtype=torch.float64), []
        for t in range(n):
            s = c["decay"] * s + u[t]
            rows.append(s)
        return torch.stack(rows)

    for stop, (layer, borrow) in enumerate(((0, False), (1, False), (0, False), (0, True), (1, False))):
        p = f"layers.{layer}."
        h = plain.rms_norm(x, w[p + "ln1.scale"].double(), c["eps"])
        if layer == 0:
            y, kv = attention(p + "self_attn.", h, kv_of_stop0 if borrow else None)
            if stop == 0:
                kv_of_stop0 = kv
        else:
            y = decay(p + "self_attn.", h)
        x = x + y
        h = plain.rms_norm(x, w[p + "ln2.scale"].double(), c["eps"])
        x = x + plain.swiglu_mlp({k: v.double() for k, v in w.items()}, p, h)
    logits = c["logit_scale"] * plain.linear(plain.rms_norm(x, w["final_ln.scale"].double(), c["eps"]),
                                             w["head.weight"].double())
    return c["logit_softcap"] * torch.tanh(logits / c["logit_softcap"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_routed_feed_forward_is_registered_and_built(dtype):
    """A feed-forward with routing, defined above in this file, goes through the registry and runs
    on the framework's products; 100 tokens (the many-row path) and 5 (the few-row path)."""
    torch.manual_seed(11)
    H, I, E = 64, 96, 3
    spec = RoutedSpec(hidden_size=H, intermediate_size=I, num_experts=E)
    part = P.build_part(P.FEED_FORWARDS, "feed-forward", spec, DT[dtype], DEV)
    names = part.tensors("m.mlp.")
    assert len(names) == 1 + 2 * E
    w = {n: (torch.randn(shape) * 0.2).to(DT[dtype]) for n, shape in names.items()}
    part.bind("m.mlp.", w)
    router = w["m.mlp.router.weight"].double()
    for T in (100, 5):
        x = torch.randn(T, H)
        # push every token towards one expert, so that no rounding decides the routing
        target = torch.arange(T) % E
        x = (x + 3.0 * router[target].float() / router[target].float().norm(dim=1, keepdim=True)).to(DT[dtype])
        logits = x.double() @ router.t()
        top2 = logits.topk(2, dim=-1).values
        assert float((top2[:, 0] - top2[:, 1]).min()) > 0.05
        choice = logits.argmax(-1)
        want = torch.zeros(T, H, dtype=torch.float64)
        for e in range(E):
            rows = choice == e
            up, down = w[f"m.mlp.experts.{e}.up.weight"].double(), w[f"m.mlp.experts.{e}.down.weight"].double()
            want[rows] = torch.relu(x[rows].double() @ up.t()) @ down.t()
        assert len(set(choice.tolist())) == E
        got = part.forward(None, x.to(DEV))
        assert (got.double().cpu() - want).abs().max() <= TOL[dtype] * max(1.0, float(want.abs().max()))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_is_registered_built_and_stepped(tmp_path, dtype):
    assert "ToyForCausalLM" in pae.known_architectures()
    config = pae.read_config_dict(TOY)
    folder = pae.write_model_folder(config, 5, str(tmp_path / "toy"), std=0.08, norm_std=0.1)
    model = pae.load_model(folder, dtype)
    assert not model.graph_safe  # the toy parts run host loops: steps are launched eagerly
    # random mode draws a tensor as the part that declares it says, whatever it is called: this
    # architecture's norm weights are `...ln1.scale`, and they come out about one
    drawn = pae.random_model(config, 5, dtype, std=0.08, norm_std=0.1)
    for norm_part in (drawn.blocks[0].mixer_norm, drawn.blocks[1].feed_forward_norm, drawn.final_norm):
        assert 0.05 < float((norm_part.weight.float() - 1).abs().max()) < 0.6
    assert {"layers.0.ln1.scale", "layers.1.ln2.scale", "final_ln.scale", "layers.0.self_attn.wq.weight"} <= set(drawn.expected_tensors())
    paged, states = model.cache_specs()
    assert [p is not None for p in paged] == [True, False, True, False, False]  # stop 3 borrows stop 0's cache
    assert [s is not None for s in states] == [False, True, False, False, True]
    cache = model.new_cache(8, 32, 3)
    assert len(cache.groups) == 1 and cache.groups[0].entries == [0, 2]
    runner = pae.StepRunner(model, cache)
    weights = pae.load_weights(folder, model.expected_tensors())
    w = {k: v.float() for k, v in weights.items()}
    gen = torch.Generator().manual_seed(2)
    seqs = {s: torch.randint(0, 97, (n,), generator=gen).tolist() for s, n in ((0, 30), (1, 19), (2, 7))}
    want = {s: toy_plain_logits(w, TOY, ids).float() for s, ids in seqs.items()}
    tol = helpers_tol(dtype, max(float(v.abs().max()) for v in want.values()))
    done = {s: 0 for s in seqs}
    for s in seqs:
        assert cache.create_sequence(s)
    plans = ([(0, 11), (1, 19)], [(0, 1), (2, 2)], [(0, 2), (2, 5)], [(0, 16)])
    for plan in plans:
        entries = []
        for s, n in plan:
            cache.reserve(s, n)
            entries.append(pae.StepEntry(s, tuple(seqs[s][done[s]:done[s] + n]), tuple(range(n))))
        got = runner.run(entries).cpu()
        ref = torch.cat([want[s][done[s]:done[s] + n] for s, n in plan])
        assert float((got - ref).abs().max()) <= tol
        for s, n in plan:
            done[s] += n
    # a freed request's state slot is zeroed for the next one: the same tokens give the same logits
    cache.free_sequence(2)
    assert cache.create_sequence(7)
    cache.reserve(7, 7)
    again = runner.run([pae.StepEntry(7, tuple(seqs[2]), tuple(range(7)))]).cpu()
    assert float((again - want[2]).abs().max()) <= tol


def helpers_tol(dtype, top):
    from tests import helpers
    ref = torch.tensor(top)
    # the toy architecture is drawn four times wider than the tiny models: the reference's 4 ulp
    return helpers.fp32_atol(ref) * 4 if dtype == "float32" else 4 * helpers.bf16_ulp(ref)


# ------------------------------------------------------------------ a mixer with a cached tensor of its own
@dataclass(frozen=True)
class LatentSpec(PartSpec):
    hidden_size: int = 0
    latent_size: int = 0
    window: int = 0
    kind: str = "toy_latent"


@P.register_mixer("toy_latent")
class LatentMeanMixer(P.Part):
    """Caches one latent vector per token, l_t = W_in x_t, in pages of its own shape [PAGE][latent]
    (no keys, no values, no heads), and returns W_out applied to the mean of the latents of the last
    `window` tokens.  Host loops and library calls: a test part."""

    def paged_spec(self):
        return PagedSpec((PagedTensor("latent", (PAGE, self.spec.latent_size)),), self.spec.window)

    def tensors(self, prefix):
        s = self.spec
        return {prefix + "in.weight": (s.latent_size, s.hidden_size), prefix + "out.weight": (s.hidden_size, s.latent_size)}

    def bind(self, prefix, weights):
        self.w_in = weights[prefix + "in.weight"].to(device=self.device, dtype=torch.float32)
        self.w_out = weights[prefix + "out.weight"].to(device=self.device, dtype=torch.float32)

    def forward(self, ctx, x):
        pages = ctx.cache.pages_of(ctx.cache_entry)["latent"]  # [block][page][latent]
        tables = ctx.block_tables[ctx.cache.group_of(ctx.cache_entry)].cpu()
        bs, window = ctx.cache.block_size, self.spec.window
        latents = x.float() @ self.w_in.t()
        out = torch.empty((x.shape[0], self.spec.hidden_size), dtype=torch.float32, device=x.device)
        for row, (start, n, past) in enumerate(zip(ctx.q_starts, ctx.q_lens, ctx.past_lens)):
            for i in range(n):  # store first: a token sees itself
                pos = past + i
                pages[int(tables[row, pos // bs]), pos % bs] = latents[start + i].to(pages.dtype)
            for i in range(n):
                pos = past + i
                seen = [pages[int(tables[row, p // bs]), p % bs].float() for p in range(max(0, pos - window + 1), pos + 1)]
                out[start + i] = torch.stack(seen).mean(0) @ self.w_out.t()
        return out.to(x.dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_mixer_with_one_cached_tensor_per_token(dtype):
    """The cache manager builds the pool a mixer declares, whatever its tensors are called and
    shaped; a window gives pages back, and they are used again by the next request."""
    torch.manual_seed(4)
    H, L, window, bs = 40, 24, 10, 4
    spec = LatentSpec(hidden_size=H, latent_size=L, window=window)
    part = P.build_part(P.MIXERS, "mixer", spec, DT[dtype], DEV)
    w = {n: (torch.randn(shape) * 0.3) for n, shape in part.tensors("m.").items()}
    part.bind("m.", w)
    cache = CacheManager([part.paged_spec()], [None], bs, 6, 2, DT[dtype], DEV)
    assert set(cache.groups[0].pools) == {"latent"}
    assert tuple(cache.groups[0].pools["latent"].shape) == (1, 6 + 1, bs, L)
    assert cache.storage_bytes() == 6 * bs * L * torch.empty((), dtype=DT[dtype]).element_size()

    def expected(x):
        lat = (x.float() @ w["m.in.weight"].t()).to(DT[dtype]).float()  # as stored
        rows = [lat[max(0, t - window + 1):t + 1].mean(0) @ w["m.out.weight"].t() for t in range(x.shape[0])]
        return torch.stack(rows)

    used = set()
    for seq, portions in ((0, (7, 1, 9, 2, 6, 8)), (1, (20, 1, 1))):  # 33 tokens need 9 pages without the window
        x = torch.randn(sum(portions), H).to(DT[dtype])
        want = expected(x)
        assert cache.create_sequence(seq)
        done = 0
        for n in portions:
            assert cache.reserve(seq, n).ok
            used |= {b for b in cache.block_table(0, seq) if b >= 0}
            ctx = make_ctx(cache, DT[dtype], [seq], [n])
            got = part.forward(ctx, x[done:done + n].to(DEV))
            assert (got.float().cpu() - want[done:done + n]).abs().max() <= TOL[dtype] * max(1.0, float(want.abs().max()))
            done += n
            cache.release_passed(seq)
        cache.free_sequence(seq)
    assert cache.free_blocks() == (6,) and used == set(range(6))


# ------------------------------------------------------------------ a norm and a block arrangement of the test's own
@P.register_norm("toy_center")
class CenterNorm(P.Part):
    """y = w * (x - mean(x)) / sqrt(var(x) + eps): a norm that subtracts the mean (a test part, written
    with library calls).  It has no `folded()`, so the products around it must hand over plain outputs
    even in steps of a few rows, where an RMS norm would be carried by them."""

    def tensors(self, prefix):
        return {prefix + "weight": (self.spec.size,)}

    def bind(self, prefix, weights):
        self.weight = weights[prefix + "weight"].to(device=self.device, dtype=torch.float32)

    def forward(self, stream, rows=None):
        pending = stream.pending
        delta = None if pending is None else (pending.sum(0) if pending.dim() == 3 else pending.float())
        if rows is None:
            stream.owed = stream.owed_to = None  # rows prepared for another norm are of no use here
            if delta is not None:
                stream.residual += delta
                stream.pending = None
            x = stream.residual
        else:  # some rows only: the stream stays as it is
            x = (stream.residual if delta is None else stream.residual + delta)[rows.long()]
        centred = x - x.mean(-1, keepdim=True)
        y = centred * torch.rsqrt(centred.pow(2).mean(-1, keepdim=True) + self.spec.eps) * self.weight
        return y.to(self.dtype)


@P.register_block("toy_parallel")
class ParallelBlock:
    """h = h + mixer(norm(h)) + feed_forward(norm(h)): both branches read the same normalised rows
    and the layer has one norm.  Both outputs are left pending as two float32 terms for the next
    norm to add; no branch is offered a sink."""

    def __init__(self, layer_spec, dtype, device):
        self.spec = layer_spec
        self.mixer_norm = P.build_part(P.NORMS, "norm", layer_spec.mixer_norm, dtype, device)
        self.mixer = P.build_part(P.MIXERS, "mixer", layer_spec.mixer, dtype, device)
        self.feed_forward = P.build_part(P.FEED_FORWARDS, "feed-forward", layer_spec.feed_forward, dtype, device)

    graph_safe = False
    graph_max_rows = None

    def _named(self):
        s = self.spec
        return ((self.mixer_norm, s.prefix + s.mixer_norm_prefix), (self.mixer, s.prefix + s.mixer_prefix),
                (self.feed_forward, s.prefix + s.feed_forward_prefix))

    def parts(self):
        return [part for part, _ in self._named()]

    def tensors(self):
        out = {}
        for part, prefix in self._named():
            out.update(part.tensors(prefix))
        return out

    def bind(self, weights):
        for part, prefix in self._named():
            part.bind(prefix, weights)

    def forward(self, ctx, stream):
        x = P.plain_rows(self.mixer_norm.forward(stream))
        ctx.sink = None
        terms = []
        for part in (self.mixer, self.feed_forward):
            y = part.forward(ctx, x)
            terms.append(y.sum(0) if y.dim() == 3 else y.float())
        stream.pending = torch.stack(terms)


class ParallelToyConfig:
    """Two layers: a parallel block around the centring norm, then the ordinary block with RMS norms;
    the final norm centres again."""

    def __init__(self, cfg):
        self.cfg = dict(cfg)

    def to_json_dict(self):
        return dict(self.cfg)

    def plan(self):
        c = self.cfg
        H, hd = c["hidden_size"], c["head_dim"]
        centre = NormSpec(size=H, eps=c["eps"], kind="toy_center")
        rms = NormSpec(size=H, eps=c["eps"])
        attn = MixerSpec(hidden_size=H, num_heads=c["heads"], num_kv_heads=c["kv_heads"], head_dim=hd,
                         scale=hd ** -0.5, qkv_bias=True, position=PositionSpec(rotary_dim=hd, theta=c["theta"]))
        ffn = FeedForwardSpec(hidden_size=H, intermediate_size=c["inter"])
        layers = (LayerSpec("model.layers.0.", attn, ffn, centre, centre, arrangement="toy_parallel"),
                  LayerSpec("model.layers.1.", attn, ffn, rms, rms))
        return ModelPlan("ParallelToyForCausalLM", H, c["vocab"], layers, (ScheduleEntry(0), ScheduleEntry(1)), centre,
                         "model.embed_tokens.weight", "lm_head.weight", "model.norm.")


pae.register_architecture("ParallelToyForCausalLM", ParallelToyConfig)
PARALLEL_TOY = dict(architectures=["ParallelToyForCausalLM"], hidden_size=64, head_dim=16, heads=4, kv_heads=2, inter=80,
                    vocab=131, eps=1e-5, theta=10000.0)


def parallel_toy_plain_logits(w, c, ids):
    """The architecture above written out plainly (float64, whole sequence, no cache)."""
    w = {k: v.double() for k, v in w.items()}
    cfg = dict(num_attention_heads=c["heads"], num_key_value_heads=c["kv_heads"], head_dim=c["head_dim"],
               hidden_size=c["hidden_size"], rope_theta=c["theta"])
    pos = torch.arange(len(ids))

    def centre(x, weight):
        d = x - x.mean(-1, keepdim=True)
        return d * torch.rsqrt(d.pow(2).mean(-1, keepdim=True) + c["eps"]) * weight

    x = w["model.embed_tokens.weight"][ids]
    h = centre(x, w["model.layers.0.input_layernorm.weight"])
    x = x + plain.self_attention(w, "model.layers.0.", cfg, h, pos, None) + plain.swiglu_mlp(w, "model.layers.0.", h)
    h = plain.rms_norm(x, w["model.layers.1.input_layernorm.weight"], c["eps"])
    x = x + plain.self_attention(w, "model.layers.1.", cfg, h, pos, None)
    h = plain.rms_norm(x, w["model.layers.1.post_attention_layernorm.weight"], c["eps"])
    x = x + plain.swiglu_mlp(w, "model.layers.1.", h)
    return plain.linear(centre(x, w["model.norm.weight"]), w["lm_head.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_norm_and_block_arrangement_are_registered_built_and_stepped(tmp_path, dtype):
    """A norm and an arrangement of a layer's parts defined in this file, beside the built-in ones in
    the same model: portions of prompts, single tokens (where the built-in norms are carried by the
    products around them and the toy norm is not) and both together."""
    assert "toy_parallel" in P.BLOCKS and "toy_center" in P.NORMS
    config = pae.read_config_dict(PARALLEL_TOY)
    folder = pae.write_model_folder(config, 8, str(tmp_path / "parallel_toy"), std=0.08, norm_std=0.1)
    model = pae.load_model(folder, dtype)
    names = model.expected_tensors()
    assert "model.layers.0.input_layernorm.weight" in names
    assert "model.layers.0.post_attention_layernorm.weight" not in names  # the parallel block has one norm
    assert not model.graph_safe
    cache = model.new_cache(16, 12, 3)
    runner = pae.StepRunner(model, cache)
    w = {k: v.float() for k, v in pae.load_weights(folder, names).items()}
    gen = torch.Generator().manual_seed(4)
    seqs = {s: torch.randint(0, 131, (n,), generator=gen).tolist() for s, n in ((0, 40), (1, 23), (2, 9))}
    want = {s: parallel_toy_plain_logits(w, PARALLEL_TOY, ids).float() for s, ids in seqs.items()}
    tol = helpers_tol(dtype, max(float(v.abs().max()) for v in want.values()))
    done = {s: 0 for s in seqs}
    for s in seqs:
        assert cache.create_sequence(s)
    plans = ([(0, 30), (1, 20)], [(0, 1), (1, 1), (2, 7)], [(0, 1), (1, 1), (2, 1)], [(0, 1), (1, 1), (2, 1)], [(0, 7)])
    for plan in plans:
        entries = []
        for s, n in plan:
            cache.reserve(s, n)
            entries.append(pae.StepEntry(s, tuple(seqs[s][done[s]:done[s] + n]), tuple(range(n))))
        got = runner.run(entries).cpu()
        ref = torch.cat([want[s][done[s]:done[s] + n] for s, n in plan])
        assert float((got - ref).abs().max()) <= tol, plan
        for s, n in plan:
            done[s] += n
