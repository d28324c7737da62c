"""Each model part alone against the plain implementation, and a toy
architecture defined HERE (a mixer with state of its own, another position
encoding, a feed-forward with routing, a block that runs twice, a layer that
reads another layer's cache) that is registered, built and stepped without any
change to the package."""
import dataclasses
import math

import pytest
import torch

from litellmengine_amd.cache import CacheManager
from litellmengine_amd.config import register_architecture
from litellmengine_amd.engine import ModelRunner, StepEntry
from litellmengine_amd.models import DecoderLM, PlanEntry, make_context, random_model
from litellmengine_amd.parts import (Embedding, FeedForward, GatedMLP, Linear, Mixer, PagedAttention,
                                     PositionEncoding, PreNormBlock, RMSNorm, RotaryHalfSplit, StateSpec)
from litellmengine_amd.weights import TensorSpec, random_weights
from tests.plain import qwen3_plain as plain
from tests.tiny import random_tokens

pytestmark = pytest.mark.gpu
D = torch.float64
TOL = {torch.float32: 3e-5, torch.bfloat16: 4e-2}


def bound(part, dtype, seed=0):
    """Give `part` seeded random weights (rounded to bfloat16 so that both types see
    the same values); returns (context, weights as float64 on the CPU)."""
    ctx = make_context(dtype)
    w = random_weights(part.tensor_specs(), seed, torch.bfloat16, "cpu", include_optional=True)
    part.bind({k: v.to(ctx.device) for k, v in w.items()}, ctx)
    return ctx, {k: v.to(D) for k, v in w.items()}


def x_of(shape, dtype, seed, scale=1.0):
    x = (torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale).to(torch.bfloat16)
    return x.to(dtype).cuda(), x.to(D)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_linear_norm_embedding_mlp(dtype):
    lin = Linear(["a.weight", "b.weight"], 72, [40, 24])
    ctx, w = bound(lin, dtype)
    x, xp = x_of((5, 72), dtype, 1)
    want = torch.cat([plain.linear(xp, w["a.weight"]), plain.linear(xp, w["b.weight"])], dim=1)
    assert (lin.forward(x).cpu().double() - want).abs().max() < TOL[dtype]

    norm = RMSNorm("n.weight", 72, 1e-5)
    ctx, w = bound(norm, dtype)
    hidden = torch.randn(5, 72).cuda()
    delta, dp = x_of((5, 72), dtype, 2)
    want_h = hidden.cpu().double() + dp
    got = norm.forward(hidden, delta)
    assert (hidden.cpu().double() - want_h).abs().max() < 1e-6
    assert (got.cpu().double() - plain.rms_norm(want_h, w["n.weight"], 1e-5)).abs().max() < TOL[dtype] * 4

    emb = Embedding("e.weight", 101, 56)
    ctx, w = bound(emb, dtype)
    ids = torch.tensor([0, 100, 7], dtype=torch.int32).cuda()
    assert torch.equal(emb.forward(ids).cpu().double(), plain.embedding([0, 100, 7], w["e.weight"]))

    mlp = GatedMLP("m.", 72, 136)
    ctx, w = bound(mlp, dtype)
    x, xp = x_of((6, 72), dtype, 3, 3.0)
    want = plain.gated_mlp(xp, w["m.gate_proj.weight"], w["m.up_proj.weight"], w["m.down_proj.weight"])
    assert (mlp.forward(x).cpu().double() - want).abs().max() < TOL[dtype]


def one_block_model(block, hidden, vocab=50):
    return DecoderLM(None, Embedding("e.weight", vocab, hidden), [block], [PlanEntry(0)],
                     RMSNorm("fn.weight", hidden, 1e-6), Linear(["head.weight"], hidden, [vocab]), tied_head=False)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [None, 5])
def test_attention_mixer_and_block_alone(dtype, window):
    """The attention mixer inside one pre-norm block, stepped in two portions and
    then one token, against plain.decoder_layer on the whole sequence."""
    H, nq, nkv, d, I = 72, 6, 2, 16, 100
    p = "model.layers.0."
    block = PreNormBlock(
        RMSNorm(p + "input_layernorm.weight", H, 1e-5),
        PagedAttention(p + "self_attn.", H, nq, nkv, d, RotaryHalfSplit(d, 5e4), qk_norm_eps=1e-5, window=window),
        RMSNorm(p + "post_attention_layernorm.weight", H, 1e-5),
        GatedMLP(p + "mlp.", H, I),
    )
    model = one_block_model(block, H)
    ctx, w = bound(model, dtype)
    model.ctx = ctx
    cache = CacheManager(model, page_size=4, num_pages=8, max_requests=2, dtype=dtype, device=ctx.device)
    runner = ModelRunner(model, cache)
    T = 19
    ids = random_tokens(T, 50, 4)
    cfg = dict(num_attention_heads=nq, num_key_value_heads=nkv, head_dim=d, rms_norm_eps=1e-5, rope_theta=5e4)
    h = plain.decoder_layer(plain.embedding(ids, w["e.weight"]), list(range(T)), w, 0, cfg, window)
    want = plain.fast_linear(plain.rms_norm(h, w["fn.weight"], 1e-6), w["head.weight"])
    slot = runner.admit()
    got = torch.cat([runner.step([StepEntry(slot, ids[a:b], list(range(b - a)))]).cpu() for a, b in ((0, 11), (11, 18), (18, 19))])
    assert (got.double() - want).abs().max() < TOL[dtype]


# ---------------------------------------------------------------------------------------
# a toy architecture, defined in this test only
# ---------------------------------------------------------------------------------------
class RunningMeanMixer(Mixer):
    """y_t = W mean(x_0 .. x_t): needs no keys or values, only a running sum and a
    count per request — fixed-size state that the cache manager carries."""

    def __init__(self, name, hidden):
        self.name, self.hidden = name, hidden

    def tensor_specs(self):
        return {self.name: TensorSpec((self.hidden, self.hidden))}

    def state_spec(self):
        return StateSpec((self.hidden + 1,), torch.float32)

    def bind(self, weights, ctx):
        self.ctx = ctx
        self.weight = weights[self.name].to(ctx.dtype).contiguous()

    def forward(self, x, step, cache):
        out = torch.empty_like(x)
        for q in step.seqs:
            rows = slice(q.q_start, q.q_start + q.q_len)
            state = cache.state[q.slot]
            sums = state[:-1] + torch.cumsum(x[rows].float(), dim=0)
            counts = state[-1] + torch.arange(1, q.q_len + 1, device=x.device, dtype=torch.float32)
            out[rows] = (sums / counts[:, None]).to(x.dtype)
            state[:-1] = sums[-1]
            state[-1] = counts[-1]
        return self.ctx.ops.linear(out, self.weight)


class LearnedAdditivePosition(PositionEncoding):
    """q += table[pos], k += table[pos]: not a rotation, so the mixer takes the
    unfused path (norm, `apply`, then the page write)."""

    def __init__(self, name, max_positions, head_dim):
        self.name, self.max_positions, self.head_dim = name, max_positions, head_dim

    def tensor_specs(self):
        return {self.name: TensorSpec((self.max_positions, self.head_dim))}

    def bind(self, weights, ctx):
        self.ctx = ctx
        self.table = weights[self.name].to(ctx.dtype).contiguous()

    def apply(self, q, k, positions):
        t = self.table[positions.long()][:, None, :]
        return q + t, k + t


class TopOneRoutedFF(FeedForward):
    """A feed-forward with routing: router logits in 32-bit, every token goes to its best
    expert (a plain two-layer perceptron with SiLU), scaled by that expert's probability."""

    def __init__(self, prefix, hidden, width, experts):
        self.prefix, self.hidden, self.width, self.experts = prefix, hidden, width, experts

    def tensor_specs(self):
        specs = {self.prefix + "router": TensorSpec((self.experts, self.hidden))}
        for e in range(self.experts):
            specs[f"{self.prefix}e{e}.up"] = TensorSpec((self.width, self.hidden))
            specs[f"{self.prefix}e{e}.down"] = TensorSpec((self.hidden, self.width))
        return specs

    def bind(self, weights, ctx):
        self.ctx = ctx
        self.router = weights[self.prefix + "router"].float() * ROUTER_GAIN
        self.up = [weights[f"{self.prefix}e{e}.up"].to(ctx.dtype).contiguous() for e in range(self.experts)]
        self.down = [weights[f"{self.prefix}e{e}.down"].to(ctx.dtype).contiguous() for e in range(self.experts)]

    def forward(self, x):
        probs = torch.softmax(x.float() @ self.router.t(), dim=-1)
        best = probs.argmax(dim=-1)
        out = torch.zeros_like(x)
        for e in range(self.experts):
            rows = (best == e).nonzero().flatten()
            if rows.numel():
                h = torch.nn.functional.silu(self.ctx.ops.linear(x[rows].contiguous(), self.up[e]).float()).to(x.dtype)
                y = self.ctx.ops.linear(h, self.down[e]).float() * probs[rows, e][:, None]
                out[rows] = y.to(x.dtype)
        return out


ROUTER_GAIN = 40.0  # wide margins between the experts' logits, so that rounding does not re-route a token


class AttentionWithPosition(PagedAttention):
    def tensor_specs(self):
        return {**super().tensor_specs(), **self.position.tensor_specs()}


@dataclasses.dataclass(frozen=True)
class ToyConfig:
    architecture: str
    vocab_size: int
    hidden_size: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    ffn: int
    eps: float
    max_positions: int

    @classmethod
    def from_dict(cls, d):
        return cls(d["architectures"][0], d["vocab_size"], d["hidden_size"], d["num_heads"], d["num_kv_heads"],
                   d["head_dim"], d["ffn"], d["eps"], d["max_positions"])


def build_toy(c: ToyConfig) -> DecoderLM:
    def attention(i):
        return AttentionWithPosition(f"l{i}.attn.", c.hidden_size, c.num_heads, c.num_kv_heads, c.head_dim,
                                     LearnedAdditivePosition(f"l{i}.attn.pos", c.max_positions, c.head_dim),
                                     qk_norm_eps=c.eps)

    def block(i, mixer):
        ff = TopOneRoutedFF(f"l{i}.moe.", c.hidden_size, c.ffn, 3) if i == 2 else GatedMLP(f"l{i}.mlp.", c.hidden_size, c.ffn)
        return PreNormBlock(RMSNorm(f"l{i}.n1", c.hidden_size, c.eps), mixer, RMSNorm(f"l{i}.n2", c.hidden_size, c.eps), ff)

    blocks = [block(0, RunningMeanMixer("l0.mean.weight", c.hidden_size)), block(1, attention(1)), block(2, attention(2))]
    # block 0 runs twice (its second run has state of its own); block 2 reads the keys and values of block 1
    plan = [PlanEntry(0), PlanEntry(1), PlanEntry(0), PlanEntry(2, cache=1, writes=False)]
    return DecoderLM(c, Embedding("emb", c.vocab_size, c.hidden_size), blocks, plan, RMSNorm("fn", c.hidden_size, c.eps),
                     Linear(["head"], c.hidden_size, [c.vocab_size]), tied_head=False)


def toy_plain(ids, w, c: ToyConfig):
    T = len(ids)
    n = lambda x, name: plain.rms_norm(x, w[name], c.eps)

    def mlp(x, i):
        if i == 2:  # routed: best expert by router logits, scaled by its probability
            probs = torch.softmax(plain.linear(x, w["l2.moe.router"] * ROUTER_GAIN), dim=-1)
            out = torch.zeros_like(x)
            for t in range(x.shape[0]):
                e = int(probs[t].argmax())
                h = torch.nn.functional.silu(plain.linear(x[t : t + 1], w[f"l2.moe.e{e}.up"]))
                out[t] = plain.linear(h, w[f"l2.moe.e{e}.down"])[0] * probs[t, e]
            return out
        return plain.gated_mlp(x, w[f"l{i}.mlp.gate_proj.weight"], w[f"l{i}.mlp.up_proj.weight"], w[f"l{i}.mlp.down_proj.weight"])

    def mean_block(x):
        xin = n(x, "l0.n1")
        m = torch.cumsum(xin, 0) / torch.arange(1, T + 1, dtype=D)[:, None]
        r = x + plain.linear(m, w["l0.mean.weight"])
        return r + mlp(n(r, "l0.n2"), 0)

    def qkv(x, i):
        pos = w[f"l{i}.attn.pos"][:T][:, None, :]
        q = plain.linear(x, w[f"l{i}.attn.q_proj.weight"]).reshape(T, c.num_heads, c.head_dim)
        k = plain.linear(x, w[f"l{i}.attn.k_proj.weight"]).reshape(T, c.num_kv_heads, c.head_dim)
        v = plain.linear(x, w[f"l{i}.attn.v_proj.weight"]).reshape(T, c.num_kv_heads, c.head_dim)
        q = plain.rms_norm(q, w[f"l{i}.attn.q_norm.weight"], c.eps) + pos
        k = plain.rms_norm(k, w[f"l{i}.attn.k_norm.weight"], c.eps) + pos
        return q, k, v

    def attn_block(x, i, kv=None):
        q, k, v = qkv(n(x, f"l{i}.n1"), i)
        if kv is not None:
            k, v = kv
        a = plain.causal_gqa_attention(q, k, v).reshape(T, -1)
        r = x + plain.linear(a, w[f"l{i}.attn.o_proj.weight"])
        return r + mlp(n(r, f"l{i}.n2"), i), (k, v)

    h = plain.embedding(ids, w["emb"])
    h = mean_block(h)
    h, kv1 = attn_block(h, 1)
    h = mean_block(h)
    h, _ = attn_block(h, 2, kv1)
    return plain.fast_linear(n(h, "fn"), w["head"])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_toy_architecture_registers_builds_and_steps(dtype):
    register_architecture("ToyForCausalLM", ToyConfig, build_toy)
    c = ToyConfig.from_dict(dict(architectures=["ToyForCausalLM"], vocab_size=61, hidden_size=40, num_heads=4,
                                 num_kv_heads=2, head_dim=16, ffn=56, eps=1e-5, max_positions=64))
    model = build_toy(c)
    ctx, w = bound(model, dtype, seed=9)
    model.ctx = ctx
    cache = CacheManager(model, page_size=4, num_pages=12, max_requests=3, dtype=dtype, device=ctx.device)
    assert len(cache.groups) == 1 and cache.groups[0].cache_ids == [1]  # one cache layer, shared by two entries
    assert sorted(cache.states) == [0, 2]  # the block that runs twice has two state rows
    runner = ModelRunner(model, cache)
    seqs = {"x": random_tokens(21, 61, 1), "y": random_tokens(13, 61, 2)}
    want = {k: toy_plain(v, w, c) for k, v in seqs.items()}
    sx, sy = runner.admit(), runner.admit()
    got = {"x": [], "y": []}
    # portions of x beside portions and single tokens of y
    for (ax, bx), (ay, by) in (((0, 9), (0, 2)), ((9, 10), (2, 11)), ((10, 21), (11, 12)), ((21, 21), (12, 13))):
        entries, names = [], []
        if bx > ax:
            entries.append(StepEntry(sx, seqs["x"][ax:bx], list(range(bx - ax))))
            names.append(("x", bx - ax))
        if by > ay:
            entries.append(StepEntry(sy, seqs["y"][ay:by], list(range(by - ay))))
            names.append(("y", by - ay))
        out = runner.step(entries).cpu()
        at = 0
        for name, cnt in names:
            got[name].append(out[at : at + cnt])
            at += cnt
    for k in seqs:
        err = (torch.cat(got[k]).double() - want[k]).abs().max().item()
        assert err < TOL[dtype], (k, err)
    # a slot that is used again starts from zeroed state
    runner.release(sx)
    s2 = runner.admit()
    assert s2 == sx
    again = runner.step([StepEntry(s2, seqs["y"], list(range(13)))]).cpu()
    assert (again.double() - want["y"]).abs().max() < TOL[dtype]


# ---------------------------------------------------------------------------------------
# a mixer whose per-token cache is no key/value pair: one latent vector a token
# ---------------------------------------------------------------------------------------
class LatentMeanMixer(Mixer):
    """c_t = W_down x_t is cached (one vector of `rank` elements per token, in pages);
    y_t = W_up mean(c_0 .. c_t), the mean read back from the pages through the block table."""

    def __init__(self, prefix, hidden, rank, window=None):
        self.prefix, self.hidden, self.rank, self.window = prefix, hidden, rank, window

    def tensor_specs(self):
        return {self.prefix + "down": TensorSpec((self.rank, self.hidden)),
                self.prefix + "up": TensorSpec((self.hidden, self.rank))}

    def cache_spec(self):
        from litellmengine_amd.parts import CacheField, CacheSpec

        return CacheSpec((CacheField("latent", 1, self.rank),), self.window)

    def bind(self, weights, ctx):
        self.ctx = ctx
        self.down = weights[self.prefix + "down"].to(ctx.dtype).contiguous()
        self.up = weights[self.prefix + "up"].to(ctx.dtype).contiguous()

    def forward(self, x, step, cache):
        c = self.ctx.ops.linear(x, self.down)
        pages = cache.field("latent")  # [page, 1, page_size, rank]
        P = pages.shape[2]
        if cache.writes:
            where = cache.group.slot_mapping.long()
            pages[where // P, 0, where % P] = c
        y = torch.empty_like(c)
        for q in step.seqs:
            table = cache.group.block_table[q.slot].long()
            for t in range(q.q_len):
                pos = q.past_len + t
                lo = max(0, pos - self.window + 1) if self.window else 0
                at = torch.arange(lo, pos + 1, device=x.device)
                seen = pages[table[at // P], 0, at % P].float()
                y[q.q_start + t] = seen.mean(dim=0).to(y.dtype)
        return self.ctx.ops.linear(y, self.up)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_cache_record_that_is_no_key_value_pair(dtype):
    """The cache manager pages whatever record a mixer declares: here one latent vector per
    token, once for all positions and once behind a window (two groups: pages of the second
    are given back and used again).  Portions, single tokens and a second request in pages
    that the first has freed, against the running mean computed whole."""
    hidden, rank, window, page = 40, 12, 7, 4
    mixers = [LatentMeanMixer("l0.mix.", hidden, rank), LatentMeanMixer("l1.mix.", hidden, rank, window)]
    blocks = [PreNormBlock(RMSNorm(f"l{i}.n1", hidden, 1e-5), m, RMSNorm(f"l{i}.n2", hidden, 1e-5),
                           GatedMLP(f"l{i}.mlp.", hidden, 56)) for i, m in enumerate(mixers)]
    model = DecoderLM(None, Embedding("emb", 61, hidden), blocks, [PlanEntry(0), PlanEntry(1)],
                      RMSNorm("fn", hidden, 1e-5), Linear(["head"], hidden, [61]), tied_head=False)
    ctx, w = bound(model, dtype, seed=4)
    model.ctx = ctx
    cache = CacheManager(model, page_size=page, num_pages=8, max_requests=2, dtype=dtype, device=ctx.device)
    assert len(cache.groups) == 2 and all(g.kv is None for g in cache.groups)
    assert cache.groups[0].data.shape == (1, 8 + 1, page * rank)

    def whole(ids):
        T = len(ids)
        h = plain.embedding(ids, w["emb"])
        for i, win in enumerate((None, window)):
            c = plain.linear(plain.rms_norm(h, w[f"l{i}.n1"], 1e-5), w[f"l{i}.mix.down"])
            y = torch.stack([c[max(0, t - win + 1) if win else 0 : t + 1].mean(dim=0) for t in range(T)])
            h = h + plain.linear(y, w[f"l{i}.mix.up"])
            h = h + plain.gated_mlp(plain.rms_norm(h, w[f"l{i}.n2"], 1e-5), w[f"l{i}.mlp.gate_proj.weight"],
                                    w[f"l{i}.mlp.up_proj.weight"], w[f"l{i}.mlp.down_proj.weight"])
        return plain.fast_linear(plain.rms_norm(h, w["fn"], 1e-5), w["head"])

    runner = ModelRunner(model, cache)
    assert not runner.use_graphs  # the mixer reads the host's view of the batch
    for seed, cuts in ((1, [9, 1, 1, 6, 1, 9]), (2, [2, 13, 1, 1, 1, 5])):
        ids = random_tokens(sum(cuts), 61, seed)
        want = whole(ids)
        slot, at, got = runner.admit(), 0, []
        for n in cuts:
            got.append(runner.step([StepEntry(slot, ids[at : at + n], list(range(n)))]).cpu())
            at += n
        err = (torch.cat(got).double() - want).abs().max().item()
        assert err < TOL[dtype], (seed, err)
        assert cache.groups[1].pool.num_held <= (window + page - 1) // page + 1  # the window let pages go
        runner.release(slot)
    assert all(g.pool.num_held == 0 for g in cache.groups)


# ---------------------------------------------------------------------------------------
# a mixer with state of its own that decodes through captured graphs
# ---------------------------------------------------------------------------------------
class GraphSafeRunningMean(RunningMeanMixer):
    """The running mean again, from the step's device arrays alone (no host-side view of the
    batch), so that decode steps may be captured and replayed.  Every run of forward() advances
    the state: a capture that ran a request's step more than once would count its token twice."""

    graph_safe = True

    def forward(self, x, step, cache):
        seq = step.token_seq.long()                      # [N] request of each token, within this batch
        rows = step.seq_slots.long()                     # [S] state row of each request (padding: the spare row)
        first = step.cu_tokens.long()[:-1]               # [S] first token of each request
        xf = x.float()
        run = torch.cumsum(xf, dim=0)
        before = torch.cat([torch.zeros_like(run[:1]), run])[first]  # [S, H] sum of the tokens before each request
        state = cache.state[rows]                        # [S, H + 1]
        sums = state[seq, :-1] + run - before[seq]
        index = torch.arange(x.shape[0], device=x.device)
        counts = state[seq, -1] + (index - first[seq] + 1).float()
        last = step.cu_tokens.long()[1:] - 1
        cache.state[rows] = torch.cat([sums[last], counts[last, None]], dim=1)
        return self.ctx.ops.linear((sums / counts[:, None]).to(x.dtype), self.weight)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_mixer_with_state_decodes_through_graphs(dtype):
    """Two requests: prompts in portions, then fifteen single tokens each through captured
    graphs (two batch buckets: the second request ends first), against the running mean computed
    whole and against the same steps without graphs.  The state of a request moves once per step:
    the runs that warm a graph's kernels up before its capture touch the spare state row only."""
    hidden, vocab = 40, 61
    outs = {}
    for use_graphs in (True, False):
        block = PreNormBlock(RMSNorm("l0.n1", hidden, 1e-5), GraphSafeRunningMean("l0.mean.weight", hidden),
                             RMSNorm("l0.n2", hidden, 1e-5), GatedMLP("l0.mlp.", hidden, 56))
        model = one_block_model(block, hidden, vocab)
        ctx, w = bound(model, dtype, seed=6)
        model.ctx = ctx
        cache = CacheManager(model, page_size=16, num_pages=4, max_requests=3, dtype=dtype, device=ctx.device)
        assert cache.states[0].shape == (3 + 1, hidden + 1)  # a spare row for the rows that pad a batch
        runner = ModelRunner(model, cache, use_graphs=use_graphs)
        assert runner.use_graphs == use_graphs
        seqs = [random_tokens(30, vocab, 11), random_tokens(18, vocab, 12)]
        slots = [runner.admit(), runner.admit()]
        got = [[], []]
        got[0].append(runner.step([StepEntry(slots[0], seqs[0][:9], list(range(9)))]))
        out = runner.step([StepEntry(slots[0], seqs[0][9:15], list(range(6))), StepEntry(slots[1], seqs[1][:7], list(range(7)))])
        got[0].append(out[:6])
        got[1].append(out[6:])
        at = [15, 7]
        while at[0] < 30:
            live = [i for i in (0, 1) if at[i] < len(seqs[i])]
            out = runner.step([StepEntry(slots[i], [seqs[i][at[i]]], [0]) for i in live])
            for n, i in enumerate(live):
                got[i].append(out[n : n + 1].clone())
                at[i] += 1
        if use_graphs:
            assert runner.num_captures == 2, "batches of two and of one: two graphs"
        outs[use_graphs] = [torch.cat(g).cpu().double() for g in got]

    def whole(ids):
        T = len(ids)
        x = plain.embedding(ids, w["e.weight"])
        m = torch.cumsum(plain.rms_norm(x, w["l0.n1"], 1e-5), 0) / torch.arange(1, T + 1, dtype=D)[:, None]
        r = x + plain.linear(m, w["l0.mean.weight"])
        r = r + plain.gated_mlp(plain.rms_norm(r, w["l0.n2"], 1e-5), w["l0.mlp.gate_proj.weight"],
                                w["l0.mlp.up_proj.weight"], w["l0.mlp.down_proj.weight"])
        return plain.fast_linear(plain.rms_norm(r, w["fn.weight"], 1e-6), w["head.weight"])

    for i, ids in enumerate(seqs):
        want = whole(ids)
        for use_graphs in (True, False):
            err = (outs[use_graphs][i] - want).abs().max().item()
            assert err < TOL[dtype], (i, use_graphs, err)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("packed", [False, True], ids=["three tensors", "one stacked tensor"])
def test_attention_with_biases_and_other_tensor_names(dtype, packed):
    """The attention mixer with what another architecture's checkpoint may bring: a bias on
    the q/k/v and on the output projection, the three projections stacked in one tensor, norm
    weights under other names.  Parameters of the part, no change to it; stepped in portions
    and single tokens (small steps: the products beside a folded norm run too) against the plain formulas."""
    H, nq, nkv, d, I, T = 64, 4, 2, 32, 96, 17
    p = "blk.attn."
    names = ["Wqkv.weight"] if packed else ["query.weight", "key.weight", "value.weight"]
    mixer = PagedAttention(p, H, nq, nkv, d, RotaryHalfSplit(d, 1e4), qk_norm_eps=1e-5, qkv_names=names, o_name="dense.weight",
                           qkv_bias=True, o_bias=True, qk_norm_names=["ln_q.weight", "ln_k.weight"])
    assert not mixer.folds_norm and mixer.qkv.has_bias and mixer.o.has_bias
    expected = {p + n for n in names} | {p + n[:-6] + "bias" for n in names}
    expected |= {p + "dense.weight", p + "dense.bias", p + "ln_q.weight", p + "ln_k.weight"}
    assert set(mixer.tensor_specs()) == expected
    block = PreNormBlock(RMSNorm("blk.n1", H, 1e-5), mixer, RMSNorm("blk.n2", H, 1e-5), GatedMLP("blk.mlp.", H, I))
    model = one_block_model(block, H)
    ctx, w = bound(model, dtype, seed=3)
    model.ctx = ctx
    cache = CacheManager(model, page_size=16, num_pages=4, max_requests=2, dtype=dtype, device=ctx.device)
    runner = ModelRunner(model, cache)
    ids = random_tokens(T, 50, 8)
    x0 = plain.embedding(ids, w["e.weight"])
    xn = plain.rms_norm(x0, w["blk.n1"], 1e-5)
    if packed:
        qkv = plain.linear(xn, w[p + "Wqkv.weight"]) + w[p + "Wqkv.bias"]
        q, k, v = qkv[:, : nq * d], qkv[:, nq * d : (nq + nkv) * d], qkv[:, (nq + nkv) * d :]
    else:
        q, k, v = (plain.linear(xn, w[p + n + ".weight"]) + w[p + n + ".bias"] for n in ("query", "key", "value"))
    q = plain.rope_half_split(plain.rms_norm(q.reshape(T, nq, d), w[p + "ln_q.weight"], 1e-5), range(T), 1e4)
    k = plain.rope_half_split(plain.rms_norm(k.reshape(T, nkv, d), w[p + "ln_k.weight"], 1e-5), range(T), 1e4)
    a = plain.causal_gqa_attention(q, k, v.reshape(T, nkv, d)).reshape(T, nq * d)
    r = x0 + plain.linear(a, w[p + "dense.weight"]) + w[p + "dense.bias"]
    r = r + plain.gated_mlp(plain.rms_norm(r, w["blk.n2"], 1e-5), w["blk.mlp.gate_proj.weight"],
                            w["blk.mlp.up_proj.weight"], w["blk.mlp.down_proj.weight"])
    want = plain.fast_linear(plain.rms_norm(r, w["fn.weight"], 1e-6), w["head.weight"])
    slot = runner.admit()
    got = torch.cat([runner.step([StepEntry(slot, ids[a0:b0], list(range(b0 - a0)))]).cpu()
                     for a0, b0 in ((0, 9), (9, 10), (10, 11), (11, 17))])
    assert (got.double() - want).abs().max() < TOL[dtype]
