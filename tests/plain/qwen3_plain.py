"""Plain, slow Qwen3 dense implementation: the oracle of the test-suite.

Whole sequences, no cache, one function per part, nothing shared with the
engine's code.  Every formula is read from the reference's sources (paths are
relative to the reference checkout) and cited next to the function that
implements it.  Everything runs on the CPU in the dtype handed in (float64 by
default, so that a 32-bit engine can be measured against something tighter).
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Sequence

import torch


# --------------------------------------------------------------------------
# parts
# --------------------------------------------------------------------------
def embedding(ids: Sequence[int], table: torch.Tensor) -> torch.Tensor:
    """out[t, :] = table[ids[t], :]; an id outside [0, V) is an error.

    src/layers/embedding.cu:75-87
    """
    vocab = table.shape[0]
    for i in ids:
        if i < 0 or i >= vocab:
            raise ValueError(f"token id {i} outside [0, {vocab})")
    return torch.stack([table[int(i)] for i in ids])


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """y = x * (1 / sqrt(mean(x^2) + eps)) * w over the last axis.

    The weight multiplies directly (no 1 + w), no bias, no mean subtraction.
    src/layers/rms_norm.cu:81-93
    """
    n = x.shape[-1]
    sum_sq = (x * x).sum(dim=-1, keepdim=True)
    inv_rms = 1.0 / torch.sqrt(sum_sq / n + eps)
    return x * inv_rms * weight


def linear(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """y[m, o] = sum_i x[m, i] * W[o, i]; W is [out, in] row-major, no bias in Qwen3.

    src/layers/linear.cu:91-123 (CPU loop), src/model/qwen3.cpp:375-377
    """
    out = torch.zeros(x.shape[0], weight.shape[0], dtype=x.dtype)
    for o in range(weight.shape[0]):
        out[:, o] = (x * weight[o]).sum(dim=-1)
    return out


def rope_half_split(x: torch.Tensor, positions: Sequence[int], theta: float) -> torch.Tensor:
    """Rotary position encoding, half-split pairing, on x [T, heads, d].

    inv_freq_i = theta ** (-2 i / d), angle = pos * inv_freq_i, and for i < d/2
      y[i]       = x[i] * cos - x[i + d/2] * sin
      y[i + d/2] = x[i + d/2] * cos + x[i] * sin
    src/layers/rotary.cu:81-83 (frequency), :96-116 (pairing and signs)
    """
    T, heads, d = x.shape
    if d % 2:
        raise ValueError("head_dim must be even")  # src/layers/rotary.cu:249-251
    half = d // 2
    y = torch.empty_like(x)
    for t in range(T):
        pos = float(positions[t])
        for i in range(half):
            inv_freq = theta ** (-(2.0 * i) / d)
            ang = pos * inv_freq
            c, s = math.cos(ang), math.sin(ang)
            x1 = x[t, :, i]
            x2 = x[t, :, i + half]
            y[t, :, i] = x1 * c - x2 * s
            y[t, :, i + half] = x2 * c + x1 * s
    return y


def causal_gqa_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    window: Optional[int] = None,
) -> torch.Tensor:
    """Causal grouped-query attention over one whole sequence.

    q [T, nq, d], k and v [T, nkv, d] -> [T, nq, d].  kv head of q head h is
    h // (nq // nkv) (consecutive q heads share one kv head); scores are
    (q . k_j) / sqrt(d); query t sees keys j <= t; softmax over those keys.
    src/ops/attention.cu:204-248 (the streamed form there equals this two-pass one)

    `window` has no counterpart in the reference (it knows full attention only):
    with a window w, query t sees keys t - w < j <= t, i.e. itself and the w - 1
    keys before it.
    """
    T, nq, d = q.shape
    nkv = k.shape[1]
    group = nq // nkv
    scale = 1.0 / math.sqrt(d)
    out = torch.zeros_like(q)
    for t in range(T):
        lo = 0 if window is None else max(0, t - window + 1)
        for h in range(nq):
            kvh = h // group
            scores = torch.stack([(q[t, h] * k[j, kvh]).sum() * scale for j in range(lo, t + 1)])
            m = scores.max()
            p = torch.exp(scores - m)
            p = p / p.sum()
            acc = torch.zeros(d, dtype=q.dtype)
            for n, j in enumerate(range(lo, t + 1)):
                acc = acc + p[n] * v[j, kvh]
            out[t, h] = acc
    return out


def silu_and_mul(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """act = gate / (1 + exp(-gate)) * up.   src/ops/silu_and_mul.cu:44-46,76-79"""
    return gate / (1.0 + torch.exp(-gate)) * up


def gated_mlp(x, w_gate, w_up, w_down) -> torch.Tensor:
    """down(silu(gate(x)) * up(x)), no biases.   src/model/qwen3.cpp:143-152"""
    return linear(silu_and_mul(linear(x, w_gate), linear(x, w_up)), w_down)


def attention_block(
    x: torch.Tensor,
    positions: Sequence[int],
    w: Dict[str, torch.Tensor],
    prefix: str,
    nq: int,
    nkv: int,
    d: int,
    eps: float,
    theta: float,
    window: Optional[int] = None,
) -> torch.Tensor:
    """q/k/v projections -> per-head RMSNorm of q and k over d (one weight [d]
    for all heads, before the rotation; v untouched) -> rotation of q and k ->
    attention -> output projection.

    src/model/qwen3.cpp:375-377 (projections), :391-407 (q_norm/k_norm on
    [T*heads, d]), :443-449 (rotation), :498-557 (attention), :565-567 (o_proj)
    """
    T = x.shape[0]
    q = linear(x, w[prefix + "q_proj.weight"]).reshape(T, nq, d)
    k = linear(x, w[prefix + "k_proj.weight"]).reshape(T, nkv, d)
    v = linear(x, w[prefix + "v_proj.weight"]).reshape(T, nkv, d)
    q = rms_norm(q, w[prefix + "q_norm.weight"], eps)
    k = rms_norm(k, w[prefix + "k_norm.weight"], eps)
    q = rope_half_split(q, positions, theta)
    k = rope_half_split(k, positions, theta)
    a = causal_gqa_attention(q, k, v, window)
    return linear(a.reshape(T, nq * d), w[prefix + "o_proj.weight"])


def decoder_layer(x, positions, w, i, cfg, window=None) -> torch.Tensor:
    """Pre-norm residual block: r = x + Attn(norm_in(x)); y = r + MLP(norm_post(r)).

    src/model/qwen3.cpp:948-968
    """
    p = f"model.layers.{i}."
    eps = cfg["rms_norm_eps"]
    a = attention_block(
        rms_norm(x, w[p + "input_layernorm.weight"], eps),
        positions,
        w,
        p + "self_attn.",
        cfg["num_attention_heads"],
        cfg["num_key_value_heads"],
        cfg["head_dim"],
        eps,
        cfg["rope_theta"],
        window,
    )
    r = x + a
    m = gated_mlp(
        rms_norm(r, w[p + "post_attention_layernorm.weight"], eps),
        w[p + "mlp.gate_proj.weight"],
        w[p + "mlp.up_proj.weight"],
        w[p + "mlp.down_proj.weight"],
    )
    return r + m


def layer_windows(cfg: dict) -> List[Optional[int]]:
    """Per-layer window from `layer_types` + `sliding_window` (config.json keys;
    the reference reads neither, so every layer there is full attention)."""
    n = cfg["num_hidden_layers"]
    types = cfg.get("layer_types") or ["full_attention"] * n
    return [cfg.get("sliding_window") if t == "sliding_attention" else None for t in types]


def model_logits(ids: Sequence[int], w: Dict[str, torch.Tensor], cfg: dict) -> torch.Tensor:
    """Logits [T, V] of one whole sequence, positions 0..T-1.

    embed -> layers -> final norm -> lm_head on every row, no bias or scaling.
    src/model/qwen3.cpp:1242-1278 (model), :1501 (head).  A tied model without
    lm_head.weight uses the embedding table (the reference refuses that case,
    src/model/qwen3.cpp:1413-1423).
    """
    positions = list(range(len(ids)))
    h = embedding(ids, w["model.embed_tokens.weight"])
    windows = layer_windows(cfg)
    for i in range(cfg["num_hidden_layers"]):
        h = decoder_layer(h, positions, w, i, cfg, windows[i])
    h = rms_norm(h, w["model.norm.weight"], cfg["rms_norm_eps"])
    head = w.get("lm_head.weight")
    if head is None:
        if not cfg.get("tie_word_embeddings", False):
            raise KeyError("lm_head.weight")
        head = w["model.embed_tokens.weight"]
    return fast_linear(h, head)


def fast_linear(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """Same product as `linear`, by the library (used where the loop is too slow)."""
    return x @ weight.t()


# --------------------------------------------------------------------------
# picking tokens
# --------------------------------------------------------------------------
def greedy_pick(logits_row: torch.Tensor) -> int:
    """First maximum wins.   src/ops/argmax.cu:49-59"""
    best, best_v = 0, float(logits_row[0])
    for i in range(1, logits_row.shape[0]):
        v = float(logits_row[i])
        if v > best_v:
            best, best_v = i, v
    return best


def temperature_pick(logits_row: torch.Tensor, temperature: float, u: float) -> int:
    """p = softmax(logits / T); the pick is the first id whose running sum of p
    exceeds u * sum(p), the last id with p > 0 if rounding leaves none.  (The
    reference parses --temperature and then only warns, src/main.cpp:175-178;
    this rule is this engine's own.)"""
    z = logits_row.double() / temperature
    p = torch.exp(z - z.max())
    cdf = torch.cumsum(p, 0)
    target = u * float(cdf[-1])
    idx = int(torch.searchsorted(cdf, torch.tensor(target, dtype=cdf.dtype), right=True))
    return min(idx, logits_row.shape[0] - 1)


# --------------------------------------------------------------------------
# reading a model folder (own reader: json + safetensors, no engine code)
# --------------------------------------------------------------------------
def read_model_dir(path: str, dtype=torch.float64):
    from safetensors import safe_open

    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    cfg.setdefault("num_key_value_heads", cfg["num_attention_heads"])
    cfg.setdefault("head_dim", cfg["hidden_size"] // cfg["num_attention_heads"])
    cfg.setdefault("rms_norm_eps", 1e-6)  # src/model/model_config.cpp:71-75
    cfg.setdefault("rope_theta", 10000.0)  # src/model/model_config.cpp:77-81
    w = {}
    with safe_open(os.path.join(path, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            w[name] = f.get_tensor(name).to(dtype)
    return cfg, w


def generate_greedy(ids: Sequence[int], w, cfg, max_new: int, eos: int = -1) -> List[int]:
    """Full recompute each step; EOS is appended and then ends the request
    (src/engine/request_manager.cpp:140-155)."""
    seq = list(ids)
    new: List[int] = []
    while len(new) < max_new:
        tok = greedy_pick(model_logits_fast(seq, w, cfg)[-1])
        seq.append(tok)
        new.append(tok)
        if eos >= 0 and tok == eos:
            break
    return new


# --------------------------------------------------------------------------
# a vectorised twin of model_logits (same formulas, library products) used for
# long sequences; test_plain.py checks it against the loop version above
# --------------------------------------------------------------------------
def _rope_fast(x, positions, theta, float32_angles=False):
    """`float32_angles`: the angle as the reference forms it, a float32 product of the position and
    a float32 frequency (src/layers/rotary.cu:81-83, :96-99).  At position p that product is off by
    up to p * 2^-24 radians from the exact angle, which far into a long sequence is more than all
    other rounding of a float32 run together; tests at thousands of positions compare like with like."""
    T, heads, d = x.shape
    half = d // 2
    i = torch.arange(half, dtype=torch.float64)
    inv_freq = theta ** (-(2.0 * i) / d)
    if float32_angles:
        ang = (torch.tensor(list(positions), dtype=torch.float32)[:, None] * inv_freq.float()[None, :]).double()
    else:
        ang = torch.tensor(list(positions), dtype=torch.float64)[:, None] * inv_freq[None, :]
    c = torch.cos(ang).to(x.dtype)[:, None, :]
    s = torch.sin(ang).to(x.dtype)[:, None, :]
    x1, x2 = x[..., :half], x[..., half:]
    return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], dim=-1)


def _attention_fast(q, k, v, window):
    T, nq, d = q.shape
    nkv = k.shape[1]
    group = nq // nkv
    k = k.repeat_interleave(group, dim=1)
    v = v.repeat_interleave(group, dim=1)
    scores = torch.einsum("thd,shd->hts", q, k) / math.sqrt(d)
    t = torch.arange(T)
    allowed = t[None, :] <= t[:, None]
    if window is not None:
        allowed = allowed & (t[None, :] > t[:, None] - window)
    scores = scores.masked_fill(~allowed[None], float("-inf"))
    p = torch.softmax(scores, dim=-1)
    return torch.einsum("hts,shd->thd", p, v)


def first_layer_attention_probs(ids, w, cfg) -> torch.Tensor:
    """Softmax weights [nq, T, T] of the first layer (tests use it to see how peaked
    the attention of a model is)."""
    T = len(ids)
    nq, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    eps, theta = cfg["rms_norm_eps"], cfg["rope_theta"]
    p = "model.layers.0."
    h = w["model.embed_tokens.weight"][torch.tensor(list(ids), dtype=torch.long)]
    x = rms_norm(h, w[p + "input_layernorm.weight"], eps)
    q = fast_linear(x, w[p + "self_attn.q_proj.weight"]).reshape(T, nq, d)
    k = fast_linear(x, w[p + "self_attn.k_proj.weight"]).reshape(T, nkv, d)
    q = _rope_fast(rms_norm(q, w[p + "self_attn.q_norm.weight"], eps), range(T), theta)
    k = _rope_fast(rms_norm(k, w[p + "self_attn.k_norm.weight"], eps), range(T), theta)
    k = k.repeat_interleave(nq // nkv, dim=1)
    scores = torch.einsum("thd,shd->hts", q, k) / math.sqrt(d)
    t = torch.arange(T)
    allowed = t[None, :] <= t[:, None]
    window = layer_windows(cfg)[0]
    if window is not None:
        allowed = allowed & (t[None, :] > t[:, None] - window)
    return torch.softmax(scores.masked_fill(~allowed[None], float("-inf")), dim=-1)


def model_logits_fast(ids, w, cfg, positions=None, rows=None, float32_angles=False) -> torch.Tensor:
    """`rows`: only these positions go through the final norm and the head (long sequences,
    wide vocabularies); the result then has one row for each of them, in their order.
    `float32_angles`: see _rope_fast."""
    T = len(ids)
    positions = list(range(T)) if positions is None else positions
    nq, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    eps, theta = cfg["rms_norm_eps"], cfg["rope_theta"]
    h = w["model.embed_tokens.weight"][torch.tensor(list(ids), dtype=torch.long)]
    windows = layer_windows(cfg)
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        x = rms_norm(h, w[p + "input_layernorm.weight"], eps)
        q = fast_linear(x, w[p + "self_attn.q_proj.weight"]).reshape(T, nq, d)
        k = fast_linear(x, w[p + "self_attn.k_proj.weight"]).reshape(T, nkv, d)
        v = fast_linear(x, w[p + "self_attn.v_proj.weight"]).reshape(T, nkv, d)
        q = _rope_fast(rms_norm(q, w[p + "self_attn.q_norm.weight"], eps), positions, theta, float32_angles)
        k = _rope_fast(rms_norm(k, w[p + "self_attn.k_norm.weight"], eps), positions, theta, float32_angles)
        a = _attention_fast(q, k, v, windows[i]).reshape(T, nq * d)
        h = h + fast_linear(a, w[p + "self_attn.o_proj.weight"])
        x = rms_norm(h, w[p + "post_attention_layernorm.weight"], eps)
        g = fast_linear(x, w[p + "mlp.gate_proj.weight"])
        u = fast_linear(x, w[p + "mlp.up_proj.weight"])
        h = h + fast_linear(silu_and_mul(g, u), w[p + "mlp.down_proj.weight"])
    if rows is not None:
        h = h[torch.tensor(list(rows), dtype=torch.long)]
    h = rms_norm(h, w["model.norm.weight"], eps)
    head = w.get("lm_head.weight")
    if head is None:
        if not cfg.get("tie_word_embeddings", False):
            raise KeyError("lm_head.weight")
        head = w["model.embed_tokens.weight"]
    return fast_linear(h, head)
