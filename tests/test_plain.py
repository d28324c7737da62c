"""What pins the plain implementation beside the reference's text: vectors the
reference's own tests hold, special cases that reduce to a library routine, and
invariants, each chosen so that a plausible mistake fails it."""
import math

import pytest
import torch

from tests.plain import qwen3_plain as plain
from tests.tiny import CONFIGS, make_model_dir, random_tokens

D = torch.float64


def test_rms_norm_vector_and_library():
    # tests/test_rms_norm.cpp:57-64: rows {1,2,3,4} and {2,0,-2,4}, w {1,1.5,2,0.5}
    x = torch.tensor([[1.0, 2, 3, 4], [2, 0, -2, 4]], dtype=D)
    w = torch.tensor([1.0, 1.5, 2.0, 0.5], dtype=D)
    got = plain.rms_norm(x, w, 1e-6)
    r0 = 1 / math.sqrt(7.5 + 1e-6)
    assert torch.allclose(got[0], torch.tensor([1, 3, 6, 2], dtype=D) * r0)
    assert torch.allclose(got, torch.nn.functional.rms_norm(x, (4,), w, 1e-6))
    # unit weight: the output has RMS 1 (a "1 + w" or mean-subtracting norm fails one of these)
    y = plain.rms_norm(torch.randn(5, 32, dtype=D) + 3.0, torch.ones(32, dtype=D), 0.0)
    assert torch.allclose((y * y).mean(-1), torch.ones(5, dtype=D))


def test_linear_vector():
    # tests/test_linear.cpp:63-78: W is [out, in]
    x = torch.tensor([[1.0, 2, 3], [4, 5, 6]], dtype=D)
    w = torch.tensor([[1.0, 2, 3], [4, 5, 6], [-1, 0, 1], [2, -3, 4]], dtype=D)
    assert torch.equal(plain.linear(x, w), torch.tensor([[14.0, 32, 2, 8], [32, 77, 2, 17]], dtype=D))
    assert torch.allclose(plain.linear(x, w), torch.nn.functional.linear(x, w))


def test_silu_and_mul_vector():
    # tests/test_silu_and_mul.cpp:48-56
    g = torch.tensor([-3.0, -1, 0, 1, 2, 4, 0.5, -0.5], dtype=D)
    u = torch.tensor([1.0, 2, -1, 0.5, 3, -2, 4, -3], dtype=D)
    assert torch.allclose(plain.silu_and_mul(g, u), torch.nn.functional.silu(g) * u)


def test_rope_vector_pairing_and_sign():
    # tests/test_rotary.cpp:98-122: positions {0, 2}, d = 4, theta 1e4
    q = torch.tensor([[[1.0, 2, 3, 4], [-1, 0.5, 2, -0.5]], [[0, 1, -2, 3], [4, -1, 0.25, -0.75]]], dtype=D)
    got = plain.rope_half_split(q, [0, 2], 10000.0)
    assert torch.equal(got[0], q[0])  # position 0 is the identity
    # head 0 of token 1 by hand: pairs (x0, x2) with angle 2 and (x1, x3) with angle 2 * 1e4^(-1/2) = 0.02
    x = q[1, 0]
    c0, s0, c1, s1 = math.cos(2.0), math.sin(2.0), math.cos(0.02), math.sin(0.02)
    want = torch.tensor([x[0] * c0 - x[2] * s0, x[1] * c1 - x[3] * s1, x[2] * c0 + x[0] * s0, x[3] * c1 + x[1] * s1], dtype=D)
    assert torch.allclose(got[1, 0], want)  # interleaved pairing or a flipped sign fails here
    # each pair keeps its norm
    assert torch.allclose(got[1, 0, 0] ** 2 + got[1, 0, 2] ** 2, x[0] ** 2 + x[2] ** 2)


def test_rope_depends_on_distance_only():
    g = torch.Generator().manual_seed(0)
    q = torch.randn(1, 1, 16, generator=g, dtype=D)
    k = torch.randn(1, 1, 16, generator=g, dtype=D)
    dots = []
    for shift in (0, 5, 1000):
        rq = plain.rope_half_split(q, [7 + shift], 1e6)
        rk = plain.rope_half_split(k, [3 + shift], 1e6)
        dots.append((rq * rk).sum())
    assert torch.allclose(dots[0], dots[1]) and torch.allclose(dots[0], dots[2], atol=1e-9)


def test_attention_matches_library_and_special_cases():
    g = torch.Generator().manual_seed(1)
    T, nq, nkv, d = 7, 4, 2, 8
    q, k, v = (torch.randn(T, n, d, generator=g, dtype=D) for n in (nq, nkv, nkv))
    got = plain.causal_gqa_attention(q, k, v)
    # library attention with a causal mask, k/v repeated so that consecutive q heads share a kv head
    kk, vv = k.repeat_interleave(2, dim=1), v.repeat_interleave(2, dim=1)
    want = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1), is_causal=True
    ).transpose(0, 1)
    assert torch.allclose(got, want)
    # a strided head mapping (h % nkv) would differ
    kk2, vv2 = k.repeat(1, 2, 1), v.repeat(1, 2, 1)
    other = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(0, 1), kk2.transpose(0, 1), vv2.transpose(0, 1), is_causal=True
    ).transpose(0, 1)
    assert not torch.allclose(got, other)
    # tests/test_attention.cpp:220-281: a single token returns its value row
    one = plain.causal_gqa_attention(q[:1], k[:1], v[:1])
    assert torch.allclose(one[0], v[0].repeat_interleave(2, dim=0))
    # window 1 = every token sees itself only; a window >= T changes nothing
    assert torch.allclose(plain.causal_gqa_attention(q, k, v, window=1), vv)
    assert torch.allclose(plain.causal_gqa_attention(q, k, v, window=T), got)
    # window 3: token 5 must ignore key 2 however large its score would be
    k_big = k.clone()
    k_big[2] = q[5, :2].mean(0) * 100
    a = plain.causal_gqa_attention(q, k_big, v, window=3)[5]
    b = plain.causal_gqa_attention(q, k, v, window=3)[5]
    assert torch.allclose(a, b)


def test_reference_attention_vector():
    # q, k, v of tests/test_attention.cpp:122-170 (T=3, nq=4, nkv=2, d=4), head 0 of token 1 by hand
    q = torch.tensor([[[1.0, 0, 0.5, -1], [0.5, 1, -0.5, 2], [-1, 0.5, 1.5, 0], [2, -1, 0, 0.5]],
                      [[0, 1, 2, -0.5], [1.5, -0.5, 0, 1], [-0.5, 2, -1, 0.5], [1, 1, 0.5, -1.5]],
                      [[2, -1, 1, 0], [-1, 0, 1, 2], [0.5, -0.5, 2, 1], [1.5, 0.5, -1, 0]]], dtype=D)
    k = torch.tensor([[[1.0, 0, -1, 0.5], [0.5, -0.5, 1, 2]], [[0, 1.5, 0.5, -1], [1, 1, -0.5, 0]],
                      [[-1, 0.5, 2, 1], [0, -1.5, 1.5, 0.5]]], dtype=D)
    v = torch.tensor([[[1.0, 2, 3, 4], [-1, 0.5, 1.5, 2.5]], [[0, -1, 2, -2], [3, 1, -0.5, 0]],
                      [[2, 0, -1, 1], [-2, 2, 0.5, -1.5]]], dtype=D)
    got = plain.causal_gqa_attention(q, k, v)
    s0 = (q[1, 0] * k[0, 0]).sum() / 2.0  # -2.25 / 2
    s1 = (q[1, 0] * k[1, 0]).sum() / 2.0  # 3.0 / 2
    p = torch.softmax(torch.stack([s0, s1]), 0)
    assert torch.allclose(got[1, 0], p[0] * v[0, 0] + p[1] * v[1, 0])
    # head 2 uses kv head 1
    s = torch.stack([(q[2, 2] * k[j, 1]).sum() / 2.0 for j in range(3)])
    p = torch.softmax(s, 0)
    assert torch.allclose(got[2, 2], p[0] * v[0, 1] + p[1] * v[1, 1] + p[2] * v[2, 1])


def reference_tiny_model():
    """Weights of tests/test_qwen3_model.cpp:593-676 (V=5, H=3, nq=2, nkv=1, d=2, I=4, one layer)."""
    t = lambda rows: torch.tensor(rows, dtype=D)
    p = "model.layers.0."
    w = {
        "model.embed_tokens.weight": t([[0.5, -1, 1.5], [1, 0, -0.5], [-1, 2, 0.25], [0, -0.75, 1.25], [2, 1, -1.5]]),
        p + "input_layernorm.weight": t([1.0, 0.75, 1.25]),
        p + "post_attention_layernorm.weight": t([0.8, 1.1, 0.9]),
        p + "self_attn.q_proj.weight": t([[0.5, -1, 0.25], [1, 0, -0.5], [-0.75, 0.5, 1], [2, -1, 0]]),
        p + "self_attn.k_proj.weight": t([[1, 0.5, -1], [-0.5, 1.5, 0.25]]),
        p + "self_attn.v_proj.weight": t([[0.25, -1, 2], [1.5, 0, -0.5]]),
        p + "self_attn.o_proj.weight": t([[1, -0.5, 0.25, 2], [-1, 1.5, 0.5, -0.25], [0, 0.75, -1, 1]]),
        p + "self_attn.q_norm.weight": t([1.0, 1.5]),
        p + "self_attn.k_norm.weight": t([0.75, 1.25]),
        p + "mlp.gate_proj.weight": t([[0.5, -1, 0.25], [1, 0, -0.5], [-0.75, 0.5, 1], [2, -1, 0]]),
        p + "mlp.up_proj.weight": t([[1, 2, -1], [-0.5, 0.25, 1.5], [2, -1, 0.5], [0, 1, -2]]),
        p + "mlp.down_proj.weight": t([[1, -1, 0.5, 2], [0, 1.5, -0.5, 1], [-1, 0.25, 1, -0.75]]),
        "model.norm.weight": t([1.2, 0.9, 1.1]),
        "lm_head.weight": t([[1, 0, 0], [0, 1, 0], [0, 0, 1], [1, 1, 1], [0.5, -0.5, 0]]),
    }
    cfg = dict(num_hidden_layers=1, hidden_size=3, num_attention_heads=2, num_key_value_heads=1, head_dim=2,
               intermediate_size=4, vocab_size=5, rms_norm_eps=1e-6, rope_theta=10000.0, tie_word_embeddings=False)
    return cfg, w


def test_whole_model_first_token_by_hand():
    """ids {2, 0, 3} (tests/test_qwen3_model.cpp:593-599).  The first token sees
    only itself and sits at position 0, so attention returns v and rotation is
    the identity: its logits follow from norms and products alone."""
    cfg, w = reference_tiny_model()
    logits = plain.model_logits([2, 0, 3], w, cfg)
    p = "model.layers.0."
    x = w["model.embed_tokens.weight"][2]
    n = lambda t, wt: t / torch.sqrt((t * t).mean() + 1e-6) * wt
    h = n(x, w[p + "input_layernorm.weight"])
    v = w[p + "self_attn.v_proj.weight"] @ h  # one kv head, both q heads get it
    a = w[p + "self_attn.o_proj.weight"] @ torch.cat([v, v])
    r = x + a
    h2 = n(r, w[p + "post_attention_layernorm.weight"])
    g, u = w[p + "mlp.gate_proj.weight"] @ h2, w[p + "mlp.up_proj.weight"] @ h2
    y = r + w[p + "mlp.down_proj.weight"] @ (torch.nn.functional.silu(g) * u)
    want = w["lm_head.weight"] @ n(y, w["model.norm.weight"])
    assert torch.allclose(logits[0], want)
    # zero projections: logits = lm_head(norm(embed)), tests/test_qwen3_causal_lm.cpp:263-285
    w0 = {k: (torch.zeros_like(t) if "proj" in k else t) for k, t in w.items()}
    z = plain.model_logits([2, 0, 3], w0, cfg)
    e = w["model.embed_tokens.weight"][torch.tensor([2, 0, 3])]
    assert torch.allclose(z, plain.rms_norm(e, w["model.norm.weight"], 1e-6) @ w["lm_head.weight"].t())


def test_qk_norm_comes_before_rotation():
    """Norm then rotate (src/model/qwen3.cpp:406-449).  With a non-uniform norm
    weight the two orders differ, so a swapped order is caught."""
    cfg, w = reference_tiny_model()
    x = torch.tensor([[0.3, -1.2, 0.8], [1.0, 0.5, -0.7]], dtype=D)
    a = plain.attention_block(x, [3, 4], w, "model.layers.0.self_attn.", 2, 1, 2, 1e-6, 1e4)
    # recompute with the other order
    q = plain.linear(x, w["model.layers.0.self_attn.q_proj.weight"]).reshape(2, 2, 2)
    k = plain.linear(x, w["model.layers.0.self_attn.k_proj.weight"]).reshape(2, 1, 2)
    v = plain.linear(x, w["model.layers.0.self_attn.v_proj.weight"]).reshape(2, 1, 2)
    q2 = plain.rms_norm(plain.rope_half_split(q, [3, 4], 1e4), w["model.layers.0.self_attn.q_norm.weight"], 1e-6)
    k2 = plain.rms_norm(plain.rope_half_split(k, [3, 4], 1e4), w["model.layers.0.self_attn.k_norm.weight"], 1e-6)
    b = plain.linear(plain.causal_gqa_attention(q2, k2, v).reshape(2, 4), w["model.layers.0.self_attn.o_proj.weight"])
    assert not torch.allclose(a, b)
    q1 = plain.rope_half_split(plain.rms_norm(q, w["model.layers.0.self_attn.q_norm.weight"], 1e-6), [3, 4], 1e4)
    k1 = plain.rope_half_split(plain.rms_norm(k, w["model.layers.0.self_attn.k_norm.weight"], 1e-6), [3, 4], 1e4)
    c = plain.linear(plain.causal_gqa_attention(q1, k1, v).reshape(2, 4), w["model.layers.0.self_attn.o_proj.weight"])
    assert torch.allclose(a, c)


@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_fast_twin_equals_loop_version(tmp_path, which):
    d = make_model_dir(tmp_path, which)
    cfg, w = plain.read_model_dir(d)
    ids = random_tokens(9 if which != "C" else 26, cfg["vocab_size"], 3)
    slow = plain.model_logits(ids, w, cfg)
    fast = plain.model_logits_fast(ids, w, cfg)
    assert (slow - fast).abs().max() < 1e-10


def test_shift_of_all_positions_changes_nothing(tmp_path):
    d = make_model_dir(tmp_path, "B")
    cfg, w = plain.read_model_dir(d)
    ids = random_tokens(12, cfg["vocab_size"], 4)
    a = plain.model_logits_fast(ids, w, cfg)
    b = plain.model_logits_fast(ids, w, cfg, positions=list(range(100, 112)))
    assert (a - b).abs().max() < 1e-9


def test_greedy_and_temperature_pick():
    # tests/test_argmax.cpp:52-67: ties go to the smaller id
    assert plain.greedy_pick(torch.tensor([1.0, 5.0, 5.0, 2.0])) == 1
    row = torch.log(torch.tensor([0.1, 0.2, 0.3, 0.4]))
    assert [plain.temperature_pick(row, 1.0, u) for u in (0.0, 0.05, 0.1, 0.29, 0.3, 0.59, 0.61, 0.999)] == [0, 0, 1, 1, 2, 2, 3, 3]
    # a low temperature sharpens: p ~ x^4 -> 0.4^4 / sum = 0.72
    assert plain.temperature_pick(row, 0.25, 0.3) == 3


def test_designed_chain_generation():
    """tests/test_generation.cpp:60-66: a model designed so that 0 -> 1 -> 2 -> 4 (eos).
    Built here from one-hot-like weights: zero projections, so the logits are
    lm_head(norm(embed)), and lm_head row t+1 points at embedding row t."""
    V, H = 5, 5
    e = torch.eye(V, H, dtype=D)
    head = torch.zeros(V, H, dtype=D)
    for src, dst in {0: 1, 1: 2, 2: 4, 3: 0, 4: 4}.items():
        head[dst, src] = 1.0
    cfg = dict(num_hidden_layers=1, hidden_size=H, num_attention_heads=1, num_key_value_heads=1, head_dim=2,
               intermediate_size=2, vocab_size=V, rms_norm_eps=1e-6, rope_theta=1e4, tie_word_embeddings=False)
    p = "model.layers.0."
    z = lambda *s: torch.zeros(*s, dtype=D)
    w = {"model.embed_tokens.weight": e, "lm_head.weight": head, "model.norm.weight": torch.ones(H, dtype=D),
         p + "input_layernorm.weight": torch.ones(H, dtype=D), p + "post_attention_layernorm.weight": torch.ones(H, dtype=D),
         p + "self_attn.q_proj.weight": z(2, H), p + "self_attn.k_proj.weight": z(2, H), p + "self_attn.v_proj.weight": z(2, H),
         p + "self_attn.o_proj.weight": z(H, 2), p + "self_attn.q_norm.weight": torch.ones(2, dtype=D),
         p + "self_attn.k_norm.weight": torch.ones(2, dtype=D), p + "mlp.gate_proj.weight": z(2, H),
         p + "mlp.up_proj.weight": z(2, H), p + "mlp.down_proj.weight": z(H, 2)}
    assert plain.generate_greedy([0], w, cfg, 8, eos=4) == [1, 2, 4]  # eos is appended, then it stops
    assert plain.generate_greedy([0], w, cfg, 2, eos=4) == [1, 2]
