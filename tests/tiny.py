"""Tiny Qwen3 configurations for the tests.  Between them every size and option
differs: layers, width, head counts and group size, head size (q width equal to
the width or not), feed-forward width, vocabulary (a power of two or odd),
rotary base, eps, tied or untied head, all-keys layers or layers with a window."""
from __future__ import annotations

import os

import torch

from litellmengine_amd.config import Qwen3Config
from litellmengine_amd.weights import write_model_dir

TINY_A = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=2, hidden_size=64,
    num_attention_heads=4, num_key_value_heads=2, head_dim=16, intermediate_size=128, vocab_size=256,
    rope_theta=10000.0, rms_norm_eps=1e-6, tie_word_embeddings=True,
)
TINY_B = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=3, hidden_size=96,
    num_attention_heads=8, num_key_value_heads=2, head_dim=32, intermediate_size=200, vocab_size=503,
    rope_theta=1000000.0, rms_norm_eps=1e-5, tie_word_embeddings=False,
)
# layers with a window beside layers that see everything: two cache groups
TINY_C = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=4, hidden_size=80,
    num_attention_heads=6, num_key_value_heads=3, head_dim=48, intermediate_size=136, vocab_size=311,
    rope_theta=500000.0, rms_norm_eps=3e-6, tie_word_embeddings=False, sliding_window=20,
    layer_types=["sliding_attention", "full_attention", "sliding_attention", "sliding_attention"],
)
# heads of 64 and a width that is a multiple of 8: in bfloat16 the small steps of this one take the
# fused paths of decoding (norm folded into the products, q/k norm + rotation + cache write inside
# the attention launch), which the sizes above never reach; a window on one layer
TINY_D = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=3, hidden_size=136,
    num_attention_heads=4, num_key_value_heads=2, head_dim=64, intermediate_size=168, vocab_size=419,
    rope_theta=250000.0, rms_norm_eps=2e-6, tie_word_embeddings=True, sliding_window=33,
    layer_types=["full_attention", "sliding_attention", "full_attention"],
)
CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D}
PAGE_SIZES = {"A": 4, "B": 8, "C": 16, "D": 16}


def make_model_dir(tmp_path, which: str, seed: int = 1234, dtype=torch.float32) -> str:
    cfg = Qwen3Config.from_dict(CONFIGS[which])
    path = os.path.join(str(tmp_path), f"tiny_{which}_{seed}")
    write_model_dir(cfg, path, seed, dtype)
    return path


def sharpen_attention(model_dir: str, factor: float) -> None:
    """Multiply the q and k norm weights of a model folder by `factor`: scores grow by
    factor^2, so every query picks out one or two keys, near or far, instead of averaging
    all of them.  A key that is lost, doubled or read from the wrong page then moves the
    logits by far more than rounding does."""
    from safetensors.torch import load_file, save_file

    path = os.path.join(model_dir, "model.safetensors")
    tensors = load_file(path)
    for name in tensors:
        if name.endswith("q_norm.weight") or name.endswith("k_norm.weight"):
            tensors[name] = (tensors[name].float() * factor).to(tensors[name].dtype)
    save_file(tensors, path, metadata={"format": "pt"})


def random_tokens(n: int, vocab: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
