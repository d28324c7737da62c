"""Qwen3 dense: how its configuration becomes parts.

Names of tensors are the checkpoint's (src/model/qwen3.cpp:87-90, :181-187,
:860-876, :1075-1088, :1413-1416).  Each layer is a pre-norm block of paged
GQA attention (per-head q/k RMSNorm, half-split rotary over the whole head)
and a SiLU-gated MLP; one eps serves all four norms
(src/model/qwen3.cpp:160-161, :852-853, :1064).  A tied model may come without
`lm_head.weight` (then the head is the embedding table; the reference refuses
that case, :1413-1423) or with it.
"""
from __future__ import annotations

from ..config.model_config import Qwen3Config
from ..config.registry import register_architecture
from ..parts import Embedding, GatedMLP, Linear, PagedAttention, PreNormBlock, RMSNorm, RotaryHalfSplit
from .decoder import DecoderLM, PlanEntry


def build_qwen3(config: Qwen3Config) -> DecoderLM:
    c = config
    blocks = []
    for i in range(c.num_hidden_layers):
        p = f"model.layers.{i}."
        attention = PagedAttention(
            prefix=p + "self_attn.",
            hidden_size=c.hidden_size,
            num_q_heads=c.num_attention_heads,
            num_kv_heads=c.num_key_value_heads,
            head_dim=c.head_dim,
            position=RotaryHalfSplit(c.head_dim, c.rope_theta),
            qk_norm_eps=c.rms_norm_eps,
            window=c.window_of_layer(i),
        )
        blocks.append(
            PreNormBlock(
                RMSNorm(p + "input_layernorm.weight", c.hidden_size, c.rms_norm_eps),
                attention,
                RMSNorm(p + "post_attention_layernorm.weight", c.hidden_size, c.rms_norm_eps),
                GatedMLP(p + "mlp.", c.hidden_size, c.intermediate_size),
            )
        )
    return DecoderLM(
        config=c,
        embedding=Embedding("model.embed_tokens.weight", c.vocab_size, c.hidden_size),
        blocks=blocks,
        plan=[PlanEntry(i) for i in range(c.num_hidden_layers)],
        final_norm=RMSNorm("model.norm.weight", c.hidden_size, c.rms_norm_eps),
        head=Linear(["lm_head.weight"], c.hidden_size, [c.vocab_size], optional=c.tie_word_embeddings),
        tied_head=c.tie_word_embeddings,
    )


def qwen3_chat_template(user_prompt: str, enable_thinking: bool = False) -> str:
    """One user turn, then the start of the assistant's; with thinking off the empty
    think block is already written (src/tokenizer/qwen3_chat_template.cpp:7-24)."""
    text = "<|im_start|>user\n" + user_prompt + "<|im_end|>\n<|im_start|>assistant\n"
    return text + ("<think>\n" if enable_thinking else "<think>\n\n</think>\n\n")


register_architecture(Qwen3Config.ARCHITECTURE, Qwen3Config, build_qwen3, chat_template=qwen3_chat_template)
