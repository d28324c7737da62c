"""Configurations drawn at random, every size within what config.json allows: head sizes in
steps of 16 up to 256, one to three kv heads, groups of 1 to 16, widths and feed-forward widths
that are multiples of 8, of 4 or of 2 only, odd vocabularies, windows on some layers, pages of 1
to 64 tokens.  Each goes through the replay loop of bin/trace_run (in this process) in all four
ways of cutting, with a pool so small that pages are used again, and every row is compared with
the plain implementation: float32 always (with the attention sharpened for some, so that a key
that is lost or read from a wrong page moves the logits), bfloat16 where the attention is not
sharpened (sharpened, the type's own rounding reaches 0.07 of the largest logit in whole prompts
and token by token alike)."""
import io
import random

import pytest
import torch

from tests.tiny import random_tokens, sharpen_attention
from tests.trace_util import (TraceBuilder, changing_portions, check_dumps, mixed, plain_logits, tail_one_by_one,
                              whole)

pytestmark = pytest.mark.gpu

# float32: about five times the worst error seen over 240 such draws (1.8e-6, sharpened 1.0e-5);
# bfloat16: the tolerance of the fixed configurations' traces (the worst of those draws was 8.9e-3)
TOL = {"float32": 1e-5, "float32 sharpened": 5e-5, "bfloat16": 2e-2}


def draw(seed: int):
    rng = random.Random(seed)
    d = rng.choice([16, 32, 48, 64, 80, 96, 128, 160, 256])
    nkv = rng.choice([1, 2, 3])
    group = rng.choice([1, 2, 3, 4, 5, 8, 16])
    if d * nkv * group > 4096:
        group = max(1, 4096 // (d * nkv))
    layers = rng.choice([1, 2, 3])
    spec = dict(
        architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=layers,
        hidden_size=rng.choice([40, 64, 70, 72, 96, 102, 136, 200, 264]), num_attention_heads=nkv * group,
        num_key_value_heads=nkv, head_dim=d, intermediate_size=rng.choice([36, 72, 76, 100, 136, 168, 200]),
        vocab_size=rng.choice([50, 97, 256, 311, 1001]), rope_theta=rng.choice([1e4, 5e5, 1e6]),
        rms_norm_eps=rng.choice([1e-6, 1e-5, 3e-6]), tie_word_embeddings=rng.random() < 0.5,
    )
    window = rng.choice([None, None, 9, 20, 33, 64])
    if window:
        spec["sliding_window"] = window
        spec["layer_types"] = [rng.choice(["sliding_attention", "full_attention"]) for _ in range(layers)]
        if "sliding_attention" not in spec["layer_types"]:
            spec["layer_types"][0] = "sliding_attention"
    page = rng.choice([1, 3, 4, 8, 16, 16, 32, 48, 64])
    sharp = rng.random() < 0.4
    lengths = {r: rng.randint(20, 130) for r in "abcdef"}
    return spec, page, sharp, lengths


@pytest.mark.parametrize("seed", range(1000, 1024))
def test_a_configuration_drawn_at_random(tmp_path, seed):
    from litellmengine_amd.config import Qwen3Config
    from litellmengine_amd.entrypoints.trace_run import replay
    from litellmengine_amd.models import load_model
    from litellmengine_amd.weights import write_model_dir

    spec, page, sharp, lengths = draw(seed)
    cfg = Qwen3Config.from_dict(spec)
    model_dir = str(tmp_path / "model")
    write_model_dir(cfg, model_dir, seed, torch.bfloat16)
    if sharp:
        sharpen_attention(model_dir, 2.0)
    requests = {r: random_tokens(n, cfg.vocab_size, seed * 10 + i) for i, (r, n) in enumerate(lengths.items())}
    tb = TraceBuilder()
    whole(tb, "a#whole", requests["a"])
    tail_one_by_one(tb, "b#tail", requests["b"], tail=min(32, lengths["b"] - 2))
    changing_portions(tb, "c#cut", requests["c"], seed=seed)
    mixed(tb, {r + "#mix": t for r, t in requests.items()}, seed=seed)
    want = plain_logits(model_dir, requests)
    # the pool: what the live requests hold at most, each rounded up to whole pages
    pool = -(-tb.max_tokens // page) * page + 4 * page
    said = f"seed {seed}: {spec}, pages of {page}, sharpened {sharp}:"
    for dtype in ("float32", "bfloat16"):
        if sharp and dtype == "bfloat16":
            continue
        out = str(tmp_path / dtype)
        model = load_model(model_dir, dtype, device="cuda:0")
        replay(model, out, pool, page, 16, io.StringIO(tb.text()), io.StringIO())
        worst = check_dumps(out, tb, want, TOL[dtype + " sharpened" if sharp else dtype])
        said += f" {dtype} {worst:.2e}"
    print(said)
