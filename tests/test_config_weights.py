"""Configuration, registry and weight loading (CPU)."""
import json
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

from litellmengine_amd.config import ConfigError, Qwen3Config, get_architecture, load_config, registered_architectures
from litellmengine_amd.models import expected_tensors, load_model
from litellmengine_amd.weights import WeightError, checkpoint_header, load_checkpoint, write_model_dir
from tests.tiny import CONFIGS, make_model_dir
from tests.torch_ops import TorchOps


def test_defaults_follow_the_reference():
    # src/model/model_config.cpp:45-87
    c = Qwen3Config.from_dict(dict(architectures=["Qwen3ForCausalLM"], vocab_size=10, hidden_size=32,
                                   intermediate_size=64, num_hidden_layers=2, num_attention_heads=4))
    assert c.num_key_value_heads == 4 and c.head_dim == 8
    assert c.rms_norm_eps == 1e-6 and c.rope_theta == 10000.0
    assert c.tie_word_embeddings is False and c.max_position_embeddings == 32768
    assert c.layer_types == ("full_attention",) * 2 and c.sliding_window is None


def test_explicit_head_dim_and_round_trip():
    c = Qwen3Config.from_dict(CONFIGS["B"])
    assert c.head_dim == 32 and c.num_attention_heads * c.head_dim != c.hidden_size
    assert Qwen3Config.from_dict(c.to_dict()) == c
    c3 = Qwen3Config.from_dict(CONFIGS["C"])
    assert c3.window_of_layer(0) == 20 and c3.window_of_layer(1) is None
    assert Qwen3Config.from_dict(c3.to_dict()) == c3


@pytest.mark.parametrize("change,word", [
    (dict(vocab_size=0), "vocab_size"), (dict(num_key_value_heads=3), "divisible"), (dict(rms_norm_eps=0.0), "rms_norm_eps"),
    (dict(rope_theta=-1.0), "rope_theta"), (dict(head_dim=15), "even"), (dict(attention_bias=True), "attention_bias"),
    (dict(hidden_act="gelu"), "hidden_act"), (dict(layer_types=["full_attention"]), "layer_types"),
    (dict(layer_types=["sliding_attention"] * 3), "sliding_window"), (dict(hidden_size="96"), "integer"),
    (dict(rope_scaling={"type": "yarn"}), "rope_scaling"),
])
def test_bad_configs_are_refused(change, word):
    d = dict(CONFIGS["B"])
    d.update(change)
    with pytest.raises(ConfigError, match=word):
        Qwen3Config.from_dict(d)


def test_missing_field_names_the_field():
    d = dict(CONFIGS["A"])
    del d["intermediate_size"]
    with pytest.raises(ConfigError, match="Missing required config field: intermediate_size"):
        Qwen3Config.from_dict(d)


def test_registry(tmp_path):
    assert "Qwen3ForCausalLM" in registered_architectures()
    with pytest.raises(ConfigError, match="unknown architecture 'LlamaForCausalLM'.*Qwen3ForCausalLM"):
        get_architecture("LlamaForCausalLM")
    d = make_model_dir(tmp_path, "A")
    assert isinstance(load_config(d), Qwen3Config)
    with open(os.path.join(d, "config.json")) as f:
        cfg = json.load(f)
    del cfg["architectures"]
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    with pytest.raises(ConfigError, match="architectures"):
        load_config(d)
    with pytest.raises(ConfigError, match="Failed to open config file"):
        load_config(str(tmp_path / "nowhere"))


def test_tensor_names_and_count():
    # 11 tensors per layer + embed + norm (+ lm_head when untied); 311 for 28 layers with a head,
    # tests/test_real_qwen3_weight_loading.cpp:88
    arch = get_architecture("Qwen3ForCausalLM")
    specs = expected_tensors(arch, Qwen3Config.from_dict(CONFIGS["B"]))
    assert len(specs) == 11 * 3 + 3
    assert specs["model.layers.2.self_attn.q_proj.weight"].shape == (256, 96)
    assert specs["model.layers.0.self_attn.k_norm.weight"].shape == (32,)
    assert specs["model.layers.1.mlp.down_proj.weight"].shape == (96, 200)
    assert specs["lm_head.weight"].shape == (503, 96) and not specs["lm_head.weight"].optional
    tied = expected_tensors(arch, Qwen3Config.from_dict(CONFIGS["A"]))
    assert tied["lm_head.weight"].optional


def test_random_weights_are_seeded_and_distributed(tmp_path):
    a = load_file(os.path.join(make_model_dir(tmp_path, "B", seed=5), "model.safetensors"))
    b = load_file(os.path.join(make_model_dir(tmp_path / "again", "B", seed=5), "model.safetensors"))
    c = load_file(os.path.join(make_model_dir(tmp_path, "B", seed=6), "model.safetensors"))
    assert all(torch.equal(a[k], b[k]) for k in a)
    assert not torch.equal(a["model.embed_tokens.weight"], c["model.embed_tokens.weight"])
    e = a["model.embed_tokens.weight"]
    assert abs(e.std().item() - 0.02) < 0.002 and abs(e.mean().item()) < 0.002
    n = a["model.layers.0.input_layernorm.weight"]
    assert n.min() >= 0.9 and n.max() <= 1.1 and n.std() > 0.02
    assert "lm_head.weight" in a
    tied = load_file(os.path.join(make_model_dir(tmp_path, "A"), "model.safetensors"))
    assert "lm_head.weight" not in tied


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    d = make_model_dir(tmp_path, "A")
    path = os.path.join(d, "model.safetensors")
    t = load_file(path)
    del t["model.layers.1.mlp.up_proj.weight"]
    del t["model.norm.weight"]
    t["model.layers.0.self_attn.q_proj.bias"] = torch.zeros(64)
    t["model.layers.0.self_attn.k_norm.weight"] = torch.ones(8)
    t["model.layers.0.mlp.gate_proj.weight"] = torch.zeros(128, 64, dtype=torch.int32)
    save_file(t, path)
    with pytest.raises(WeightError) as e:
        load_model(d, "float32", device="cpu", ops=TorchOps())
    msg = str(e.value)
    assert "missing tensors (2): model.layers.1.mlp.up_proj.weight, model.norm.weight" in msg
    assert "unexpected tensors (1): model.layers.0.self_attn.q_proj.bias" in msg
    assert "model.layers.0.self_attn.k_norm.weight: stored [8], model wants [16]" in msg
    assert "model.layers.0.mlp.gate_proj.weight: stored as I32" in msg


def test_untied_model_needs_its_head_and_tied_takes_either(tmp_path):
    d = make_model_dir(tmp_path, "B")
    path = os.path.join(d, "model.safetensors")
    t = load_file(path)
    del t["lm_head.weight"]
    save_file(t, path)
    with pytest.raises(WeightError, match="missing tensors \\(1\\): lm_head.weight"):
        load_model(d, "float32", device="cpu", ops=TorchOps())
    d = make_model_dir(tmp_path, "A")
    m = load_model(d, "float32", device="cpu", ops=TorchOps())
    assert m.head.weight is m.embedding.weight
    path = os.path.join(d, "model.safetensors")
    t = load_file(path)
    t["lm_head.weight"] = torch.randn(256, 64)
    save_file(t, path)
    m = load_model(d, "float32", device="cpu", ops=TorchOps())
    assert torch.equal(m.head.weight, t["lm_head.weight"])


def test_storage_types(tmp_path):
    d = make_model_dir(tmp_path, "A", dtype=torch.bfloat16)
    path = os.path.join(d, "model.safetensors")
    t = load_file(path)
    t["model.norm.weight"] = t["model.norm.weight"].float()  # stored in 32-bit: stays so
    t["model.layers.0.mlp.up_proj.weight"] = t["model.layers.0.mlp.up_proj.weight"].half()
    save_file(t, path)
    specs = expected_tensors(get_architecture("Qwen3ForCausalLM"), load_config(d))
    w = load_checkpoint(d, specs, torch.bfloat16, "cpu")
    assert w["model.norm.weight"].dtype == torch.float32
    assert w["model.layers.0.mlp.up_proj.weight"].dtype == torch.bfloat16
    assert w["model.embed_tokens.weight"].dtype == torch.bfloat16
    w32 = load_checkpoint(d, specs, torch.float32, "cpu")
    assert all(x.dtype == torch.float32 for x in w32.values())


def test_sharded_checkpoint(tmp_path):
    d = make_model_dir(tmp_path, "A")
    path = os.path.join(d, "model.safetensors")
    t = load_file(path)
    names = sorted(t)
    half = len(names) // 2
    save_file({n: t[n] for n in names[:half]}, os.path.join(d, "model-00001-of-00002.safetensors"))
    save_file({n: t[n] for n in names[half:]}, os.path.join(d, "model-00002-of-00002.safetensors"))
    os.unlink(path)
    wm = {n: "model-00001-of-00002.safetensors" for n in names[:half]}
    wm.update({n: "model-00002-of-00002.safetensors" for n in names[half:]})
    with open(os.path.join(d, "model.safetensors.index.json"), "w") as f:
        json.dump({"weight_map": wm}, f)
    assert set(checkpoint_header(d)) == set(names)
    os.unlink(os.path.join(d, "model-00002-of-00002.safetensors"))
    with pytest.raises(WeightError, match="shard files that do not exist"):
        checkpoint_header(d)


def test_sizes_that_no_kernel_takes_are_refused_when_the_model_is_built():
    """src/model/qwen3.cpp:19-75 validates at construction; so does the builder here: a head the
    attention kernels cannot hold is refused before any weight is read, naming the key."""
    import pytest

    from litellmengine_amd.config import ConfigError, Qwen3Config
    from litellmengine_amd.config.registry import get_architecture
    from tests.tiny import TINY_A

    build = get_architecture("Qwen3ForCausalLM").build
    build(Qwen3Config.from_dict(dict(TINY_A, head_dim=256)))
    with pytest.raises(ValueError, match="head_dim 272"):
        build(Qwen3Config.from_dict(dict(TINY_A, head_dim=272)))
    with pytest.raises(ConfigError, match="head_dim must be even"):
        Qwen3Config.from_dict(dict(TINY_A, head_dim=15))
