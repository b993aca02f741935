"""Configuration and registry (no GPU)."""
import json

import pytest

from synaptix_amd import Qwen3Config, ConfigError, load_config, known_architectures
from synaptix_amd.config import resolve_architecture
from helpers import TINY_A, TINY_B

# the JSON sample of the reference's own test (crates/synaptix-models/llm/qwen3/src/config.rs:168-193)
REFERENCE_JSON = """{
 "vocab_size": 151936, "hidden_size": 2048, "intermediate_size": 6144, "num_hidden_layers": 28,
 "num_attention_heads": 16, "num_key_value_heads": 8, "head_dim": 128, "max_position_embeddings": 40960,
 "rms_norm_eps": 1e-06, "rope_theta": 1000000, "hidden_act": "silu", "attention_bias": false,
 "bos_token_id": 151643, "eos_token_id": 151645, "tie_word_embeddings": true, "use_sliding_window": false,
 "sliding_window": null, "model_type": "qwen3"}"""


def test_reference_sample_and_defaults():
    cfg = Qwen3Config.from_dict(json.loads(REFERENCE_JSON))
    assert cfg.intermediate_size == 6144 and cfg.eos_token_id == 151645
    assert cfg == Qwen3Config()                       # the sample is the default model (config.rs:28-50)
    assert (cfg.q_total_dim, cfg.kv_total_dim, cfg.group_size) == (2048, 1024, 2)
    assert cfg.rope_theta == 1e6 and isinstance(cfg.rope_theta, float)


def test_head_dim_is_not_hidden_over_heads():
    cfg = Qwen3Config.from_dict(TINY_B)
    assert cfg.num_attention_heads * cfg.head_dim == 256 != cfg.hidden_size
    assert Qwen3Config.from_dict({"hidden_size": 2560, "num_attention_heads": 32}).head_dim == 128


@pytest.mark.parametrize("patch,needle", [
    ({"num_key_value_heads": 3}, "GQA"), ({"num_key_value_heads": 0}, "GQA"), ({"hidden_size": 0}, "hidden_size"),
    ({"head_dim": 0}, "head_dim"), ({"head_dim": 15}, "even"), ({"hidden_act": "gelu"}, "hidden_act"),
    ({"use_sliding_window": True}, "sliding"), ({"attention_bias": True}, "bias"), ({"vocab_size": 0}, "vocab_size"),
    ({"num_hidden_layers": 0}, "num_hidden_layers"), ({"rms_norm_eps": 0.0}, "rms_norm_eps"),
    ({"rope_theta": -1.0}, "rope_theta"), ({"hidden_size": "64"}, "hidden_size"), ({"eos_token_id": [1, 2]}, "eos_token_id"),
])
def test_invalid_configs_are_named(patch, needle):
    with pytest.raises(ConfigError, match=needle):
        Qwen3Config.from_dict({**TINY_A, **patch})


def test_registry(tmp_path):
    assert "Qwen3ForCausalLM" in known_architectures()
    assert resolve_architecture({"architectures": ["Qwen3ForCausalLM"]}).config_cls is Qwen3Config
    assert resolve_architecture({"model_type": "qwen3"}).name == "Qwen3ForCausalLM"
    with pytest.raises(ConfigError, match="unknown architecture 'LlamaForCausalLM'.*Qwen3ForCausalLM"):
        resolve_architecture({"architectures": ["LlamaForCausalLM"], "model_type": "qwen3"})
    with pytest.raises(ConfigError, match="unknown architecture"):
        resolve_architecture({})
    (tmp_path / "config.json").write_text(json.dumps({**TINY_A, "architectures": ["Qwen3ForCausalLM"], "extra": 1}))
    arch, cfg = load_config(str(tmp_path))
    assert cfg.hidden_size == 64 and cfg.rope_theta == 1e4 and arch.name == "Qwen3ForCausalLM"
    with pytest.raises(ConfigError, match="read"):
        load_config(str(tmp_path / "nowhere"))
    (tmp_path / "config.json").write_text("{ not json")
    with pytest.raises(ConfigError, match="parse"):
        load_config(str(tmp_path))


def test_round_trip_and_model_shape():
    cfg = Qwen3Config.from_dict(TINY_B)
    assert Qwen3Config.from_dict(cfg.to_dict()) == cfg
    model = resolve_architecture(cfg.to_dict()).build(cfg)
    specs = model.tensor_specs()
    assert len(specs) == 3 * 11 + 3                      # 11 a layer, embedding, final norm, lm_head
    assert specs["model.layers.2.self_attn.q_proj.weight"].shape == (256, 128)
    assert specs["model.layers.0.self_attn.k_norm.weight"].shape == (32,)
    assert specs["lm_head.weight"].shape == (1000, 128)
    tied = resolve_architecture({"model_type": "qwen3"}).build(Qwen3Config.from_dict(TINY_A))
    assert "lm_head.weight" not in tied.tensor_specs() and tied.ignored_tensors() == ["lm_head.weight"]
    assert [r.block for r in model.schedule] == [0, 1, 2] and model.n_caches == 3


def test_eps_and_theta_are_held_as_32_bit():
    import numpy as np
    cfg = Qwen3Config.from_dict({**TINY_A, "rms_norm_eps": 1e-6})
    assert cfg.eps_f32 == float(np.float32(1e-6)) != 1e-6


def test_a_feed_forward_names_its_activation_and_refuses_one_without_a_kernel():
    from synaptix_amd.parts import GatedMlp
    assert GatedMlp("x.", 64, 128, "silu").activation == "silu"
    with pytest.raises(ValueError, match="activation 'gelu_pytorch_tanh'"):
        GatedMlp("x.", 64, 128, "gelu_pytorch_tanh")
