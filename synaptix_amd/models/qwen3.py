"""The Qwen3 dense decoder put together from parts, and its entry in the registry.

Mapping as crates/synaptix-models/llm/qwen3/src/config.rs:89-125: plain norm gain, SiLU, no
sandwich norms, q/k norm with the layers' eps, scale 1/sqrt(head_dim), one rotation over the
whole head, every layer attends to all keys, no embedding or logit scale.
Tensor names: crates/synaptix-models/llm/common/src/model.rs:723,742,770,780-876.
"""
from __future__ import annotations

from ..config.qwen3 import Qwen3Config
from ..config.registry import register_architecture
from ..parts import RmsNorm, RotaryHalfSplit, GqaAttention, GatedMlp, PreNormBlock
from .decoder import DecoderModel, LayerRun, TokenEmbedding, OutputHead


def build_qwen3(cfg: Qwen3Config, max_positions: int | None = None) -> DecoderModel:
    capacity = max_positions or cfg.max_position_embeddings
    eps = cfg.eps_f32
    rope = RotaryHalfSplit(cfg.theta_f32, cfg.head_dim, capacity)   # one table shared by all layers
    embedding = TokenEmbedding("model.embed_tokens.weight", cfg.vocab_size, cfg.hidden_size)
    blocks = []
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}."
        blocks.append(PreNormBlock(
            RmsNorm(p + "input_layernorm.weight", cfg.hidden_size, eps),
            GqaAttention(p + "self_attn.", cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads,
                         cfg.head_dim, position=rope, qk_norm_eps=eps, window=None),
            RmsNorm(p + "post_attention_layernorm.weight", cfg.hidden_size, eps),
            GatedMlp(p + "mlp.", cfg.hidden_size, cfg.intermediate_size, cfg.hidden_act),
        ))
    schedule = [LayerRun(i, i) for i in range(cfg.num_hidden_layers)]
    final_norm = RmsNorm("model.norm.weight", cfg.hidden_size, eps)
    head = OutputHead("lm_head.weight", cfg.vocab_size, cfg.hidden_size,
                      tied_to=embedding if cfg.tie_word_embeddings else None)
    return DecoderModel(cfg, embedding, blocks, schedule, final_norm, head)


QWEN3 = register_architecture("Qwen3ForCausalLM", Qwen3Config, build_qwen3, model_types=("qwen3",))
