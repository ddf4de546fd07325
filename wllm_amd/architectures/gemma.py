"""Gemma 1 as a plan of parts.

Every layer is the same pre-norm block (src/wllm/models/gemma.py:83-93):
(1 + w) RMSNorm (gemma.py:41-51), attention with rotated queries and keys over
all earlier keys, scale 1/sqrt(head_dim) (src/wllm/models/llama.py:85-115,242),
(1 + w) RMSNorm, gelu-tanh gated feed-forward (gemma.py:54-62).  Embeddings are
multiplied by sqrt(hidden_size) held in the model's dtype (gemma.py:158-162,
llama.py:397,651); the head is the embedding table when tied (llama.py:443-446).
Tensor names are the checkpoint's (llama.py:1-4).
"""
from __future__ import annotations

import math

from wllm_amd.architectures.gemma_config import GemmaConfig
from wllm_amd.config.registry import register_architecture
from wllm_amd.parts.specs import (
    AttentionSpec,
    BlockSpec,
    EmbeddingSpec,
    GatedMLPSpec,
    HeadSpec,
    ModelPlan,
    NormSpec,
    PositionSpec,
    ScheduleEntry,
)


def gemma_plan(cfg: GemmaConfig) -> ModelPlan:
    def norm(name: str) -> NormSpec:
        return NormSpec(size=cfg.hidden_size, eps=cfg.rms_norm_eps, weight=name, weight_offset=1.0)

    layers = []
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}."
        a = p + "self_attn."
        bias = cfg.attention_bias
        layers.append(BlockSpec(
            arrangement="pre_norm",
            mixer=AttentionSpec(
                hidden_size=cfg.hidden_size,
                num_heads=cfg.num_attention_heads,
                num_kv_heads=cfg.num_key_value_heads,
                head_dim=cfg.head_dim,
                scale=1.0 / math.sqrt(cfg.head_dim),
                window=None,
                position=PositionSpec(kind="rope", rotary_dim=cfg.head_dim, theta=cfg.rope_theta, pairing="half"),
                q_weight=a + "q_proj.weight", k_weight=a + "k_proj.weight",
                v_weight=a + "v_proj.weight", o_weight=a + "o_proj.weight",
                q_bias=a + "q_proj.bias" if bias else None,
                k_bias=a + "k_proj.bias" if bias else None,
                v_bias=a + "v_proj.bias" if bias else None,
            ),
            feed_forward=GatedMLPSpec(
                hidden_size=cfg.hidden_size,
                intermediate_size=cfg.intermediate_size,
                activation="gelu_tanh",
                gate_weight=p + "mlp.gate_proj.weight",
                up_weight=p + "mlp.up_proj.weight",
                down_weight=p + "mlp.down_proj.weight",
            ),
            mixer_norm=norm(p + "input_layernorm.weight"),
            feed_forward_norm=norm(p + "post_attention_layernorm.weight"),
        ))
    return ModelPlan(
        embedding=EmbeddingSpec(
            vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size, weight="model.embed_tokens.weight",
            scale=math.sqrt(cfg.hidden_size), scale_in_model_dtype=True),
        layers=tuple(layers),
        schedule=tuple(ScheduleEntry(layer=i) for i in range(cfg.num_hidden_layers)),
        final_norm=norm("model.norm.weight"),
        head=HeadSpec(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size,
                      weight=None if cfg.tie_word_embeddings else "lm_head.weight",
                      tied_checkpoint_name="lm_head.weight"),
        max_positions=cfg.max_position_embeddings,
        # the rotation's frequencies are not persistent in the reference (llama.py:56);
        # checkpoints written by other tools sometimes carry them
        ignored_tensor_suffixes=("rotary_emb.inv_freq",),
    )


register_architecture("GemmaForCausalLM", GemmaConfig.from_dict, gemma_plan)
