"""The Qwen2.5 dense decoder assembled from parts (flow_engine/model.py:88-112).

Per layer: RMSNorm, grouped-query attention with q/k/v biases and no o bias,
rotate-half RoPE over the whole head, RMSNorm, SwiGLU; a final RMSNorm; a head
that is tied to the embedding when config.json says so. Tensor names are the
checkpoint's own (flow_engine/model.py:39-43,71-73,91-94,100-102,109-110).
"""
from __future__ import annotations

from ..config.model_config import Qwen2Config
from ..config.registry import register_architecture
from ..parts import (DecoderModel, GroupedQueryAttention, OutputHead, PreNormBlock, RMSNorm,
                     RotaryEmbedding, SwiGLU, TokenEmbedding)


def build_qwen2(config: Qwen2Config, packed=True):
    c = config
    rotary = RotaryEmbedding(c.head_dim, c.rope_theta)
    embedding = TokenEmbedding("model.embed_tokens", c.vocab_size, c.hidden_size)
    blocks = []
    for i in range(c.num_hidden_layers):
        p = f"model.layers.{i}."
        blocks.append(PreNormBlock(
            RMSNorm(p + "input_layernorm", c.hidden_size, c.rms_norm_eps),
            GroupedQueryAttention(p + "self_attn.", c.hidden_size, c.num_attention_heads,
                                  c.num_key_value_heads, c.head_dim, rotary, qkv_bias=c.attention_bias,
                                  o_bias=False, packed=packed),
            RMSNorm(p + "post_attention_layernorm", c.hidden_size, c.rms_norm_eps),
            SwiGLU(p + "mlp.", c.hidden_size, c.intermediate_size, packed=packed)))
    final_norm = RMSNorm("model.norm", c.hidden_size, c.rms_norm_eps)
    head = OutputHead("lm_head", c.vocab_size, c.hidden_size,
                      tied_to=embedding if c.tie_word_embeddings else None)
    return DecoderModel(c, embedding, blocks, final_norm, head)


register_architecture(Qwen2Config.ARCHITECTURE, Qwen2Config.MODEL_TYPE, Qwen2Config, build_qwen2, replace=True)
