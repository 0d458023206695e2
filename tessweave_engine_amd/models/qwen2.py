"""The Qwen2.5 dense decoder: its typed configuration and its model assembled from parts.

Configuration: the numbers config.json of a `Qwen2ForCausalLM` gives, with the reference's keys, defaults
and the rejections that must happen before any weight is read (flow_engine/config.py:23-52). Every size
and constant the model code uses comes from it; the parts take them as parameters.

Model (flow_engine/model.py:88-112), per layer: RMSNorm, grouped-query attention with q/k/v biases and no
o bias, rotate-half RoPE over the whole head, RMSNorm, SwiGLU; a final RMSNorm; a head that is tied to the
embedding when config.json says so. Tensor names are the checkpoint's own
(flow_engine/model.py:39-43,71-73,91-94,100-102,109-110).
"""
from __future__ import annotations

from dataclasses import asdict, dataclass

from ..config.model_config import ConfigError, eos_tuple
from ..config.registry import register_architecture
from ..parts import (DecoderModel, GroupedQueryAttention, OutputHead, PreNormBlock, RMSNorm,
                     RotaryEmbedding, SwiGLU, TokenEmbedding)


@dataclass(frozen=True)
class Qwen2Config:
    """The Qwen2.5 dense decoder's numbers (config.json of a `Qwen2ForCausalLM`).

    Defaults follow flow_engine/config.py:38-49: kv heads default to the query
    heads, head_dim to hidden/heads, rms_norm_eps 1e-6, rope_theta 10000, untied
    head; q/k/v biases are always on for qwen2 whatever `attention_bias` says
    (flow_engine/config.py:49).
    """
    architecture: str
    model_type: str
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float
    rope_theta: float
    max_position_embeddings: int
    tie_word_embeddings: bool
    attention_bias: bool
    eos_token_ids: tuple = ()

    ARCHITECTURE = "Qwen2ForCausalLM"
    MODEL_TYPE = "qwen2"

    @classmethod
    def from_dict(cls, d):
        if d.get("model_type") != cls.MODEL_TYPE:
            raise ConfigError(f"model_type {d.get('model_type')!r} is not {cls.MODEL_TYPE!r}")
        # Unsupported semantics are refused before any weight is read
        # (flow_engine/config.py:25-37).
        if d.get("quantization_config"):
            raise ConfigError("quantized checkpoints are not supported")
        scaling = d.get("rope_scaling")
        if scaling and scaling.get("rope_type", scaling.get("type")) != "default":
            raise ConfigError("scaled RoPE is not implemented; refusing a silent approximation")
        if d.get("use_sliding_window"):
            raise ConfigError("sliding-window attention is not enabled for this architecture")
        if d.get("hidden_act", "silu") != "silu" or d.get("mlp_bias"):
            raise ConfigError("only an unbiased SwiGLU (silu) feed-forward is supported")
        if d.get("num_local_experts") or d.get("num_experts") or d.get("auto_map"):
            raise ConfigError("experts and remote-code checkpoints are not supported")
        for key in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                    "num_attention_heads", "max_position_embeddings"):
            if key not in d:
                raise ConfigError(f"config.json lacks the required key {key!r}")
        hidden, heads = int(d["hidden_size"]), int(d["num_attention_heads"])
        if heads <= 0:
            raise ConfigError("num_attention_heads must be positive")
        kv_heads = int(d.get("num_key_value_heads") or heads)
        head_dim = int(d.get("head_dim") or hidden // heads)
        if min(hidden, kv_heads, head_dim) <= 0 or heads % kv_heads or hidden != heads * head_dim or head_dim % 2:
            raise ConfigError("invalid attention dimensions: need hidden == heads*head_dim, "
                              "heads % kv_heads == 0 and an even head_dim")
        cfg = cls(
            architecture=cls.ARCHITECTURE, model_type=d["model_type"],
            vocab_size=int(d["vocab_size"]), hidden_size=hidden,
            intermediate_size=int(d["intermediate_size"]),
            num_hidden_layers=int(d["num_hidden_layers"]),
            num_attention_heads=heads, num_key_value_heads=kv_heads, head_dim=head_dim,
            rms_norm_eps=float(d.get("rms_norm_eps", 1e-6)),
            rope_theta=float(d.get("rope_theta", 10000.0)),
            max_position_embeddings=int(d["max_position_embeddings"]),
            tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
            attention_bias=True,
            eos_token_ids=eos_tuple(d.get("eos_token_id")),
        )
        if min(cfg.vocab_size, cfg.intermediate_size, cfg.num_hidden_layers,
               cfg.max_position_embeddings) <= 0:
            raise ConfigError("model dimensions must be positive")
        if not cfg.rms_norm_eps > 0 or not cfg.rope_theta > 0:
            raise ConfigError("rms_norm_eps and rope_theta must be positive")
        return cfg

    def to_dict(self):
        """config.json contents that `from_dict` reads back to an equal object."""
        return {
            "architectures": [self.architecture], "model_type": self.model_type,
            "vocab_size": self.vocab_size, "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads, "head_dim": self.head_dim,
            "rms_norm_eps": self.rms_norm_eps, "rope_theta": self.rope_theta,
            "max_position_embeddings": self.max_position_embeddings,
            "tie_word_embeddings": self.tie_word_embeddings, "hidden_act": "silu",
            "use_sliding_window": False,
            "eos_token_id": list(self.eos_token_ids) if self.eos_token_ids else None,
        }

    def kv_bytes_per_token(self, element_bytes):
        """2 * layers * kv_heads * head_dim * bytes (flow_engine/config.py:64-65), over the checkpoint's head
        size. The device holds heads in multiples of 16 elements: what the cache really takes is
        `model.cache_layout().bytes_per_token`, which `inspect` prints beside this where the two differ."""
        return 2 * self.num_hidden_layers * self.num_key_value_heads * self.head_dim * element_bytes

    def describe(self):
        return asdict(self)



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
